"""Randomised computation graphs with shared sub-expressions, built through Boat's tape API on the GPU library and
checked against float64 reverse-mode differentiation of the same graph written independently in numpy.

The reference's own backward walks depth first and counts a shared non-leaf node once per path
(src/autodiff.c:299-455); this library walks the tape in reverse topological order, so the values here are the true
gradients.  A float64 evaluation with explicit per-op adjoints (textbook formulas, nothing taken from the library)
is the checker; a wrong visiting order, a dropped accumulation or a wrong operand in any op's backward shows up in
at least one of the graphs.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

R, C = 6, 6          # every node is an R x C matrix, so any two nodes can meet in any binary op (matmul included)


def softmax64(x):
    e = np.exp(x - x.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


# name -> (arity, forward, adjoint(inputs, output, upstream) -> gradients of the inputs)
OPS = {
    "add": (2, lambda a, b: a + b, lambda i, y, g: (g, g)),
    "sub": (2, lambda a, b: a - b, lambda i, y, g: (g, -g)),
    "mul": (2, lambda a, b: a * b, lambda i, y, g: (g * i[1], g * i[0])),
    "matmul": (2, lambda a, b: a @ b, lambda i, y, g: (g @ i[1].T, i[0].T @ g)),
    "tanh": (1, np.tanh, lambda i, y, g: (g * (1 - y * y),)),
    "sigmoid": (1, lambda a: 1 / (1 + np.exp(-a)), lambda i, y, g: (g * y * (1 - y),)),
    "softmax": (1, softmax64, lambda i, y, g: (y * (g - (g * y).sum(-1, keepdims=True)),)),
    "log_softmax": (1, lambda a: np.log(softmax64(a)), lambda i, y, g: (g - np.exp(y) * g.sum(-1, keepdims=True),)),
    "gelu": (1, None, None),     # filled in below (needs erf)
}


def _erf(x):
    from math import erf
    return np.vectorize(erf)(x)


OPS["gelu"] = (1, lambda a: 0.5 * a * (1 + _erf(a / np.sqrt(2))),
               lambda i, y, g: (g * (0.5 * (1 + _erf(i[0] / np.sqrt(2))) + i[0] * np.exp(-0.5 * i[0] ** 2) / np.sqrt(2 * np.pi)),))

API_NAME = {"add": "boat_var_add", "sub": "boat_var_sub", "mul": "boat_var_mul", "matmul": "boat_var_matmul",
            "tanh": "boat_var_tanh", "sigmoid": "boat_var_sigmoid", "gelu": "boat_hip_var_gelu"}


def random_graph(rng, n_leaves, n_ops):
    """A list of (op, input node indices); node k < n_leaves is leaf k.  Later nodes pick any earlier node, so sub-graphs
    are shared freely; the last node is the output."""
    names = list(OPS)
    nodes = []
    for k in range(n_ops):
        op = names[int(rng.integers(len(names)))]
        have = n_leaves + k
        ins = tuple(int(rng.integers(have)) for _ in range(OPS[op][0]))
        nodes.append((op, ins))
    return nodes


def reference_gradients(leaves, nodes, seed_grad):
    vals = [x.astype(np.float64) for x in leaves]
    for op, ins in nodes:
        vals.append(OPS[op][1](*[vals[i] for i in ins]))
    adj = [np.zeros_like(v) for v in vals]
    adj[-1] = seed_grad.astype(np.float64)
    for k in range(len(nodes) - 1, -1, -1):
        op, ins = nodes[k]
        out = len(leaves) + k
        grads = OPS[op][2]([vals[i] for i in ins], vals[out], adj[out])
        for i, g in zip(ins, grads):
            adj[i] = adj[i] + g
    return vals[-1], adj[:len(leaves)]


def library_gradients(api, leaves, nodes, seed_grad):
    handles = []
    for x in leaves:
        t = api.tensor(x)
        handles.append(api.boat_variable_create(t, True))
        api.boat_tensor_unref(t)
    for op, ins in nodes:
        args = [handles[i] for i in ins]
        if op == "softmax":
            v = api.boat_var_softmax(args[0], -1)
        elif op == "log_softmax":
            v = api.boat_var_log_softmax(args[0], -1)
        else:
            v = getattr(api, API_NAME[op])(*args)
        assert v, op
        handles.append(v)
    out = api.numpy(api.boat_variable_data(handles[-1]))
    tg = api.tensor(seed_grad)
    api.boat_variable_backward(handles[-1], tg)
    api.boat_tensor_unref(tg)
    grads = []
    for h, x in zip(handles[:len(leaves)], leaves):
        g = api.boat_variable_grad(h)
        grads.append(api.numpy(g) if g else np.zeros_like(x))
    for h in reversed(handles):
        api.boat_variable_free(h)
    return out, grads


@pytest.mark.parametrize("seed", range(24))
def test_random_graph_gradients_match_float64_adjoints(boat, seed):
    rng = np.random.default_rng(1000 + seed)
    n_leaves, n_ops = int(rng.integers(2, 5)), int(rng.integers(3, 13))
    nodes = random_graph(rng, n_leaves, n_ops)
    leaves = [(0.6 * rng.standard_normal((R, C))).astype(np.float32) for _ in range(n_leaves)]
    seed_grad = rng.standard_normal((R, C)).astype(np.float32)
    want_out, want = reference_gradients(leaves, nodes, seed_grad)
    got_out, got = library_gradients(boat, leaves, nodes, seed_grad)
    scale = max(1.0, np.abs(want_out).max())
    assert np.abs(got_out - want_out).max() <= 2e-4 * scale, (seed, nodes)
    for k, (g, w) in enumerate(zip(got, want)):
        tol = 5e-4 * max(1.0, np.abs(w).max())
        assert np.abs(g - w).max() <= tol, (seed, k, nodes, float(np.abs(g - w).max()), float(np.abs(w).max()))


# ---- the same with dense layers and ReLU among the ops ----
# A dense layer's bias gradient is taken by the rule of the activation (or loss) that consumes its output when nothing else
# reads that output, and by the dense rule itself otherwise: random graphs put dense outputs in front of activations with
# and without a second reader, and the layers' own gradients (dW = x^T g, db = column sums of g) are checked as well.
def _dense_graph(rng, n_leaves, n_ops):
    names = list(OPS) + ["dense", "dense", "relu", "relu"]        # dense and relu drawn more often
    nodes = []
    for k in range(n_ops):
        op = names[int(rng.integers(len(names)))]
        have = n_leaves + k
        if op == "dense":
            w = (0.5 * rng.standard_normal((C, C))).astype(np.float32)
            b = (0.5 * rng.standard_normal(C)).astype(np.float32)
            nodes.append((op, (int(rng.integers(have)),), (w, b)))
        else:
            arity = 1 if op == "relu" else OPS[op][0]
            ins = [int(rng.integers(have)) for _ in range(arity)]
            dense_nodes = [n_leaves + j for j, nd in enumerate(nodes) if nd[0] == "dense"]
            if dense_nodes and rng.random() < 0.6:      # often straight behind a dense layer, as a first or a second reader
                ins[0] = dense_nodes[int(rng.integers(len(dense_nodes)))]
            nodes.append((op, tuple(ins), None))
    # every node that nobody reads is added to the output, so that all layers take part in the backward walk
    used = {i for _, ins, _ in nodes for i in ins}
    for k in range(len(nodes) - 1):
        if n_leaves + k not in used:
            nodes.append(("add", (n_leaves + k, n_leaves + len(nodes) - 1), None))
    return nodes


def _dense_reference(leaves, nodes, seed_grad):
    vals = [x.astype(np.float64) for x in leaves]
    for op, ins, par in nodes:
        a = [vals[i] for i in ins]
        if op == "dense":
            vals.append(a[0] @ par[0].astype(np.float64) + par[1].astype(np.float64))
        elif op == "relu":
            vals.append(np.maximum(a[0], 0.0))
        else:
            vals.append(OPS[op][1](*a))
    adj = [np.zeros_like(v) for v in vals]
    adj[-1] = seed_grad.astype(np.float64)
    layer_grads = {}
    for k in range(len(nodes) - 1, -1, -1):
        op, ins, par = nodes[k]
        out = len(leaves) + k
        a = [vals[i] for i in ins]
        if op == "dense":
            grads = (adj[out] @ par[0].astype(np.float64).T,)
            layer_grads[k] = (a[0].T @ adj[out], adj[out].sum(0))
        elif op == "relu":
            grads = (adj[out] * (a[0] > 0),)
        else:
            grads = OPS[op][2](a, vals[out], adj[out])
        for i, g in zip(ins, grads):
            adj[i] = adj[i] + g
    return vals[-1], adj[:len(leaves)], layer_grads


def _dense_library(api, leaves, nodes, seed_grad):
    handles, layers = [], {}
    for x in leaves:
        t = api.tensor(x)
        handles.append(api.boat_variable_create(t, True))
        api.boat_tensor_unref(t)
    for k, (op, ins, par) in enumerate(nodes):
        args = [handles[i] for i in ins]
        if op == "dense":
            layer = api.boat_dense_layer_create(C, C, True)
            api.write(api.boat_dense_layer_get_weight(layer), par[0])
            api.write(api.boat_dense_layer_get_bias(layer), par[1])
            layers[k] = layer
            v = api.boat_var_dense(args[0], layer)
        elif op == "relu":
            v = api.boat_var_relu(args[0])
        elif op == "softmax":
            v = api.boat_var_softmax(args[0], -1)
        elif op == "log_softmax":
            v = api.boat_var_log_softmax(args[0], -1)
        else:
            v = getattr(api, API_NAME[op])(*args)
        assert v, op
        handles.append(v)
    out = api.numpy(api.boat_variable_data(handles[-1]))
    tg = api.tensor(seed_grad)
    api.boat_variable_backward(handles[-1], tg)
    api.boat_tensor_unref(tg)
    grads = []
    for h, x in zip(handles[:len(leaves)], leaves):
        g = api.boat_variable_grad(h)
        grads.append(api.numpy(g) if g else np.zeros_like(x))
    layer_grads = {}
    for k, layer in layers.items():
        gw, gb = api.boat_dense_layer_get_grad_weight(layer), api.boat_dense_layer_get_grad_bias(layer)
        layer_grads[k] = (api.numpy(gw) if gw else np.zeros((C, C), np.float32), api.numpy(gb) if gb else np.zeros(C, np.float32))
    for h in reversed(handles):
        api.boat_variable_free(h)
    for layer in layers.values():
        api.boat_dense_layer_free(layer)
    return out, grads, layer_grads


@pytest.mark.parametrize("pointers_kept", [True, False])
@pytest.mark.parametrize("seed", range(30))
def test_random_graphs_with_dense_layers(boat, seed, pointers_kept):
    rng = np.random.default_rng(5000 + seed)
    n_leaves, n_ops = int(rng.integers(1, 4)), int(rng.integers(3, 13))
    nodes = _dense_graph(rng, n_leaves, n_ops)
    leaves = [(0.6 * rng.standard_normal((R, C))).astype(np.float32) for _ in range(n_leaves)]
    seed_grad = rng.standard_normal((R, C)).astype(np.float32)
    want_out, want, want_layers = _dense_reference(leaves, nodes, seed_grad)
    boat.boat_hip_set_coherent_pointers(1 if pointers_kept else 0)
    try:
        got_out, got, got_layers = _dense_library(boat, leaves, nodes, seed_grad)
    finally:
        boat.boat_hip_set_coherent_pointers(1)
    shape = [(op, ins) for op, ins, _ in nodes]
    assert np.abs(got_out - want_out).max() <= 2e-4 * max(1.0, np.abs(want_out).max()), (seed, shape)
    for k, (g, w) in enumerate(zip(got, want)):
        assert np.abs(g - w).max() <= 5e-4 * max(1.0, np.abs(w).max()), (seed, k, shape)
    reached = set()          # layers the output depends on: the others keep no gradient
    stack = [len(leaves) + len(nodes) - 1]
    while stack:
        n = stack.pop()
        if n < len(leaves) or n in reached:
            continue
        reached.add(n)
        stack.extend(nodes[n - len(leaves)][1])
    for k, (gw, gb) in got_layers.items():
        if len(leaves) + k not in reached:
            assert not gw.any() and not gb.any(), (seed, k, shape)
            continue
        ww, wb = want_layers[k]
        assert np.abs(gw - ww).max() <= 5e-4 * max(1.0, np.abs(ww).max()), (seed, k, "dW", shape)
        assert np.abs(gb - wb).max() <= 5e-4 * max(1.0, np.abs(wb).max()), (seed, k, "db", shape)
