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
