"""The training path driven through Boat's own C API on libboat_amd.so (GPU) and compared with the
oracle on the same seeded inputs -- the same scenarios that pin the oracle to the compiled
reference in test_oracle_vs_reference.py, so the chain GPU == oracle == reference closes.
"""
import ctypes as C

import numpy as np
import pytest

import boat_cases as bc
from oracle_lib import max_rel, rel_fro
from test_oracle_vs_reference import ATT_CASES, make_attention_inputs, oracle_mlp_steps

pytestmark = pytest.mark.gpu

TOL_EW, TOL_RED, TOL_GEMM = 1e-5, 1e-4, 1e-3


def test_known_answers_of_the_reference_unit_tests(boat):
    # tests/unit/test_autodiff.c:116-374
    c, da, db = bc.binary_grads(boat, "mul", [2, 3], [4, 5])
    assert c.tolist() == [8, 15] and da.tolist() == [4, 5] and db.tolist() == [2, 3]
    c, da, db = bc.binary_grads(boat, "div", [6, 12], [2, 3])
    assert da.tolist() == [0.5, np.float32(1 / 3)] and db.tolist() == [-1.5, np.float32(-12 / 9)]
    y, dx = bc.unary_grads(boat, "relu", [-1, 0, 2])
    assert y.tolist() == [0, 0, 2] and dx.tolist() == [0, 0, 1]
    c, da, db = bc.dot_grads(boat, [1, 2, 3], [4, 5, 6])
    assert c.tolist() == [32] and da.tolist() == [4, 5, 6] and db.tolist() == [1, 2, 3]
    c, da, db = bc.binary_grads(boat, "add", [1, 2], [3, 4])
    assert c.tolist() == [4, 6] and da.tolist() == [1, 1] and db.tolist() == [1, 1]
    c, da, db = bc.binary_grads(boat, "sub", [1, 2], [3, 4])
    assert da.tolist() == [1, 1] and db.tolist() == [-1, -1]
    # tests/test_dense_forward.c:79-91
    x = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    w = np.array([[0.1, 0.2], [0.3, 0.4], [0.5, 0.6]], np.float32)
    y = bc.dense_forward(boat, x, w, np.array([0.1, 0.2], np.float32))
    assert np.allclose(y, [[2.3, 3.0], [5.0, 6.6]], rtol=1e-6)


def test_variable_semantics(boat):
    t = boat.tensor(np.ones((2, 2), np.float32))
    v = boat.boat_variable_create(t, True)
    assert not boat.boat_variable_grad(v)                      # no gradient before backward (test_autodiff.c:20)
    boat.boat_variable_backward_full(v)
    assert np.all(boat.numpy(boat.boat_variable_grad(v)) == 1)
    boat.boat_variable_backward_full(v)                        # leaf gradients accumulate across calls
    assert np.all(boat.numpy(boat.boat_variable_grad(v)) == 2)
    boat.boat_variable_zero_grad(v)
    assert not boat.boat_variable_grad(v)                      # zero_grad drops the tensor (autodiff.c:285-292)
    g = boat.boat_hip_variable_ensure_grad(v)                  # persistent gradient buffer for optimizers
    boat.boat_variable_backward_full(v)
    boat.boat_variable_zero_grad(v)
    assert boat.boat_variable_grad(v) == g and not boat.numpy(g).any()
    nv = boat.boat_variable_create(t, False)
    boat.boat_variable_backward_full(nv)                       # silently ignored without requires_grad
    assert not boat.boat_variable_grad(nv)
    boat.boat_variable_free(v)
    boat.boat_variable_free(nv)
    boat.boat_tensor_unref(t)


@pytest.mark.parametrize("op", ["mul", "div", "add", "sub"])
def test_binary_grads(boat, oracle, rng, op):
    a = rng.standard_normal((5, 7)).astype(np.float32)
    b = (rng.standard_normal((5, 7)) + 3).astype(np.float32)
    dy = rng.standard_normal((5, 7)).astype(np.float32)
    _, da, db = bc.binary_grads(boat, op, a, b, dy)
    if op == "mul":
        wa, wb = oracle.mul_backward(a, b, dy)
    elif op == "div":
        wa, wb = oracle.div_backward(a, b, dy)
    else:
        wa, wb = dy, (dy if op == "add" else dy * np.float32(-1))
    assert np.array_equal(da, wa) and np.array_equal(db, wb)


@pytest.mark.parametrize("op", ["relu", "sigmoid", "tanh", "softmax", "log_softmax"])
def test_unary_grads(boat, oracle, rng, op):
    x = (2 * rng.standard_normal((6, 10))).astype(np.float32)
    dy = rng.standard_normal((6, 10)).astype(np.float32)
    y, dx = bc.unary_grads(boat, op, x, dy)
    wy = getattr(oracle, op + "_forward")(x)
    wdx = getattr(oracle, op + "_backward")(x if op == "relu" else wy, dy)
    assert np.max(np.abs(y - wy)) <= TOL_RED * max(1, np.abs(wy).max())
    assert np.max(np.abs(dx - wdx)) <= TOL_RED * max(1, np.abs(wdx).max())


def test_sum_and_matmul_grads(boat, oracle, rng):
    x = rng.standard_normal(1000).astype(np.float32)
    y, dx = bc.unary_grads(boat, "sum", x)
    assert abs(y[0] - oracle.sum(x)) <= TOL_RED * np.abs(x).sum() and np.all(dx == 1)
    a = rng.standard_normal((9, 12)).astype(np.float32)
    b = rng.standard_normal((12, 7)).astype(np.float32)
    dy = rng.standard_normal((9, 7)).astype(np.float32)
    c, da, db = bc.matmul_grads(boat, a, b, dy)
    assert rel_fro(c, oracle.matmul(a, b)) <= TOL_GEMM
    assert rel_fro(da, oracle.matmul(dy, oracle.transpose_last2(b))) <= TOL_GEMM
    assert rel_fro(db, oracle.matmul(oracle.transpose_last2(a), dy)) <= TOL_GEMM


def test_matmul_layouts_and_transpose(boat, oracle, rng):
    a = rng.standard_normal((2, 3, 5, 4)).astype(np.float32)
    b = rng.standard_normal((2, 3, 4, 6)).astype(np.float32)
    assert rel_fro(bc.matmul(boat, a, b), oracle.matmul(a, b)) <= TOL_GEMM
    assert np.array_equal(bc.transpose(boat, a, 2, 3), oracle.transpose_last2(a))
    m = rng.standard_normal((6, 11)).astype(np.float32)
    assert np.array_equal(bc.transpose(boat, m, 0, 1), m.T)


def test_fanout_gives_the_true_gradient(boat):
    """z = y + y, y = a*b.  The reference reports 4b (its recursion revisits y); each op is visited once here."""
    a, b = np.array([1.5, -2.0], np.float32), np.array([3.0, 0.5], np.float32)
    da, db = bc.fanout(boat, a, b)
    assert np.array_equal(da, 2 * b) and np.array_equal(db, 2 * a)


def test_dense_backward_accumulates(boat, oracle, rng):
    m, k, n = 9, 13, 6
    w = rng.standard_normal((k, n)).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    x1, x2 = (rng.standard_normal((m, k)).astype(np.float32) for _ in range(2))
    dy1, dy2 = (rng.standard_normal((m, n)).astype(np.float32) for _ in range(2))
    (dx1, gw1, gb1), (dx2, gw2, gb2) = bc.dense_backward_twice(boat, w, b, x1, dy1, x2, dy2)
    o1 = oracle.dense_backward(x1, w, dy1)
    o2 = oracle.dense_backward(x2, w, dy2, o1[1], o1[2])
    for got, want in zip((dx1, gw1, gb1, dx2, gw2, gb2), o1 + o2):
        assert rel_fro(got, want) <= TOL_GEMM


def test_zero_grad_keeps_its_meaning_when_the_zeros_are_never_written(boat, oracle, rng):
    """With pointers not kept, boat_optimizer_zero_grad clears a gradient by dropping its contents: the next backward
    writes it (the same numbers as adding to zeros, dense.c:255-291), a second backward adds, a reader in between sees
    zeros, and an optimizer step right after zero_grad uses zero gradients (adam.c:203-222)."""
    m, k, n = 12, 20, 7
    w = rng.standard_normal((k, n)).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    dy = rng.standard_normal((m, n)).astype(np.float32)
    _, gw, gb = oracle.dense_backward(x, w, dy)
    boat.boat_hip_set_coherent_pointers(0)
    try:
        layer = bc._make_dense(boat, w, b)
        opt = boat.boat_adam_optimizer_create(1e-2, 0.9, 0.999, 1e-8)
        tgw, tgb = boat.boat_dense_layer_get_grad_weight(layer), boat.boat_dense_layer_get_grad_bias(layer)
        boat.boat_optimizer_add_parameter(opt, boat.boat_dense_layer_get_weight(layer), tgw)
        boat.boat_optimizer_add_parameter(opt, boat.boat_dense_layer_get_bias(layer), tgb)
        tx, tdy = boat.tensor(x), boat.tensor(dy)

        def backward():
            ty = boat.boat_dense_layer_forward(layer, tx)
            tdx = boat.boat_dense_layer_backward(layer, tdy)
            boat.boat_tensor_unref(ty)
            boat.boat_tensor_unref(tdx)

        backward()
        boat.boat_optimizer_zero_grad(opt)
        backward()                                             # written, not added to stale contents
        assert rel_fro(boat.numpy(tgw), gw) <= TOL_GEMM and rel_fro(boat.numpy(tgb), gb) <= TOL_GEMM
        once_w, once_b = boat.numpy(tgw).copy(), boat.numpy(tgb).copy()
        backward()                                             # no zero_grad in between: accumulates
        assert np.array_equal(boat.numpy(tgw), once_w + once_w) and np.array_equal(boat.numpy(tgb), once_b + once_b)
        boat.boat_optimizer_zero_grad(opt)
        assert not boat.numpy(tgw).any() and not boat.numpy(tgb).any()      # a reader in between sees zeros
        backward()
        assert np.array_equal(boat.numpy(tgw), once_w) and np.array_equal(boat.numpy(tgb), once_b)
        boat.boat_optimizer_zero_grad(opt)
        before = boat.numpy(boat.boat_dense_layer_get_weight(layer)).copy()
        boat.boat_optimizer_step(opt)                          # a step on cleared gradients: m, v decay, the update is m/(sqrt(v)+eps)
        after = boat.numpy(boat.boat_dense_layer_get_weight(layer))
        assert np.isfinite(after).all() and np.abs(after - before).max() <= 1e-2 * 1.0001
        boat.boat_optimizer_zero_grad(opt)
        only_b = boat.numpy(tgb)                                # one of the pair looked at, the other still dropped
        assert not only_b.any()
        backward()
        assert np.array_equal(boat.numpy(tgw), once_w) and np.array_equal(boat.numpy(tgb), once_b)
        boat.boat_optimizer_free(opt)
        boat.boat_dense_layer_free(layer)
        boat.boat_tensor_unref(tx)
        boat.boat_tensor_unref(tdy)
    finally:
        boat.boat_hip_set_coherent_pointers(1)


def test_dense_error_paths(boat):
    layer = boat.boat_dense_layer_create(4, 3, True)
    bad = boat.tensor(np.zeros((2, 3), np.float32))
    assert not boat.boat_dense_layer_backward(layer, bad)              # no forward yet (dense.c:191)
    x = boat.tensor(np.zeros((2, 4), np.float32))
    y = boat.boat_dense_layer_forward(layer, x)
    wrong = boat.tensor(np.zeros((5, 3), np.float32))
    assert not boat.boat_dense_layer_backward(layer, wrong)            # batch mismatch (dense.c:212-217)
    assert not boat.boat_dense_layer_forward(layer, bad)               # wrong feature count
    assert not boat.boat_adam_optimizer_create(0.0, 0.9, 0.999, 1e-8)  # adam.c:45-53
    assert not boat.boat_adam_optimizer_create(0.1, 1.0, 0.999, 1e-8)
    assert not boat.boat_adam_optimizer_create(0.1, 0.9, 0.0, 1e-8)
    for t in (bad, x, y, wrong):
        boat.boat_tensor_unref(t)
    boat.boat_dense_layer_free(layer)


def test_loss_chain_recognised_on_the_tape_gives_the_op_by_op_bits(boat):
    """The example's loss chain (log_softmax, mul by the one-hot matrix, sum, mul by -1/B) at the root of a backward walk
    runs as one kernel that keeps the four gradient rules' operations: every gradient and updated parameter of the MLP step
    equals, bit for bit, what the op-by-op walk gives (reference-exact mode walks op by op; on a chain its results are the
    default walk's)."""
    rng = np.random.default_rng(99)
    x = rng.random((64, 784), dtype=np.float32)
    labels = rng.integers(0, 10, 64)
    w1 = rng.uniform(-0.08, 0.08, (784, 128)).astype(np.float32)
    w2 = rng.uniform(-0.2, 0.2, (128, 10)).astype(np.float32)
    b1, b2 = np.zeros(128, np.float32), np.zeros(10, np.float32)
    fused = bc.mlp_ce_adam(boat, x, labels, w1, b1, w2, b2, steps=2)
    boat.boat_hip_set_reference_exact(1)
    try:
        plain = bc.mlp_ce_adam(boat, x, labels, w1, b1, w2, b2, steps=2)
    finally:
        boat.boat_hip_set_reference_exact(0)
    for a, b in zip(fused, plain):
        for key in a:
            assert np.array_equal(a[key], b[key]), key


@pytest.mark.parametrize("dims,batch,steps", [((20, 16, 10), 8, 3), ((784, 128, 10), 64, 2)])
def test_mlp_ce_adam_training_steps(boat, oracle, dims, batch, steps):
    """Config 1: MLP 784->128->10, batch 64, forward + boat_variable_backward_full + Adam."""
    rng = np.random.default_rng(1234 + dims[0])
    d_in, d_h, d_out = dims
    x = rng.random((batch, d_in), dtype=np.float32)
    labels = rng.integers(0, d_out, batch)
    lim1, lim2 = np.sqrt(6.0 / (d_in + d_h)), np.sqrt(6.0 / (d_h + d_out))
    w1 = rng.uniform(-lim1, lim1, (d_in, d_h)).astype(np.float32)
    w2 = rng.uniform(-lim2, lim2, (d_h, d_out)).astype(np.float32)
    b1, b2 = np.zeros(d_h, np.float32), np.zeros(d_out, np.float32)
    hp = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8)
    got = bc.mlp_ce_adam(boat, x, labels, w1, b1, w2, b2, steps=steps, **hp)
    want = oracle_mlp_steps(oracle, x, labels, w1, b1, w2, b2, steps, **hp)
    g, w = got[0], want[0]
    assert abs(g["loss"] - w["loss"]) <= TOL_RED * abs(w["loss"])
    for key in ("gw1", "gw2"):
        assert rel_fro(g[key], w[key]) <= TOL_GEMM, key
    for key in ("gb1", "gb2"):
        assert np.max(np.abs(g[key] - w[key])) <= TOL_RED * max(1e-3, np.abs(w[key]).max()), key
    # Updated parameters.  The first Adam step moves every weight by ~lr*sign(g), so weights whose gradient is
    # pure rounding noise may flip; compare where the gradient is resolved and bound the rest by 2*lr.
    for t in range(steps):
        for key, gkey in (("w1", "gw1"), ("b1", "gb1"), ("w2", "gw2"), ("b2", "gb2")):
            diff = np.abs(got[t][key] - want[t][key])
            assert diff.max() <= 2.1e-3 * (t + 1), (t, key)
            resolved = np.abs(want[0][gkey]) > 1e-4 * np.abs(want[0][gkey]).max()
            if t == 0:
                assert np.max(diff[resolved]) <= 1e-5 * max(1.0, np.abs(want[t][key]).max()), (t, key)


def test_adam_trajectory_bit_exact(boat, oracle, rng):
    shapes = [(4, 3), (7,), (1,)]
    params = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    grads = [[(rng.standard_normal(s) * 10 ** rng.uniform(-4, 1)).astype(np.float32) for s in shapes] for _ in range(10)]
    got, zeroed = bc.adam_trajectory(boat, params, grads, lr=1e-2, lr_change=(5, 3e-3))
    p = [a.copy() for a in params]
    m = [np.zeros_like(a) for a in params]
    v = [np.zeros_like(a) for a in params]
    for t, gstep in enumerate(grads):
        lr = 3e-3 if t >= 5 else 1e-2
        for i in range(3):
            p[i], m[i], v[i] = oracle.adam_update(p[i], gstep[i], m[i], v[i], lr, 0.9, 0.999, 1e-8, t)
            assert np.array_equal(p[i].reshape(shapes[i]), got[t][i]), (t, i)
    assert all(not z.any() for z in zeroed)
    got, _ = bc.adam_trajectory(boat, [np.array([5.0], np.float32)], [[np.array([2.0], np.float32)]], lr=0.01)
    assert abs(float(got[0][0][0]) - 4.99) < 1e-6


@pytest.mark.parametrize("shape", [(2, 5, 48), (7, 64), (4, 768), (3, 2, 1024), (2, 3, 4, 16)])
def test_layernorm_forward(boat, oracle, rng, shape):
    x = rng.standard_normal(shape).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(shape[-1])).astype(np.float32)
    beta = (0.1 * rng.standard_normal(shape[-1])).astype(np.float32)
    y = bc.layernorm_forward(boat, x, gamma, beta, 1e-5)
    rows = shape[0] * shape[1] if len(shape) >= 3 else shape[0]      # rows the reference's loops visit (norm.c:279-281)
    flat = x.reshape(-1, shape[-1])
    want = np.zeros_like(flat)
    want[:rows] = oracle.layernorm_forward(flat[:rows], gamma, beta, 1e-5)[0]
    assert np.max(np.abs(y.reshape(want.shape) - want)) <= TOL_RED * np.abs(want).max()


def test_layernorm_backward_hook(boat, oracle, rng):
    """boat_layernorm_backward is a stub in the reference: checked against the float64 closed form."""
    from boat_amd.capi import LayerNormConfig
    x = rng.standard_normal((3, 5, 64)).astype(np.float32)
    dy = rng.standard_normal((3, 5, 64)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(64)).astype(np.float32)
    cfg = LayerNormConfig(64, 1e-5, True, True)
    norm = boat.boat_layernorm_create(C.byref(cfg))
    assert not boat.boat_layernorm_backward(norm, boat.tensor(dy))        # before forward: NULL
    boat.write(boat.boat_hip_layernorm_get_weight(norm), gamma)
    tx, tdy = boat.tensor(x), boat.tensor(dy)
    ty = boat.boat_layernorm_forward(norm, tx)
    _, mean, rstd = oracle.layernorm_forward(x, gamma, None, 1e-5)
    wdx, wdg, wdb = oracle.layernorm_backward_f64(x, gamma, dy, mean, rstd)
    for call in (1, 2):                                                   # parameter grads accumulate
        tdx = boat.boat_layernorm_backward(norm, tdy)
        assert np.max(np.abs(boat.numpy(tdx) - wdx)) <= TOL_RED * np.abs(wdx).max()
        assert np.max(np.abs(boat.numpy(boat.boat_hip_layernorm_get_grad_weight(norm)) - call * wdg)) <= call * TOL_RED * np.abs(wdg).max()
        assert np.max(np.abs(boat.numpy(boat.boat_hip_layernorm_get_grad_bias(norm)) - call * wdb)) <= call * TOL_RED * np.abs(wdb).max()
        boat.boat_tensor_unref(tdx)
    boat.boat_layernorm_free(norm)


def test_rmsnorm_layer_hooks(boat, oracle, rng):
    """boat_rmsnorm_*: forward as the reference (the oracle is bit-exact to it), backward and update implemented here
    (stubs there, norm.c:404-421) and checked against the float64 closed form; the stateless forms agree with the layer."""
    from boat_amd.capi import RmsNormConfig
    x = rng.standard_normal((3, 5, 64)).astype(np.float32)
    dy = rng.standard_normal((3, 5, 64)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(64)).astype(np.float32)
    assert not boat.boat_rmsnorm_create(C.byref(RmsNormConfig(0, 1e-6, True)))          # norm.c:137-139
    norm = boat.boat_rmsnorm_create(C.byref(RmsNormConfig(64, 1e-6, True)))
    tx, tdy = boat.tensor(x), boat.tensor(dy)
    assert not boat.boat_rmsnorm_backward(norm, tdy)                                      # before forward: NULL
    assert not boat.boat_rmsnorm_forward(norm, boat.tensor(np.zeros((2, 63), np.float32)))   # wrong width: NULL (norm.c:333-335)
    assert np.array_equal(boat.numpy(boat.boat_hip_rmsnorm_get_weight(norm)), np.ones(64, np.float32))
    boat.write(boat.boat_hip_rmsnorm_get_weight(norm), w)
    ty = boat.boat_rmsnorm_forward(norm, tx)
    wy, _ = oracle.rmsnorm_forward(x, w, 1e-6)
    assert np.max(np.abs(boat.numpy(ty) - wy)) <= TOL_RED * np.abs(wy).max()
    wdx, wdw = oracle.rmsnorm_backward_f64(x, w, dy, 1e-6)
    for call in (1, 2):                                                                   # the parameter gradient accumulates
        tdx = boat.boat_rmsnorm_backward(norm, tdy)
        assert np.max(np.abs(boat.numpy(tdx) - wdx)) <= TOL_RED * np.abs(wdx).max()
        got = boat.numpy(boat.boat_hip_rmsnorm_get_grad_weight(norm))
        assert np.max(np.abs(got - call * wdw)) <= call * TOL_RED * np.abs(wdw).max()
        boat.boat_tensor_unref(tdx)
    boat.boat_rmsnorm_update(norm, 0.5)                                                   # SGD step, then the gradient is cleared
    assert np.max(np.abs(boat.numpy(boat.boat_hip_rmsnorm_get_weight(norm)) - (w - 0.5 * 2 * wdw))) <= 1e-3
    assert not boat.numpy(boat.boat_hip_rmsnorm_get_grad_weight(norm)).any()
    boat.boat_rmsnorm_free(norm)
    # stateless forms: last dimension, no affine
    shape = (C.c_int64 * 1)(64)
    plain_y, _ = oracle.rmsnorm_forward(x, None, 1e-6)
    t = boat.boat_rms_norm(tx, shape, 1, 1e-6)
    assert np.max(np.abs(boat.numpy(t) - plain_y)) <= TOL_RED * np.abs(plain_y).max()
    tg = boat.boat_rms_norm_grad(tdy, tx, t, shape, 1, 1e-6)
    pdx, _ = oracle.rmsnorm_backward_f64(x, None, dy, 1e-6)
    assert np.max(np.abs(boat.numpy(tg) - pdx)) <= TOL_RED * np.abs(pdx).max()
    tl = boat.boat_layer_norm(tx, shape, 1, 1e-5)
    ly, _, _ = oracle.layernorm_forward(x, None, None, 1e-5)
    assert np.max(np.abs(boat.numpy(tl) - ly)) <= TOL_RED * np.abs(ly).max()
    assert not boat.boat_rms_norm(tx, shape, 2, 1e-6) and not boat.boat_layer_norm(None, shape, 1, 1e-5)
    for t_ in (t, tg, tl, ty, tx, tdy):
        boat.boat_tensor_unref(t_)


@pytest.mark.parametrize("shape,causal", [((2, 3, 16, 8), False), ((2, 2, 40, 16), True), ((2, 4, 128, 64), False), ((1, 2, 200, 64), True)])
def test_public_attention_core(boat, oracle, rng, shape, causal):
    """boat_scaled_dot_product_attention (attention.c:1082-1092) against the oracle's restatement of the same routine."""
    q, k, v = (rng.standard_normal(shape).astype(np.float32) for _ in range(3))
    scale = float(1.0 / np.sqrt(np.float32(shape[-1])))
    out = bc.sdpa_public(boat, q, k, v, scale, causal)
    want, _, _ = oracle.sdpa_forward(q, k, v, scale, causal)
    assert out.shape == shape and rel_fro(out, want) <= TOL_GEMM and np.max(np.abs(out - want)) <= 1e-5
    assert bc.sdpa_public(boat, q, k[:, :1], v, scale, causal) is None                    # shapes must agree (attention.c:929-933)


def test_multihead_attention_is_a_throwaway_layer(boat, rng):
    """boat_multihead_attention (attention.c:830-880) = create a layer with fresh rand() weights and bias, run self-attention,
    free it: with the generator seeded the same way it must equal that sequence done by hand."""
    import ctypes.util
    from boat_amd.capi import AttentionConfig
    libc = C.CDLL(ctypes.util.find_library("c"))
    x = rng.standard_normal((2, 12, 32)).astype(np.float32)
    tx = boat.tensor(x)
    libc.srand(1234)
    t = boat.boat_multihead_attention(tx, 4, 0.0, True, None)
    got = boat.numpy(t)
    libc.srand(1234)
    att = boat.boat_attention_create(C.byref(AttentionConfig(32, 4, 8, 0.0, True, True, False, 10000.0)))
    t2 = boat.boat_attention_forward(att, tx, tx, tx, None)
    assert got.shape == x.shape and np.array_equal(got, boat.numpy(t2))
    assert not boat.boat_multihead_attention(tx, 5, 0.0, False, None)                     # 32 % 5 != 0
    assert not boat.boat_multihead_attention(boat.tensor(x[0]), 4, 0.0, False, None)      # not 3-D
    boat.boat_attention_free(att)
    for t_ in (t, t2, tx):
        boat.boat_tensor_unref(t_)


def test_symbols_that_are_stubs_in_the_reference_too(boat, rng):
    """NULL / no effect in the reference (autodiff.c:595-603, attention.c:1094-1120, linear.c:409-413, activation.c:304-308,
    model.c:368-379), the same here; plus the small host-side helpers of the cited header ranges."""
    x = rng.standard_normal((2, 4, 8)).astype(np.float32)
    tx = boat.tensor(x)
    v = boat.boat_variable_create(tx, True)
    dims = (C.c_int64 * 1)(0)
    assert not boat.boat_var_max(v, dims, 1, False) and not boat.boat_var_min(v, dims, 1, False)
    assert not boat.boat_rotary_position_encoding(tx, 4, 8, 10000.0)
    boat.boat_apply_rotary_embedding(tx, tx, 4, 8, 10000.0)
    assert np.array_equal(boat.numpy(tx), x)
    assert not boat.boat_inverse(tx) and not boat.boat_selu(tx)
    assert not boat.boat_model_load(b"/nonexistent") 
    model = boat.boat_model_create()
    assert boat.boat_model_save(model, b"/tmp/never_written.boat") is False
    # user data travels with the model and its destructor runs once, at replacement or when the model is freed (model.c:382-397, 119-121)
    from boat_amd.capi import FREE_FN
    freed = []
    cb = FREE_FN(lambda p: freed.append(p))
    assert not boat.boat_model_get_user_data(model)
    boat.boat_model_set_user_data(model, 0x1000, cb)
    assert boat.boat_model_get_user_data(model) == 0x1000 and freed == []
    boat.boat_model_set_user_data(model, 0x2000, cb)
    assert freed == [0x1000]
    boat.boat_model_free(model)
    assert freed == [0x1000, 0x2000]
    g = boat.boat_graph_create()
    m2 = boat.boat_model_create_with_graph(g)
    assert boat.boat_model_graph(m2) == g and not boat.boat_model_create_with_graph(None)
    g2 = boat.boat_graph_create()
    boat.boat_model_set_graph(m2, g2)                                                     # frees g, owns g2
    assert boat.boat_model_graph(m2) == g2
    boat.boat_model_free(m2)
    # error state and aligned host blocks
    boat.boat_set_error(3, b"x")
    boat.boat_reset_error()
    assert boat.boat_get_last_error() == 0
    p = boat.boat_memory_allocate_aligned(100, 256, 0, b"t", 1)
    assert p and p % 256 == 0
    C.memset(p, 7, 100)
    boat.boat_memory_free_aligned(p)
    block = C.c_void_p(boat.boat_memory_allocate(64, 0, b"t", 2))
    boat.boat_memory_free_safe(C.byref(block))
    assert block.value is None
    boat.boat_memory_free_safe(C.byref(block))                                            # NULL inside: nothing happens
    boat.boat_variable_free(v)
    boat.boat_tensor_unref(tx)


@pytest.mark.parametrize("case", ATT_CASES, ids=lambda c: f"B{c['B']}S{c['S']}H{c['H']}{'c' if c['causal'] else ''}{'b' if c['bias'] else ''}")
def test_attention_layer(boat, oracle, case):
    xs, w, b, dys = make_attention_inputs(case, 99)
    out, results = bc.attention(boat, *xs, w, b, case["heads"], case["causal"], dys)
    o_out, cache = oracle.attention_forward(*xs, w, b, case["heads"], case["causal"])
    assert rel_fro(out, o_out) <= TOL_GEMM
    for dy, rec in zip(dys, results):
        g = oracle.attention_backward(*xs, w, b is not None, cache, dy, case["heads"])
        for got, want in ((rec["dq"], g["d_query"]), (rec["dk"], g["d_key"]), (rec["dv"], g["d_value"])):
            assert rel_fro(got, want) <= TOL_GEMM
        for n in "qkvo":
            assert rel_fro(rec["gw" + n], g["gw" + n]) <= TOL_GEMM, n
            if b is not None:
                assert rel_fro(rec["gb" + n], g["gb" + n]) <= TOL_GEMM, n


@pytest.mark.parametrize("causal", [False, True])
def test_attention_layer_with_and_without_score_cache(boat, oracle, causal):
    """Head size 64, 128 keys: the layer keeps the scaled scores of its forward pass and its backward kernel reads them
    (the reference keeps its attention weights, src/layers/attention.c:424-431, 584-598); with the limit at 0 the
    backward kernel recomputes Q.K^T.  Both against the oracle, and against each other to fp32 rounding."""
    case = dict(B=2, S=128, H=128, heads=2, causal=causal, bias=True)
    xs, w, b, dys = make_attention_inputs(case, 5)
    o_out, cache = oracle.attention_forward(*xs, w, b, 2, causal)
    runs = []
    for limit in (1 << 30, 0):
        boat.boat_hip_set_attention_score_cache_limit(limit)
        try:
            runs.append(bc.attention(boat, *xs, w, b, 2, causal, dys))
        finally:
            boat.boat_hip_set_attention_score_cache_limit(1 << 30)
    for out, results in runs:
        assert rel_fro(out, o_out) <= TOL_GEMM
        for dy, rec in zip(dys, results):
            g = oracle.attention_backward(*xs, w, True, cache, dy, 2)
            for got, want in ((rec["dq"], g["d_query"]), (rec["dk"], g["d_key"]), (rec["dv"], g["d_value"])):
                assert rel_fro(got, want) <= TOL_GEMM
    assert np.array_equal(runs[0][0], runs[1][0])                      # the forward arithmetic is the same
    for a, c in zip(runs[0][1], runs[1][1]):
        for key in ("dq", "dk", "dv", "gwq", "gwk", "gwv", "gwo"):
            assert rel_fro(a[key], c[key]) <= 2e-5, key


def test_attention_through_the_tape_self_attention(boat, oracle):
    """boat_var_attention(x, x, x): the three input gradients land in the same leaf (autodiff.c:2458-2532)."""
    case = dict(B=2, S=8, H=32, heads=4, causal=False, bias=True)
    xs, w, b, dys = make_attention_inputs(case, 7)
    x = xs[0]
    from boat_amd.capi import AttentionConfig
    cfg = AttentionConfig(32, 4, 8, 0.0, False, True, False, 10000.0)
    att = boat.boat_attention_create(C.byref(cfg))
    for n in "qkvo":
        boat.write(getattr(boat, f"boat_attention_get_weight_{n}")(att), w[n])
        boat.write(getattr(boat, f"boat_attention_get_bias_{n}")(att), b[n])
    tx = boat.tensor(x)
    vx = boat.boat_variable_create(tx, True)
    vy = boat.boat_var_attention(vx, vx, vx, att, None)
    tdy = boat.tensor(dys[0])
    boat.boat_variable_backward(vy, tdy)
    _, cache = oracle.attention_forward(x, x, x, w, b, 4, False)
    g = oracle.attention_backward(x, x, x, w, True, cache, dys[0], 4)
    want = g["d_query"] + g["d_key"] + g["d_value"]
    assert rel_fro(boat.numpy(boat.boat_variable_grad(vx)), want) <= TOL_GEMM
    boat.boat_variable_free(vy)
    boat.boat_variable_free(vx)
    boat.boat_attention_free(att)


def test_model_backward_over_layer_vtables(boat, oracle, rng):
    """boat_model_backward is a stub in the reference; here it walks layers[n-1..0] through ops->backward."""
    m, d_in, d_h, d_out = 16, 24, 32, 8
    x = rng.standard_normal((m, d_in)).astype(np.float32)
    dy = rng.standard_normal((m, d_out)).astype(np.float32)
    w1 = rng.standard_normal((d_in, d_h)).astype(np.float32) * 0.2
    w2 = rng.standard_normal((d_h, d_out)).astype(np.float32) * 0.2
    l1 = boat.boat_dense_layer_create(d_in, d_h, True)
    l2 = boat.boat_dense_layer_create(d_h, d_out, True)
    boat.write(boat.boat_dense_layer_get_weight(l1), w1)
    boat.write(boat.boat_dense_layer_get_weight(l2), w2)
    model = boat.boat_model_create()
    for layer in (boat.boat_hip_layer_from_dense(l1), boat.boat_hip_layer_relu(), boat.boat_hip_layer_from_dense(l2)):
        boat.boat_model_add_layer(model, layer)
    assert boat.boat_model_layer_count(model) == 3
    tx, tdy = boat.tensor(x), boat.tensor(dy)
    ty = boat.boat_model_forward(model, tx)
    tdx = boat.boat_model_backward(model, tdy)
    h = oracle.dense_forward(x, w1, np.zeros(d_h, np.float32))
    r = oracle.relu_forward(h)
    assert rel_fro(boat.numpy(ty), oracle.dense_forward(r, w2, np.zeros(d_out, np.float32))) <= TOL_GEMM
    dr, gw2, _ = oracle.dense_backward(r, w2, dy)
    dh = oracle.relu_backward(h, dr)
    dx, gw1, _ = oracle.dense_backward(x, w1, dh)
    assert rel_fro(boat.numpy(tdx), dx) <= TOL_GEMM
    assert rel_fro(boat.numpy(boat.boat_dense_layer_get_grad_weight(l1)), gw1) <= TOL_GEMM
    assert rel_fro(boat.numpy(boat.boat_dense_layer_get_grad_weight(l2)), gw2) <= TOL_GEMM
    boat.boat_model_update(model, 0.1)                                   # SGD step, gradients cleared (dense.c:297-329)
    assert rel_fro(boat.numpy(boat.boat_dense_layer_get_weight(l2)), w2 - np.float32(0.1) * gw2) <= TOL_GEMM
    assert not boat.numpy(boat.boat_dense_layer_get_grad_weight(l2)).any()
    boat.boat_model_free(model)


def test_relu_and_softmax_layer_hooks_pass_gradients_through(boat):
    # src/layers/relu.c:58-72, src/layers/softmax.c:43-58
    relu = boat.boat_relu_layer_create()
    g = boat.tensor(np.array([[-1.0, 2.0]], np.float32))
    back = boat.boat_relu_layer_backward(relu, g)
    assert back == g
    boat.boat_tensor_unref(back)
    sm = boat.boat_softmax_layer_create(-1)
    back = boat.boat_softmax_layer_backward(sm, g)
    assert back == g
    boat.boat_tensor_unref(back)
    y = boat.boat_relu_layer_forward(relu, g)
    assert boat.numpy(y).tolist() == [[0.0, 2.0]]
    boat.boat_relu_layer_free(relu)
    boat.boat_softmax_layer_free(sm)


def test_device_tensors_and_fused_losses(boat, oracle, rng):
    from boat_amd.capi import DEVICE_HIP
    a = rng.standard_normal((4, 6)).astype(np.float32)
    ta = boat.tensor(a, device=DEVICE_HIP)                               # lives in HBM only
    assert boat.boat_tensor_device(ta) == DEVICE_HIP
    tb = boat.boat_mul_scalar(ta, 2.0)
    assert boat.boat_tensor_device(tb) == DEVICE_HIP and np.array_equal(boat.numpy(tb), a * 2)
    cpu = boat.tensor(a)
    assert not boat.boat_add(ta, cpu)                                    # mixed devices refused (arithmetic.c:136-143)
    z = (2 * rng.standard_normal((8, 10))).astype(np.float32)
    labels = rng.integers(0, 10, 8).astype(np.int32)
    onehot = np.zeros((8, 10), np.float32)
    onehot[np.arange(8), labels] = 1
    dz = C.c_void_p()
    tl = boat.boat_hip_softmax_cross_entropy(boat.tensor(z), boat.tensor(labels), C.byref(dz))
    wl, wdz = oracle.ce_chain(z, onehot)
    assert abs(boat.numpy(tl)[0] - wl) <= TOL_RED * abs(wl) and np.max(np.abs(boat.numpy(dz) - wdz)) <= 1e-7
    p, t = rng.standard_normal((3, 5)).astype(np.float32), rng.standard_normal((3, 5)).astype(np.float32)
    gm = C.c_void_p()
    tl = boat.boat_hip_mse_loss(boat.tensor(p), boat.tensor(t), C.byref(gm))
    assert abs(boat.numpy(tl)[0] - oracle.mse_loss(p, t)) <= TOL_RED and np.array_equal(boat.numpy(gm), oracle.mse_grad(p, t))


# ---- convolution / pooling / flatten hooks and the MNIST CNN on the tape ----

def test_conv_known_answer_and_hooks(boat):
    # tests/test_conv_forward.c:20-165, weights injected with boat_conv_layer_set_weight as the reference's test does
    x = np.arange(1, 10, dtype=np.float32).reshape(1, 1, 3, 3)
    w = np.array([1, 0, 0, 1], np.float32).reshape(1, 1, 2, 2)
    for stride, pad, want_shape in ((1, 0, (1, 1, 2, 2)), (1, 1, (1, 1, 4, 4)), (2, 0, (1, 1, 1, 1))):
        layer = boat.boat_conv_layer_create(1, 1, 2, stride, pad)
        tw = boat.tensor(w)
        boat.boat_conv_layer_set_weight(layer, tw)
        boat.boat_tensor_unref(tw)
        tx = boat.tensor(x)
        ty = boat.boat_conv_layer_forward(layer, tx)
        y = boat.numpy(ty)
        assert y.shape == want_shape
        if pad == 0 and stride == 1:
            assert y.reshape(-1).tolist() == [6, 8, 12, 14]
        boat.boat_tensor_unref(ty)
        boat.boat_tensor_unref(tx)
        boat.boat_conv_layer_free(layer)
    # error paths: backward before forward, wrong rank, wrong channel count (conv.c:326-360, 475-500)
    layer = boat.boat_conv_layer_create(2, 3, 3, 1, 1)
    g = boat.tensor(np.zeros((1, 3, 4, 4), np.float32))
    with bc.scratch_cwd():
        assert not boat.boat_conv_layer_backward(layer, g)
        bad = boat.tensor(np.zeros((4, 4), np.float32))
        assert not boat.boat_conv_layer_forward(layer, bad)
        bad2 = boat.tensor(np.zeros((1, 5, 4, 4), np.float32))
        assert not boat.boat_conv_layer_forward(layer, bad2)
    for t in (g, bad, bad2):
        boat.boat_tensor_unref(t)
    assert not boat.boat_conv_layer_create(0, 3, 3, 1, 1)
    # gradient tensors keep their identity across backward calls, so an optimizer may hold them
    gw_before = boat.boat_conv_layer_get_grad_weight(layer)
    tx = boat.tensor(np.ones((1, 2, 4, 4), np.float32))
    ty = boat.boat_conv_layer_forward(layer, tx)
    tdy = boat.tensor(np.ones((1, 3, 4, 4), np.float32))
    for _ in range(2):
        boat.boat_tensor_unref(boat.boat_conv_layer_backward(layer, tdy))
    assert boat.boat_conv_layer_get_grad_weight(layer) == gw_before
    assert boat.numpy(boat.boat_conv_layer_get_grad_bias(layer)).tolist() == [16, 16, 16]       # overwritten, not doubled
    for t in (tdy, ty, tx):
        boat.boat_tensor_unref(t)
    boat.boat_conv_layer_free(layer)


def test_conv_forward_on_the_matrix_cores_is_opt_in(boat, oracle, rng):
    """boat_conv_layer_forward is bit-identical to the reference's loop order by default (src/layers/conv.c:326-437); after
    boat_hip_conv_forward_matrix_cores(1) a 3x3 layer wide enough to gain (here 16 -> 32 channels) runs as one MFMA
    contraction and agrees to fp32 rounding; layers the switch does not cover (few channels, other kernel sizes) stay
    bit-identical."""
    x = rng.standard_normal((4, 16, 10, 9)).astype(np.float32)
    w = (0.2 * rng.standard_normal((32, 16, 3, 3))).astype(np.float32)
    b = rng.standard_normal(32).astype(np.float32)
    want = oracle.conv2d_forward(x, w, b, 1, 1)
    y_default, _ = bc.conv_layer(boat, x, w, b, 1, 1, [])
    assert np.array_equal(y_default, want)
    x_small = rng.standard_normal((2, 3, 8, 8)).astype(np.float32)
    w_small = (0.2 * rng.standard_normal((5, 3, 3, 3))).astype(np.float32)
    b_small = rng.standard_normal(5).astype(np.float32)
    boat.boat_hip_conv_forward_matrix_cores(1)
    try:
        y_mfma, grads = bc.conv_layer(boat, x, w, b, 1, 1, [np.ones_like(want)])
        y_small, _ = bc.conv_layer(boat, x_small, w_small, b_small, 1, 1, [])
    finally:
        boat.boat_hip_conv_forward_matrix_cores(0)
    assert np.max(np.abs(y_mfma - want)) <= 1e-5 * np.abs(want).max()
    assert grads[0][2].tolist() == [4.0 * 10 * 9] * 32                      # the backward hooks are untouched
    assert not np.array_equal(y_mfma, want)                                # it did take the other kernel
    assert np.array_equal(y_small, oracle.conv2d_forward(x_small, w_small, b_small, 1, 1))
    y_again, _ = bc.conv_layer(boat, x, w, b, 1, 1, [])
    assert np.array_equal(y_again, want)


def test_flatten_layer_round_trip(boat, rng):
    x = rng.standard_normal((3, 2, 4, 5)).astype(np.float32)
    layer = boat.boat_flatten_layer_create()
    tx = boat.tensor(x)
    ty = boat.boat_flatten_layer_forward(layer, tx)
    assert boat.shape(ty) == (3, 40) and np.array_equal(boat.numpy(ty), x.reshape(3, 40))
    tb = boat.boat_flatten_layer_backward(layer, ty)
    assert boat.shape(tb) == x.shape and np.array_equal(boat.numpy(tb), x)
    for t in (tb, ty, tx):
        boat.boat_tensor_unref(t)
    boat.boat_flatten_layer_free(layer)


@pytest.mark.parametrize("size", ["small", "mnist"])
def test_cnn_chain_on_the_tape(boat, oracle, size):
    """conv-relu-pool x2, flatten, dense-relu-dense, cross-entropy chain (examples/mnist/mnist_autodiff.c:536-557)
    against the oracle: the reference's mirrored-tap input gradient with the switch on, the true gradient without."""
    from test_oracle_vs_reference import CNN_KEYS, cnn_params, oracle_cnn_grads
    rng = np.random.default_rng(2718)
    if size == "small":
        B, ic, c1, c2, side, hidden, classes = 3, 2, 4, 6, 8, 12, 5
    else:
        B, ic, c1, c2, side, hidden, classes = 8, 1, 32, 64, 28, 128, 10
    x = rng.random((B, ic, side, side), dtype=np.float32)
    labels = rng.integers(0, classes, B)
    p = cnn_params(rng, ic, c1, c2, side, hidden, classes)
    if size == "mnist":
        for k in ("cw2", "w1", "w2"):
            p[k] = (p[k] * 0.2).astype(np.float32)
    for flip in (True, False):
        boat.boat_hip_conv_reference_input_grad(int(flip))
        try:
            got = bc.cnn_ce_grads(boat, x, labels, p)
        finally:
            boat.boat_hip_conv_reference_input_grad(0)
        want = oracle_cnn_grads(oracle, x, labels, p, flip_taps=flip)
        assert abs(got["loss"] - want["loss"]) <= TOL_RED * abs(want["loss"])
        for key in CNN_KEYS:
            assert rel_fro(got[key], want[key]) <= TOL_GEMM, (key, flip)
            assert np.max(np.abs(got[key] - want[key])) <= 10 * TOL_RED * np.abs(want[key]).max(), (key, flip)


def test_cnn_training_with_registered_optimizer(boat):
    """Adam registered once with the layers' gradient tensors; three steps reduce the loss (the reference replaces the
    conv gradient tensors on every backward, conv.c:523-532, and would update from stale ones)."""
    rng = np.random.default_rng(99)
    B = 8
    x = rng.random((B, 1, 12, 12), dtype=np.float32)
    labels = rng.integers(0, 4, B)
    onehot = np.zeros((B, 4), np.float32)
    onehot[np.arange(B), labels] = 1
    conv = boat.boat_conv_layer_create(1, 4, 3, 1, 1)
    pool = boat.boat_pool_layer_create(2, 2, 0)
    dense = boat.boat_dense_layer_create(4 * 6 * 6, 4, True)
    opt = boat.boat_adam_optimizer_create(1e-2, 0.9, 0.999, 1e-8)
    boat.boat_hip_optimizer_add_conv(opt, conv)
    boat.boat_hip_optimizer_add_dense(opt, dense)
    losses = []
    for _ in range(4):
        vx = boat.boat_variable_create(tx := boat.tensor(x), True)
        a = boat.boat_var_conv(vx, conv)
        r = boat.boat_var_relu(a)
        q = boat.boat_var_pool(r, pool)
        f = boat.boat_var_flatten(q)
        z = boat.boat_var_dense(f, dense)
        ls = boat.boat_var_log_softmax(z, 1)
        voh = boat.boat_variable_create(toh := boat.tensor(onehot), False)
        m = boat.boat_var_mul(voh, ls)
        s = boat.boat_var_sum(m, None, 0, False)
        vf = boat.boat_variable_create(tf := boat.tensor(np.array([-1.0 / B], np.float32)), False)
        loss = boat.boat_var_mul(vf, s)
        losses.append(float(boat.numpy(boat.boat_variable_data(loss))[0]))
        boat.boat_optimizer_zero_grad(opt)
        with bc.scratch_cwd():
            boat.boat_variable_backward_full(loss)
        boat.boat_optimizer_step(opt)
        for v in (loss, vf, s, m, voh, ls, z, f, q, r, a, vx):
            boat.boat_variable_free(v)
        for t in (tx, toh, tf):
            boat.boat_tensor_unref(t)
    assert losses[-1] < losses[0], losses
    boat.boat_optimizer_free(opt)
    boat.boat_conv_layer_free(conv)
    boat.boat_pool_layer_free(pool)
    boat.boat_dense_layer_free(dense)


@pytest.mark.parametrize("kind", ["mse", "ce", "huber"])
@pytest.mark.parametrize("shape", [(7, 10), (64, 10), (3, 5, 1000), (1,)])
def test_loss_objects(boat, oracle, rng, kind, shape):
    if kind == "ce":
        pred = rng.random(shape, dtype=np.float32)
        pred.reshape(-1)[0] = 0.0
        target = (rng.random(shape) < 0.2).astype(np.float32)
    else:
        pred = (2 * rng.standard_normal(shape)).astype(np.float32)
        target = rng.standard_normal(shape).astype(np.float32)
    v1, v2 = bc.loss_values(boat, kind, pred, target, 0.75)
    want = oracle.loss_value(kind, pred, target, 0.75)
    assert v1 == v2 and abs(v1 - want) <= TOL_RED * max(abs(want), 1e-6)
    assert bc.loss_values(boat, "huber", pred, target, -1.0) is None
    # shape or dtype mismatch: 0 without a message (mse.c:49-68)
    loss = boat.boat_mse_loss_create()
    a, b = boat.tensor(np.zeros((2, 3), np.float32)), boat.tensor(np.ones((3, 2), np.float32))
    assert boat.boat_loss_compute(loss, a, b) == 0.0 and boat.boat_loss_compute(loss, a, None) == 0.0
    boat.boat_tensor_unref(a)
    boat.boat_tensor_unref(b)
    boat.boat_loss_free(loss)


def test_tape_listing_and_dot_export(boat, rng):
    a = bc._var(boat, rng.standard_normal((2, 3)).astype(np.float32), True)
    b = bc._var(boat, rng.standard_normal((2, 3)).astype(np.float32), True)
    c = boat.boat_var_mul(a, b)
    d = boat.boat_var_relu(c)
    e = boat.boat_var_sum(d, None, 0, False)
    dot = boat.boat_autodiff_graph_to_dot(e)
    text = C.string_at(dot).decode()
    C.CDLL(None).free(C.c_void_p(dot))
    assert text.startswith("digraph") and text.count("->") == 4 and "mul [2,3]" in text and "sum [1]" in text
    assert text.index("mul") < text.index("relu") < text.index("sum")       # recording order
    assert not boat.boat_autodiff_graph_to_dot(a) and not boat.boat_autodiff_graph_to_dot(None)
    boat.boat_autodiff_print_graph(e)
    boat.boat_autodiff_print_graph(None)
    boat.boat_autodiff_set_grad_checkpointing(True)
    for v in (e, d, c, b, a):
        boat.boat_variable_free(v)
