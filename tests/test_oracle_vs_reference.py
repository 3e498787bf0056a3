"""Pins the oracle: every routine of oracle/boat_oracle.c must reproduce the compiled reference
(oracle/_ref/libboat_ref.so, built from the reference's own C sources) BIT FOR BIT on seeded
inputs, and the reference's own known-answer tests must hold for both.

Runs on the CPU.  Skipped when the reference library was not built (no reference tree); the
committed golden vectors (test_golden.py) then keep the same pins.
"""
import numpy as np
import pytest

import boat_cases as bc


def same(a, b):
    return a is not None and b is not None and a.shape == b.shape and np.array_equal(a, b)


# ---- known answers the reference's own tests assert (tests/unit/test_autodiff.c:116-374) ----

def test_known_answers_reference_unit_tests(ref, oracle):
    c, da, db = bc.binary_grads(ref, "mul", [2, 3], [4, 5])
    assert c.tolist() == [8, 15] and da.tolist() == [4, 5] and db.tolist() == [2, 3]
    o_da, o_db = oracle.mul_backward([2, 3], [4, 5], [1, 1])
    assert same(o_da, da) and same(o_db, db)

    c, da, db = bc.binary_grads(ref, "div", [6, 12], [2, 3])
    assert c.tolist() == [3, 4]
    assert da.tolist() == [0.5, np.float32(1 / 3)] and db.tolist() == [-1.5, np.float32(-12 / 9)]
    o_da, o_db = oracle.div_backward([6, 12], [2, 3], [1, 1])
    assert same(o_da, da) and same(o_db, db)

    y, dx = bc.unary_grads(ref, "relu", [-1, 0, 2])
    assert y.tolist() == [0, 0, 2] and dx.tolist() == [0, 0, 1]          # gradient at exactly 0 is 0
    assert same(oracle.relu_backward([-1, 0, 2], [1, 1, 1]), dx)

    c, da, db = bc.dot_grads(ref, [1, 2, 3], [4, 5, 6])
    assert c.tolist() == [32] and da.tolist() == [4, 5, 6] and db.tolist() == [1, 2, 3]

    c, da, db = bc.binary_grads(ref, "add", [1, 2], [3, 4])
    assert da.tolist() == [1, 1] and db.tolist() == [1, 1]
    c, da, db = bc.binary_grads(ref, "sub", [1, 2], [3, 4])
    assert da.tolist() == [1, 1] and db.tolist() == [-1, -1]


def test_known_answer_dense_forward(ref, oracle):
    # tests/test_dense_forward.c:79-91
    x = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    w = np.array([[0.1, 0.2], [0.3, 0.4], [0.5, 0.6]], np.float32)
    b = np.array([0.1, 0.2], np.float32)
    y_ref = bc.dense_forward(ref, x, w, b)
    assert np.allclose(y_ref, x.astype(np.float64) @ w.astype(np.float64) + b, rtol=1e-6)
    assert same(oracle.dense_forward(x, w, b), y_ref)


# ---- seeded bit-exact comparisons ----

@pytest.mark.parametrize("shape_a,shape_b", [((7, 5), (5, 9)), ((2, 3, 5, 4), (2, 3, 4, 6)), ((3, 8, 2), (3, 2, 5))])
def test_matmul_bit_exact(ref, oracle, rng, shape_a, shape_b):
    a = rng.standard_normal(shape_a).astype(np.float32)
    b = rng.standard_normal(shape_b).astype(np.float32)
    assert same(oracle.matmul(a, b), bc.matmul(ref, a, b))


def test_transpose_bit_exact(ref, oracle, rng):
    a = rng.standard_normal((6, 11)).astype(np.float32)
    assert same(oracle.transpose_last2(a), bc.transpose(ref, a, 0, 1))
    a4 = rng.standard_normal((2, 3, 5, 4)).astype(np.float32)
    assert same(oracle.transpose_last2(a4), bc.transpose(ref, a4, 2, 3))


@pytest.mark.parametrize("op", ["mul", "div"])
def test_binary_grads_bit_exact(ref, oracle, rng, op):
    a = rng.standard_normal((5, 7)).astype(np.float32)
    b = (rng.standard_normal((5, 7)) + 3.0).astype(np.float32)
    dy = rng.standard_normal((5, 7)).astype(np.float32)
    _, da, db = bc.binary_grads(ref, op, a, b, dy)
    o_da, o_db = (oracle.mul_backward if op == "mul" else oracle.div_backward)(a, b, dy)
    assert same(o_da, da) and same(o_db, db)


@pytest.mark.parametrize("op", ["relu", "sigmoid", "tanh"])
def test_activation_bit_exact(ref, oracle, rng, op):
    x = rng.standard_normal((5, 7)).astype(np.float32)
    x[0, :3] = [0.0, -0.0, 1e-30]
    dy = rng.standard_normal((5, 7)).astype(np.float32)
    y, dx = bc.unary_grads(ref, op, x, dy)
    o_y = getattr(oracle, op + "_forward")(x)
    assert same(o_y, y)
    saved = x if op == "relu" else y
    assert same(getattr(oracle, op + "_backward")(saved, dy), dx)


@pytest.mark.parametrize("shape", [(6, 10), (3, 33), (2, 4, 5)])
@pytest.mark.parametrize("op", ["softmax", "log_softmax"])
def test_softmax_family_bit_exact(ref, oracle, rng, op, shape):
    x = (3 * rng.standard_normal(shape)).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    y, dx = bc.unary_grads(ref, op, x, dy)
    assert same(getattr(oracle, op + "_forward")(x), y)
    assert same(getattr(oracle, op + "_backward")(y, dy), dx)
    # the invariant the reference's tests check (test_autodiff.c:393-397,437-441)
    p = y if op == "softmax" else np.exp(y)
    assert np.allclose(p.sum(-1), 1.0, atol=1e-5)


def test_sum_bit_exact(ref, oracle, rng):
    x = rng.standard_normal(1000).astype(np.float32)
    y, dx = bc.unary_grads(ref, "sum", x)
    assert y[0] == np.float32(oracle.sum(x)) and np.all(dx == 1.0)


def test_dense_backward_accumulates_bit_exact(ref, oracle, rng):
    m, k, n = 9, 13, 6
    w = rng.standard_normal((k, n)).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    x1, x2 = (rng.standard_normal((m, k)).astype(np.float32) for _ in range(2))
    dy1, dy2 = (rng.standard_normal((m, n)).astype(np.float32) for _ in range(2))
    (dx1, gw1, gb1), (dx2, gw2, gb2) = bc.dense_backward_twice(ref, w, b, x1, dy1, x2, dy2)
    o_dx1, o_gw1, o_gb1 = oracle.dense_backward(x1, w, dy1)
    o_dx2, o_gw2, o_gb2 = oracle.dense_backward(x2, w, dy2, o_gw1, o_gb1)
    assert same(o_dx1, dx1) and same(o_gw1, gw1) and same(o_gb1, gb1)
    assert same(o_dx2, dx2) and same(o_gw2, gw2) and same(o_gb2, gb2)
    # grads really accumulate (+=) across calls
    assert not np.array_equal(gw1, gw2)
    assert np.allclose(gb2, dy1.sum(0) + dy2.sum(0), rtol=1e-5, atol=1e-5)


def oracle_mlp_steps(oracle, x, labels, w1, b1, w2, b2, steps, lr, beta1, beta2, eps):
    """The config-1 step restated with oracle primitives."""
    B, classes = x.shape[0], w2.shape[1]
    onehot = np.zeros((B, classes), np.float32)
    onehot[np.arange(B), labels] = 1.0
    params = [w1.copy(), b1.copy(), w2.copy(), b2.copy()]
    m = [np.zeros_like(p) for p in params]
    v = [np.zeros_like(p) for p in params]
    hist = []
    for t in range(steps):
        w1_, b1_, w2_, b2_ = params
        h = oracle.dense_forward(x, w1_, b1_)
        r = oracle.relu_forward(h)
        z = oracle.dense_forward(r, w2_, b2_)
        loss, dz = oracle.ce_chain(z, onehot)
        dr, gw2, gb2 = oracle.dense_backward(r, w2_, dz)
        dh = oracle.relu_backward(h, dr)
        _, gw1, gb1 = oracle.dense_backward(x, w1_, dh)
        grads = [gw1, gb1, gw2, gb2]
        for i in range(4):
            p, mm, vv = oracle.adam_update(params[i], grads[i], m[i], v[i], lr, beta1, beta2, eps, t)
            params[i], m[i], v[i] = p.reshape(params[i].shape), mm.reshape(params[i].shape), vv.reshape(params[i].shape)
        hist.append(dict(loss=loss, gw1=gw1, gb1=gb1, gw2=gw2, gb2=gb2,
                         w1=params[0].copy(), b1=params[1].copy(), w2=params[2].copy(), b2=params[3].copy()))
    return hist


@pytest.mark.parametrize("dims,batch,steps", [((20, 16, 10), 8, 3), ((784, 128, 10), 64, 1)])
def test_mlp_ce_adam_steps_bit_exact(ref, oracle, dims, batch, steps):
    rng = np.random.default_rng(1234 + dims[0])
    d_in, d_h, d_out = dims
    x = rng.random((batch, d_in), dtype=np.float32)
    labels = rng.integers(0, d_out, batch)
    lim1, lim2 = np.sqrt(6.0 / (d_in + d_h)), np.sqrt(6.0 / (d_h + d_out))
    w1 = rng.uniform(-lim1, lim1, (d_in, d_h)).astype(np.float32)
    w2 = rng.uniform(-lim2, lim2, (d_h, d_out)).astype(np.float32)
    b1, b2 = np.zeros(d_h, np.float32), np.zeros(d_out, np.float32)
    hp = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8)
    got = bc.mlp_ce_adam(ref, x, labels, w1, b1, w2, b2, steps=steps, **hp)
    want = oracle_mlp_steps(oracle, x, labels, w1, b1, w2, b2, steps, **hp)
    for g, w in zip(got, want):
        assert np.float32(g["loss"]) == np.float32(w["loss"])
        for key in ("gw1", "gb1", "gw2", "gb2", "w1", "b1", "w2", "b2"):
            assert same(w[key], g[key]), key
    # sanity: the fused identity dlogits = (softmax - onehot)/B holds to rounding
    assert abs(got[0]["loss"] - np.log(d_out)) < 1.0


def test_adam_trajectory_bit_exact(ref, oracle, rng):
    shapes = [(4, 3), (7,), (1,)]
    params = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    grads = [[(rng.standard_normal(s) * 10 ** rng.uniform(-4, 1)).astype(np.float32) for s in shapes] for _ in range(10)]
    hp = dict(lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8)
    got, zeroed = bc.adam_trajectory(ref, params, grads, lr_change=(5, 3e-3), **hp)
    p = [a.copy() for a in params]
    m = [np.zeros_like(a) for a in params]
    v = [np.zeros_like(a) for a in params]
    for t, gstep in enumerate(grads):
        lr = 3e-3 if t >= 5 else 1e-2
        for i in range(3):
            pi, mi, vi = oracle.adam_update(p[i], gstep[i], m[i], v[i], lr, 0.9, 0.999, 1e-8, t)
            p[i], m[i], v[i] = pi, mi, vi
            assert same(p[i].reshape(shapes[i]), got[t][i]), (t, i)
    assert all(np.all(z == 0) for z in zeroed)


def oracle_sq_trajectory(oracle, kind, params, grads, lr, alpha, eps, lr_change=None):
    """RMSprop / Adagrad trajectories restated with the oracle: list over steps of lists of arrays."""
    p = [np.asarray(a, np.float32).copy() for a in params]
    st = [np.zeros_like(a) for a in p]
    out = []
    for t, gstep in enumerate(grads):
        if lr_change and t >= lr_change[0]:
            lr = lr_change[1]
        for i in range(len(p)):
            if kind == "rmsprop":
                pi, si = oracle.rmsprop_update(p[i], gstep[i], st[i], lr, alpha, eps)
            else:
                pi, si = oracle.adagrad_update(p[i], gstep[i], st[i], lr, eps)
            p[i], st[i] = pi.reshape(p[i].shape), si.reshape(p[i].shape)
        out.append([a.copy() for a in p])
    return out


@pytest.mark.parametrize("kind", ["rmsprop", "adagrad"])
def test_rmsprop_adagrad_trajectory_bit_exact(ref, oracle, rng, kind, capfd):
    # tests/unit/test_optimizer_rmsprop.c / test_optimizer_adagrad.c only assert "the parameter moved";
    # here whole trajectories of three tensors over ten steps, with a learning-rate change, must agree exactly
    shapes = [(4, 3), (7,), (1,)]
    params = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    grads = [[(rng.standard_normal(s) * 10 ** rng.uniform(-4, 1)).astype(np.float32) for s in shapes] for _ in range(10)]
    got, zeroed = bc.adam_trajectory(ref, params, grads, lr=1e-2, beta1=0.99, eps=1e-8, lr_change=(5, 3e-3), kind=kind)
    want = oracle_sq_trajectory(oracle, kind, params, grads, 1e-2, 0.99, 1e-8, lr_change=(5, 3e-3))
    for t in range(10):
        for i in range(3):
            assert same(want[t][i], got[t][i]), (t, i)
    assert all(np.all(z == 0) for z in zeroed)
    # closed form of the first step from zero state: RMSprop dp = -lr*g/(sqrt((1-a))*|g| + eps); Adagrad dp = -lr*g/(|g| + eps)
    g0, p0 = np.float64(grads[0][1]), np.float64(params[1])
    den = np.sqrt(1 - 0.99) * np.abs(g0) + 1e-8 if kind == "rmsprop" else np.abs(g0) + 1e-8
    assert np.allclose(got[0][1], p0 - 1e-2 * g0 / den, rtol=1e-5, atol=1e-7)
    # creation validation (rmsprop.c:33-57, adagrad.c:41-50)
    assert not ref.boat_rmsprop_optimizer_create(0.0, 0.9, 1e-8) and not ref.boat_rmsprop_optimizer_create(0.1, 1.0, 1e-8)
    assert not ref.boat_adagrad_optimizer_create(0.1, 0.0) and not ref.boat_adagrad_optimizer_create(-1.0, 1e-8)


def test_adam_first_step_closed_form(ref, oracle):
    # from m = v = 0: p -= lr*g/(|g|+eps)  =>  p=5, g=2, lr=.01 -> 4.99 (tests/unit/test_optimizer_adam.c:96-108)
    got, _ = bc.adam_trajectory(ref, [np.array([5.0], np.float32)], [[np.array([2.0], np.float32)]], lr=0.01)
    assert abs(float(got[0][0][0]) - 4.99) < 1e-6
    p, m, v = oracle.adam_update(np.array([5.0]), np.array([2.0]), np.zeros(1), np.zeros(1), 0.01, 0.9, 0.999, 1e-8, 0)
    assert same(p, got[0][0])
    # zero gradient leaves the parameter alone (:203-205)
    got, _ = bc.adam_trajectory(ref, [np.array([1.5], np.float32)], [[np.array([0.0], np.float32)]], lr=0.01)
    assert float(got[0][0][0]) == 1.5


@pytest.mark.parametrize("shape", [(2, 5, 48), (7, 64), (4, 768)])
def test_layernorm_forward_bit_exact(ref, oracle, rng, shape):
    x = rng.standard_normal(shape).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(shape[-1])).astype(np.float32)
    beta = (0.1 * rng.standard_normal(shape[-1])).astype(np.float32)
    y = bc.layernorm_forward(ref, x, gamma, beta, 1e-5)
    o_y, mean, rstd = oracle.layernorm_forward(x, gamma, beta, 1e-5)
    assert same(o_y, y)
    # closed form in float64
    xd = x.astype(np.float64)
    mu = xd.mean(-1, keepdims=True)
    var = xd.var(-1, keepdims=True)
    assert np.allclose(y, (xd - mu) / np.sqrt(var + 1e-5) * gamma + beta, atol=1e-5)
    assert np.allclose(mean, mu.ravel(), atol=1e-6) and np.allclose(rstd, 1 / np.sqrt(var.ravel() + 1e-5), rtol=1e-5)


def test_reference_ignores_a_contexts_disabled_grad_flag(ref):
    # src/autodiff.c:625-632 stores the flag; nothing reads it: the op is recorded and backward reaches the leaf
    a, b = np.array([1.5, -2.0], np.float32), np.array([3.0, 0.5], np.float32)
    assert same(bc.grad_under_disabled_context(ref, a, b), b)


@pytest.mark.parametrize("shape", [(2, 5, 48), (7, 64), (4, 768), (33,)])
def test_rmsnorm_forward_bit_exact(ref, oracle, rng, shape):
    # src/layers/norm.c:212-229,319-395: eps is added to the root, not under it
    x = (rng.standard_normal(shape) * 10 ** rng.uniform(-2, 1)).astype(np.float32)
    for eps, affine in ((1e-6, True), (1e-2, False)):
        y = bc.rmsnorm_forward(ref, x, eps, affine)
        o_y, inv = oracle.rmsnorm_forward(x, np.ones(shape[-1], np.float32) if affine else None, eps)
        assert same(o_y, y)
        xd = x.astype(np.float64).reshape(-1, shape[-1])
        want = xd / (np.sqrt((xd * xd).mean(-1, keepdims=True)) + eps)
        assert np.allclose(y.reshape(want.shape), want, rtol=2e-6, atol=1e-7)
        assert np.allclose(inv, 1 / (np.sqrt((xd * xd).mean(-1)) + eps), rtol=2e-6)
        # had eps been under the root the rows would differ by far more than rounding at eps = 1e-2
        wrong = xd / np.sqrt((xd * xd).mean(-1, keepdims=True) + eps)
        if eps == 1e-2:
            assert np.max(np.abs(wrong - want)) > 1e-4


def test_rmsnorm_rows_the_reference_visits(ref, oracle, rng):
    # norm.c:360-362: a 4-D input is treated as [shape0, shape1, hidden]: only the first shape0*shape1 rows are written
    x = rng.standard_normal((2, 3, 2, 8)).astype(np.float32)
    y = bc.rmsnorm_forward(ref, x, 1e-6)
    o_y, _ = oracle.rmsnorm_forward(x.reshape(-1, 8)[:6], np.ones(8, np.float32), 1e-6)
    assert same(y.reshape(-1, 8)[:6], o_y) and not y.reshape(-1, 8)[6:].any()


@pytest.mark.parametrize("shape,causal", [((2, 3, 16, 8), False), ((1, 2, 40, 16), True), ((1, 1, 5, 4), True)])
def test_public_sdpa_bit_exact(ref, oracle, rng, shape, causal):
    # boat_scaled_dot_product_attention (attention.c:1082-1092) is the routine the layer's forward runs per head
    q, k, v = (rng.standard_normal(shape).astype(np.float32) for _ in range(3))
    scale = float(1.0 / np.sqrt(np.float32(shape[-1])))
    out = bc.sdpa_public(ref, q, k, v, scale, causal)
    o_out, _, attn = oracle.sdpa_forward(q, k, v, scale, causal)
    assert same(o_out, out)
    # textbook softmax(scale*QK^T)V in float64
    sc = np.einsum("bhid,bhjd->bhij", q.astype(np.float64), k.astype(np.float64)) * scale
    if causal:
        sc = np.where(np.triu(np.ones(sc.shape[-2:], bool), 1), -np.inf, sc)
    pr = np.exp(sc - sc.max(-1, keepdims=True))
    pr /= pr.sum(-1, keepdims=True)
    assert np.allclose(out, pr @ v.astype(np.float64), atol=2e-6)
    # operands that are not 4-D come back as a copy of value (attention.c:905-917)
    assert same(bc.sdpa_public(ref, q[0], k[0], v[0], scale, causal), v[0])


def test_layernorm_pattern_input(ref, oracle):
    # tests/test_layernorm_simple.c: pattern (i % 10) * 0.1, H = 768, eps 1e-5
    x = ((np.arange(2 * 3 * 768) % 10) * 0.1).astype(np.float32).reshape(2, 3, 768)
    y = bc.layernorm_forward(ref, x, np.ones(768, np.float32), np.zeros(768, np.float32), 1e-5)
    o_y, _, _ = oracle.layernorm_forward(x, np.ones(768, np.float32), np.zeros(768, np.float32), 1e-5)
    assert same(o_y, y)
    assert np.allclose(y.mean(-1), 0, atol=1e-5) and np.allclose(y.var(-1), 1, atol=1e-3)


ATT_CASES = [
    dict(B=2, S=4, H=32, heads=4, causal=False, bias=True),    # tests/unit/test_attention_gradient_check.c config
    dict(B=2, S=4, H=32, heads=4, causal=True, bias=True),
    dict(B=1, S=16, H=64, heads=4, causal=False, bias=False),
    dict(B=1, S=16, H=64, heads=4, causal=True, bias=True),
    dict(B=2, S=70, H=96, heads=3, causal=True, bias=True),     # head size 32 from 64 keys on: the GEMM-based device path
    dict(B=1, S=40, H=128, heads=2, causal=False, bias=True),   # head size 64, 40 keys: the fused device kernels, ragged length
]


def make_attention_inputs(case, seed):
    rng = np.random.default_rng(seed)
    B, S, H = case["B"], case["S"], case["H"]
    xs = [rng.standard_normal((B, S, H)).astype(np.float32) for _ in range(3)]
    w = {n: (rng.standard_normal((H, H)) / np.sqrt(H)).astype(np.float32) for n in "qkvo"}
    b = {n: (0.1 * rng.standard_normal(H)).astype(np.float32) for n in "qkvo"} if case["bias"] else None
    dys = [rng.standard_normal((B, S, H)).astype(np.float32) for _ in range(2)]
    return xs, w, b, dys


@pytest.mark.parametrize("case", ATT_CASES, ids=lambda c: f"B{c['B']}S{c['S']}H{c['H']}{'c' if c['causal'] else ''}{'b' if c['bias'] else ''}")
def test_attention_layer_bit_exact(ref, oracle, case):
    xs, w, b, dys = make_attention_inputs(case, 99)
    out, results = bc.attention(ref, *xs, w, b, case["heads"], case["causal"], dys)
    o_out, cache = oracle.attention_forward(*xs, w, b, case["heads"], case["causal"])
    assert same(o_out, out)
    for dy, rec in zip(dys, results):          # second call: parameter grads overwritten, not accumulated
        g = oracle.attention_backward(*xs, w, b is not None, cache, dy, case["heads"])
        assert same(g["d_query"], rec["dq"]) and same(g["d_key"], rec["dk"]) and same(g["d_value"], rec["dv"])
        for n in "qkvo":
            assert same(g["gw" + n], rec["gw" + n]), n
            if b is not None:
                assert same(g["gb" + n], rec["gb" + n]), n


def test_sdpa_core_via_identity_projections(ref, oracle):
    """With W = I and no bias the layer is bare SDPA on the reshaped [B*nh, S, hd] blocks: pins the
    head split (plain reshape, no transpose), the scale on the scores and the double row-dot."""
    B, S, H, heads = 1, 8, 16, 2
    rng = np.random.default_rng(5)
    xs = [rng.standard_normal((B, S, H)).astype(np.float32) for _ in range(3)]
    eye = {n: np.eye(H, dtype=np.float32) for n in "qkvo"}
    dy = rng.standard_normal((B, S, H)).astype(np.float32)
    out, (rec,) = bc.attention(ref, *xs, eye, None, heads, False, [dy])
    hd = H // heads
    q, k, v = (x.reshape(B * heads, S, hd) for x in xs)       # the reference's reshape, not a head transpose
    scale = np.float32(1.0) / np.sqrt(np.float32(hd))
    o, lse, attn = oracle.sdpa_forward(q, k, v, scale)
    assert same(o.reshape(B, S, H), out)
    dq, dk, dv = oracle.sdpa_backward(q, k, v, attn, dy.reshape(B * heads, S, hd), scale)
    assert same(dq.reshape(B, S, H), rec["dq"]) and same(dk.reshape(B, S, H), rec["dk"]) and same(dv.reshape(B, S, H), rec["dv"])
    # textbook SDPA backward in float64 on each contiguous block
    qd, kd, vd, gd = (a.astype(np.float64) for a in (q, k, v, dy.reshape(B * heads, S, hd)))
    sc = np.einsum("bid,bjd->bij", qd, kd) / np.sqrt(hd)
    p = np.exp(sc - sc.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    dp = np.einsum("bid,bjd->bij", gd, vd)
    ds = p * (dp - (dp * p).sum(-1, keepdims=True)) / np.sqrt(hd)
    assert np.allclose(dq, np.einsum("bij,bjd->bid", ds, kd), atol=1e-5)
    assert np.allclose(dk, np.einsum("bij,bid->bjd", ds, qd), atol=1e-5)
    assert np.allclose(dv, np.einsum("bij,bid->bjd", p, gd), atol=1e-5)
    assert np.allclose(lse, np.log(np.exp(sc).sum(-1)), atol=1e-5)


def test_fanout_divergence_is_documented(ref):
    """z = y + y, y = a*b: the reference's depth-first recursion visits y once per consumer and
    reports dz/da = 4b; the true gradient is 2b.  Recorded as a known reference behaviour."""
    a, b = np.array([1.5, -2.0], np.float32), np.array([3.0, 0.5], np.float32)
    da, db = bc.fanout(ref, a, b)
    assert np.array_equal(da, 4 * b) and np.array_equal(db, 4 * a)


# ---- convolution / max pooling / the MNIST CNN chain (src/layers/conv.c, pool.c, flatten.c) ----

def test_known_answer_conv_forward(ref, oracle):
    # tests/test_conv_forward.c:20-91: 3x3 ramp image, 2x2 kernel [[1,0],[0,1]], zero bias -> [6, 8, 12, 14]
    x = np.arange(1, 10, dtype=np.float32).reshape(1, 1, 3, 3)
    w = np.array([1, 0, 0, 1], np.float32).reshape(1, 1, 2, 2)
    b = np.zeros(1, np.float32)
    y, _ = bc.conv_layer(ref, x, w, b, 1, 0, [])
    assert y.reshape(-1).tolist() == [6, 8, 12, 14]
    assert same(oracle.conv2d_forward(x, w, b, 1, 0), y)
    # :93-165: padding 1 gives 4x4, stride 2 gives 1x1
    assert bc.conv_layer(ref, x, w, b, 1, 1, [])[0].shape == (1, 1, 4, 4)
    assert bc.conv_layer(ref, x, w, b, 2, 0, [])[0].shape == (1, 1, 1, 1)
    assert oracle.conv2d_forward(x, w, b, 1, 1).shape == (1, 1, 4, 4)
    assert oracle.conv2d_forward(x, w, b, 2, 0).shape == (1, 1, 1, 1)


CONV_CASES = [  # B, ic, h, w, oc, k, stride, pad
    (2, 3, 7, 6, 4, 3, 1, 1),
    (3, 1, 8, 8, 5, 3, 1, 0),
    (2, 2, 9, 7, 3, 2, 2, 1),
    (1, 4, 5, 5, 2, 5, 1, 2),
    (2, 3, 10, 10, 2, 3, 3, 0),
]


def conv_inputs(case, seed):
    B, ic, h, w, oc, k, stride, pad = case
    rng = np.random.default_rng(seed)
    ho, wo = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    return dict(x=rng.standard_normal((B, ic, h, w)).astype(np.float32),
                w=(0.3 * rng.standard_normal((oc, ic, k, k))).astype(np.float32),
                b=rng.standard_normal(oc).astype(np.float32),
                dy1=rng.standard_normal((B, oc, ho, wo)).astype(np.float32),
                dy2=rng.standard_normal((B, oc, ho, wo)).astype(np.float32))


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(map(str, c)))
def test_conv_layer_bit_exact(ref, oracle, case):
    stride, pad = case[6], case[7]
    d = conv_inputs(case, 77)
    y, calls = bc.conv_layer(ref, d["x"], d["w"], d["b"], stride, pad, [d["dy1"], d["dy2"]])
    assert same(oracle.conv2d_forward(d["x"], d["w"], d["b"], stride, pad), y)
    for dy, (dx, gw, gb) in zip((d["dy1"], d["dy2"]), calls):
        o_dx, o_gw, o_gb = oracle.conv2d_backward(d["x"], d["w"], dy, stride, pad, flip_taps=True)
        assert same(o_dx, dx) and same(o_gw, gw) and same(o_gb, gb)
    # parameter gradients are overwritten, not accumulated, by the second call (conv.c:523-532)
    assert not np.array_equal(calls[0][1], calls[1][1])


def conv_f64(x, w, b, stride, pad):
    """Textbook cross-correlation in float64 from numpy slices (independent of the oracle's loops)."""
    x, w = x.astype(np.float64), w.astype(np.float64)
    B, ic, h, wd = x.shape
    oc, _, k, _ = w.shape
    ho, wo = (h + 2 * pad - k) // stride + 1, (wd + 2 * pad - k) // stride + 1
    xp = np.zeros((B, ic, h + 2 * pad, wd + 2 * pad))
    xp[:, :, pad:pad + h, pad:pad + wd] = x
    y = np.zeros((B, oc, ho, wo))
    for kh in range(k):
        for kw in range(k):
            patch = xp[:, :, kh:kh + stride * ho:stride, kw:kw + stride * wo:stride]
            y += np.einsum("bchw,oc->bohw", patch, w[:, :, kh, kw])
    return y + (0 if b is None else b.astype(np.float64)[None, :, None, None])


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(map(str, c)))
def test_conv_true_gradients_float64(oracle, case):
    """flip_taps=False is the gradient of the forward: adjoint identities against an independent float64 forward.
    <conv(u; w), dy> = <u, dx(dy)> for any u, and <conv(x; q), dy> = <q, gw(dy)> for any q (conv is bilinear)."""
    stride, pad = case[6], case[7]
    d = conv_inputs(case, 78)
    dx, gw, gb = oracle.conv2d_backward(d["x"], d["w"], d["dy1"], stride, pad, flip_taps=False)
    rng = np.random.default_rng(5)
    dy = d["dy1"].astype(np.float64)
    assert np.allclose(oracle.conv2d_forward(d["x"], d["w"], d["b"], stride, pad), conv_f64(d["x"], d["w"], d["b"], stride, pad),
                       rtol=1e-5, atol=1e-5)
    for _ in range(3):
        u = rng.standard_normal(d["x"].shape)
        q = rng.standard_normal(d["w"].shape)
        lhs_x = np.sum(conv_f64(u, d["w"], None, stride, pad) * dy)
        lhs_w = np.sum(conv_f64(d["x"], q, None, stride, pad) * dy)
        assert abs(lhs_x - np.sum(u * dx)) <= 1e-4 * (abs(lhs_x) + 1)
        assert abs(lhs_w - np.sum(q * gw)) <= 1e-4 * (abs(lhs_w) + 1)
    assert np.allclose(gb, dy.sum((0, 2, 3)), rtol=1e-5, atol=1e-5)
    # unit probes: dx at one input element equals the directional derivative along that element
    u = np.zeros(d["x"].shape)
    u[0, 0, 1, 2] = 1.0
    assert abs(np.sum(conv_f64(u, d["w"], None, stride, pad) * dy) - dx[0, 0, 1, 2]) <= 1e-4 * (abs(dx[0, 0, 1, 2]) + 1)
    # the reference's pairing is a different operator whenever the kernel is not symmetric under a 180 degree turn
    dx_flip = oracle.conv2d_backward(d["x"], d["w"], d["dy1"], stride, pad, flip_taps=True)[0]
    assert not np.allclose(dx_flip, dx, rtol=1e-3, atol=1e-3)
    turned = np.ascontiguousarray(d["w"][:, :, ::-1, ::-1])
    assert same(oracle.conv2d_backward(d["x"], turned, d["dy1"], stride, pad, flip_taps=False)[0], dx_flip)


POOL_CASES = [  # B, ch, h, w, pool, stride, pad
    (2, 3, 8, 8, 2, 2, 0),
    (1, 2, 7, 9, 3, 2, 1),
    (2, 1, 6, 6, 3, 1, 0),     # overlapping windows: several outputs route to one input
    (1, 2, 5, 5, 2, 2, 1),
]


@pytest.mark.parametrize("case", POOL_CASES, ids=lambda c: "x".join(map(str, c)))
def test_pool_layer_bit_exact(ref, oracle, case):
    B, ch, h, w, pool, stride, pad = case
    rng = np.random.default_rng(91)
    x = rng.standard_normal((B, ch, h, w)).astype(np.float32)
    x[0, 0, :2, :2] = 1.5                     # a tie: the first maximum in scan order wins
    ho, wo = (h + 2 * pad - pool) // stride + 1, (w + 2 * pad - pool) // stride + 1
    dy = rng.standard_normal((B, ch, ho, wo)).astype(np.float32)
    y, dx = bc.pool_layer(ref, x, pool, stride, pad, dy)
    o_y, arg = oracle.maxpool2d_forward(x, pool, stride, pad)
    assert same(o_y, y)
    assert same(oracle.maxpool2d_backward(dy, arg, x.shape), dx)
    # invariants: outputs are maxima of their windows; the gradient is conserved
    assert np.all(o_y.reshape(-1) == x.reshape(-1)[arg.reshape(-1)])
    assert np.isclose(dx.sum(dtype=np.float64), dy.sum(dtype=np.float64), rtol=1e-5, atol=1e-5)


def cnn_params(rng, ic, c1, c2, side, hidden, classes):
    feat = c2 * (side // 4) ** 2
    return dict(cw1=(0.3 * rng.standard_normal((c1, ic, 3, 3))).astype(np.float32), cb1=(0.1 * rng.standard_normal(c1)).astype(np.float32),
                cw2=(0.2 * rng.standard_normal((c2, c1, 3, 3))).astype(np.float32), cb2=(0.1 * rng.standard_normal(c2)).astype(np.float32),
                w1=(0.2 * rng.standard_normal((feat, hidden))).astype(np.float32), b1=(0.1 * rng.standard_normal(hidden)).astype(np.float32),
                w2=(0.3 * rng.standard_normal((hidden, classes))).astype(np.float32), b2=np.zeros(classes, np.float32))


def oracle_cnn_grads(oracle, x, labels, p, flip_taps):
    """The chain of bc.cnn_ce_grads restated with oracle primitives."""
    B, classes = x.shape[0], p["w2"].shape[1]
    onehot = np.zeros((B, classes), np.float32)
    onehot[np.arange(B), labels] = 1.0
    a1 = oracle.conv2d_forward(x, p["cw1"], p["cb1"], 1, 1)
    r1 = oracle.relu_forward(a1)
    q1, i1 = oracle.maxpool2d_forward(r1, 2, 2, 0)
    a2 = oracle.conv2d_forward(q1, p["cw2"], p["cb2"], 1, 1)
    r2 = oracle.relu_forward(a2)
    q2, i2 = oracle.maxpool2d_forward(r2, 2, 2, 0)
    fl = q2.reshape(B, -1)
    h = oracle.dense_forward(fl, p["w1"], p["b1"])
    rh = oracle.relu_forward(h)
    z = oracle.dense_forward(rh, p["w2"], p["b2"])
    loss, dz = oracle.ce_chain(z, onehot)
    drh, g_w2, g_b2 = oracle.dense_backward(rh, p["w2"], dz)
    dh = oracle.relu_backward(h, drh)
    dfl, g_w1, g_b1 = oracle.dense_backward(fl, p["w1"], dh)
    dr2 = oracle.maxpool2d_backward(dfl.reshape(q2.shape), i2, r2.shape)
    da2 = oracle.relu_backward(a2, dr2)
    dq1, g_cw2, g_cb2 = oracle.conv2d_backward(q1, p["cw2"], da2, 1, 1, flip_taps)
    dr1 = oracle.maxpool2d_backward(dq1, i1, r1.shape)
    da1 = oracle.relu_backward(a1, dr1)
    dx, g_cw1, g_cb1 = oracle.conv2d_backward(x, p["cw1"], da1, 1, 1, flip_taps)
    return dict(loss=loss, logits=z, dx=dx, g_cw1=g_cw1, g_cb1=g_cb1, g_cw2=g_cw2, g_cb2=g_cb2,
                g_w1=g_w1, g_b1=g_b1, g_w2=g_w2, g_b2=g_b2)


CNN_KEYS = ("logits", "dx", "g_cw1", "g_cb1", "g_cw2", "g_cb2", "g_w1", "g_b1", "g_w2", "g_b2")


def test_cnn_chain_bit_exact(ref, oracle):
    """examples/mnist/mnist_autodiff.c:536-557 at a small size: conv-relu-pool x2, flatten, dense-relu-dense, CE chain."""
    rng = np.random.default_rng(314)
    x = rng.random((3, 2, 8, 8), dtype=np.float32)
    labels = rng.integers(0, 5, 3)
    p = cnn_params(rng, 2, 4, 6, 8, 12, 5)
    got = bc.cnn_ce_grads(ref, x, labels, p)
    want = oracle_cnn_grads(oracle, x, labels, p, flip_taps=True)
    assert np.float32(got["loss"]) == np.float32(want["loss"])
    for key in CNN_KEYS:
        assert same(want[key], got[key]), key


def test_checkpoint_written_through_the_reference_api(ref, tmp_path):
    """The example's checkpoint routines (examples/mnist/mnist_autodiff.c:775-995) restated over the C API in
    boat_cases.CnnLayers: the reference writes exactly the documented records, and a model created with other weights
    that reads the file computes the logits of the model that wrote it."""
    rng = np.random.default_rng(271)
    x = rng.random((2, 2, 8, 8), dtype=np.float32)
    p = cnn_params(rng, 2, 3, 5, 8, 7, 4)
    holder = bc.CnnLayers(ref, p)
    path = str(tmp_path / "model.bin")
    holder.save(path)
    with open(path, "rb") as f:
        assert f.read() == bc.checkpoint_bytes(p)
    other = bc.CnnLayers(ref, {k: np.full_like(v, 0.01) for k, v in p.items()})
    want = holder.logits(x)
    assert not same(other.logits(x), want)
    assert other.load(path)
    assert same(other.logits(x), want)


# ---- loss objects (src/loss/*.c) ----

@pytest.mark.parametrize("kind", ["mse", "ce", "huber"])
def test_loss_values_bit_exact(ref, oracle, rng, kind):
    shape = (7, 10)
    if kind == "ce":
        z = rng.standard_normal(shape)
        pred = (np.exp(z) / np.exp(z).sum(1, keepdims=True)).astype(np.float32)
        pred[0, 0], pred[0, 1] = 0.0, 1.0                      # both clip bounds
        target = np.eye(10, dtype=np.float32)[rng.integers(0, 10, 7)]
    else:
        pred = (2 * rng.standard_normal(shape)).astype(np.float32)
        target = rng.standard_normal(shape).astype(np.float32)
    v1, v2 = bc.loss_values(ref, kind, pred, target, 0.75)
    want = oracle.loss_value(kind, pred, target, 0.75)
    assert np.float32(v1) == np.float32(want) and np.float32(v2) == np.float32(want)
    # closed forms in float64
    d = pred.astype(np.float64) - target
    if kind == "mse":
        assert abs(want - (d * d).mean()) <= 1e-5 * (d * d).mean()
    elif kind == "huber":
        a = np.abs(d)
        assert abs(want - np.where(a <= 0.75, 0.5 * a * a, 0.75 * (a - 0.375)).mean()) <= 1e-5
    else:
        assert abs(want + (target * np.log(np.clip(pred.astype(np.float64), 1e-7, 1 - 1e-7))).mean()) <= 1e-5
    assert bc.loss_values(ref, "huber", pred, target, 0.0) is None
