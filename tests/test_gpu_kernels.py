"""Parity of every HIP kernel, called through the C-ABI of include/boat_hip.h, with the CPU oracle on the
same seeded inputs.  Tolerances are the ones the path states:
  elementwise / activation / Adam   max relative error <= 1e-5   (Adam and the exp-free ops are checked bit for bit)
  reductions / LayerNorm            <= 1e-4
  GEMM / attention gradients        <= 1e-3 relative Frobenius norm
"""
import ctypes as C

import numpy as np
import pytest

from oracle_lib import FP32_ATTENTION_BOUND, fp32_gemm_bound, max_rel, rel_fro

pytestmark = pytest.mark.gpu

TOL_EW = 1e-5
TOL_RED = 1e-4
TOL_GEMM = 1e-3


_KEEP = []


def dev(hip, a):
    """Upload and keep the device array alive until the test ends: a temporary used only for its .ptr
    would be returned to the allocator cache (and reused by the next upload) before the kernel is launched."""
    d = hip.to_device(np.ascontiguousarray(a, dtype=np.float32))
    _KEEP.append(d)
    return d


@pytest.fixture(autouse=True)
def _release_device_arrays():
    yield
    _KEEP.clear()


# ------------------------------------------------------------------ runtime

def test_runtime_buffers_and_cache(hip):
    assert b"gfx950" in hip.bh_device_name()
    assert hip.bh_device_cu_count() >= 200
    b = hip.bh_buffer_create(4096, 1)
    assert b and hip.bh_buffer_refcount(b) == 1 and hip.bh_buffer_nbytes(b) == 4096
    hip.bh_buffer_ref(b)
    assert hip.bh_buffer_refcount(b) == 2
    host = np.empty(1024, np.float32)
    hip.check(hip.bh_memcpy_d2h(host.ctypes.data, hip.bh_buffer_ptr(b), 4096))
    assert not host.any()
    hip.bh_buffer_unref(b)
    hip.bh_buffer_unref(b)
    # a freed block is reused for the next request of the same size
    p1 = hip.bh_malloc(1 << 20)
    hip.bh_free(p1)
    p2 = hip.bh_malloc(1 << 20)
    assert p1 == p2
    hip.bh_free(p2)
    # error path: bad arguments are refused, nothing runs
    assert hip.bh_gemm(0, 0, 4, 4, 4, None, 4, None, 4, None, 4, None, 0, 1) == -1
    assert b"null pointer" in hip.bh_last_error()


# -------------------------------------------------------------- elementwise

@pytest.mark.parametrize("n", [1, 3, 4, 1023, 4096, 100003])
def test_elementwise_bit_exact(hip, oracle, rng, n):
    a = rng.standard_normal(n).astype(np.float32)
    b = (rng.standard_normal(n) + 3).astype(np.float32)
    dy = rng.standard_normal(n).astype(np.float32)
    da, db, ddy = dev(hip, a), dev(hip, b), dev(hip, dy)
    out = hip.empty(n)
    for op, fn in enumerate([np.add, np.subtract, np.multiply, np.divide]):
        hip.check(hip.bh_binary(op, da.ptr, db.ptr, out.ptr, n))
        assert np.array_equal(out.numpy(), fn(a, b))
    hip.check(hip.bh_scalar_op(2, da.ptr, -0.015625, out.ptr, n))
    assert np.array_equal(out.numpy(), oracle.mul_scalar(a, -0.015625))
    acc = dev(hip, b)
    hip.check(hip.bh_add_inplace(acc.ptr, da.ptr, n))
    assert np.array_equal(acc.numpy(), b + a)
    hip.check(hip.bh_div_backward_b(da.ptr, db.ptr, ddy.ptr, out.ptr, n))
    assert np.array_equal(out.numpy(), oracle.div_backward(a, b, dy)[1])
    hip.check(hip.bh_fill(out.ptr, 1.0, n))
    assert np.all(out.numpy() == 1.0)


def test_elementwise_unaligned_pointers(hip, rng):
    n = 1001
    a = rng.standard_normal(n + 1).astype(np.float32)
    da = dev(hip, a)
    out = hip.empty(n + 1)
    hip.check(hip.bh_memset_zero(out.ptr, 4 * (n + 1)))
    hip.check(hip.bh_scalar_op(2, da.ptr + 4, 2.0, out.ptr + 4, n))      # 4-byte aligned only
    got = out.numpy()
    assert got[0] == 0 and np.array_equal(got[1:], a[1:] * 2)


def test_broadcast_binary(hip, rng):
    a = rng.standard_normal((3, 1, 5)).astype(np.float32)
    b = rng.standard_normal((4, 1)).astype(np.float32)
    want = a * b
    da, db, out = dev(hip, a), dev(hip, b), hip.empty(want.shape)
    L3 = C.c_int64 * 3
    hip.check(hip.bh_binary_broadcast(2, da.ptr, L3(3, 1, 5), db.ptr, L3(1, 4, 1), out.ptr, L3(3, 4, 5), 3))
    assert np.array_equal(out.numpy(), want)


@pytest.mark.parametrize("n", [5, 4096, 70001])
def test_activations(hip, oracle, rng, n):
    x = rng.standard_normal(n).astype(np.float32) * 2
    x[:3] = [0.0, -0.0, 1e-30][: min(3, n)]
    dy = rng.standard_normal(n).astype(np.float32)
    dx_, ddy, y, g = dev(hip, x), dev(hip, dy), hip.empty(n), hip.empty(n)
    # relu: exp-free, bit exact
    hip.check(hip.bh_activation_forward(hip.ACT_RELU, dx_.ptr, y.ptr, n))
    assert np.array_equal(y.numpy(), oracle.relu_forward(x))
    hip.check(hip.bh_activation_backward(hip.ACT_RELU, dx_.ptr, ddy.ptr, g.ptr, n, 0))
    assert np.array_equal(g.numpy(), oracle.relu_backward(x, dy))
    for act, name in ((hip.ACT_SIGMOID, "sigmoid"), (hip.ACT_TANH, "tanh")):
        hip.check(hip.bh_activation_forward(act, dx_.ptr, y.ptr, n))
        want = getattr(oracle, name + "_forward")(x)
        # The reference's tanh, (e^x - e^-x)/(e^x + e^-x), cancels for small |x|: there its own result carries
        # expf's last-bit noise amplified by 1/|x|, so the relative bound is taken against max(|y|, 0.05).
        assert max_rel(y.numpy(), want, floor=0.05 if name == "tanh" else 1e-6) <= TOL_EW
        dc = dev(hip, want)
        hip.check(hip.bh_activation_backward(act, dc.ptr, ddy.ptr, g.ptr, n, 0))
        assert np.array_equal(g.numpy(), getattr(oracle, name + "_backward")(want, dy))   # from the same saved output
    # gelu (no reference implementation): double-precision closed form
    hip.check(hip.bh_activation_forward(hip.ACT_GELU, dx_.ptr, y.ptr, n))
    assert np.max(np.abs(y.numpy() - oracle.gelu_forward_f64(x))) <= 1e-6
    hip.check(hip.bh_activation_backward(hip.ACT_GELU, dx_.ptr, ddy.ptr, g.ptr, n, 0))
    want = oracle.gelu_backward_f64(x, dy)
    assert np.max(np.abs(g.numpy() - want)) <= 1e-5 * max(1.0, np.abs(want).max())
    # accumulate form adds into dx
    hip.check(hip.bh_activation_backward(hip.ACT_GELU, dx_.ptr, ddy.ptr, g.ptr, n, 1))
    assert np.allclose(g.numpy(), 2 * want, rtol=1e-5, atol=1e-6)


def test_bias_mse_sgd(hip, oracle, rng):
    rows, cols = 37, 53
    y = rng.standard_normal((rows, cols)).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    dy_, db = dev(hip, y), dev(hip, b)
    hip.check(hip.bh_bias_add_rows(dy_.ptr, db.ptr, rows, cols))
    assert np.array_equal(dy_.numpy(), y + b)
    t = rng.standard_normal((rows, cols)).astype(np.float32)
    dp, dt, g, loss = dev(hip, y), dev(hip, t), hip.empty((rows, cols)), hip.empty(1)
    hip.check(hip.bh_mse_grad(dp.ptr, dt.ptr, g.ptr, rows * cols))
    assert np.array_equal(g.numpy(), oracle.mse_grad(y, t))
    hip.check(hip.bh_mse_loss(dp.ptr, dt.ptr, loss.ptr, rows * cols))
    assert abs(loss.numpy()[0] - oracle.mse_loss(y, t)) <= TOL_RED * oracle.mse_loss(y, t)
    p, gr = dev(hip, y), dev(hip, t)
    hip.check(hip.bh_sgd_update(p.ptr, gr.ptr, 0.1, rows * cols, 1))
    assert np.array_equal(p.numpy(), y - np.float32(0.1) * t) and not gr.numpy().any()


# --------------------------------------------------------------------- adam

@pytest.mark.parametrize("n", [1, 7, 4096, 1 << 20, (1 << 20) + 3])
def test_adam_bit_exact_over_steps(hip, oracle, rng, n):
    p = (0.02 * rng.standard_normal(n)).astype(np.float32)
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    dp, dm, dv = dev(hip, p), dev(hip, m), dev(hip, v)
    for t in range(3):
        g = (1e-3 * rng.standard_normal(n)).astype(np.float32)
        dg = dev(hip, g)
        hip.check(hip.bh_adam_update(dp.ptr, dg.ptr, dm.ptr, dv.ptr, n, 1e-3, 0.9, 0.999, 1e-8, t))
        p, m, v = oracle.adam_update(p, g, m, v, 1e-3, 0.9, 0.999, 1e-8, t)
        assert np.array_equal(dp.numpy(), p) and np.array_equal(dm.numpy(), m) and np.array_equal(dv.numpy(), v)


def test_adam_multi_tensor_bit_exact(hip, oracle, rng):
    sizes = [12, 1, 4099, 128 * 784, 10] + [33] * 60          # more tensors than one launch table holds
    ps = [rng.standard_normal(s).astype(np.float32) for s in sizes]
    gs = [(rng.standard_normal(s) * 0.1).astype(np.float32) for s in sizes]
    ms = [np.abs(rng.standard_normal(s)).astype(np.float32) * 0.01 for s in sizes]
    vs = [np.abs(rng.standard_normal(s)).astype(np.float32) * 0.001 for s in sizes]
    d = [[dev(hip, a) for a in group] for group in (ps, gs, ms, vs)]
    PA = C.c_void_p * len(sizes)
    tabs = [PA(*[x.ptr for x in group]) for group in d]
    ns = (C.c_int64 * len(sizes))(*sizes)
    hip.check(hip.bh_adam_update_multi(*tabs, ns, len(sizes), 3e-4, 0.9, 0.999, 1e-8, 41))
    for i in range(len(sizes)):
        p, m, v = oracle.adam_update(ps[i], gs[i], ms[i], vs[i], 3e-4, 0.9, 0.999, 1e-8, 41)
        assert np.array_equal(d[0][i].numpy(), p), i
        assert np.array_equal(d[2][i].numpy(), m) and np.array_equal(d[3][i].numpy(), v)


@pytest.mark.parametrize("n", [1, 7, 4096, (1 << 20) + 3])
def test_rmsprop_adagrad_bit_exact_over_steps(hip, oracle, rng, n):
    for kind in ("rmsprop", "adagrad"):
        p = rng.standard_normal(n).astype(np.float32)
        st = np.zeros(n, np.float32)
        dp, dst = dev(hip, p), dev(hip, st)
        for step in range(3):
            g = (rng.standard_normal(n) * 10 ** rng.uniform(-3, 0)).astype(np.float32)
            dg = dev(hip, g)
            if kind == "rmsprop":
                hip.check(hip.bh_rmsprop_update(dp.ptr, dg.ptr, dst.ptr, n, 1e-2, 0.99, 1e-8))
                p, st = oracle.rmsprop_update(p, g, st, 1e-2, 0.99, 1e-8)
            else:
                hip.check(hip.bh_adagrad_update(dp.ptr, dg.ptr, dst.ptr, n, 1e-2, 1e-8))
                p, st = oracle.adagrad_update(p, g, st, 1e-2, 1e-8)
            assert np.array_equal(dp.numpy(), p) and np.array_equal(dst.numpy(), st), (kind, step)


def test_adam_zero_gradient_is_a_no_op(hip):
    p = hip.to_device(np.full(1000, 1.5, np.float32))
    g, m, v = hip.zeros(1000), hip.zeros(1000), hip.zeros(1000)
    hip.check(hip.bh_adam_update(p.ptr, g.ptr, m.ptr, v.ptr, 1000, 0.01, 0.9, 0.999, 1e-8, 0))
    assert np.all(p.numpy() == 1.5)


# ------------------------------------------------------- reductions, softmax

@pytest.mark.parametrize("n", [1, 63, 4096, 4097, 100000])
def test_sum_all(hip, oracle, rng, n):
    x = rng.standard_normal(n).astype(np.float32)
    out = hip.empty(1)
    hip.check(hip.bh_sum_all(dev(hip, x).ptr, out.ptr, n))
    assert abs(out.numpy()[0] - x.astype(np.float64).sum()) <= TOL_RED * max(1.0, np.abs(x).sum())


@pytest.mark.parametrize("rows,cols", [(1, 1), (64, 10), (8, 128), (1000, 37), (4096, 512)])
def test_colsum(hip, rng, rows, cols):
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    base = rng.standard_normal(cols).astype(np.float32)
    out = dev(hip, base)
    hip.check(hip.bh_colsum(dev(hip, x).ptr, out.ptr, rows, cols, 0))
    want = x.astype(np.float64).sum(0)
    assert np.max(np.abs(out.numpy() - want)) <= TOL_RED * np.abs(x).sum(0).max()
    hip.check(hip.bh_colsum(dev(hip, x).ptr, out.ptr, rows, cols, 1))
    assert np.max(np.abs(out.numpy() - 2 * want)) <= 2 * TOL_RED * np.abs(x).sum(0).max()


@pytest.mark.parametrize("groups", [3, 4])
@pytest.mark.parametrize("rows,cols", [(8192, 1024), (1000, 37), (300, 4096), (64, 10)])
def test_colsum_grouped(hip, rng, rows, cols, groups):
    """bh_colsum_grouped: three or four matrices in one pair of launches give bh_colsum's bits for each, with and without
    accumulation (few rows fall back to bh_colsum itself)."""
    import ctypes as C
    xs = [rng.standard_normal((rows, cols)).astype(np.float32) for _ in range(groups)]
    dxs = [dev(hip, x) for x in xs]
    outs = [hip.zeros(cols) for _ in range(groups)]
    singles = [hip.zeros(cols) for _ in range(groups)]
    tab = lambda arrs: (C.c_void_p * groups)(*[a.ptr for a in arrs])
    for acc in (0, 1):
        hip.check(hip.bh_colsum_grouped(tab(dxs), tab(outs), groups, rows, cols, acc))
        for g in range(groups):
            hip.check(hip.bh_colsum(dxs[g].ptr, singles[g].ptr, rows, cols, acc))
            assert np.array_equal(outs[g].numpy(), singles[g].numpy()), (acc, g)
            want = (1 + acc) * xs[g].sum(0, dtype=np.float64)
            assert np.max(np.abs(outs[g].numpy() - want)) <= TOL_RED * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("rows,cols", [(64, 128), (1, 5), (256, 33), (257, 64), (1000, 37), (300, 4096), (8192, 1024), (1030, 516), (4100, 2052)])
def test_activation_backward_with_column_sums(hip, rng, rows, cols):
    """bh_activation_backward_colsum: dx and the column sums of dx in one pass are, bit for bit, bh_activation_backward
    followed by bh_colsum (few rows; the scalar form of the partial kernel; its vector forms with four wavefronts per row
    chunk, up to 8M elements, and with one, beyond), with and without accumulation."""
    saved = (2 * rng.standard_normal((rows, cols))).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    ds, ddy = dev(hip, saved), dev(hip, dy)
    for act in (hip.ACT_RELU, hip.ACT_GELU, hip.ACT_SIGMOID, hip.ACT_TANH):
        sv = dev(hip, 1 / (1 + np.exp(-saved))) if act in (hip.ACT_SIGMOID, hip.ACT_TANH) else ds   # those two save the output
        base = rng.standard_normal(cols).astype(np.float32)
        dx_a, dx_b, sum_a, sum_b = hip.empty((rows, cols)), hip.empty((rows, cols)), dev(hip, base), dev(hip, base)
        for acc in (0, 1):
            hip.check(hip.bh_activation_backward_colsum(act, sv.ptr, ddy.ptr, dx_a.ptr, sum_a.ptr, rows, cols, acc))
            hip.check(hip.bh_activation_backward(act, sv.ptr, ddy.ptr, dx_b.ptr, rows * cols, 0))
            hip.check(hip.bh_colsum(dx_b.ptr, sum_b.ptr, rows, cols, acc))
            assert np.array_equal(dx_a.numpy(), dx_b.numpy()), (act, acc)
            assert np.array_equal(sum_a.numpy(), sum_b.numpy()), (act, acc)
        want = 2 * dx_b.numpy().astype(np.float64).sum(0)
        assert np.max(np.abs(sum_a.numpy() - want)) <= TOL_RED * max(1.0, np.abs(dx_b.numpy()).sum(0).max())


@pytest.mark.parametrize("rows,cols", [(64, 10), (3, 33), (5, 1), (7, 1000), (300, 257), (129, 1025), (40, 2049)])
def test_softmax_family(hip, oracle, rng, rows, cols):
    x = (3 * rng.standard_normal((rows, cols))).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    dx_, ddy, y, g = dev(hip, x), dev(hip, dy), hip.empty((rows, cols)), hip.empty((rows, cols))
    for fwd, bwd, name in ((hip.bh_softmax_forward, hip.bh_softmax_backward, "softmax"),
                           (hip.bh_log_softmax_forward, hip.bh_log_softmax_backward, "log_softmax")):
        hip.check(fwd(dx_.ptr, y.ptr, rows, cols))
        want = getattr(oracle, name + "_forward")(x)
        assert np.max(np.abs(y.numpy() - want)) <= TOL_RED * max(1.0, np.abs(want).max())
        dwant = dev(hip, want)
        hip.check(bwd(dwant.ptr, ddy.ptr, g.ptr, rows, cols))
        gw = getattr(oracle, name + "_backward")(want, dy)
        assert np.max(np.abs(g.numpy() - gw)) <= TOL_RED * max(1.0, np.abs(gw).max())


@pytest.mark.parametrize("rows,cols", [(64, 10), (3, 33), (5, 1), (7, 1000)])
def test_loss_chain_backward_kernel(hip, oracle, rng, rows, cols):
    """bh_log_softmax_weighted_backward against the oracle's log-softmax backward of dls = (seed*f)*w and, bit for bit,
    against the separate kernel on the same dls (the fused kernel keeps the rules' operations), with and without a seed."""
    z = (3 * rng.standard_normal((rows, cols))).astype(np.float32)
    y = oracle.log_softmax_forward(z)
    w = np.zeros((rows, cols), np.float32)
    w[np.arange(rows), rng.integers(0, cols, rows)] = 1.0
    w[0] = rng.standard_normal(cols).astype(np.float32)          # any weights, not only one-hot rows
    f, seed = np.array([-1.0 / rows], np.float32), np.array([0.75], np.float32)
    dz = hip.empty((rows, cols))
    for s in (None, seed):
        c = np.float32((np.float32(1.0) if s is None else s[0]) * f[0])
        hip.check(hip.bh_log_softmax_weighted_backward(dev(hip, y).ptr, dev(hip, w).ptr, dev(hip, s).ptr if s is not None else None,
                                                       dev(hip, f).ptr, dz.ptr, rows, cols))
        dls = (c * w).astype(np.float32)
        want = oracle.log_softmax_backward(y, dls)
        got = dz.numpy()
        assert np.max(np.abs(got - want)) <= TOL_RED * max(1e-6, np.abs(want).max())
        dchain = hip.empty((rows, cols))
        hip.check(hip.bh_log_softmax_backward(dev(hip, y).ptr, dev(hip, dls).ptr, dchain.ptr, rows, cols))
        assert np.array_equal(got, dchain.numpy())


@pytest.mark.parametrize("rows,cols", [(64, 10), (1, 3), (256, 32), (17, 130), (100, 81), (257, 10), (300, 100)])
def test_loss_chain_backward_kernel_with_column_sums(hip, oracle, rng, rows, cols):
    """bh_log_softmax_weighted_backward_colsum: dz and its column sums in one launch (small batches) are, bit for bit,
    bh_log_softmax_weighted_backward followed by bh_colsum; larger matrices take those two."""
    z = (3 * rng.standard_normal((rows, cols))).astype(np.float32)
    y = dev(hip, oracle.log_softmax_forward(z))
    w = dev(hip, rng.standard_normal((rows, cols)).astype(np.float32))
    f, seed = dev(hip, np.array([-1.0 / rows], np.float32)), dev(hip, np.array([0.75], np.float32))
    base = rng.standard_normal(cols).astype(np.float32)
    dz_a, dz_b, sum_a, sum_b = hip.empty((rows, cols)), hip.empty((rows, cols)), dev(hip, base), dev(hip, base)
    for acc in (0, 1):
        hip.check(hip.bh_log_softmax_weighted_backward_colsum(y.ptr, w.ptr, seed.ptr, f.ptr, dz_a.ptr, sum_a.ptr, rows, cols, acc))
        hip.check(hip.bh_log_softmax_weighted_backward(y.ptr, w.ptr, seed.ptr, f.ptr, dz_b.ptr, rows, cols))
        hip.check(hip.bh_colsum(dz_b.ptr, sum_b.ptr, rows, cols, acc))
        assert np.array_equal(dz_a.numpy(), dz_b.numpy()), acc
        assert np.array_equal(sum_a.numpy(), sum_b.numpy()), acc
    want = 2 * dz_b.numpy().astype(np.float64).sum(0)
    assert np.max(np.abs(sum_a.numpy() - want)) <= TOL_RED * max(1e-6, np.abs(dz_b.numpy()).sum(0).max())


@pytest.mark.parametrize("rows,cols", [(64, 10), (8, 10), (5, 130)])
def test_fused_softmax_ce_matches_tape_chain(hip, oracle, rng, rows, cols):
    z = (2 * rng.standard_normal((rows, cols))).astype(np.float32)
    labels = rng.integers(0, cols, rows).astype(np.int32)
    onehot = np.zeros((rows, cols), np.float32)
    onehot[np.arange(rows), labels] = 1
    loss_want, dz_want = oracle.ce_chain(z, onehot)
    dz, loss = hip.empty((rows, cols)), hip.empty(1)
    dlabels = hip.to_device(labels)
    hip.check(hip.bh_softmax_ce_grad(dev(hip, z).ptr, dlabels.ptr, dz.ptr, loss.ptr, rows, cols))
    assert abs(loss.numpy()[0] - loss_want) <= TOL_RED * abs(loss_want)
    assert np.max(np.abs(dz.numpy() - dz_want)) <= TOL_EW * np.abs(dz_want).max() + 1e-9
    # closed form: (softmax - onehot)/B
    p = np.exp(z.astype(np.float64) - z.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    assert np.allclose(dz.numpy(), (p - onehot) / rows, atol=1e-7)


# ---------------------------------------------------------------- layernorm

LN_SHAPES = [(1, 4), (7, 64), (10, 48), (33, 768), (64, 1024), (17, 4096), (5, 8192), (6, 50), (3, 9000),
             (40, 2048), (21, 2044), (9, 2040)]


@pytest.mark.parametrize("rows,hidden", LN_SHAPES)
def test_layernorm_forward(hip, oracle, rng, rows, hidden):
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(hidden)).astype(np.float32)
    y, mean, rstd = hip.empty((rows, hidden)), hip.empty(rows), hip.empty(rows)
    hip.check(hip.bh_layernorm_forward(dev(hip, x).ptr, dev(hip, gamma).ptr, dev(hip, beta).ptr, y.ptr, mean.ptr, rstd.ptr,
                                       rows, hidden, 1e-5))
    wy, wm, wr = oracle.layernorm_forward(x, gamma, beta, 1e-5)
    assert np.max(np.abs(y.numpy() - wy)) <= TOL_RED * np.abs(wy).max()
    assert np.max(np.abs(mean.numpy() - wm)) <= 1e-6 and max_rel(rstd.numpy(), wr) <= TOL_RED
    # no affine
    hip.check(hip.bh_layernorm_forward(dev(hip, x).ptr, None, None, y.ptr, None, None, rows, hidden, 1e-5))
    wy, _, _ = oracle.layernorm_forward(x, None, None, 1e-5)
    assert np.max(np.abs(y.numpy() - wy)) <= TOL_RED * np.abs(wy).max()


@pytest.mark.parametrize("rows,hidden", LN_SHAPES + [(1000, 1024), (300, 4096)])
def test_layernorm_backward_with_added_gradient(hip, oracle, rng, rows, hidden):
    """bh_layernorm_backward_add: dx = LayerNorm input gradient + add, the same kernel's arithmetic plus one fp32 add per
    element (bit for bit what bh_layernorm_backward followed by an add gives); parameter gradients unchanged."""
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    dy = rng.standard_normal((rows, hidden)).astype(np.float32)
    add = rng.standard_normal((rows, hidden)).astype(np.float32)
    _, mean, rstd = oracle.layernorm_forward(x, gamma, None, 1e-5)
    args = (dev(hip, x).ptr, dev(hip, gamma).ptr, dev(hip, dy).ptr, dev(hip, mean).ptr, dev(hip, rstd).ptr)
    dx0, dg0, db0 = hip.empty((rows, hidden)), hip.zeros(hidden), hip.zeros(hidden)
    hip.check(hip.bh_layernorm_backward(*args, dx0.ptr, dg0.ptr, db0.ptr, rows, hidden, 0))
    dx1, dg1, db1 = hip.empty((rows, hidden)), hip.zeros(hidden), hip.zeros(hidden)
    hip.check(hip.bh_layernorm_backward_add(*args, dev(hip, add).ptr, dx1.ptr, dg1.ptr, db1.ptr, rows, hidden, 0))
    assert np.array_equal(dx1.numpy(), dx0.numpy() + add)
    assert np.array_equal(dg1.numpy(), dg0.numpy()) and np.array_equal(db1.numpy(), db0.numpy())
    wdx, _, _ = oracle.layernorm_backward_f64(x, gamma, dy, mean, rstd)
    assert np.max(np.abs(dx1.numpy() - (wdx + add))) <= TOL_RED * np.abs(wdx + add).max()
    with pytest.raises(RuntimeError):      # in place is refused
        hip.check(hip.bh_layernorm_backward_add(*args, dx1.ptr, dx1.ptr, dg1.ptr, db1.ptr, rows, hidden, 0))


@pytest.mark.parametrize("rows,hidden", LN_SHAPES + [(1000, 1024), (300, 4096)])
def test_layernorm_backward(hip, oracle, rng, rows, hidden):
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    dy = rng.standard_normal((rows, hidden)).astype(np.float32)
    _, mean, rstd = oracle.layernorm_forward(x, gamma, None, 1e-5)
    dx, dg, db = hip.empty((rows, hidden)), hip.zeros(hidden), hip.zeros(hidden)
    args = (dev(hip, x).ptr, dev(hip, gamma).ptr, dev(hip, dy).ptr, dev(hip, mean).ptr, dev(hip, rstd).ptr)
    hip.check(hip.bh_layernorm_backward(*args, dx.ptr, dg.ptr, db.ptr, rows, hidden, 0))
    wdx, wdg, wdb = oracle.layernorm_backward_f64(x, gamma, dy, mean, rstd)
    assert np.max(np.abs(dx.numpy() - wdx)) <= TOL_RED * np.abs(wdx).max()
    assert np.max(np.abs(dg.numpy() - wdg)) <= TOL_RED * max(1.0, np.abs(wdg).max())
    assert np.max(np.abs(db.numpy() - wdb)) <= TOL_RED * max(1.0, np.abs(wdb).max())
    # accumulate into the parameter gradients
    hip.check(hip.bh_layernorm_backward(*args, dx.ptr, dg.ptr, db.ptr, rows, hidden, 1))
    assert np.max(np.abs(dg.numpy() - 2 * wdg)) <= 2 * TOL_RED * max(1.0, np.abs(wdg).max())
    assert np.max(np.abs(db.numpy() - 2 * wdb)) <= 2 * TOL_RED * max(1.0, np.abs(wdb).max())


@pytest.mark.parametrize("rows,hidden", LN_SHAPES + [(1000, 1024), (300, 4096)])
def test_rmsnorm_forward_backward(hip, oracle, rng, rows, hidden):
    """RMSNorm (eps outside the root, src/layers/norm.c:212-229,366-389): forward against the oracle's fp32 restatement,
    backward (a stub in the reference) against the float64 closed form; the LayerNorm tolerance applies."""
    x = (rng.standard_normal((rows, hidden)) * 10 ** rng.uniform(-1, 1)).astype(np.float32)
    x[0] = 0.0                                       # a row of zeros: scale 1/eps, output and gradient term stay finite
    w = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    dy = rng.standard_normal((rows, hidden)).astype(np.float32)
    for eps, weight in ((1e-6, w), (1e-2, None)):
        dw_ = None if weight is None else dev(hip, weight).ptr
        y, inv = hip.empty((rows, hidden)), hip.empty(rows)
        hip.check(hip.bh_rmsnorm_forward(dev(hip, x).ptr, dw_, y.ptr, inv.ptr, rows, hidden, eps))
        wy, winv = oracle.rmsnorm_forward(x, weight, eps)
        assert np.max(np.abs(y.numpy() - wy)) <= TOL_RED * max(np.abs(wy).max(), 1e-30)
        assert max_rel(inv.numpy(), winv) <= TOL_RED
        dx, dg = hip.empty((rows, hidden)), hip.zeros(hidden)
        args = (dev(hip, x).ptr, dw_, dev(hip, dy).ptr, dev(hip, winv).ptr)
        hip.check(hip.bh_rmsnorm_backward(*args, dx.ptr, dg.ptr, rows, hidden, eps, 0))
        wdx, wdw = oracle.rmsnorm_backward_f64(x, weight, dy, eps)
        assert np.max(np.abs(dx.numpy() - wdx)) <= TOL_RED * np.abs(wdx).max()
        assert np.max(np.abs(dg.numpy() - wdw)) <= TOL_RED * max(1.0, np.abs(wdw).max())
        hip.check(hip.bh_rmsnorm_backward(*args, dx.ptr, dg.ptr, rows, hidden, eps, 1))
        assert np.max(np.abs(dg.numpy() - 2 * wdw)) <= 2 * TOL_RED * max(1.0, np.abs(wdw).max())


# --------------------------------------------------------------------- gemm

def gemm_case(hip, rng, ta, tb, m, n, k, accumulate=False, bias=False, batch=1, force=None, direct=None):
    a = rng.standard_normal((batch, k, m) if ta else (batch, m, k)).astype(np.float32)
    b = rng.standard_normal((batch, n, k) if tb else (batch, k, n)).astype(np.float32)
    c0 = rng.standard_normal((batch, m, n)).astype(np.float32)
    bv = rng.standard_normal(n).astype(np.float32) if bias else None
    A = a.transpose(0, 2, 1) if ta else a
    B = b.transpose(0, 2, 1) if tb else b
    want = np.matmul(A.astype(np.float64), B.astype(np.float64))
    if bias:
        want = want + bv
    if accumulate:
        want = want + c0
    dc = dev(hip, c0)
    if force is not None:
        hip.bh_gemm_force_config(force)
    if direct is not None:
        hip.bh_gemm_force_direct(direct)
    try:
        hip.check(hip.bh_gemm(int(ta), int(tb), m, n, k, dev(hip, a).ptr, a.shape[2], dev(hip, b).ptr, b.shape[2], dc.ptr, n,
                              dev(hip, bv).ptr if bias else None, int(accumulate), batch))
    finally:
        hip.bh_gemm_force_config(-1)
        hip.bh_gemm_force_direct(-1)
    got = dc.numpy()
    assert rel_fro(got, want) <= TOL_GEMM, (ta, tb, m, n, k, rel_fro(got, want))
    # the contract above would also pass a narrowed matrix path (tf32 lands near 3e-4); full fp32 stays under this
    assert rel_fro(got, want) <= fp32_gemm_bound(k), (ta, tb, m, n, k, rel_fro(got, want), fp32_gemm_bound(k))
    return got, want


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(64, 128, 784), (64, 784, 128), (784, 128, 64), (64, 10, 128), (128, 10, 64),
                                   (64, 128, 10), (1, 1, 1), (33, 17, 5), (256, 256, 64), (384, 640, 200),
                                   (512, 512, 512), (300, 260, 1028)])
def test_gemm_heuristic_path(hip, rng, ta, tb, m, n, k):
    gemm_case(hip, rng, ta, tb, m, n, k)


@pytest.mark.parametrize("force", [1, 2, 3, 4, 7])
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(256, 256, 16), (256, 512, 64), (128, 128, 8), (260, 132, 36), (512, 768, 100), (1024, 1024, 256)])
def test_gemm_mfma_tiles(hip, rng, force, ta, tb, m, n, k):
    # operands staged through registers (any contraction length) and, where k % 16 == 0, streamed straight to LDS
    gemm_case(hip, rng, ta, tb, m, n, k, force=force, direct=0)
    gemm_case(hip, rng, ta, tb, m, n, k, force=force, direct=1)


@pytest.mark.parametrize("force", [1, 2, 3, 4, 7])
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_direct_to_lds_edges_epilogues_and_split_k(hip, rng, force, ta, tb):
    gemm_case(hip, rng, ta, tb, 260, 132, 48, force=force, direct=1, accumulate=True, bias=True)   # ragged edge tiles
    gemm_case(hip, rng, ta, tb, 4, 2048, 32, force=force, direct=1)                                # a single row block
    gemm_case(hip, rng, ta, tb, 1028, 8, 16, force=force, direct=1)                                # one k-tile
    gemm_case(hip, rng, ta, tb, 256, 384, 2048, force=force, direct=1, accumulate=True)            # split-K
    gemm_case(hip, rng, ta, tb, 128, 256, 64, force=force, direct=1, batch=3)


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("k", [32, 64, 96, 160, 1024])
def test_gemm_big_tile_with_one_or_two_k_tiles_per_barrier(hip, rng, ta, tb, k):
    """The 256x256 tile keeps two k-tiles per LDS stage when the contraction is a multiple of 32 (mode 1) and one
    otherwise or on request (mode 3).  Both walk k in the same order, so the results are the same bits."""
    state = rng.bit_generator.state
    one, _ = gemm_case(hip, rng, ta, tb, 520, 300, k, force=2, direct=3, accumulate=True, bias=True)
    rng.bit_generator.state = state
    two, _ = gemm_case(hip, rng, ta, tb, 520, 300, k, force=2, direct=1, accumulate=True, bias=True)
    assert np.array_equal(one, two)


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (33, 17, 5), (64, 64, 128), (65, 63, 129), (37, 130, 225), (200, 70, 1000),
                                   (256, 512, 64)])
def test_gemm_small_problem_kernel(hip, rng, ta, tb, m, n, k):
    gemm_case(hip, rng, ta, tb, m, n, k, force=5)
    gemm_case(hip, rng, ta, tb, m, n, k, force=5, accumulate=True, bias=True)
    gemm_case(hip, rng, ta, tb, m, n, k, force=0)                    # the bounds-checked fallback on the same shapes


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (33, 17, 5), (64, 128, 784), (64, 784, 128), (784, 128, 64), (64, 10, 128),
                                   (128, 10, 64), (64, 128, 10), (65, 63, 129), (37, 130, 225), (200, 70, 1000), (32, 32, 4096)])
def test_gemm_tiny_problem_kernel(hip, rng, ta, tb, m, n, k):
    """The staging-free single-trip kernel (forced: the heuristic only picks it for a few million multiply-adds): both
    wavefront counts, 16-byte and 4-byte fetches (k % 4), ragged tiles, k tails, bias and accumulation."""
    gemm_case(hip, rng, ta, tb, m, n, k, force=6)
    gemm_case(hip, rng, ta, tb, m, n, k, force=6, accumulate=True, bias=True)


def test_gemm_tiny_problem_kernel_batched_and_deterministic(hip, rng):
    gemm_case(hip, rng, 0, 0, 5, 4, 6, batch=6, force=6)
    gemm_case(hip, rng, 1, 1, 70, 40, 300, batch=3, force=6, accumulate=True)
    got1, _ = gemm_case(hip, rng := np.random.default_rng(5), 0, 1, 64, 128, 784, force=6)
    got2, _ = gemm_case(hip, np.random.default_rng(5), 0, 1, 64, 128, 784, force=6)
    assert np.array_equal(got1, got2)          # partial tiles are summed in wavefront order, not arrival order


def test_gemm_small_problem_kernel_batched(hip, rng):
    gemm_case(hip, rng, 0, 0, 5, 4, 6, batch=6, force=5)
    gemm_case(hip, rng, 1, 1, 70, 40, 300, batch=3, force=5, accumulate=True)


def test_gemm_epilogues_and_batch(hip, rng):
    gemm_case(hip, rng, 0, 0, 256, 384, 128, bias=True)
    gemm_case(hip, rng, 1, 0, 384, 256, 128, accumulate=True)
    gemm_case(hip, rng, 0, 1, 130, 70, 64, accumulate=True, bias=True)
    gemm_case(hip, rng, 0, 0, 128, 128, 64, batch=6)
    gemm_case(hip, rng, 0, 0, 5, 4, 6, batch=6)                      # the [2,3,5,4].[2,3,4,6] layout case
    gemm_case(hip, rng, 1, 0, 256, 256, 4096, accumulate=True)       # split-K with accumulation
    gemm_case(hip, rng, 1, 0, 128, 384, 2048, bias=True)             # split-K with bias


def _ptr_table(arrays):
    import ctypes as C
    return (C.c_void_p * len(arrays))(*[a.ptr if a is not None else None for a in arrays])


@pytest.mark.parametrize("force", [None, 1, 2, 3, 4])
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k,accumulate,bias,shared_a,groups", [
    (512, 384, 256, False, True, True, 3),   # the forward projections' form: one input, three weights, three biases
    (260, 132, 96, True, True, False, 3),    # ragged edge tiles, accumulate
    (256, 384, 2048, True, False, True, 3),  # split-K: partials of the three groups folded by one launch
    (40, 24, 12, False, False, False, 3),    # no table kernel for this shape: the groups run one after the other
    (256, 256, 2048, False, False, False, 4),   # four groups (the weight gradients of an attention layer's four projections), split-K
    (260, 132, 96, True, True, False, 4),
    (384, 256, 64, False, True, False, 2),
])
def test_gemm_grouped_equals_separate_launches(hip, rng, force, ta, tb, m, n, k, accumulate, bias, shared_a, groups):
    """bh_gemm_grouped (two to four products of one shape in one launch, operands from pointer tables) against float64 and
    against the same products through bh_gemm: bit for bit where the contraction is too short to be cut (the grouped
    kernels walk a product as bh_gemm does), to fp32 rounding otherwise (the number of cuts is chosen for the group as a
    whole, and partial sums are added in another order)."""
    a = [rng.standard_normal((k, m) if ta else (m, k)).astype(np.float32) for _ in range(1 if shared_a else groups)]
    if shared_a:
        a = a * groups
    b = [rng.standard_normal((n, k) if tb else (k, n)).astype(np.float32) for _ in range(groups)]
    c0 = [rng.standard_normal((m, n)).astype(np.float32) for _ in range(groups)]
    bv = [rng.standard_normal(n).astype(np.float32) if (bias and g != 1) else None for g in range(groups)]   # one group without bias
    da = [dev(hip, a[0])] * groups if shared_a else [dev(hip, x) for x in a]
    db = [dev(hip, x) for x in b]
    dbias = [dev(hip, x) if x is not None else None for x in bv]
    lda, ldb = a[0].shape[1], b[0].shape[1]
    results = []
    for tables_off in (0, 1):
        dc = [dev(hip, x) for x in c0]
        if force is not None:
            hip.bh_gemm_force_config(force)
        hip.bh_gemm_no_tables(tables_off)
        try:
            hip.check(hip.bh_gemm_grouped(ta, tb, m, n, k, groups, _ptr_table(da), lda, _ptr_table(db), ldb, _ptr_table(dc), n,
                                          _ptr_table(dbias) if bias else None, int(accumulate)))
        finally:
            hip.bh_gemm_force_config(-1)
            hip.bh_gemm_no_tables(0)
        results.append([x.numpy() for x in dc])
    for g in range(groups):
        A = a[g].T if ta else a[g]
        B = b[g].T if tb else b[g]
        want = A.astype(np.float64) @ B.astype(np.float64)
        if bv[g] is not None:
            want = want + bv[g]
        if accumulate:
            want = want + c0[g]
        assert rel_fro(results[0][g], want) <= fp32_gemm_bound(k), (g, rel_fro(results[0][g], want))
        if k < 256:
            assert np.array_equal(results[0][g], results[1][g]), g
        else:
            assert rel_fro(results[0][g], results[1][g]) <= 2 * fp32_gemm_bound(k), g


@pytest.mark.parametrize("force", [None, 1, 2, 3, 4])
@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k,accumulate,bias", [(512, 256, 128, False, False), (300, 260, 64, True, True), (256, 128, 1024, False, True),
                                                   (48, 40, 20, True, False)])
def test_gemm_ksegments(hip, rng, force, ta, tb, m, n, k, accumulate, bias):
    """bh_gemm_ksegments: c (+)= a0.b0 + a1.b1 + a2.b2 as one contraction over three operand pairs (the summed input
    gradient of self-attention), against float64 at the bound only fp32 accumulation meets, and against the
    pair-by-pair fallback to fp32 rounding."""
    segs = 3
    a = [rng.standard_normal((k, m) if ta else (m, k)).astype(np.float32) for _ in range(segs)]
    b = [rng.standard_normal((n, k) if tb else (k, n)).astype(np.float32) for _ in range(segs)]
    c0 = rng.standard_normal((m, n)).astype(np.float32)
    bv = rng.standard_normal(n).astype(np.float32) if bias else None
    want = sum((x.T if ta else x).astype(np.float64) @ (y.T if tb else y).astype(np.float64) for x, y in zip(a, b))
    if bias:
        want = want + bv
    if accumulate:
        want = want + c0
    da, db = [dev(hip, x) for x in a], [dev(hip, x) for x in b]
    dbias = dev(hip, bv) if bias else None
    got = []
    for tables_off in (0, 1):
        dc = dev(hip, c0)
        if force is not None:
            hip.bh_gemm_force_config(force)
        hip.bh_gemm_no_tables(tables_off)
        try:
            hip.check(hip.bh_gemm_ksegments(ta, tb, m, n, k, segs, _ptr_table(da), a[0].shape[1], _ptr_table(db), b[0].shape[1], dc.ptr, n,
                                            dbias.ptr if bias else None, int(accumulate)))
        finally:
            hip.bh_gemm_force_config(-1)
            hip.bh_gemm_no_tables(0)
        got.append(dc.numpy())
        assert rel_fro(got[-1], want) <= fp32_gemm_bound(segs * k), (tables_off, rel_fro(got[-1], want))
    assert rel_fro(got[0], got[1]) <= 2 * fp32_gemm_bound(segs * k)


def test_gemm_grouped_at_the_block_shapes(hip, rng):
    """The three grouped launches of a self-attention layer at d_model 1024 and 8192 rows (forward projections, summed
    input gradient, weight gradients with split contraction), sampled against float64."""
    rows, h = 8192, 1024
    x = rng.standard_normal((rows, h)).astype(np.float32)
    w = [(0.02 * rng.standard_normal((h, h))).astype(np.float32) for _ in range(3)]
    bias = [rng.standard_normal(h).astype(np.float32) for _ in range(3)]
    dy = [rng.standard_normal((rows, h)).astype(np.float32) for _ in range(3)]
    dx_, dw, db, ddy = dev(hip, x), [dev(hip, t) for t in w], [dev(hip, t) for t in bias], [dev(hip, t) for t in dy]
    y = [hip.empty((rows, h)) for _ in range(3)]
    hip.check(hip.bh_gemm_grouped(0, 0, rows, h, h, 3, _ptr_table([dx_] * 3), h, _ptr_table(dw), h, _ptr_table(y), h, _ptr_table(db), 0))
    gin = hip.empty((rows, h))
    hip.check(hip.bh_gemm_ksegments(0, 1, rows, h, h, 3, _ptr_table(ddy), h, _ptr_table(dw), h, gin.ptr, h, None, 0))
    gw = [hip.empty((h, h)) for _ in range(3)]
    hip.check(hip.bh_gemm_grouped(1, 0, h, h, rows, 3, _ptr_table([dx_] * 3), h, _ptr_table(ddy), h, _ptr_table(gw), h, None, 0))
    r = np.sort(rng.choice(rows, 24, replace=False))
    c = np.sort(rng.choice(h, 24, replace=False))
    x64 = x.astype(np.float64)
    for g in range(3):
        assert rel_fro(y[g].numpy()[r], x64[r] @ w[g].astype(np.float64) + bias[g]) <= fp32_gemm_bound(h), g
        assert rel_fro(gw[g].numpy()[c], x64[:, c].T @ dy[g].astype(np.float64)) <= fp32_gemm_bound(rows), g
    want = sum(dy[g][r].astype(np.float64) @ w[g].astype(np.float64).T for g in range(3))
    assert rel_fro(gin.numpy()[r], want) <= fp32_gemm_bound(3 * h)


def test_gemm_matches_reference_loop_order_within_tolerance(hip, oracle, rng):
    a = rng.standard_normal((96, 200)).astype(np.float32)
    b = rng.standard_normal((200, 160)).astype(np.float32)
    c = hip.empty((96, 160))
    hip.check(hip.bh_gemm(0, 0, 96, 160, 200, dev(hip, a).ptr, 200, dev(hip, b).ptr, 160, c.ptr, 160, None, 0, 1))
    assert rel_fro(c.numpy(), oracle.matmul(a, b)) <= TOL_GEMM


@pytest.mark.parametrize("m,k,n", [(9, 13, 6), (64, 784, 128), (64, 128, 10), (512, 256, 384)])
def test_dense_backward_entry_point(hip, oracle, rng, m, k, n):
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.standard_normal((k, n)).astype(np.float32)
    dy = rng.standard_normal((m, n)).astype(np.float32)
    gw0 = rng.standard_normal((k, n)).astype(np.float32)
    gb0 = rng.standard_normal(n).astype(np.float32)
    dx, gw, gb = hip.empty((m, k)), dev(hip, gw0), dev(hip, gb0)
    hip.check(hip.bh_dense_backward(dev(hip, x).ptr, dev(hip, w).ptr, dev(hip, dy).ptr, dx.ptr, gw.ptr, gb.ptr, m, k, n, 1))
    wdx, wgw, wgb = oracle.dense_backward(x, w, dy, gw0, gb0)
    assert rel_fro(dx.numpy(), wdx) <= TOL_GEMM and rel_fro(gw.numpy(), wgw) <= TOL_GEMM
    assert np.max(np.abs(gb.numpy() - wgb)) <= TOL_RED * max(1.0, np.abs(wgb).max())
    # invariant: db == column sum of dY
    hip.check(hip.bh_dense_backward(dev(hip, x).ptr, dev(hip, w).ptr, dev(hip, dy).ptr, dx.ptr, gw.ptr, gb.ptr, m, k, n, 0))
    assert np.allclose(gb.numpy(), dy.sum(0), rtol=1e-4, atol=1e-4)


def test_transpose(hip, oracle, rng):
    a = rng.standard_normal((3, 45, 70)).astype(np.float32)
    out = hip.empty((3, 70, 45))
    hip.check(hip.bh_transpose_last2(dev(hip, a).ptr, out.ptr, 3, 45, 70))
    assert np.array_equal(out.numpy(), oracle.transpose_last2(a))


# ---------------------------------------------------------------- attention

SDPA_SHAPES = [(8, 4, 8), (4, 16, 16), (2, 8, 8), (3, 33, 20), (2, 64, 64), (3, 130, 32), (2, 200, 128), (2, 96, 20), (4, 128, 64), (2, 256, 64), (3, 100, 64),
               (2, 512, 64), (1, 1024, 64), (2, 32, 64), (2, 77, 64), (1, 129, 64), (2, 191, 64), (1, 1000, 64),
               # the matrix-core kernels' other head sizes: whole tiles, ragged lengths, the shortest sequence
               (2, 128, 32), (2, 256, 32), (1, 1024, 32), (3, 77, 32), (2, 32, 32), (1, 513, 32),
               (2, 128, 128), (2, 384, 128), (1, 1024, 128), (2, 100, 128), (2, 32, 128), (1, 257, 128)]


@pytest.mark.parametrize("causal", [0, 1])
@pytest.mark.parametrize("bh,s,d", SDPA_SHAPES)
@pytest.mark.parametrize("general", [0, 1, 2])      # heuristic; row kernels; GEMM-based path
def test_sdpa_forward_backward(hip, oracle, rng, bh, s, d, causal, general):
    q, k, v, go = (rng.standard_normal((bh, s, d)).astype(np.float32) for _ in range(4))
    scale = float(np.float32(1.0) / np.sqrt(np.float32(d)))
    wo, wlse, wattn = oracle.sdpa_forward(q, k, v, scale, causal)
    wdq, wdk, wdv = oracle.sdpa_backward(q, k, v, wattn, go, scale)
    dq_, dk_, dv_ = dev(hip, q), dev(hip, k), dev(hip, v)
    out, lse = hip.empty((bh, s, d)), hip.empty((bh, s))
    hip.bh_sdpa_force_general(general)
    try:
        hip.check(hip.bh_sdpa_forward(dq_.ptr, dk_.ptr, dv_.ptr, scale, causal, out.ptr, lse.ptr, None, bh, s, d))
        assert rel_fro(out.numpy(), wo) <= TOL_GEMM
        assert np.max(np.abs(lse.numpy() - wlse)) <= 1e-4
        gq, gk, gv = hip.empty((bh, s, d)), hip.empty((bh, s, d)), hip.empty((bh, s, d))
        hip.check(hip.bh_sdpa_backward(dq_.ptr, dk_.ptr, dv_.ptr, out.ptr, lse.ptr, dev(hip, go).ptr, scale, causal,
                                       gq.ptr, gk.ptr, gv.ptr, bh, s, d))
    finally:
        hip.bh_sdpa_force_general(0)
    assert rel_fro(gq.numpy(), wdq) <= TOL_GEMM and rel_fro(gk.numpy(), wdk) <= TOL_GEMM and rel_fro(gv.numpy(), wdv) <= TOL_GEMM
    # beyond the contract: only full-fp32 products and sums come this close to the fp32 oracle (a narrowed matrix path
    # would sit near 3e-4 and still pass the line above)
    errs = [rel_fro(out.numpy(), wo), rel_fro(gq.numpy(), wdq), rel_fro(gk.numpy(), wdk), rel_fro(gv.numpy(), wdv)]
    assert max(errs) <= FP32_ATTENTION_BOUND, errs


@pytest.mark.parametrize("bh,s,d", [(3, 12, 8), (2, 80, 24)])      # row kernels; GEMM-based path (s >= 64)
def test_sdpa_attention_matrix_output(hip, oracle, rng, bh, s, d):
    q, k, v = (rng.standard_normal((bh, s, d)).astype(np.float32) for _ in range(3))
    out, lse, attn = hip.empty((bh, s, d)), hip.empty((bh, s)), hip.empty((bh, s, s))
    hip.check(hip.bh_sdpa_forward(dev(hip, q).ptr, dev(hip, k).ptr, dev(hip, v).ptr, 0.35, 1, out.ptr, lse.ptr, attn.ptr, bh, s, d))
    wo, _, wattn = oracle.sdpa_forward(q, k, v, 0.35, 1)
    assert np.max(np.abs(attn.numpy() - wattn)) <= 1e-6
    assert np.allclose(attn.numpy().sum(-1), 1.0, atol=1e-5)
    assert rel_fro(out.numpy(), wo) <= TOL_GEMM


@pytest.mark.parametrize("general", [0, 1, 2])
@pytest.mark.parametrize("causal", [0, 1])
def test_sdpa_large_scores_stay_finite(hip, oracle, rng, causal, general):
    """Scores of several hundred (one key dominates each row, most exponentials underflow): max-subtracted softmax in
    every path, so outputs, log-sum-exp and gradients stay finite and match the float64-accurate oracle."""
    bh, s, d = 2, 160, 64
    q, k, v, go = (rng.standard_normal((bh, s, d)).astype(np.float32) for _ in range(4))
    q *= 9.0
    k *= 9.0
    scale = 1.0
    wo, wlse, wattn = oracle.sdpa_forward(q, k, v, scale, causal)
    wdq, wdk, wdv = oracle.sdpa_backward(q, k, v, wattn, go, scale)
    assert np.abs(wlse).max() > 300
    dq_, dk_, dv_ = dev(hip, q), dev(hip, k), dev(hip, v)
    out, lse = hip.empty((bh, s, d)), hip.empty((bh, s))
    gq, gk, gv = hip.empty((bh, s, d)), hip.empty((bh, s, d)), hip.empty((bh, s, d))
    hip.bh_sdpa_force_general(general)
    try:
        hip.check(hip.bh_sdpa_forward(dq_.ptr, dk_.ptr, dv_.ptr, scale, causal, out.ptr, lse.ptr, None, bh, s, d))
        hip.check(hip.bh_sdpa_backward(dq_.ptr, dk_.ptr, dv_.ptr, out.ptr, lse.ptr, dev(hip, go).ptr, scale, causal,
                                       gq.ptr, gk.ptr, gv.ptr, bh, s, d))
    finally:
        hip.bh_sdpa_force_general(0)
    for got, want in ((out, wo), (gq, wdq), (gk, wdk), (gv, wdv)):
        g = got.numpy()
        assert np.isfinite(g).all()
        assert rel_fro(g, want) <= TOL_GEMM
    assert np.max(np.abs(lse.numpy() - wlse)) <= 1e-4 * np.abs(wlse).max()


def test_sdpa_more_head_blocks_than_a_grid_dimension_holds(hip, oracle, rng):
    """66000 [32, 64] blocks: the MFMA kernels number their workgroups along one grid dimension, so the 65535 limit of the
    other two does not apply; first and last blocks against float64, forward and backward."""
    bh, s, d = 66000, 32, 64
    q, k, v, go = (rng.standard_normal((bh, s, d), dtype=np.float32) for _ in range(4))
    dq_, dk_, dv_, dgo = dev(hip, q), dev(hip, k), dev(hip, v), dev(hip, go)
    o, lse = hip.empty((bh, s, d)), hip.empty((bh, s))
    scale = 0.125
    hip.check(hip.bh_sdpa_forward(dq_.ptr, dk_.ptr, dv_.ptr, scale, 1, o.ptr, lse.ptr, None, bh, s, d))
    gq, gk, gv = hip.empty((bh, s, d)), hip.empty((bh, s, d)), hip.empty((bh, s, d))
    hip.check(hip.bh_sdpa_backward(dq_.ptr, dk_.ptr, dv_.ptr, o.ptr, lse.ptr, dgo.ptr, scale, 1, gq.ptr, gk.ptr, gv.ptr, bh, s, d))
    got_o, got = o.numpy(), [x.numpy() for x in (gq, gk, gv)]
    for sl in (slice(0, 3), slice(bh - 3, bh), slice(65534, 65537)):
        want_o, _, wattn = oracle.sdpa_forward(q[sl], k[sl], v[sl], scale, 1)
        wq, wk, wv = oracle.sdpa_backward(q[sl], k[sl], v[sl], wattn, go[sl], scale)
        assert rel_fro(got_o[sl], want_o) <= TOL_GEMM
        for g, w in zip(got, (wq, wk, wv)):
            assert rel_fro(g[sl], w) <= TOL_GEMM


@pytest.mark.parametrize("causal", [0, 1])
@pytest.mark.parametrize("bh,s", [(3, 128), (2, 384), (1, 1024), (520, 256), (128, 1024)])
def test_sdpa_with_score_cache(hip, oracle, rng, bh, s, causal):
    """bh_sdpa_forward_cached leaves the scaled scores, bh_sdpa_backward_cached reads them instead of recomputing Q.K^T:
    same outputs as the plain pair to fp32 rounding, against the oracle's attention backward
    (src/layers/attention.c:1417-1520) at the bound only fp32 accumulation meets; (520, 256) also takes the mirrored
    second launch, (128, 1024) is benchmark configuration 4 (a 537 MB cache, sampled heads against the oracle).  Shapes
    without the path are refused."""
    d = 64
    q, k, v, go = (rng.standard_normal((bh, s, d), dtype=np.float32) for _ in range(4))
    dq_, dk_, dv_, dgo = dev(hip, q), dev(hip, k), dev(hip, v), dev(hip, go)
    scale = 0.125
    assert hip.bh_sdpa_score_cache_bytes(bh, s, d) == 4 * bh * s * s
    o, lse, cache = hip.empty((bh, s, d)), hip.empty((bh, s)), hip.to_device(np.full((bh, s, s), np.nan, np.float32))
    hip.check(hip.bh_sdpa_forward_cached(dq_.ptr, dk_.ptr, dv_.ptr, scale, causal, o.ptr, lse.ptr, cache.ptr, bh, s, d))
    o2, lse2 = hip.empty((bh, s, d)), hip.empty((bh, s))
    hip.check(hip.bh_sdpa_forward(dq_.ptr, dk_.ptr, dv_.ptr, scale, causal, o2.ptr, lse2.ptr, None, bh, s, d))
    assert np.array_equal(o.numpy(), o2.numpy()) and np.array_equal(lse.numpy(), lse2.numpy())   # same arithmetic, one more store
    gq, gk, gv = hip.empty((bh, s, d)), hip.empty((bh, s, d)), hip.empty((bh, s, d))
    hip.check(hip.bh_sdpa_backward_cached(dq_.ptr, dk_.ptr, dv_.ptr, o.ptr, lse.ptr, cache.ptr, dgo.ptr, scale, causal,
                                          gq.ptr, gk.ptr, gv.ptr, bh, s, d))
    got = [x.numpy() for x in (gq, gk, gv)]
    assert all(np.isfinite(g).all() for g in got)
    for sl in (slice(0, 2), slice(bh - 1, bh)):
        _, _, wattn = oracle.sdpa_forward(q[sl], k[sl], v[sl], scale, causal)
        for g, w in zip(got, oracle.sdpa_backward(q[sl], k[sl], v[sl], wattn, go[sl], scale)):
            assert rel_fro(g[sl], w) <= FP32_ATTENTION_BOUND
    rq, rk, rv = hip.empty((bh, s, d)), hip.empty((bh, s, d)), hip.empty((bh, s, d))
    hip.check(hip.bh_sdpa_backward(dq_.ptr, dk_.ptr, dv_.ptr, o.ptr, lse.ptr, dgo.ptr, scale, causal, rq.ptr, rk.ptr, rv.ptr, bh, s, d))
    for g, x in zip(got, (rq, rk, rv)):
        assert rel_fro(g, x.numpy()) <= FP32_ATTENTION_BOUND


@pytest.mark.parametrize("causal", [0, 1])
@pytest.mark.parametrize("bh,s,d", [(2, 256, 64), (3, 512, 64), (2, 300, 64), (1, 1000, 64), (2, 77, 64), (2, 32, 64), (1, 1024, 64),
                                    (2, 256, 32), (3, 520, 32), (1, 1024, 32), (2, 77, 32), (2, 32, 32)])
def test_sdpa_backward_with_256_key_workgroups(hip, oracle, rng, bh, s, d, causal):
    """The backward kernel's form with eight wavefronts and 256 keys per workgroup, which the library picks for launches
    that fill the chip twice over, forced on small shapes (whole tiles, ragged lengths, a sequence shorter than one
    tile): the oracle's attention backward (src/layers/attention.c:1417-1520) at the bound only fp32 accumulation meets,
    dK and dV bit for bit those of the 128-key form (the same products in the same order), dQ to rounding (its
    contraction over the keys is cut differently)."""
    q, k, v, go = (rng.standard_normal((bh, s, d)).astype(np.float32) for _ in range(4))
    scale = float(np.float32(1.0) / np.sqrt(np.float32(d)))
    _, _, wattn = oracle.sdpa_forward(q, k, v, scale, causal)
    want = oracle.sdpa_backward(q, k, v, wattn, go, scale)
    dq_, dk_, dv_, dgo = dev(hip, q), dev(hip, k), dev(hip, v), dev(hip, go)
    out, lse = hip.empty((bh, s, d)), hip.empty((bh, s))
    hip.check(hip.bh_sdpa_forward(dq_.ptr, dk_.ptr, dv_.ptr, scale, causal, out.ptr, lse.ptr, None, bh, s, d))
    got = {}
    try:
        for mode in (0, 1):
            hip.check(hip.bh_sdpa_force_wide(mode))
            g = [hip.to_device(np.full((bh, s, d), np.nan, np.float32)) for _ in range(3)]
            hip.check(hip.bh_sdpa_backward(dq_.ptr, dk_.ptr, dv_.ptr, out.ptr, lse.ptr, dgo.ptr, scale, causal,
                                           g[0].ptr, g[1].ptr, g[2].ptr, bh, s, d))
            got[mode] = [x.numpy() for x in g]
    finally:
        hip.check(hip.bh_sdpa_force_wide(-1))
    for g, w in zip(got[1], want):
        assert rel_fro(g, w) <= FP32_ATTENTION_BOUND
    assert np.array_equal(got[0][1], got[1][1]) and np.array_equal(got[0][2], got[1][2])
    assert rel_fro(got[1][0], got[0][0]) <= 1e-6


@pytest.mark.parametrize("bh,s", [(3, 256), (2, 512), (1, 1024)])
def test_sdpa_score_cache_with_256_key_workgroups(hip, oracle, rng, bh, s):
    """The score-cache backward in its 256-key form (unmasked, whole 256-key tiles), forced: against the oracle and the
    128-key form."""
    d, scale = 64, 0.125
    q, k, v, go = (rng.standard_normal((bh, s, d), dtype=np.float32) for _ in range(4))
    dq_, dk_, dv_, dgo = dev(hip, q), dev(hip, k), dev(hip, v), dev(hip, go)
    o, lse, cache = hip.empty((bh, s, d)), hip.empty((bh, s)), hip.empty((bh, s, s))
    hip.check(hip.bh_sdpa_forward_cached(dq_.ptr, dk_.ptr, dv_.ptr, scale, 0, o.ptr, lse.ptr, cache.ptr, bh, s, d))
    got = {}
    try:
        for mode in (0, 1):
            hip.check(hip.bh_sdpa_force_wide(mode))
            g = [hip.to_device(np.full((bh, s, d), np.nan, np.float32)) for _ in range(3)]
            hip.check(hip.bh_sdpa_backward_cached(dq_.ptr, dk_.ptr, dv_.ptr, o.ptr, lse.ptr, cache.ptr, dgo.ptr, scale, 0,
                                                  g[0].ptr, g[1].ptr, g[2].ptr, bh, s, d))
            got[mode] = [x.numpy() for x in g]
    finally:
        hip.check(hip.bh_sdpa_force_wide(-1))
    _, _, wattn = oracle.sdpa_forward(q, k, v, scale, 0)
    for g, w in zip(got[1], oracle.sdpa_backward(q, k, v, wattn, go, scale)):
        assert rel_fro(g, w) <= FP32_ATTENTION_BOUND
    assert np.array_equal(got[0][1], got[1][1]) and np.array_equal(got[0][2], got[1][2])
    assert rel_fro(got[1][0], got[0][0]) <= 1e-6


def test_sdpa_score_cache_refuses_other_shapes(hip):
    assert hip.bh_sdpa_score_cache_bytes(4, 100, 64) == 0 and hip.bh_sdpa_score_cache_bytes(4, 128, 32) == 0
    buf = hip.empty(4 * 128 * 64)
    with pytest.raises(RuntimeError):
        hip.check(hip.bh_sdpa_forward_cached(buf.ptr, buf.ptr, buf.ptr, 0.1, 0, buf.ptr, buf.ptr, buf.ptr, 4, 100, 64))
    with pytest.raises(RuntimeError):
        hip.check(hip.bh_sdpa_backward_cached(buf.ptr, buf.ptr, buf.ptr, buf.ptr, buf.ptr, buf.ptr, buf.ptr, 0.1, 0,
                                              buf.ptr, buf.ptr, buf.ptr, 4, 128, 32))


@pytest.mark.parametrize("bh,s,d", [(512, 384, 64), (512, 300, 64), (256, 512, 64), (600, 256, 64), (512, 384, 32), (600, 300, 32),
                                    (256, 384, 128), (300, 300, 128),
                                    (512, 700, 64), (512, 768, 32)])     # three 256-key tiles: the middle one belongs to the first launch
def test_sdpa_backward_mirrored_second_launch(hip, oracle, rng, bh, s, d):
    """Enough heads for the unmasked backward to run as two launches that share one set of dQ partials (the second
    takes the key tiles in mirrored order and adds to what the first stored): odd tile counts (the middle tile belongs
    to the first launch), a ragged length, an even count; sampled heads against float64, a second call gives the same
    bits (nothing of the first call's partials survives into it).  All three head sizes of the matrix-core kernels."""
    q, k, v, go = (rng.standard_normal((bh, s, d), dtype=np.float32) for _ in range(4))
    dq_, dk_, dv_, dgo = dev(hip, q), dev(hip, k), dev(hip, v), dev(hip, go)
    o, lse = hip.empty((bh, s, d)), hip.empty((bh, s))
    scale = float(1.0 / np.sqrt(d))
    hip.check(hip.bh_sdpa_forward(dq_.ptr, dk_.ptr, dv_.ptr, scale, 0, o.ptr, lse.ptr, None, bh, s, d))
    gq, gk, gv = hip.empty((bh, s, d)), hip.empty((bh, s, d)), hip.empty((bh, s, d))
    hip.check(hip.bh_sdpa_backward(dq_.ptr, dk_.ptr, dv_.ptr, o.ptr, lse.ptr, dgo.ptr, scale, 0, gq.ptr, gk.ptr, gv.ptr, bh, s, d))
    got = [x.numpy() for x in (gq, gk, gv)]
    for sl in (slice(0, 2), slice(bh // 2, bh // 2 + 2), slice(bh - 2, bh)):
        _, _, wattn = oracle.sdpa_forward(q[sl], k[sl], v[sl], scale, 0)
        for g, w in zip(got, oracle.sdpa_backward(q[sl], k[sl], v[sl], wattn, go[sl], scale)):
            assert rel_fro(g[sl], w) <= FP32_ATTENTION_BOUND
    hip.check(hip.bh_sdpa_backward(dq_.ptr, dk_.ptr, dv_.ptr, o.ptr, lse.ptr, dgo.ptr, scale, 0, gq.ptr, gk.ptr, gv.ptr, bh, s, d))
    for g, x in zip(got, (gq, gk, gv)):
        assert np.array_equal(g, x.numpy())


# ------------------------------------------------------------------ convolution / max pooling

CONV_SHAPES = [  # batch, ic, h, w, oc, k, stride, pad
    (2, 3, 7, 6, 4, 3, 1, 1), (3, 1, 8, 8, 5, 3, 1, 0), (2, 2, 9, 7, 3, 2, 2, 1), (1, 4, 5, 5, 2, 5, 1, 2),
    (2, 3, 10, 10, 2, 3, 3, 0), (1, 1, 1, 1, 1, 1, 1, 0),
    (16, 1, 28, 28, 32, 3, 1, 1), (8, 32, 14, 14, 64, 3, 1, 1),      # the two layers of the MNIST network
]


@pytest.mark.parametrize("shape", CONV_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_conv2d_forward_backward(hip, oracle, rng, shape):
    B, ic, h, w, oc, k, stride, pad = shape
    ho, wo = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    x = rng.standard_normal((B, ic, h, w)).astype(np.float32)
    wt = (0.3 * rng.standard_normal((oc, ic, k, k))).astype(np.float32)
    b = rng.standard_normal(oc).astype(np.float32)
    dy = rng.standard_normal((B, oc, ho, wo)).astype(np.float32)
    dx_, dw_, db_, ddy = dev(hip, x), dev(hip, wt), dev(hip, b), dev(hip, dy)
    y = hip.empty((B, oc, ho, wo))
    hip.check(hip.bh_conv2d_forward(dx_.ptr, dw_.ptr, db_.ptr, y.ptr, B, ic, h, w, oc, k, stride, pad))
    assert np.array_equal(y.numpy(), oracle.conv2d_forward(x, wt, b, stride, pad))       # same operation order: bit exact
    hip.check(hip.bh_conv2d_forward(dx_.ptr, dw_.ptr, None, y.ptr, B, ic, h, w, oc, k, stride, pad))
    assert np.array_equal(y.numpy(), oracle.conv2d_forward(x, wt, None, stride, pad))
    for flip in (0, 1):
        gx, gw, gb = hip.empty(x.shape), hip.empty(wt.shape), hip.empty(oc)
        hip.check(hip.bh_conv2d_backward(dx_.ptr, dw_.ptr, ddy.ptr, gx.ptr, gw.ptr, gb.ptr, B, ic, h, w, oc, k, stride, pad, 0, flip))
        o_dx, o_gw, o_gb = oracle.conv2d_backward(x, wt, dy, stride, pad, flip_taps=bool(flip))
        for got, want in ((gx, o_dx), (gw, o_gw), (gb, o_gb)):
            assert np.max(np.abs(got.numpy() - want)) <= TOL_RED * np.abs(want).max(), flip
    # accumulate: a second call adds to the parameter gradients and leaves dx assigned
    first_gw, first_gb = gw.numpy(), gb.numpy()
    hip.check(hip.bh_conv2d_backward(dx_.ptr, dw_.ptr, ddy.ptr, None, gw.ptr, gb.ptr, B, ic, h, w, oc, k, stride, pad, 1, 0))
    assert np.array_equal(gw.numpy(), 2 * first_gw) and np.array_equal(gb.numpy(), 2 * first_gb)     # g + g is exact


@pytest.mark.parametrize("shape", [(64, 1, 28, 28, 32, 3, 1, 1), (64, 32, 14, 14, 64, 3, 1, 1), (64, 4, 28, 28, 16, 5, 1, 2),
                                   (4, 8, 14, 14, 16, 5, 1, 2)], ids=lambda s: "x".join(map(str, s)))
def test_conv2d_forward_output_channel_tiles(hip, oracle, rng, shape):
    """Launches large enough for the forward kernel to keep eight or four output channels per lane (small ones fall
    to two): whatever the tile, the sums run in the reference's order, so the result is bit exact."""
    B, ic, h, w, oc, k, stride, pad = shape
    ho, wo = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    x = rng.standard_normal((B, ic, h, w)).astype(np.float32)
    wt = (0.3 * rng.standard_normal((oc, ic, k, k))).astype(np.float32)
    b = rng.standard_normal(oc).astype(np.float32)
    y = hip.empty((B, oc, ho, wo))
    hip.check(hip.bh_conv2d_forward(dev(hip, x).ptr, dev(hip, wt).ptr, dev(hip, b).ptr, y.ptr, B, ic, h, w, oc, k, stride, pad))
    assert np.array_equal(y.numpy(), oracle.conv2d_forward(x, wt, b, stride, pad))


CONV_MFMA_SHAPES = [  # batch, ic, h, w, oc, k (3 or 5), stride, pad: ragged channel counts, odd channel counts, strides, two LDS stages
    (2, 3, 7, 6, 4, 3, 1, 1), (3, 1, 8, 8, 5, 3, 1, 0), (2, 3, 10, 10, 2, 3, 3, 0), (1, 5, 3, 3, 70, 3, 1, 1),
    (8, 32, 14, 14, 64, 3, 1, 1), (64, 32, 14, 14, 64, 3, 1, 1), (3, 33, 9, 11, 65, 3, 2, 1), (2, 70, 6, 6, 40, 3, 1, 2),
    # more than 256 workgroups: the kernel's two-wavefronts-per-position-tile form
    (40, 33, 20, 21, 65, 3, 1, 1), (64, 64, 28, 28, 64, 3, 1, 1), (30, 70, 31, 29, 130, 3, 2, 1), (40, 5, 21, 20, 10, 3, 1, 1),
    (33, 8, 30, 30, 3, 3, 1, 2),
    # 5x5 kernels (two 16-channel parts per 32-channel stage): one part, a short second part, an odd count behind a full
    # part and behind a full stage, several stages, stride 2, more than 256 workgroups
    (2, 3, 9, 8, 4, 5, 1, 2), (3, 1, 8, 8, 5, 5, 1, 0), (2, 16, 12, 12, 64, 5, 2, 2), (2, 17, 10, 11, 33, 5, 1, 2),
    (4, 20, 14, 14, 70, 5, 2, 1), (2, 33, 9, 9, 65, 5, 1, 2), (8, 32, 28, 28, 64, 5, 2, 2), (3, 70, 13, 12, 40, 5, 1, 0),
    (40, 48, 24, 24, 96, 5, 1, 2), (2, 15, 7, 7, 130, 5, 3, 2),
]


@pytest.mark.parametrize("shape", CONV_MFMA_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_conv2d_forward_on_the_matrix_cores(hip, oracle, rng, shape):
    """The opt-in forward (one contraction on the fp32 matrix cores) against the oracle in the reference's order
    (src/layers/conv.c:326-437): equal to fp32 rounding -- the bound is the one only full fp32 accumulation meets."""
    B, ic, h, w, oc, k, stride, pad = shape
    ho, wo = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    x = rng.standard_normal((B, ic, h, w)).astype(np.float32)
    wt = (0.3 * rng.standard_normal((oc, ic, k, k))).astype(np.float32)
    b = rng.standard_normal(oc).astype(np.float32)
    dx_, dw_, db_ = dev(hip, x), dev(hip, wt), dev(hip, b)
    for bias, bias_np in ((db_.ptr, b), (None, None)):
        y = hip.to_device(np.full((B, oc, ho, wo), np.nan, np.float32))
        hip.check(hip.bh_conv2d_forward_mfma(dx_.ptr, dw_.ptr, bias, y.ptr, B, ic, h, w, oc, k, stride, pad))
        want = oracle.conv2d_forward(x, wt, bias_np, stride, pad)
        got = y.numpy()
        assert np.isfinite(got).all()
        assert np.linalg.norm(got - want) <= fp32_gemm_bound(ic * k * k) * np.linalg.norm(want)
        assert np.max(np.abs(got - want)) <= 1e-5 * max(1.0, np.abs(want).max())
    with pytest.raises(RuntimeError):
        hip.check(hip.bh_conv2d_forward_mfma(dx_.ptr, dw_.ptr, None, y.ptr, B, ic, h + 4, w + 4, oc, 7, stride, pad))   # 3x3 and 5x5 only


def test_conv2d_forward_on_the_matrix_cores_random_shapes(hip, oracle):
    """Eighty seeded random shapes (3x3 and 5x5 kernels, channel counts on both sides of the 16- and 32-channel LDS stages and
    the 64-channel tile, odd counts, strides 1-3, paddings 0-2, images from the kernel's size up, position counts that are
    no multiple of the 64-position tile) against the oracle at the fp32 bound."""
    shapes = np.random.default_rng(20250109)
    for case in range(80):
        k = 3 if case < 40 else 5
        B = int(shapes.integers(1, 5))
        ic = int(shapes.choice([1, 2, 3, 7, 8, 16, 31, 32, 33, 48, 65, 70]))
        oc = int(shapes.choice([1, 3, 16, 31, 32, 33, 63, 64, 65, 100, 130]))
        h, w = int(shapes.integers(k, 20)), int(shapes.integers(k, 20))
        stride, pad = int(shapes.integers(1, 4)), int(shapes.integers(0, 3))
        data = np.random.default_rng(1000 + case)
        x = data.standard_normal((B, ic, h, w)).astype(np.float32)
        wt = (0.3 * data.standard_normal((oc, ic, k, k))).astype(np.float32)
        b = data.standard_normal(oc).astype(np.float32)
        ho, wo = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
        y = hip.to_device(np.full((B, oc, ho, wo), np.nan, np.float32))
        hip.check(hip.bh_conv2d_forward_mfma(dev(hip, x).ptr, dev(hip, wt).ptr, dev(hip, b).ptr, y.ptr, B, ic, h, w, oc, k, stride, pad))
        want = oracle.conv2d_forward(x, wt, b, stride, pad)
        got = y.numpy()
        shape = (B, ic, h, w, oc, k, stride, pad)
        assert np.isfinite(got).all(), shape
        assert np.max(np.abs(got - want)) <= 1e-5 * max(1.0, np.abs(want).max()), shape


def test_conv2d_refuses_bad_shapes(hip):
    p = hip.empty(16)
    assert hip.bh_conv2d_forward(p.ptr, p.ptr, None, p.ptr, 1, 1, 2, 2, 1, 3, 1, 0) == -1       # kernel larger than image
    assert hip.bh_conv2d_forward(p.ptr, p.ptr, None, p.ptr, 1, 1, 2, 2, 1, 1, 0, 0) == -1       # stride 0
    assert hip.bh_conv2d_forward(None, p.ptr, None, p.ptr, 1, 1, 2, 2, 1, 1, 1, 0) == -1
    assert hip.bh_conv2d_forward(None, None, None, None, 0, 1, 2, 2, 1, 1, 1, 0) == 0           # empty batch: nothing to do
    assert hip.bh_maxpool2d_forward(p.ptr, p.ptr, p.ptr, 1, 2, 2, 3, 1, 0) == -1


@pytest.mark.parametrize("shape", [(2, 3, 8, 8, 2, 2, 0), (1, 2, 7, 9, 3, 2, 1), (2, 1, 6, 6, 3, 1, 0), (1, 2, 5, 5, 2, 2, 1),
                                   (16, 32, 28, 28, 2, 2, 0)], ids=lambda s: "x".join(map(str, s)))
def test_maxpool2d_forward_backward(hip, oracle, rng, shape):
    B, ch, h, w, pool, stride, pad = shape
    ho, wo = (h + 2 * pad - pool) // stride + 1, (w + 2 * pad - pool) // stride + 1
    x = rng.standard_normal((B, ch, h, w)).astype(np.float32)
    x[0, 0, :2, :2] = 1.5                                    # ties: first maximum in scan order
    x = np.maximum(x, 0) if B > 2 else x                     # post-ReLU input has many tied zeros
    dy = rng.standard_normal((B, ch, ho, wo)).astype(np.float32)
    dx_, ddy = dev(hip, x), dev(hip, dy)
    y, arg, gx = hip.empty((B, ch, ho, wo)), hip.empty((B, ch, ho, wo), np.int32), hip.empty(x.shape)
    hip.check(hip.bh_maxpool2d_forward(dx_.ptr, y.ptr, arg.ptr, B * ch, h, w, pool, stride, pad))
    hip.check(hip.bh_maxpool2d_backward(ddy.ptr, arg.ptr, gx.ptr, B * ch, h, w, pool, stride, pad))
    o_y, o_arg = oracle.maxpool2d_forward(x, pool, stride, pad)
    assert np.array_equal(y.numpy(), o_y)
    plane = (np.arange(B * ch) * h * w).reshape(B, ch, 1, 1)
    assert np.array_equal(arg.numpy().astype(np.int64) + plane, o_arg)
    assert np.array_equal(gx.numpy(), oracle.maxpool2d_backward(dy, o_arg, x.shape))


def test_zero_multi(hip, rng):
    sizes = [1, 3, 4, 1000, 4097, 100352, 128, 1280, 10]
    arrs = [dev(hip, rng.standard_normal(n).astype(np.float32)) for n in sizes]
    guard = dev(hip, np.ones(8, np.float32))
    ptrs = (C.c_void_p * len(sizes))(*[a.ptr for a in arrs])
    ns = (C.c_int64 * len(sizes))(*sizes)
    hip.check(hip.bh_zero_multi(ptrs, ns, len(sizes)))
    for a in arrs:
        assert not a.numpy().any()
    assert guard.numpy().tolist() == [1.0] * 8
    # an unaligned view (offset by one float) and a zero-length entry
    base = dev(hip, np.ones(1001, np.float32))
    ptrs2 = (C.c_void_p * 2)(base.ptr + 4, base.ptr)
    ns2 = (C.c_int64 * 2)(999, 0)
    hip.check(hip.bh_zero_multi(ptrs2, ns2, 2))
    got = base.numpy()
    assert got[0] == 1 and got[1000] == 1 and not got[1:1000].any()
    assert hip.bh_zero_multi(None, None, 0) == 0


@pytest.mark.parametrize("n,offset", [(1, 0), (1000, 0), (1003, 1), (1 << 20, 0), (4099, 3)])
def test_device_to_device_copy(hip, rng, n, offset):
    """bh_memcpy_d2d: bit-preserving (NaN payloads, -0.0), any float alignment, odd byte counts through the runtime."""
    src = rng.standard_normal(n + 8).astype(np.float32)
    src[:3] = [np.nan, -0.0, np.inf]
    bits = src.view(np.uint32).copy()
    bits[0] = 0x7FC12345                                     # a NaN with a payload
    src = bits.view(np.float32)
    d_src, d_dst = dev(hip, src), dev(hip, np.zeros(n + 8, np.float32))
    hip.check(hip.bh_memcpy_d2d(d_dst.ptr + 4 * offset, d_src.ptr + 4 * offset, 4 * n))
    got = d_dst.numpy().view(np.uint32)
    assert np.array_equal(got[offset:offset + n], bits[offset:offset + n])
    assert not got[:offset].any() and not got[offset + n:].any()
    hip.check(hip.bh_memcpy_d2d(d_dst.ptr + 1, d_src.ptr + 1, 6))          # not whole floats: runtime copy
    assert np.array_equal(d_dst.numpy().view(np.uint8)[1:7], src.view(np.uint8)[1:7])


def test_gemm_with_very_wide_leading_dimensions(hip):
    """The MFMA tiles address an operand tile with 32-bit byte offsets from the tile's first row when they stream it
    straight to LDS; a leading dimension of 2^22 or more does not fit that and takes the register-staged loader.  Both
    sides of the limit, operands that are windows of much wider rows, against float64."""
    rng = np.random.default_rng(77)
    for ld, (ta, tb, m, n, k) in (((1 << 22) - 4, (0, 1, 8, 8, 64)), (1 << 22, (0, 1, 8, 8, 64)), ((1 << 22) + 8, (0, 0, 4, 128, 32)),
                                  (1 << 22, (1, 0, 128, 64, 4))):
        ra = k if ta else m
        rb = n if tb else k
        ca, cb = (m if ta else k), (k if tb else n)
        lda = ld if ra * ld * 4 <= (1 << 28) else ca
        ldb = ld if lda == ca else cb                      # one wide operand per case keeps the buffers small
        a = rng.standard_normal((ra, lda)).astype(np.float32)
        b = rng.standard_normal((rb, ldb)).astype(np.float32)
        A = a[:, :ca].T if ta else a[:, :ca]
        B = b[:, :cb].T if tb else b[:, :cb]
        want = A.astype(np.float64) @ B.astype(np.float64)
        dc = hip.zeros((m, n))
        for cfg in (-1, 1, 4, 7):                          # the heuristic, and the MFMA tiles pinned
            hip.bh_gemm_force_config(cfg)
            try:
                hip.check(hip.bh_gemm(ta, tb, m, n, k, dev(hip, a).ptr, lda, dev(hip, b).ptr, ldb, dc.ptr, n, None, 0, 1))
            finally:
                hip.bh_gemm_force_config(-1)
            assert rel_fro(dc.numpy(), want) <= TOL_GEMM, (ld, ta, tb, m, n, k, cfg)
        _KEEP.clear()


def test_gemm_random_sweep_with_padded_leading_dimensions(hip):
    """Seeded sweep over shapes, layouts, epilogues and leading dimensions wider than the rows (every kernel behind
    bh_gemm must honour lda / ldb / ldc), against float64."""
    rng = np.random.default_rng(4242)
    dims = [1, 3, 4, 16, 31, 64, 100, 128, 192, 256, 260, 384, 512, 700]
    ks = [1, 5, 16, 32, 48, 100, 128, 256, 400, 1024]
    for case in range(80):
        m, n, k = (int(rng.choice(dims)), int(rng.choice(dims)), int(rng.choice(ks)))
        ta, tb = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        pad_a, pad_b, pad_c = (int(rng.choice([0, 0, 4, 8, 3])) for _ in range(3))
        accumulate, bias = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        ra, ca = (k, m) if ta else (m, k)
        rb, cb = (n, k) if tb else (k, n)
        a = rng.standard_normal((ra, ca + pad_a)).astype(np.float32)
        b = rng.standard_normal((rb, cb + pad_b)).astype(np.float32)
        c0 = rng.standard_normal((m, n + pad_c)).astype(np.float32)
        bv = rng.standard_normal(n).astype(np.float32)
        A = a[:, :ca].T if ta else a[:, :ca]
        B = b[:, :cb].T if tb else b[:, :cb]
        want = A.astype(np.float64) @ B.astype(np.float64)
        if bias:
            want = want + bv
        if accumulate:
            want = want + c0[:, :n]
        dc = dev(hip, c0)
        hip.check(hip.bh_gemm(ta, tb, m, n, k, dev(hip, a).ptr, ca + pad_a, dev(hip, b).ptr, cb + pad_b, dc.ptr, n + pad_c,
                              dev(hip, bv).ptr if bias else None, int(accumulate), 1))
        got = dc.numpy()
        tag = (case, ta, tb, m, n, k, pad_a, pad_b, pad_c, accumulate, bias)
        assert rel_fro(got[:, :n], want) <= TOL_GEMM, tag
        assert np.array_equal(got[:, n:], c0[:, n:]), tag            # the padding of C is never written
        _KEEP.clear()


@pytest.mark.parametrize("force", [-1, 1, 2, 3, 4, 7])
def test_gemm_tiles_inside_and_on_the_edge_of_odd_outputs(hip, force):
    """Outputs whose row length is odd or padded, large enough to hold tiles that lie wholly inside them (which store
    through one pointer per lane and immediate offsets) next to tiles cut by the edge (which keep the bounds-checked
    code): every layout, with and without bias and accumulation, on every tile shape, against float64 at the bound only
    fp32 accumulation meets; the padding behind a row of C is never written."""
    rng = np.random.default_rng(97)
    hip.bh_gemm_force_config(force)
    try:
        for (m, n, k) in ((300, 257, 64), (513, 385, 48), (260, 1001, 32)):
            for ta, tb in ((0, 0), (0, 1), (1, 0)):
                for accumulate, bias, pad in ((0, 0, 0), (1, 0, 3), (0, 1, 3), (1, 1, 0)):
                    a = rng.standard_normal((k, m) if ta else (m, k)).astype(np.float32)
                    b = rng.standard_normal((n, k) if tb else (k, n)).astype(np.float32)
                    c0 = rng.standard_normal((m, n + pad)).astype(np.float32)
                    bv = rng.standard_normal(n).astype(np.float32)
                    dc = dev(hip, c0)
                    rc = hip.bh_gemm(ta, tb, m, n, k, dev(hip, a).ptr, m if ta else k, dev(hip, b).ptr, k if tb else n, dc.ptr, n + pad,
                                     dev(hip, bv).ptr if bias else None, accumulate, 1)
                    hip.check(rc)
                    A = a.T if ta else a
                    B = b.T if tb else b
                    want = A.astype(np.float64) @ B.astype(np.float64) + (bv if bias else 0) + (c0[:, :n] if accumulate else 0)
                    got = dc.numpy()
                    tag = (force, m, n, k, ta, tb, accumulate, bias, pad)
                    assert np.abs(got[:, :n] - want).max() <= 2e-6 * np.abs(want).max(), tag
                    assert np.array_equal(got[:, n:], c0[:, n:]), tag
                    _KEEP.clear()
    finally:
        hip.bh_gemm_force_config(-1)
