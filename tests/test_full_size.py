"""Parity at the full sizes of the five benchmark configurations, through properties that do not need the CPU oracle
to finish a full-size run: float64 checks on sampled rows / columns / heads / elements, exact scaling (linearity in
powers of two), independence of heads and of batch elements, and bit-exact Adam on sampled positions (the update is
elementwise, so a sample checks the same arithmetic as the whole).  Tolerances are the path's: 1e-5 elementwise,
1e-4 reductions and LayerNorm, 1e-3 relative Frobenius for GEMM and attention gradients.
"""
import math

import numpy as np
import pytest

import boat_cases as bc
from oracle_lib import rel_fro

pytestmark = pytest.mark.gpu

TOL_EW, TOL_RED, TOL_GEMM = 1e-5, 1e-4, 1e-3


def normal(rng, shape, std=1.0):
    a = rng.standard_normal(shape, dtype=np.float32)
    if std != 1.0:
        a *= np.float32(std)
    return a


def test_config2_dense_backward_full_size(hip):
    """X[8192x4096], W[4096x4096], dY[8192x4096]: sampled rows of dX and columns of dW against float64, db against the
    float64 column sum, and exact scaling: doubling dY doubles all three results bit for bit."""
    M, K, N = 8192, 4096, 4096
    rng = np.random.default_rng(2)
    X, W, dY = normal(rng, (M, K)), normal(rng, (K, N), 0.02), normal(rng, (M, N))
    dXd, dWd, dBd = hip.empty((M, K)), hip.zeros((K, N)), hip.zeros(N)
    Xd, Wd, dYd = hip.to_device(X), hip.to_device(W), hip.to_device(dY)
    hip.check(hip.bh_dense_backward(Xd.ptr, Wd.ptr, dYd.ptr, dXd.ptr, dWd.ptr, dBd.ptr, M, K, N, 0))
    dX, dW, dB = dXd.numpy(), dWd.numpy(), dBd.numpy()
    rows = rng.choice(M, 6, replace=False)
    want = dY[rows].astype(np.float64) @ W.astype(np.float64).T
    assert rel_fro(dX[rows], want) <= TOL_GEMM
    cols = rng.choice(N, 4, replace=False)
    want = X.astype(np.float64).T @ dY[:, cols].astype(np.float64)
    assert rel_fro(dW[:, cols], want) <= TOL_GEMM
    want = dY.astype(np.float64).sum(0)
    assert np.max(np.abs(dB - want)) <= TOL_RED * np.abs(want).max()
    # accumulate = 1 adds the same contribution again: exactly twice the first result
    hip.check(hip.bh_dense_backward(Xd.ptr, Wd.ptr, dYd.ptr, None, dWd.ptr, dBd.ptr, M, K, N, 1))
    assert np.array_equal(dWd.numpy(), 2 * dW) and np.array_equal(dBd.numpy(), 2 * dB)
    # linearity with a power of two is exact in floating point
    dY2 = hip.to_device(2 * dY)
    hip.check(hip.bh_dense_backward(Xd.ptr, Wd.ptr, dY2.ptr, dXd.ptr, dWd.ptr, dBd.ptr, M, K, N, 0))
    assert np.array_equal(dXd.numpy(), 2 * dX) and np.array_equal(dWd.numpy(), 2 * dW) and np.array_equal(dBd.numpy(), 2 * dB)


def gelu_grad_f64(x, dy):
    x = x.astype(np.float64)
    cdf = 0.5 * (1.0 + np.vectorize(math.erf)(x / math.sqrt(2.0)))
    pdf = np.exp(-0.5 * x * x) / math.sqrt(2.0 * math.pi)
    return dy.astype(np.float64) * (cdf + x * pdf)


def test_config3_layernorm_and_gelu_backward_full_size(hip):
    """16384 x 4096: LayerNorm dX on sampled rows, dgamma/dbeta over all rows on sampled columns (float64 closed form
    with float64 statistics), and the GELU input gradient on sampled elements."""
    R, H = 16384, 4096
    rng = np.random.default_rng(3)
    x, dy = normal(rng, (R, H)), normal(rng, (R, H))
    gamma = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(H)).astype(np.float32)
    xd, dyd, gd, bd = hip.to_device(x), hip.to_device(dy), hip.to_device(gamma), hip.to_device(beta)
    y, mean, rstd = hip.empty((R, H)), hip.empty(R), hip.empty(R)
    hip.check(hip.bh_layernorm_forward(xd.ptr, gd.ptr, bd.ptr, y.ptr, mean.ptr, rstd.ptr, R, H, 1e-5))
    dx, dg, db = hip.empty((R, H)), hip.zeros(H), hip.zeros(H)
    hip.check(hip.bh_layernorm_backward(xd.ptr, gd.ptr, dyd.ptr, mean.ptr, rstd.ptr, dx.ptr, dg.ptr, db.ptr, R, H, 0))
    mu = x.mean(1, dtype=np.float64)
    var = ((x.astype(np.float64) - mu[:, None]) ** 2).mean(1)
    rs = 1.0 / np.sqrt(var + 1e-5)
    assert np.max(np.abs(mean.numpy() - mu)) <= TOL_RED and np.max(np.abs(rstd.numpy() / rs - 1)) <= TOL_RED
    rows = rng.choice(R, 8, replace=False)
    xh = (x[rows].astype(np.float64) - mu[rows, None]) * rs[rows, None]
    g = dy[rows].astype(np.float64) * gamma
    want = rs[rows, None] * (g - g.mean(1, keepdims=True) - xh * (g * xh).mean(1, keepdims=True))
    got = dx.numpy()[rows]
    assert np.max(np.abs(got - want)) <= TOL_RED * np.abs(want).max()
    assert np.max(np.abs(y.numpy()[rows] - (xh * gamma + beta))) <= TOL_RED * 5
    cols = rng.choice(H, 16, replace=False)
    xh_c = (x[:, cols].astype(np.float64) - mu[:, None]) * rs[:, None]
    want_g = (dy[:, cols].astype(np.float64) * xh_c).sum(0)
    want_b = dy[:, cols].astype(np.float64).sum(0)
    scale = np.abs(dy[:, cols]).sum(0).max()      # the sums cancel: measure against the magnitude that was added up
    assert np.max(np.abs(dg.numpy()[cols] - want_g)) <= TOL_RED * scale
    assert np.max(np.abs(db.numpy()[cols] - want_b)) <= TOL_RED * scale
    # GELU backward, same arrays as pre-activation and upstream gradient
    hip.check(hip.bh_activation_backward(hip.ACT_GELU, xd.ptr, dyd.ptr, dx.ptr, R * H, 0))
    idx = rng.choice(R * H, 20000, replace=False)
    want = gelu_grad_f64(x.reshape(-1)[idx], dy.reshape(-1)[idx])
    got = dx.numpy().reshape(-1)[idx]
    assert np.max(np.abs(got - want)) <= TOL_EW * np.abs(want).max()


def sdpa_backward_f64(q, k, v, do, scale):
    q, k, v, do = (a.astype(np.float64) for a in (q, k, v, do))
    s = q @ k.T * scale
    p = np.exp(s - s.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    dv = p.T @ do
    dp = do @ v.T
    ds = p * (dp - (dp * p).sum(1, keepdims=True)) * scale
    return ds @ k, ds.T @ q, dv, p @ v


def test_config4_attention_backward_full_size(hip):
    """batch 8 x 16 heads, seq 1024, head_dim 64: sampled heads against the float64 textbook backward, and independence
    of heads: changing dO of one head changes nothing, bit for bit, in any other head."""
    BH, S, D = 8 * 16, 1024, 64
    rng = np.random.default_rng(4)
    q, k, v, do = (normal(rng, (BH, S, D)) for _ in range(4))
    qd, kd, vd, dod = (hip.to_device(a) for a in (q, k, v, do))
    o, lse = hip.empty((BH, S, D)), hip.empty((BH, S))
    scale = 1.0 / 8.0
    hip.check(hip.bh_sdpa_forward(qd.ptr, kd.ptr, vd.ptr, scale, 0, o.ptr, lse.ptr, None, BH, S, D))
    dq, dk, dv = hip.empty((BH, S, D)), hip.empty((BH, S, D)), hip.empty((BH, S, D))
    hip.check(hip.bh_sdpa_backward(qd.ptr, kd.ptr, vd.ptr, o.ptr, lse.ptr, dod.ptr, scale, 0, dq.ptr, dk.ptr, dv.ptr, BH, S, D))
    gq, gk, gv, go = dq.numpy(), dk.numpy(), dv.numpy(), o.numpy()
    for h in (0, 77, BH - 1):
        wq, wk, wv, wo = sdpa_backward_f64(q[h], k[h], v[h], do[h], scale)
        assert rel_fro(go[h], wo) <= TOL_GEMM
        assert rel_fro(gq[h], wq) <= TOL_GEMM and rel_fro(gk[h], wk) <= TOL_GEMM and rel_fro(gv[h], wv) <= TOL_GEMM
    do2 = do.copy()
    do2[5] *= -3.0
    hip.check(hip.bh_memcpy_h2d(dod.ptr, do2.ctypes.data, do2.nbytes))
    hip.check(hip.bh_sdpa_backward(qd.ptr, kd.ptr, vd.ptr, o.ptr, lse.ptr, dod.ptr, scale, 0, dq.ptr, dk.ptr, dv.ptr, BH, S, D))
    others = np.arange(BH) != 5
    for got, first in ((dq.numpy(), gq), (dk.numpy(), gk), (dv.numpy(), gv)):
        assert np.array_equal(got[others], first[others])
        assert rel_fro(got[5], -3.0 * first[5].astype(np.float64)) <= TOL_GEMM


def test_config5b_flat_adam_full_size(hip, oracle):
    """268,435,456 parameters, three steps: sampled positions bit for bit against the oracle (the update is elementwise),
    including the first and last elements and both sides of every 2^24 boundary."""
    n = 268435456
    rng = np.random.default_rng(5)
    chunk = 1 << 24
    p0 = normal(rng, chunk, 0.02)
    g0 = normal(rng, chunk, 1e-3)
    p, g, m, v = (hip.empty(n) for _ in range(4))
    for off in range(0, n, chunk):
        hip.check(hip.bh_memcpy_h2d(p.ptr + 4 * off, p0.ctypes.data, 4 * chunk))
        hip.check(hip.bh_memcpy_h2d(g.ptr + 4 * off, g0.ctypes.data, 4 * chunk))
    hip.check(hip.bh_memset_zero(m.ptr, 4 * n))
    hip.check(hip.bh_memset_zero(v.ptr, 4 * n))
    for t in range(3):
        hip.check(hip.bh_adam_update(p.ptr, g.ptr, m.ptr, v.ptr, n, 1e-3, 0.9, 0.999, 1e-8, t))
    sample = np.unique(np.concatenate([np.arange(0, 4096), np.arange(n - 4096, n), rng.integers(0, n, 100000),
                                       np.arange(chunk, n, chunk) - 1, np.arange(chunk, n, chunk)]))
    wp, wm, wv = p0[sample % chunk].copy(), np.zeros(sample.size, np.float32), np.zeros(sample.size, np.float32)
    for t in range(3):
        wp, wm, wv = oracle.adam_update(wp, g0[sample % chunk], wm, wv, 1e-3, 0.9, 0.999, 1e-8, t)
    # read back only the sampled elements: contiguous runs at both ends plus single elements
    got_p = np.empty(sample.size, np.float32)
    got_v = np.empty(sample.size, np.float32)
    one = np.empty(1, np.float32)
    head, tail = 4096, 4096
    buf = np.empty(4096, np.float32)
    hip.check(hip.bh_memcpy_d2h(buf.ctypes.data, p.ptr, 4 * head))
    assert np.array_equal(buf, wp[:head].reshape(-1))
    hip.check(hip.bh_memcpy_d2h(buf.ctypes.data, p.ptr + 4 * (n - tail), 4 * tail))
    assert np.array_equal(buf, wp[-tail:].reshape(-1))
    mid = sample[head:-tail]
    for j, idx in enumerate(mid[:: max(1, mid.size // 2000)]):      # ~2000 scattered single-element reads
        pos = int(np.searchsorted(sample, idx))
        hip.check(hip.bh_memcpy_d2h(one.ctypes.data, p.ptr + 4 * int(idx), 4))
        assert one[0] == wp.reshape(-1)[pos], (idx, one[0], wp.reshape(-1)[pos])
        hip.check(hip.bh_memcpy_d2h(one.ctypes.data, v.ptr + 4 * int(idx), 4))
        assert one[0] == wv.reshape(-1)[pos]
    del p, g, m, v


def test_config5a_block_step_full_size_batch_independence(boat):
    """Pre-LN block d1024 h16 ffn4096 seq 512 batch 16 (one training step through the C API): the loss is finite,
    Adam moves every parameter tensor, and the forward output and input gradient of one batch element equal those of
    the same element run alone (attention mixes positions of one element only) up to the 1/B of the mean loss."""
    from test_block import make_block
    B, S, H, ffn, heads = 16, 512, 1024, 4096, 16
    x, target, p = make_block(11, B, S, H, ffn)
    full = bc.transformer_block_steps(boat, x, target, p, heads, steps=1)[0]
    assert np.isfinite(full["loss"]) and np.isfinite(full["y"]).all() and np.isfinite(full["dx"]).all()
    for name in bc.BLOCK_PARAM_ORDER:
        assert np.isfinite(full["g_" + name]).all() and np.any(full["p_" + name] != p[name]), name
    e = 3
    alone = bc.transformer_block_steps(boat, x[e:e + 1], target[e:e + 1], p, heads, steps=1)[0]
    assert rel_fro(full["y"][e], alone["y"][0]) <= TOL_RED
    assert rel_fro(full["dx"][e] * B, alone["dx"][0]) <= TOL_GEMM          # MSE averages over B times fewer elements
    # parameter gradients add over batch elements: sum of per-element runs == full run, checked on two tensors
    acc_w2 = np.zeros_like(p["w2"], np.float64)
    acc_bq = np.zeros_like(p["bq"], np.float64)
    for i in range(B):
        one = bc.transformer_block_steps(boat, x[i:i + 1], target[i:i + 1], p, heads, steps=1)[0]
        acc_w2 += one["g_w2"]
        acc_bq += one["g_bq"]
    assert rel_fro(full["g_w2"] * B, acc_w2) <= TOL_GEMM and rel_fro(full["g_bq"] * B, acc_bq) <= TOL_GEMM


def test_more_than_two_to_the_31_elements(hip):
    """Flat kernels past the 32-bit element count (2^31 + 4099 floats, 8.6 GB per array): fill, scale, Adam and the
    sum reduction index with 64 bits.  Checked through the tail of the arrays and through sums with known values."""
    n = (1 << 31) + 4099
    tail = 4099 + 1024

    def tail_of(arr):
        out = np.empty(tail, np.float32)
        hip.check(hip.lib.bh_memcpy_d2h(out.ctypes.data, arr.ptr + 4 * (n - tail), 4 * tail), "d2h tail")
        return out

    p, g, m, v = (hip.empty((n,)) for _ in range(4))
    hip.check(hip.bh_fill(p.ptr, 0.5, n))
    hip.check(hip.bh_fill(g.ptr, 0.25, n))
    hip.check(hip.lib.bh_memset_zero(m.ptr, 4 * n))
    hip.check(hip.lib.bh_memset_zero(v.ptr, 4 * n))
    assert np.all(tail_of(p) == 0.5) and np.all(tail_of(v) == 0.0)
    total = hip.empty((1,))
    hip.check(hip.bh_sum_all(g.ptr, total.ptr, n))
    assert abs(float(total.numpy()[0]) - 0.25 * n) <= 1e-6 * 0.25 * n          # partial sums of 0.25 are exact until the final adds
    hip.check(hip.bh_scalar_op(2, g.ptr, 2.0, g.ptr, n))                       # g *= 2, in place
    assert np.all(tail_of(g) == 0.5)
    # first Adam step from zero moments: p -= lr * g / (|g| + eps) up to rounding, the same number everywhere
    hip.check(hip.bh_adam_update(p.ptr, g.ptr, m.ptr, v.ptr, n, 0.01, 0.9, 0.999, 1e-8, 0))
    pt, mt, vt = tail_of(p), tail_of(m), tail_of(v)
    assert np.all(pt == pt[0]) and abs(float(pt[0]) - 0.49) < 1e-6
    assert np.all(mt == mt[0]) and abs(float(mt[0]) - 0.05) < 1e-7 and np.all(vt == vt[0]) and abs(float(vt[0]) - 0.00025) < 1e-8
    first = np.empty(8, np.float32)
    hip.check(hip.lib.bh_memcpy_d2h(first.ctypes.data, p.ptr, 32), "d2h head")
    assert np.all(first == pt[0])


def test_gemm_operand_and_result_past_two_to_the_31_elements(hip):
    """GEMM addressing with 64-bit offsets: an A operand and a C result of 2.29e9 elements each.  Rows of A below and
    above the 2^31-element mark hold different constants, so an offset that wrapped would show as the wrong multiple
    of the column sums of B."""
    rng = np.random.default_rng(11)
    m, k, n = 70000, 32768, 64
    split = 66000                                         # row 65536 starts at element 2^31
    a = hip.empty((m, k))
    hip.check(hip.bh_fill(a.ptr, 1.0, split * k))
    hip.check(hip.bh_fill(a.ptr + 4 * split * k, 2.0, (m - split) * k))
    b = rng.standard_normal((k, n)).astype(np.float32)
    db = hip.to_device(b)
    c = hip.empty((m, n))
    hip.check(hip.bh_gemm(0, 0, m, n, k, a.ptr, k, db.ptr, n, c.ptr, n, None, 0, 1))
    got = c.numpy()
    colsum = b.astype(np.float64).sum(0)
    scale = np.abs(b).astype(np.float64).sum(0).max()
    assert np.abs(got[:split] - colsum).max() <= 1e-5 * scale
    assert np.abs(got[split:] - 2 * colsum).max() <= 2e-5 * scale
    del a, c
    # a result of m x k2 elements past 2^31: C = A2 . B2 with a short contraction; check the first and the last rows
    k2, n2 = 16, 32768
    a2 = rng.standard_normal((m, k2)).astype(np.float32)
    b2 = rng.standard_normal((k2, n2)).astype(np.float32)
    c2 = hip.empty((m, n2))
    da2, db2 = hip.to_device(a2), hip.to_device(b2)
    hip.check(hip.bh_gemm(0, 0, m, n2, k2, da2.ptr, k2, db2.ptr, n2, c2.ptr, n2, None, 0, 1))
    for r0 in (0, 65530, m - 8):
        rows = np.empty((8, n2), np.float32)
        hip.check(hip.lib.bh_memcpy_d2h(rows.ctypes.data, c2.ptr + 4 * r0 * n2, rows.nbytes), "d2h rows")
        want = a2[r0:r0 + 8].astype(np.float64) @ b2.astype(np.float64)
        assert np.abs(rows - want).max() <= 1e-5 * np.abs(want).max()
