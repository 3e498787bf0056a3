"""bh_layernorm_backward_noalloc (the entry point for callers that cannot allocate device memory) against
bh_layernorm_backward, through the C-ABI: same inputs, two calls in a row on the one scratch array, the second with a
smaller input.  Same kernels, same workgroup count for these shapes, so the results must agree bit for bit; the
LayerNorm tolerance of the path (1e-4) is asserted as well, against the float64 oracle.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL_RED = 1e-4


def _case(hip, oracle, rng, rows, hidden, accumulate):
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    dy = rng.standard_normal((rows, hidden)).astype(np.float32)
    _, mean, rstd = oracle.layernorm_forward(x, gamma, None, 1e-5)
    seed_g = rng.standard_normal(hidden).astype(np.float32)
    seed_b = rng.standard_normal(hidden).astype(np.float32)
    keep = [hip.to_device(a) for a in (x, gamma, dy, mean, rstd)]
    args = tuple(d.ptr for d in keep)

    out = {}
    for name, fn in (("alloc", hip.bh_layernorm_backward), ("noalloc", hip.bh_layernorm_backward_noalloc)):
        dx, dg, db = hip.empty((rows, hidden)), hip.to_device(seed_g), hip.to_device(seed_b)
        in_use = hip.bh_bytes_in_use()
        cached = hip.bh_bytes_cached()
        hip.check(fn(*args, dx.ptr, dg.ptr, db.ptr, rows, hidden, accumulate), name)
        if name == "noalloc":
            # nothing was taken from, or returned to, the library's allocator
            assert hip.bh_bytes_in_use() == in_use and hip.bh_bytes_cached() == cached
        out[name] = (dx.numpy(), dg.numpy(), db.numpy())
    for a, b in zip(out["alloc"], out["noalloc"]):
        assert np.array_equal(a, b)
    wdx, wdg, wdb = oracle.layernorm_backward_f64(x, gamma, dy, mean, rstd)
    if accumulate:
        wdg, wdb = wdg + seed_g, wdb + seed_b
    dx, dg, db = out["noalloc"]
    assert np.max(np.abs(dx - wdx)) <= TOL_RED * np.abs(wdx).max()
    assert np.max(np.abs(dg - wdg)) <= TOL_RED * max(1.0, np.abs(wdg).max())
    assert np.max(np.abs(db - wdb)) <= TOL_RED * max(1.0, np.abs(wdb).max())


def test_layernorm_backward_noalloc_two_calls(hip, oracle):
    rng = np.random.default_rng(20251)
    # large first (512 partials of 2 x 4096 floats fill the whole scratch array), then smaller ones that reuse its
    # front part, with leftovers of the first call behind them
    _case(hip, oracle, rng, 2048, 4096, accumulate=0)
    _case(hip, oracle, rng, 37, 1024, accumulate=0)
    _case(hip, oracle, rng, 300, 2048, accumulate=1)
    _case(hip, oracle, rng, 9, 8192, accumulate=0)
    _case(hip, oracle, rng, 5, 12, accumulate=1)


def test_layernorm_backward_noalloc_refuses_what_it_cannot_do(hip):
    rows, hidden = 4, 8196                       # beyond BH_LN_NOALLOC_MAX_HIDDEN
    x = hip.zeros((rows, hidden))
    v = hip.zeros(rows)
    dx = hip.zeros((rows, hidden))
    rc = hip.bh_layernorm_backward_noalloc(x.ptr, None, x.ptr, v.ptr, v.ptr, dx.ptr, None, None, rows, hidden, 0)
    assert rc == -1 and b"not supported" in hip.bh_last_error()
    rows, hidden = 4, 10                         # not a multiple of 4
    rc = hip.bh_layernorm_backward_noalloc(x.ptr, None, x.ptr, v.ptr, v.ptr, dx.ptr, None, None, rows, hidden, 0)
    assert rc == -1 and b"not supported" in hip.bh_last_error()
    # rows == 0 is a no-op that clears the parameter gradients
    g = hip.to_device(np.ones(8, np.float32))
    hip.check(hip.bh_layernorm_backward_noalloc(None, None, None, None, None, None, g.ptr, None, 0, 8, 0))
    assert not g.numpy().any()
