"""Committed golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py from the
compiled reference) against (a) the oracle, bit for bit, on the CPU and (b) the GPU path through
Boat's C API, within the tolerances of the path: 1e-5 max-relative for elementwise/activation/Adam,
1e-4 for reductions and LayerNorm, 1e-3 relative Frobenius for GEMM and attention gradients.

These are the pins that survive where the reference tree is absent (the GPU box).  Two fixtures do
not come from the reference, which ships stubs for them: ln_bwd_ref64 and gelu_ref64 hold float64
autograd results of an independent library.
"""
from pathlib import Path

import numpy as np
import pytest

import boat_cases as bc
from oracle_lib import max_rel, rel_fro
from test_oracle_vs_reference import oracle_mlp_steps

GOLDEN = Path(__file__).resolve().parent / "golden"
TOL_EW, TOL_RED, TOL_GEMM = 1e-5, 1e-4, 1e-3


def load(name):
    with np.load(GOLDEN / f"{name}.npz", allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def same(a, b):
    a, b = np.asarray(a), np.asarray(b)
    return a.shape == b.shape and np.array_equal(a, b)


def close_max(got, want, tol):
    """max |got-want| <= tol * max |want| (absolute floor for all-zero expectations)"""
    want = np.asarray(want, np.float64)
    scale = max(float(np.abs(want).max()) if want.size else 0.0, 1e-30)
    return float(np.max(np.abs(np.asarray(got, np.float64) - want))) <= tol * scale if want.size else True


def att_case(g):
    B, S, H, heads, causal, bias = (int(v) for v in g["meta"])
    w = {n: g["w" + n] for n in "qkvo"}
    b = {n: g["b" + n] for n in "qkvo"} if bias else None
    return (g["xq"], g["xk"], g["xv"]), w, b, heads, bool(causal), [g["dy0"], g["dy1"]]


# ------------------------------------------------------------------ oracle == golden (CPU, bit exact)

def test_oracle_elementwise_golden(oracle):
    g = load("elementwise")
    a, b, dy, x = g["a"], g["b"], g["dy"], g["x"]
    assert same(g["add_da"], dy) and same(g["add_db"], dy)
    assert same(g["sub_da"], dy) and same(g["sub_db"], -dy)
    da, db = oracle.mul_backward(a, b, dy)
    assert same(da, g["mul_da"]) and same(db, g["mul_db"])
    da, db = oracle.div_backward(a, b, dy)
    assert same(da, g["div_da"]) and same(db, g["div_db"])
    assert same(a + b, g["add_out"]) and same(a - b, g["sub_out"]) and same(a * b, g["mul_out"]) and same(a / b, g["div_out"])
    assert same(oracle.relu_forward(x), g["relu_y"]) and same(oracle.relu_backward(x, dy), g["relu_dx"])
    assert g["relu_dx"][0, 0] == 0 and g["relu_dx"][0, 1] == 0 and g["relu_dx"][0, 2] == dy[0, 2]   # 0, -0 -> 0; 1e-30 passes
    y = oracle.sigmoid_forward(x)
    assert same(y, g["sigmoid_y"]) and same(oracle.sigmoid_backward(y, dy), g["sigmoid_dx"])
    y = oracle.tanh_forward(x)
    assert same(y, g["tanh_y"]) and same(oracle.tanh_backward(y, dy), g["tanh_dx"])
    assert np.float32(oracle.sum(x)) == g["sum_y"][0] and np.all(g["sum_dx"] == 1)


def test_oracle_softmax_golden(oracle):
    g = load("softmax")
    for tag in "ab":
        x, dy = g[f"{tag}_x"], g[f"{tag}_dy"]
        y = oracle.softmax_forward(x)
        assert same(y, g[f"{tag}_softmax_y"]) and same(oracle.softmax_backward(y, dy), g[f"{tag}_softmax_dx"])
        y = oracle.log_softmax_forward(x)
        assert same(y, g[f"{tag}_log_softmax_y"]) and same(oracle.log_softmax_backward(y, dy), g[f"{tag}_log_softmax_dx"])
        assert np.allclose(g[f"{tag}_softmax_y"].sum(-1), 1, atol=1e-6)          # tests/unit/test_autodiff.c:393-397


def test_oracle_matmul_golden(oracle):
    g = load("matmul")
    assert same(oracle.matmul(g["a4"], g["b4"]), g["c4"])
    assert same(oracle.transpose_last2(g["a4"]), g["a4_t23"])
    assert same(oracle.transpose_last2(g["a2"]), g["a2_t01"])
    assert same(oracle.matmul(g["a2"], g["b2"]), g["c2"])
    # compute_backward_matmul: dA = dY.B^T, dB = A^T.dY through materialised transposes (autodiff.c:1454-1496)
    assert same(oracle.matmul(g["dy2"], oracle.transpose_last2(g["b2"])), g["da2"])
    assert same(oracle.matmul(oracle.transpose_last2(g["a2"]), g["dy2"]), g["db2"])


def test_oracle_dense_golden(oracle):
    g = load("dense_bwd_accum")
    assert same(oracle.dense_forward(g["x1"], g["w"], g["b"]), g["y1"])
    dx1, gw1, gb1 = oracle.dense_backward(g["x1"], g["w"], g["dy1"])
    dx2, gw2, gb2 = oracle.dense_backward(g["x2"], g["w"], g["dy2"], gw1, gb1)
    for got, key in ((dx1, "dx1"), (gw1, "gw1"), (gb1, "gb1"), (dx2, "dx2"), (gw2, "gw2"), (gb2, "gb2")):
        assert same(got, g[key]), key


def test_oracle_mlp_golden(oracle):
    g = load("mlp_small_3steps")
    hist = oracle_mlp_steps(oracle, g["x"], g["labels"], g["w1"], g["b1"], g["w2"], g["b2"], 3, 1e-3, 0.9, 0.999, 1e-8)
    for t, rec in enumerate(hist):
        assert np.float32(rec["loss"]) == g[f"s{t}_loss"]
        for key in ("gw1", "gb1", "gw2", "gb2", "w1", "b1", "w2", "b2"):
            assert same(rec[key], g[f"s{t}_{key}"]), (t, key)


def config1_inputs(g):
    r1 = np.random.default_rng(int(g["seed"]))
    d_in, d_h, d_out, batch = 784, 128, 10, 64
    x = r1.random((batch, d_in), dtype=np.float32)
    labels = r1.integers(0, d_out, batch)
    lim1, lim2 = np.sqrt(6.0 / (d_in + d_h)), np.sqrt(6.0 / (d_h + d_out))
    w1 = r1.uniform(-lim1, lim1, (d_in, d_h)).astype(np.float32)
    w2 = r1.uniform(-lim2, lim2, (d_h, d_out)).astype(np.float32)

    def chk(arr):
        arr = np.asarray(arr, np.float64)
        return np.array([arr.sum(), np.abs(arr).sum(), (arr * arr).sum()])

    assert np.array_equal(labels, g["labels"]) and np.allclose(np.stack([chk(x), chk(w1), chk(w2)]), g["input_checksums"], rtol=1e-12), \
        "the seeded generator no longer reproduces the fixture's inputs"
    return x, labels, w1, np.zeros(d_h, np.float32), w2, np.zeros(d_out, np.float32), chk


def test_oracle_mlp_config1_golden(oracle):
    g = load("mlp_config1_step")
    x, labels, w1, b1, w2, b2, chk = config1_inputs(g)
    rec = oracle_mlp_steps(oracle, x, labels, w1, b1, w2, b2, 1, 1e-3, 0.9, 0.999, 1e-8)[0]
    assert np.float32(rec["loss"]) == g["loss"]
    for key in ("gb1", "gb2", "gw2", "b1", "b2", "w2"):
        assert same(rec[key], g[key]), key
    assert same(rec["gw1"][:4], g["gw1_rows"]) and same(rec["w1"][:4], g["w1_rows"])
    assert np.array_equal(chk(rec["gw1"]), g["gw1_chk"]) and np.array_equal(chk(rec["w1"]), g["w1_chk"])


@pytest.mark.parametrize("idx", range(4))
def test_oracle_attention_golden(oracle, idx):
    g = load(f"attention_case{idx}")
    xs, w, b, heads, causal, dys = att_case(g)
    out, cache = oracle.attention_forward(*xs, w, b, heads, causal)
    assert same(out, g["out"])
    for t, dy in enumerate(dys):
        r = oracle.attention_backward(*xs, w, b is not None, cache, dy, heads)
        assert same(r["d_query"], g[f"c{t}_dq"]) and same(r["d_key"], g[f"c{t}_dk"]) and same(r["d_value"], g[f"c{t}_dv"])
        for n in "qkvo":
            assert same(r["gw" + n], g[f"c{t}_gw{n}"]), n
            if b is not None:
                assert same(r["gb" + n], g[f"c{t}_gb{n}"]), n


def test_oracle_sdpa_core_golden(oracle):
    g = load("sdpa_core")
    B, S, H, heads = (int(v) for v in g["meta"])
    hd = H // heads
    q, k, v, dy = (g[n].reshape(B * heads, S, hd) for n in ("xq", "xk", "xv", "dy"))
    scale = np.float32(1.0) / np.sqrt(np.float32(hd))
    o, _, attn = oracle.sdpa_forward(q, k, v, scale)
    assert same(o.reshape(B, S, H), g["out"])
    dq, dk, dv = oracle.sdpa_backward(q, k, v, attn, dy, scale)
    assert same(dq.reshape(B, S, H), g["dq"]) and same(dk.reshape(B, S, H), g["dk"]) and same(dv.reshape(B, S, H), g["dv"])


def test_oracle_layernorm_golden(oracle):
    g = load("layernorm_fwd")
    for tag in "ab":
        y, _, _ = oracle.layernorm_forward(g[f"{tag}_x"], g[f"{tag}_gamma"], g[f"{tag}_beta"], 1e-5)
        assert same(y, g[f"{tag}_y"])


def test_oracle_rmsnorm_golden(oracle):
    g = load("rmsnorm_fwd")
    for tag in "abc":
        x = g[f"{tag}_x"]
        assert same(oracle.rmsnorm_forward(x, np.ones(x.shape[-1], np.float32), 1e-6)[0], g[f"{tag}_y"]), tag
        assert same(oracle.rmsnorm_forward(x, None, 1e-3)[0], g[f"{tag}_y_plain"]), tag
    x = g["d_x"].reshape(-1, 8)                      # 4-D input: the reference visits shape0*shape1 = 6 rows only
    y = g["d_y"].reshape(-1, 8)
    assert same(oracle.rmsnorm_forward(x[:6], np.ones(8, np.float32), 1e-6)[0], y[:6]) and not y[6:].any()
    assert not g["zero_y"].any() and not oracle.rmsnorm_forward(g["zero_x"], None, 1e-6)[0].any()


def test_oracle_rmsnorm_backward_against_independent_library(oracle):
    """The reference has no RMSNorm backward (stub, norm.c:404-409): the oracle's float64 closed form is pinned by float64
    autograd vectors of an independent library for y = x/(sqrt(mean(x^2)) + eps)*w, at a small and at a large eps."""
    for tag in "ab":
        g = load(f"rmsnorm_bwd_ref64_{tag}")
        x32, w32, dy32 = (g[k].astype(np.float32) for k in ("x", "w", "dy"))
        dx, dw = oracle.rmsnorm_backward_f64(x32, w32, dy32, float(g["eps"]))
        # inputs are rounded to float32 for the oracle: compare with that rounding's effect allowed for
        assert close_max(dx, g["dx"], 1e-5) and close_max(dw, g["dw"], 1e-5), tag
        y, _ = oracle.rmsnorm_forward(x32, w32, float(g["eps"]))
        assert close_max(y, g["y"], 1e-5)
    # dropping the second term of dx (the derivative of the scale) must fail the same check
    g = load("rmsnorm_bwd_ref64_a")
    s = 1 / (np.sqrt((g["x"] ** 2).mean(-1, keepdims=True)) + float(g["eps"]))
    assert not close_max(s * g["dy"] * g["w"], g["dx"], 1e-3)


def test_oracle_public_sdpa_golden(oracle):
    g = load("sdpa_public")
    for tag in "abc":
        out, _, _ = oracle.sdpa_forward(g[f"{tag}_q"], g[f"{tag}_k"], g[f"{tag}_v"], float(g[f"{tag}_scale"]), bool(g[f"{tag}_causal"]))
        assert same(out, g[f"{tag}_out"]), tag
    assert same(g["three_d_out"], g["three_d_v"])


def c_div(a, b):
    """C's integer division truncates toward zero; numpy's // floors."""
    q = np.abs(a) // np.abs(b)
    return (q * np.sign(a) * np.sign(b)).astype(a.dtype)


def typed_expectations(a, b, scalar):
    """What one C operator per element gives (src/ops/arithmetic.c:197-282, 425-570), written with numpy."""
    dt = a.dtype
    s = dt.type(scalar)                                   # the scalar is narrowed to the element type first
    is_f = dt.kind == "f"
    want = {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b if is_f else c_div(a, np.broadcast_to(b, a.shape)),
            "mod": np.fmod(a, b),
            "add_scalar": a + s, "sub_scalar": a - s, "mul_scalar": a * s, "div_scalar": a / s if is_f else c_div(a, np.full_like(a, s))}
    for k in ("add", "sub", "mul", "div"):
        want[f"{k}_scalar_inplace"] = want[f"{k}_scalar"]
        if a.shape == b.shape:
            want[f"{k}_inplace"] = want[k]
    return {k: np.asarray(v, dt) for k, v in want.items()}


def check_typed(get, tol_pow):
    g = load("typed_ops")
    for tag, dt in (("f64", np.float64), ("i32", np.int32), ("i64", np.int64), ("f32", np.float32)):
        a, b = g[f"{tag}_a"], g[f"{tag}_b"]
        assert a.dtype == dt
        a2 = np.abs(a) + dt(0.25) if dt in (np.float64, np.float32) else a
        for prefix, aa, bb, sc in (("bc", a, b, 2.75), ("eq", a2, np.broadcast_to(b, a.shape).copy(), -1.5 if a.dtype.kind == "f" else 3.0)):
            got = get(tag, prefix, aa, bb, sc)
            for key, want in typed_expectations(aa, bb, sc).items():
                assert got[key].dtype == dt and np.array_equal(got[key], want), (tag, prefix, key)
            if a.dtype.kind == "f":
                with np.errstate(invalid="ignore"):
                    pw = np.power(aa.astype(np.float64), dt(sc))
                assert max_rel(got["pow_scalar"][np.isfinite(got["pow_scalar"])],
                               pw[np.isfinite(got["pow_scalar"])]) <= tol_pow[tag], (tag, prefix)
                assert np.array_equal(np.isnan(got["pow_scalar"]), np.isnan(pw))
            else:
                assert bool(got["pow_scalar_is_null"])


def test_typed_arithmetic_fixture_is_one_c_operator_per_element():
    """The non-float32 elementwise ops have no oracle routine: the expectation is numpy's IEEE / two's-complement operator
    per element, and this test pins that expectation on what the compiled reference produced (tests/golden/typed_ops.npz)."""
    g = load("typed_ops")
    check_typed(lambda tag, prefix, a, b, s: {k[len(tag) + len(prefix) + 2:]: g[k] for k in g if k.startswith(f"{tag}_{prefix}_")},
                {"f64": 1e-14, "f32": 1e-6})


def test_oracle_adam_golden(oracle):
    g = load("adam_traj")
    for i in range(3):
        p = g[f"p{i}"].copy()
        m, v = np.zeros_like(p), np.zeros_like(p)
        for t in range(10):
            lr = 3e-3 if t >= 5 else 1e-2
            p, m, v = oracle.adam_update(p, g[f"g{i}"][t], m, v, lr, 0.9, 0.999, 1e-8, t)
            assert same(p.reshape(g[f"p{i}"].shape), g[f"traj{i}"][t]), (i, t)


@pytest.mark.parametrize("kind", ["rmsprop", "adagrad"])
def test_oracle_rmsprop_adagrad_golden(oracle, kind):
    from test_oracle_vs_reference import oracle_sq_trajectory
    g = load(f"{kind}_traj")
    params = [g[f"p{i}"] for i in range(3)]
    grads = [[g[f"g{i}"][t] for i in range(3)] for t in range(10)]
    want = oracle_sq_trajectory(oracle, kind, params, grads, 1e-2, 0.99, 1e-8, lr_change=(5, 3e-3))
    for t in range(10):
        for i in range(3):
            assert same(want[t][i], g[f"traj{i}"][t]), (t, i)


def test_oracle_f64_closed_forms_against_library_vectors(oracle):
    """LayerNorm backward and GELU: no reference implementation; the oracle's float64 closed forms
    against float64 autograd vectors of an independent library."""
    g = load("ln_bwd_ref64")
    x32 = g["x"].astype(np.float32)
    _, mean, rstd = oracle.layernorm_forward(x32, g["gamma"].astype(np.float32), g["beta"].astype(np.float32), 1e-5)
    dx, dg, db = oracle.layernorm_backward_f64(x32, g["gamma"].astype(np.float32), g["dy"].astype(np.float32), mean, rstd)
    assert close_max(dx, g["dx"], 1e-5) and close_max(dg, g["dgamma"], 1e-5) and close_max(db, g["dbeta"], 1e-5)
    g = load("gelu_ref64")
    x32, dy32 = g["x"].astype(np.float32), g["dy"].astype(np.float32)
    assert close_max(oracle.gelu_forward_f64(x32), g["y"], 1e-6)
    assert close_max(oracle.gelu_backward_f64(x32, dy32), g["dx"], 1e-6)


def cnn_case(g):
    p = {k[2:]: g[k] for k in g if k.startswith("p_")}
    return g["x"], g["labels"], p


def test_oracle_conv_pool_cnn_golden(oracle):
    from test_oracle_vs_reference import CNN_KEYS, oracle_cnn_grads
    g = load("conv_layer")
    for i in range(3):
        stride, pad = int(g[f"c{i}_meta"][6]), int(g[f"c{i}_meta"][7])
        x, w, b = g[f"c{i}_x"], g[f"c{i}_w"], g[f"c{i}_b"]
        assert same(oracle.conv2d_forward(x, w, b, stride, pad), g[f"c{i}_y"])
        for j in range(2):
            dx, gw, gb = oracle.conv2d_backward(x, w, g[f"c{i}_dy{j + 1}"], stride, pad, flip_taps=True)
            assert same(dx, g[f"c{i}_dx{j}"]) and same(gw, g[f"c{i}_gw{j}"]) and same(gb, g[f"c{i}_gb{j}"]), (i, j)
    g = load("pool_layer")
    for i in range(4):
        k, stride, pad = (int(v) for v in g[f"p{i}_meta"])
        y, arg = oracle.maxpool2d_forward(g[f"p{i}_x"], k, stride, pad)
        assert same(y, g[f"p{i}_y"]) and same(oracle.maxpool2d_backward(g[f"p{i}_dy"], arg, g[f"p{i}_x"].shape), g[f"p{i}_dx"]), i
    g = load("cnn_chain")
    x, labels, p = cnn_case(g)
    want = oracle_cnn_grads(oracle, x, labels, p, flip_taps=True)
    assert np.float32(want["loss"]) == g["loss"]
    for key in CNN_KEYS:
        assert same(want[key], g[key]), key


def test_checkpoint_fixture_is_the_documented_layout():
    """The file the reference wrote (examples/mnist/mnist_autodiff.c:775-927 over its API) is magic, version and eight
    (null marker, ndim, dims, dtype, payload) records of the parameters; reading it back gave the same logits as the
    model the parameters were set into directly."""
    g, c = load("cnn_checkpoint"), load("cnn_chain")
    _x, _labels, p = cnn_case(c)
    assert g["content"].tobytes() == bc.checkpoint_bytes(p)
    assert same(g["x"], c["x"]) and same(g["logits"], c["logits"])


def test_fanout_fixture_documents_the_reference_behaviour():
    g = load("fanout_divergence")
    assert same(g["ref_da"], 4 * g["b"]) and same(g["ref_db"], 4 * g["a"])


# ------------------------------------------------------------------ GPU path == golden

@pytest.mark.gpu
def test_gpu_elementwise_golden(boat):
    g = load("elementwise")
    a, b, dy, x = g["a"], g["b"], g["dy"], g["x"]
    for op in ("add", "sub", "mul", "div"):
        c, da, db = bc.binary_grads(boat, op, a, b, dy)
        # the device keeps the reference's operation order for these: bit exact
        assert same(c, g[f"{op}_out"]) and same(da, g[f"{op}_da"]) and same(db, g[f"{op}_db"]), op
    y, dx = bc.unary_grads(boat, "relu", x, dy)
    assert same(y, g["relu_y"]) and same(dx, g["relu_dx"])
    for op in ("sigmoid", "tanh"):
        y, dx = bc.unary_grads(boat, op, x, dy)
        assert max_rel(y, g[f"{op}_y"]) <= TOL_EW and close_max(dx, g[f"{op}_dx"], TOL_EW), op
    y, dx = bc.unary_grads(boat, "sum", x)
    assert abs(float(y[0]) - float(g["sum_y"][0])) <= TOL_RED * np.abs(x).sum() and same(dx, g["sum_dx"])


@pytest.mark.gpu
def test_gpu_softmax_golden(boat):
    g = load("softmax")
    for tag in "ab":
        for op in ("softmax", "log_softmax"):
            y, dx = bc.unary_grads(boat, op, g[f"{tag}_x"], g[f"{tag}_dy"])
            assert close_max(y, g[f"{tag}_{op}_y"], TOL_RED), (tag, op)
            assert close_max(dx, g[f"{tag}_{op}_dx"], TOL_RED), (tag, op)


@pytest.mark.gpu
def test_gpu_matmul_and_dense_golden(boat):
    g = load("matmul")
    assert rel_fro(bc.matmul(boat, g["a4"], g["b4"]), g["c4"]) <= TOL_GEMM
    assert same(bc.transpose(boat, g["a4"], 2, 3), g["a4_t23"]) and same(bc.transpose(boat, g["a2"], 0, 1), g["a2_t01"])
    c, da, db = bc.matmul_grads(boat, g["a2"], g["b2"], g["dy2"])
    assert rel_fro(c, g["c2"]) <= TOL_GEMM and rel_fro(da, g["da2"]) <= TOL_GEMM and rel_fro(db, g["db2"]) <= TOL_GEMM
    g = load("dense_bwd_accum")
    assert rel_fro(bc.dense_forward(boat, g["x1"], g["w"], g["b"]), g["y1"]) <= TOL_GEMM
    first, second = bc.dense_backward_twice(boat, g["w"], g["b"], g["x1"], g["dy1"], g["x2"], g["dy2"])
    for got, keys in ((first, ("dx1", "gw1", "gb1")), (second, ("dx2", "gw2", "gb2"))):
        for arr, key in zip(got, keys):
            assert rel_fro(arr, g[key]) <= TOL_GEMM, key


@pytest.mark.gpu
def test_gpu_mlp_golden(boat):
    g = load("mlp_small_3steps")
    hist = bc.mlp_ce_adam(boat, g["x"], g["labels"], g["w1"], g["b1"], g["w2"], g["b2"], steps=3)
    assert abs(hist[0]["loss"] - float(g["s0_loss"])) <= TOL_RED * abs(float(g["s0_loss"]))
    for key in ("gw1", "gw2", "gb1", "gb2"):
        assert rel_fro(hist[0][key], g[f"s0_{key}"]) <= TOL_GEMM, key
    for t in range(3):   # a weight whose gradient is rounding noise may step the other way: bounded by 2*lr per step
        for key in ("w1", "b1", "w2", "b2"):
            assert np.max(np.abs(hist[t][key] - g[f"s{t}_{key}"])) <= 2.1e-3 * (t + 1), (t, key)
        assert abs(hist[t]["loss"] - float(g[f"s{t}_loss"])) <= 5e-3


@pytest.mark.gpu
def test_gpu_mlp_config1_golden(boat):
    """Benchmark configuration 1 at its real size: MLP 784-128-10, batch 64, forward + backward + one Adam step."""
    g = load("mlp_config1_step")
    x, labels, w1, b1, w2, b2, chk = config1_inputs(g)
    rec = bc.mlp_ce_adam(boat, x, labels, w1, b1, w2, b2, steps=1)[0]
    assert abs(rec["loss"] - float(g["loss"])) <= TOL_RED * abs(float(g["loss"]))
    assert rel_fro(rec["gw2"], g["gw2"]) <= TOL_GEMM and rel_fro(rec["gw1"][:4], g["gw1_rows"]) <= TOL_GEMM
    assert close_max(rec["gb1"], g["gb1"], TOL_RED) and close_max(rec["gb2"], g["gb2"], TOL_RED)
    got_chk, want_chk = chk(rec["gw1"]), g["gw1_chk"]
    assert abs(got_chk[1] - want_chk[1]) <= TOL_GEMM * want_chk[1] and abs(got_chk[2] - want_chk[2]) <= TOL_GEMM * want_chk[2]
    for key in ("w2", "b1", "b2"):
        assert np.max(np.abs(rec[key] - g[key])) <= 2.1e-3, key
    resolved = np.abs(g["gw2"]) > 1e-4 * np.abs(g["gw2"]).max()
    assert np.max(np.abs(rec["w2"] - g["w2"])[resolved]) <= 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("idx", range(4))
def test_gpu_attention_golden(boat, idx):
    g = load(f"attention_case{idx}")
    xs, w, b, heads, causal, dys = att_case(g)
    out, results = bc.attention(boat, *xs, w, b, heads, causal, dys)
    assert rel_fro(out, g["out"]) <= TOL_GEMM
    for t, rec in enumerate(results):     # the second call overwrites the parameter gradients
        for key in ("dq", "dk", "dv"):
            assert rel_fro(rec[key], g[f"c{t}_{key}"]) <= TOL_GEMM, (t, key)
        for n in "qkvo":
            assert rel_fro(rec["gw" + n], g[f"c{t}_gw{n}"]) <= TOL_GEMM, (t, n)
            if b is not None:
                assert rel_fro(rec["gb" + n], g[f"c{t}_gb{n}"]) <= TOL_GEMM, (t, n)


@pytest.mark.gpu
def test_gpu_sdpa_core_golden(boat):
    g = load("sdpa_core")
    B, S, H, heads = (int(v) for v in g["meta"])
    eye = {n: np.eye(H, dtype=np.float32) for n in "qkvo"}
    out, (rec,) = bc.attention(boat, g["xq"], g["xk"], g["xv"], eye, None, heads, False, [g["dy"]])
    assert rel_fro(out, g["out"]) <= TOL_GEMM
    for key in ("dq", "dk", "dv"):
        assert rel_fro(rec[key], g[key]) <= TOL_GEMM, key


@pytest.mark.gpu
def test_gpu_layernorm_golden(boat):
    g = load("layernorm_fwd")
    for tag in "ab":
        y = bc.layernorm_forward(boat, g[f"{tag}_x"], g[f"{tag}_gamma"], g[f"{tag}_beta"], 1e-5)
        assert close_max(y, g[f"{tag}_y"], TOL_RED), tag


@pytest.mark.gpu
def test_gpu_rmsnorm_golden(boat):
    g = load("rmsnorm_fwd")
    for tag in "abcd":
        assert close_max(bc.rmsnorm_forward(boat, g[f"{tag}_x"], 1e-6), g[f"{tag}_y"], TOL_RED), tag
        assert close_max(bc.rmsnorm_forward(boat, g[f"{tag}_x"], 1e-3, affine=False), g[f"{tag}_y_plain"], TOL_RED), tag
    assert not bc.rmsnorm_forward(boat, g["d_x"], 1e-6).reshape(-1, 8)[6:].any()     # rows the reference does not visit stay zero
    assert not bc.rmsnorm_forward(boat, g["zero_x"], 1e-6).any()


@pytest.mark.gpu
def test_gpu_public_sdpa_golden(boat):
    g = load("sdpa_public")
    for tag in "abc":                                 # c has head size 64: the matrix-core kernel
        out = bc.sdpa_public(boat, g[f"{tag}_q"], g[f"{tag}_k"], g[f"{tag}_v"], float(g[f"{tag}_scale"]), bool(g[f"{tag}_causal"]))
        assert rel_fro(out, g[f"{tag}_out"]) <= TOL_GEMM and close_max(out, g[f"{tag}_out"], 1e-5), tag
    assert same(bc.sdpa_public(boat, g["three_d_q"], g["three_d_q"], g["three_d_v"], 0.5, False), g["three_d_v"])


@pytest.mark.gpu
def test_gpu_typed_arithmetic_golden(boat):
    """float64 / int32 / int64 (and float32 through the same entry points) elementwise ops, bit for bit against the
    reference's results; pow within the tolerance of the device's pow routine."""
    g = load("typed_ops")

    def run(tag, prefix, a, b, s):
        got = bc.typed_arithmetic(boat, a, b, s)
        for key, val in got.items():
            ref_val = g[f"{tag}_{prefix}_{key}"]
            if key == "pow_scalar":
                continue
            assert np.array_equal(val, ref_val), (tag, prefix, key)
        return got
    check_typed(run, {"f64": 1e-13, "f32": 2e-6})


@pytest.mark.gpu
def test_gpu_adam_golden_bit_exact(boat):
    g = load("adam_traj")
    params = [g[f"p{i}"] for i in range(3)]
    grads = [[g[f"g{i}"][t] for i in range(3)] for t in range(10)]
    traj, zeroed = bc.adam_trajectory(boat, params, grads, lr=1e-2, lr_change=(5, 3e-3))
    for t in range(10):
        for i in range(3):
            assert same(traj[t][i], g[f"traj{i}"][t]), (t, i)
    assert all(not z.any() for z in zeroed)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["rmsprop", "adagrad"])
def test_gpu_rmsprop_adagrad_golden_bit_exact(boat, kind):
    g = load(f"{kind}_traj")
    params = [g[f"p{i}"] for i in range(3)]
    grads = [[g[f"g{i}"][t] for i in range(3)] for t in range(10)]
    traj, zeroed = bc.adam_trajectory(boat, params, grads, lr=1e-2, beta1=0.99, eps=1e-8, lr_change=(5, 3e-3), kind=kind)
    for t in range(10):
        for i in range(3):
            assert same(traj[t][i], g[f"traj{i}"][t]), (t, i)
    assert all(not z.any() for z in zeroed)
    assert not boat.boat_rmsprop_optimizer_create(0.0, 0.9, 1e-8) and not boat.boat_rmsprop_optimizer_create(0.1, 1.0, 1e-8)
    assert not boat.boat_adagrad_optimizer_create(0.1, 0.0)


@pytest.mark.gpu
def test_gpu_ln_backward_and_gelu_against_library_vectors(hip):
    g = load("ln_bwd_ref64")
    x, gamma, beta, dy = (g[k].astype(np.float32) for k in ("x", "gamma", "beta", "dy"))
    rows, hidden = x.shape
    dx_, dg_, db_ = hip.to_device(x), hip.to_device(gamma), hip.to_device(beta)
    y, mean, rstd = hip.empty((rows, hidden)), hip.empty(rows), hip.empty(rows)
    hip.check(hip.bh_layernorm_forward(dx_.ptr, dg_.ptr, db_.ptr, y.ptr, mean.ptr, rstd.ptr, rows, hidden, 1e-5))
    assert close_max(y.numpy(), g["y"], TOL_RED)
    ddy = hip.to_device(dy)
    gdx, gdg, gdb = hip.empty((rows, hidden)), hip.empty(hidden), hip.empty(hidden)
    hip.check(hip.bh_layernorm_backward(dx_.ptr, dg_.ptr, ddy.ptr, mean.ptr, rstd.ptr, gdx.ptr, gdg.ptr, gdb.ptr, rows, hidden, 0))
    assert close_max(gdx.numpy(), g["dx"], TOL_RED) and close_max(gdg.numpy(), g["dgamma"], TOL_RED) and close_max(gdb.numpy(), g["dbeta"], TOL_RED)
    g = load("gelu_ref64")
    x, dy = g["x"].astype(np.float32), g["dy"].astype(np.float32)
    dxv, ddy = hip.to_device(x), hip.to_device(dy)
    yv, gx = hip.empty(x.shape), hip.empty(x.shape)
    hip.check(hip.bh_activation_forward(hip.ACT_GELU, dxv.ptr, yv.ptr, x.size))
    hip.check(hip.bh_activation_backward(hip.ACT_GELU, dxv.ptr, ddy.ptr, gx.ptr, x.size, 0))
    assert close_max(yv.numpy(), g["y"], TOL_EW) and close_max(gx.numpy(), g["dx"], TOL_EW)


@pytest.mark.gpu
def test_gpu_conv_pool_cnn_golden(boat):
    """Convolution, pooling and the CNN chain against the compiled reference's vectors.  The reference pairs each tap of
    the input gradient with the mirrored weight (src/layers/conv.c:86-88); boat_hip_conv_reference_input_grad(1) selects
    that pairing so every number can be compared; the default (true gradient) is checked against it through the turned
    kernel: dx_true(w) == dx_reference(w turned by 180 degrees)."""
    from test_oracle_vs_reference import CNN_KEYS
    boat.boat_hip_conv_reference_input_grad(1)
    try:
        g = load("conv_layer")
        for i in range(3):
            stride, pad = int(g[f"c{i}_meta"][6]), int(g[f"c{i}_meta"][7])
            x, w, b = g[f"c{i}_x"], g[f"c{i}_w"], g[f"c{i}_b"]
            y, calls = bc.conv_layer(boat, x, w, b, stride, pad, [g[f"c{i}_dy1"], g[f"c{i}_dy2"]])
            assert same(y, g[f"c{i}_y"]), i          # forward keeps the reference's operation order: bit exact
            for j, (dx, gw, gb) in enumerate(calls):
                assert close_max(dx, g[f"c{i}_dx{j}"], TOL_RED) and close_max(gw, g[f"c{i}_gw{j}"], TOL_RED), (i, j)
                assert close_max(gb, g[f"c{i}_gb{j}"], TOL_RED), (i, j)
        c = load("cnn_chain")
        x, labels, p = cnn_case(c)
        rec = bc.cnn_ce_grads(boat, x, labels, p)
        assert abs(rec["loss"] - float(c["loss"])) <= TOL_RED * abs(float(c["loss"]))
        for key in CNN_KEYS:
            assert close_max(rec[key], c[key], TOL_GEMM if key.startswith("g_w") else TOL_RED), key
    finally:
        boat.boat_hip_conv_reference_input_grad(-1)      # back to following reference-exact mode (off: the true gradient)
    # default mode = true gradient: equals the reference's operator applied to the turned kernel
    i = 0
    stride, pad = int(g[f"c{i}_meta"][6]), int(g[f"c{i}_meta"][7])
    x, w, b, dy = g[f"c{i}_x"], g[f"c{i}_w"], g[f"c{i}_b"], g[f"c{i}_dy1"]
    boat.boat_hip_conv_reference_input_grad(1)
    dx_ref_turned = bc.conv_layer(boat, x, np.ascontiguousarray(w[:, :, ::-1, ::-1]), b, stride, pad, [dy])[1][0][0]
    boat.boat_hip_conv_reference_input_grad(-1)
    dx_true = bc.conv_layer(boat, x, w, b, stride, pad, [dy])[1][0][0]
    assert same(dx_true, dx_ref_turned)
    pl = load("pool_layer")
    for i in range(4):
        k, stride, pad = (int(v) for v in pl[f"p{i}_meta"])
        y, dx = bc.pool_layer(boat, pl[f"p{i}_x"], k, stride, pad, pl[f"p{i}_dy"])
        assert same(y, pl[f"p{i}_y"]) and same(dx, pl[f"p{i}_dx"]), i      # no arithmetic reordering: bit exact


@pytest.mark.gpu
def test_gpu_fanout_is_the_true_gradient_not_the_reference_value(boat):
    g = load("fanout_divergence")
    da, db = bc.fanout(boat, g["a"], g["b"])
    assert same(da, 2 * g["b"]) and same(db, 2 * g["a"])      # the reference reports 4b, 4a (see the fixture)


def _backward_twice_inputs():
    rng = np.random.default_rng(77)
    return [rng.standard_normal((3, 5)).astype(np.float32) for _ in range(6)]


def test_reference_backward_twice_over_a_kept_graph(ref):
    """The compiled reference on bc.backward_twice: non-leaf gradients persist between two backward calls, so the second
    walk hands on the accumulated gradient (the closed form in bc.backward_twice_expected)."""
    t = _backward_twice_inputs()
    for got, want in zip(bc.backward_twice(ref, *t), bc.backward_twice_expected(*t)):
        assert close_max(got, want, TOL_EW)


@pytest.mark.gpu
def test_gpu_backward_twice_over_a_kept_graph(boat):
    """The same scenario on this library, whose walk shares gradient tensors between variables instead of copying them:
    a second backward over the kept graph must not add into a tensor another variable holds."""
    t = _backward_twice_inputs()
    for got, want in zip(bc.backward_twice(boat, *t), bc.backward_twice_expected(*t)):
        assert close_max(got, want, TOL_EW)


@pytest.mark.gpu
def test_gpu_reference_exact_mode(boat):
    """boat_hip_set_reference_exact(1): the three deliberate divergences follow the reference at once -- the depth-first
    walk that counts a non-leaf's fan-out once per consumer (fixture fanout_divergence), the mirrored-tap convolution
    input gradient (fixtures conv_layer, cnn_chain) and the ignored disable_grad flag."""
    from test_oracle_vs_reference import CNN_KEYS
    f = load("fanout_divergence")
    a, b = f["a"], f["b"]
    assert bc.grad_under_disabled_context(boat, a, b) is None                 # default: not recorded, no gradient
    boat.boat_hip_set_reference_exact(1)
    try:
        da, db = bc.fanout(boat, a, b)
        assert same(da, f["ref_da"]) and same(db, f["ref_db"])                # 4b, 4a
        assert same(bc.grad_under_disabled_context(boat, a, b), b)            # the flag is ignored: da = b
        g = load("conv_layer")
        for i in range(3):
            stride, pad = int(g[f"c{i}_meta"][6]), int(g[f"c{i}_meta"][7])
            y, calls = bc.conv_layer(boat, g[f"c{i}_x"], g[f"c{i}_w"], g[f"c{i}_b"], stride, pad, [g[f"c{i}_dy1"]])
            assert same(y, g[f"c{i}_y"]) and close_max(calls[0][0], g[f"c{i}_dx0"], TOL_RED), i
        c = load("cnn_chain")
        x, labels, p = cnn_case(c)
        rec = bc.cnn_ce_grads(boat, x, labels, p)                             # a chain: the depth-first walk visits each op once
        for key in CNN_KEYS:
            assert close_max(rec[key], c[key], TOL_GEMM if key.startswith("g_w") else TOL_RED), key
    finally:
        boat.boat_hip_set_reference_exact(0)
    da, db = bc.fanout(boat, a, b)
    assert same(da, 2 * b) and same(db, 2 * a)


@pytest.mark.gpu
def test_gpu_checkpoint_roundtrip_golden(boat, tmp_path):
    """The example's checkpoint routines over this library: a model holding the fixture's parameters writes the very
    bytes the reference wrote; the reference's file read into a model created with other weights gives the logits
    of the model built from the parameters directly (bit for bit) and the reference's logits (to tolerance); a file
    with another magic number is refused."""
    g, c = load("cnn_checkpoint"), load("cnn_chain")
    x, labels, p = cnn_case(c)
    holder = bc.CnnLayers(boat, p)
    path = tmp_path / "model.bin"
    holder.save(str(path))
    assert path.read_bytes() == g["content"].tobytes()
    direct = holder.logits(x)
    ref_file = tmp_path / "reference.bin"
    ref_file.write_bytes(g["content"].tobytes())
    other = bc.CnnLayers(boat, {k: np.full_like(v, 0.01) for k, v in p.items()})
    assert not same(other.logits(x), direct)
    assert other.load(str(ref_file))
    loaded = other.logits(x)
    assert same(loaded, direct)
    assert close_max(loaded, g["logits"], TOL_RED)
    bad = tmp_path / "bad.bin"
    bad.write_bytes(b"\0" * 8 + g["content"].tobytes()[8:])
    assert not other.load(str(bad))                            # wrong magic: refused, nothing changed
    assert same(other.logits(x), direct)
    holder.free()
    other.free()
