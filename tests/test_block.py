"""Pre-LN transformer encoder block training step (benchmark configuration 5, scaled down): forward,
boat_variable_backward and fused Adam over the block's 16 parameter tensors.

The expected values are composed from oracle primitives that are each pinned to the compiled
reference (dense, attention, LayerNorm forward, Adam, MSE) or, where the reference ships stubs
(LayerNorm backward, GELU), to float64 closed forms.  The composition itself -- residual fan-out,
the order of the chain rule, the reference's reshape head split -- is pinned on the CPU against
float64 autograd of an independent library (torch), so a dropped residual term or a transposed
head split fails there before any GPU is involved.
"""
import numpy as np
import pytest

import boat_cases as bc
from oracle_lib import rel_fro

TOL_RED, TOL_GEMM = 1e-4, 1e-3


def make_block(seed, B, S, H, ffn, scale_w=None):
    rng = np.random.default_rng(seed)
    sw = 0.02 if scale_w is None else scale_w
    p = {"ln1_g": 1 + 0.1 * rng.standard_normal(H), "ln1_b": 0.1 * rng.standard_normal(H),
         "ln2_g": 1 + 0.1 * rng.standard_normal(H), "ln2_b": 0.1 * rng.standard_normal(H),
         "w1": sw * rng.standard_normal((H, ffn)), "b1": 0.01 * rng.standard_normal(ffn),
         "w2": sw * rng.standard_normal((ffn, H)), "b2": 0.01 * rng.standard_normal(H)}
    for n in "qkvo":
        p["w" + n] = sw * rng.standard_normal((H, H))
        p["b" + n] = 0.01 * rng.standard_normal(H)
    p = {k: v.astype(np.float32) for k, v in p.items()}
    x = rng.standard_normal((B, S, H)).astype(np.float32)
    target = rng.standard_normal((B, S, H)).astype(np.float32)
    return x, target, p


def oracle_block_steps(oracle, x, target, params, heads, steps=1, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8):
    """The block step restated with oracle primitives; same outputs as bc.transformer_block_steps."""
    B, S, H = x.shape
    T = B * S
    p = {k: v.copy() for k, v in params.items()}
    m = {k: np.zeros_like(v) for k, v in p.items()}
    v_ = {k: np.zeros_like(v) for k, v in p.items()}
    hist = []
    for t in range(steps):
        w = {n: p["w" + n] for n in "qkvo"}
        b = {n: p["b" + n] for n in "qkvo"}
        x2 = x.reshape(T, H)
        h1, mean1, rstd1 = oracle.layernorm_forward(x2, p["ln1_g"], p["ln1_b"], 1e-5)
        h1_3 = h1.reshape(B, S, H)
        att, cache = oracle.attention_forward(h1_3, h1_3, h1_3, w, b, heads)
        x1 = x + att                                            # boat_add, fp32
        x1_2 = x1.reshape(T, H)
        h2, mean2, rstd2 = oracle.layernorm_forward(x1_2, p["ln2_g"], p["ln2_b"], 1e-5)
        f1 = oracle.dense_forward(h2, p["w1"], p["b1"])
        g1 = oracle.gelu_forward_f64(f1).astype(np.float32)
        f2 = oracle.dense_forward(g1, p["w2"], p["b2"])
        y = x1 + f2.reshape(B, S, H)
        loss = oracle.mse_loss(y, target)
        dy = oracle.mse_grad(y, target)
        # backward
        dy2 = dy.reshape(T, H)
        dg1, gw2, gb2 = oracle.dense_backward(g1, p["w2"], dy2)
        df1 = oracle.gelu_backward_f64(f1, dg1).astype(np.float32)
        dh2, gw1, gb1 = oracle.dense_backward(h2, p["w1"], df1)
        dx1_ln, dgam2, dbet2 = oracle.layernorm_backward_f64(x1_2, p["ln2_g"], dh2, mean2, rstd2)
        dx1 = (dy2.astype(np.float64) + dx1_ln).astype(np.float32)              # two consumers of x1
        ga = oracle.attention_backward(h1_3, h1_3, h1_3, w, True, cache, dx1.reshape(B, S, H), heads)
        dh1 = (ga["d_query"].astype(np.float64) + ga["d_key"] + ga["d_value"]).astype(np.float32)   # q = k = v = LN1(x)
        dx_ln, dgam1, dbet1 = oracle.layernorm_backward_f64(x2, p["ln1_g"], dh1.reshape(T, H), mean1, rstd1)
        dx = (dx1.astype(np.float64) + dx_ln).astype(np.float32).reshape(B, S, H)  # two consumers of x
        grads = {"ln1_g": dgam1, "ln1_b": dbet1, "ln2_g": dgam2, "ln2_b": dbet2, "w1": gw1, "b1": gb1, "w2": gw2, "b2": gb2}
        for n in "qkvo":
            grads["w" + n] = ga["gw" + n]
            grads["b" + n] = ga["gb" + n]
        grads = {k: np.asarray(g, np.float32).reshape(p[k].shape) for k, g in grads.items()}
        rec = {"loss": loss, "y": y, "dx": dx}
        for k in bc.BLOCK_PARAM_ORDER:
            rec["g_" + k] = grads[k]
        for k in bc.BLOCK_PARAM_ORDER:
            pk, mk, vk = oracle.adam_update(p[k], grads[k], m[k], v_[k], lr, beta1, beta2, eps, t)
            p[k], m[k], v_[k] = pk.reshape(p[k].shape), mk.reshape(p[k].shape), vk.reshape(p[k].shape)
            rec["p_" + k] = p[k].copy()
        hist.append(rec)
    return hist


def torch_block_grads(x, target, params, heads):
    """float64 autograd of the same block, with the reference's head split: [B,S,H] viewed as [B*nh, S, hd]
    by plain reshape (src/layers/attention.c:393-397), scale on the scores, exact-erf GELU, MSE mean."""
    import torch
    B, S, H = x.shape
    hd = H // heads
    tp = {k: torch.tensor(v, dtype=torch.float64, requires_grad=True) for k, v in params.items()}
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tt = torch.tensor(target, dtype=torch.float64)
    F = torch.nn.functional
    h1 = F.layer_norm(tx, (H,), tp["ln1_g"], tp["ln1_b"], 1e-5)
    q = (h1.reshape(B * S, H) @ tp["wq"] + tp["bq"]).reshape(B * heads, S, hd)
    k = (h1.reshape(B * S, H) @ tp["wk"] + tp["bk"]).reshape(B * heads, S, hd)
    v = (h1.reshape(B * S, H) @ tp["wv"] + tp["bv"]).reshape(B * heads, S, hd)
    a = torch.softmax(q @ k.transpose(1, 2) / np.sqrt(hd), dim=-1)
    ao = (a @ v).reshape(B * S, H)
    x1 = tx + (ao @ tp["wo"] + tp["bo"]).reshape(B, S, H)
    h2 = F.layer_norm(x1, (H,), tp["ln2_g"], tp["ln2_b"], 1e-5)
    f = F.gelu(h2.reshape(B * S, H) @ tp["w1"] + tp["b1"], approximate="none") @ tp["w2"] + tp["b2"]
    y = x1 + f.reshape(B, S, H)
    loss = ((y - tt) ** 2).mean()
    loss.backward()
    out = {"loss": float(loss.detach()), "y": y.detach().numpy(), "dx": tx.grad.numpy()}
    for kname, t in tp.items():
        out["g_" + kname] = t.grad.numpy()
    return out


@pytest.mark.parametrize("B,S,H,heads,ffn", [(2, 8, 32, 4, 64), (1, 16, 64, 2, 96)])
def test_oracle_block_composition_against_float64_autograd(oracle, B, S, H, heads, ffn):
    x, target, params = make_block(11, B, S, H, ffn, scale_w=0.2)
    rec = oracle_block_steps(oracle, x, target, params, heads, steps=1)[0]
    want = torch_block_grads(x, target, params, heads)
    assert abs(rec["loss"] - want["loss"]) <= 1e-5 * abs(want["loss"])
    assert rel_fro(rec["y"], want["y"]) <= 1e-5
    for key in ["dx"] + ["g_" + k for k in bc.BLOCK_PARAM_ORDER]:
        assert rel_fro(rec[key], want[key]) <= 2e-4, key
    # first Adam step from zero moments moves every resolved parameter by lr against its gradient's sign
    for k in ("w1", "wq", "ln1_g"):
        g = rec["g_" + k]
        big = np.abs(g) > 1e-6
        step = rec["p_" + k] - params[k]
        assert np.allclose(step[big], -1e-3 * np.sign(g[big]), rtol=1e-2, atol=1e-7), k


@pytest.mark.gpu
@pytest.mark.parametrize("B,S,H,heads,ffn", [
    (2, 8, 32, 4, 64),        # general attention kernels (head_dim 8)
    (2, 128, 128, 2, 256),    # head_dim 64, seq 128: the matrix-core attention kernels
    (1, 256, 192, 3, 320),    # three heads, sizes that are not powers of two
])
def test_block_training_steps(boat, oracle, B, S, H, heads, ffn):
    x, target, params = make_block(5, B, S, H, ffn, scale_w=0.08)
    steps = 2
    got = bc.transformer_block_steps(boat, x, target, params, heads, steps=steps)
    want = oracle_block_steps(oracle, x, target, params, heads, steps=steps)
    g, w = got[0], want[0]
    assert abs(g["loss"] - w["loss"]) <= TOL_RED * abs(w["loss"])
    assert rel_fro(g["y"], w["y"]) <= TOL_GEMM and rel_fro(g["dx"], w["dx"]) <= TOL_GEMM
    for k in bc.BLOCK_PARAM_ORDER:
        assert rel_fro(g["g_" + k], w["g_" + k]) <= TOL_GEMM, k
    for t in range(steps):
        assert abs(got[t]["loss"] - want[t]["loss"]) <= 1e-3 * abs(want[t]["loss"])
        for k in bc.BLOCK_PARAM_ORDER:
            # each Adam step moves a parameter by at most ~lr; gradients that are rounding noise may pick the other sign
            assert np.max(np.abs(got[t]["p_" + k] - want[t]["p_" + k])) <= 2.1e-3 * (t + 1), (t, k)
            if t == 0:
                gref = w["g_" + k]
                resolved = np.abs(gref) > 1e-3 * np.abs(gref).max()
                assert np.max(np.abs(got[0]["p_" + k] - want[0]["p_" + k])[resolved]) <= 2e-5, k


# One batch element of benchmark configuration 5's block at its real sizes, pinned by float64 autograd
# (tests/golden/make_golden.py writes tests/golden/block_config5_ref64.npz from torch_block_grads above).
BLOCK_REF64 = {"seed": 11, "S": 512, "H": 1024, "ffn": 4096, "heads": 16}


def block_ref64_sample(params, n_rows=12, n_picks=512):
    """Rows of y / dx and flat positions inside every parameter gradient that the fixture holds (seeded)."""
    rng = np.random.default_rng(20251125)
    rows = np.sort(rng.choice(BLOCK_REF64["S"], n_rows, replace=False))
    picks = {}
    for name in bc.BLOCK_PARAM_ORDER:
        size = params[name].size
        picks[name] = np.sort(rng.choice(size, min(n_picks, size), replace=False))
    return rows, picks


@pytest.mark.gpu
@pytest.mark.parametrize("score_cache", [True, False])
def test_config5_block_one_element_against_float64(boat, score_cache):
    """d_model 1024, 16 heads, seq 512, FFN 4096, batch 1: the shapes that pick the split-K weight-gradient GEMMs, the
    head_dim-64 matrix-core attention kernels (with and without the score cache) and the grouped self-attention
    projections, against float64 autograd on sampled rows and entries.  The batch-independence test of
    test_full_size.py carries this to batch 16."""
    from pathlib import Path
    c = BLOCK_REF64
    with np.load(Path(__file__).resolve().parent / "golden" / "block_config5_ref64.npz", allow_pickle=False) as z:
        want = {k: z[k] for k in z.files}
    x, target, params = make_block(c["seed"], 1, c["S"], c["H"], c["ffn"])
    rows, picks = block_ref64_sample(params)
    boat.boat_hip_set_attention_score_cache_limit((1 << 30) if score_cache else 0)
    try:
        got = bc.transformer_block_steps(boat, x, target, params, c["heads"], steps=1)[0]
    finally:
        boat.boat_hip_set_attention_score_cache_limit(1 << 30)
    assert abs(got["loss"] - float(want["loss"])) <= TOL_RED * abs(float(want["loss"]))
    assert rel_fro(got["y"][0][rows], want["y_rows"]) <= TOL_GEMM
    assert rel_fro(got["dx"][0][rows], want["dx_rows"]) <= TOL_GEMM
    for name in bc.BLOCK_PARAM_ORDER:
        tol = TOL_RED if name.startswith("ln") else TOL_GEMM
        assert rel_fro(got["g_" + name].reshape(-1)[picks[name]], want["g_" + name]) <= tol, name
