#!/usr/bin/env python3
"""Benchmark of the training hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extra] [--no-cpu] [--legs ...]

A step is benchmark configuration 5, the one configuration that is literally "backward + Adam step": one training
step of a pre-LN transformer encoder block (d_model 1024, 16 heads, FFN 4096 with GELU, seq 512, batch 16: forward,
boat_variable_backward, fused Adam over the block's 12,596,224 parameters, zero_grad) driven through Boat's C API,
followed by the standalone fused Adam over 268,435,456 flat fp32 parameters.  Inputs, weights, gradients and moments
are resident in HBM before timing starts; the K timed steps are bracketed by HIP events on the library stream.

Prints ONE JSON line: the step time in ms (value); the roofline of the dominant kernel family (the fp32-MFMA GEMM
launches of the step: their algorithmic 2*m*n*k flops / their durations, both summed over the timed region, each launch
bracketed by HIP events through bh_profile_enable, against the 157.3 TFLOP/s fp32-MFMA peak); the CPU baseline (the
compiled reference's routines timed on one host core on a bounded sample and scaled by flops and by element count);
and -- under "extra" -- the step's breakdown and the other configurations of the path with their own roofline fractions.

The library keeps host pointers coherent by default (what an unchanged Boat caller needs); the legs that run through
Boat's API switch that off (boat_hip_set_coherent_pointers(0)), as a training loop that fetches pointers per batch
would, so that parameters stay resident in HBM.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_HBM_GBS = 8000.0        # MI355X HBM3E
PEAK_FP32_MFMA_TFLOPS = 157.3
METRIC = "backward+Adam step ms; GB/s & TFLOP/s as % of MI355X roofline (1 GPU)"

# HBM bytes per GEMM launch of configuration 2 (average of its dX and dW launches) measured with rocprofv3 --pmc:
# 2.000 x FETCH_SIZE (393,392 and 426,101 KiB) + 1.000 x WRITE_SIZE (131,072 and 65,536 KiB), the factors being what the
# same counters read for a streaming copy of known size (profiles/pmc_hbm_traffic_and_mfma.md).  A constant taken from
# that profile, not a measurement of this run.
GEMM_TRAFFIC_BYTES_CONFIG2 = int(((2.0 * 393392.3 + 131072.0) + (2.0 * 426101.2 + 65536.0)) / 2 * 1024)
# the bytes the same two launches need at least: dX reads dY and W and writes dX (335.5 MB), dW reads X and dY, reads and
# writes dW (402.7 MB)
GEMM_ALGORITHMIC_BYTES_CONFIG2 = int((335.5e6 + 402.7e6) / 2)
# HBM bytes per GEMM launch of the block training step, averaged over the step's 11 launches (same file, same counters)
GEMM_TRAFFIC_BYTES_STEP = 364_800_000
# what the step's 11 GEMM launches need at least (each operand read once, each output written once): 1,929 MB
GEMM_ALGORITHMIC_BYTES_STEP = 1_929_000_000 // 11


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-extra", action="store_true", help="skip the other configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--legs", default="all",
                    help="comma list of step,dense,adam,ln_gelu,sdpa,gemm,mlp,cnn,conv (default all); for profiling one workload at a time. "
                         "Without the step leg the line carries no value/roofline.")
    return ap.parse_args()


# The GPU drops its clocks while the host prepares the next leg's inputs and needs some tens of milliseconds of work to
# raise them again (attention forward: 0.34 ms per launch cold, 0.29 ms after 15 ms of launches).  Every secondary leg
# therefore repeats its warm-up batch until this much time has passed; the headline leg does exactly --warmup steps.
CLOCK_WARM_SECONDS = 0.05


def warm_clocks(sync, fn, warmup):
    """At least `warmup` untimed calls of fn(), repeated in batches until CLOCK_WARM_SECONDS have passed."""
    t_end = time.perf_counter() + CLOCK_WARM_SECONDS
    while True:
        for _ in range(max(warmup, 1)):
            fn()
        sync()
        if time.perf_counter() >= t_end:
            return


def time_steps(hip, fn, steps, warmup):
    """ms per step of fn(), timed with HIP events on the library stream, device idle on both sides."""
    warm_clocks(hip.synchronize, fn, warmup)
    t = hip.Timer()
    with t:
        for _ in range(steps):
            fn()
    hip.synchronize()
    return t.ms / steps


def bench_dense_backward(hip, steps, warmup):
    M, K, N = 8192, 4096, 4096
    rng = np.random.default_rng(20250102)
    X = hip.to_device(rng.standard_normal((M, K), dtype=np.float32))
    W = hip.to_device((0.02 * rng.standard_normal((K, N), dtype=np.float32)).astype(np.float32))
    dY = hip.to_device(rng.standard_normal((M, N), dtype=np.float32))
    dX, dW, dB = hip.empty((M, K)), hip.zeros((K, N)), hip.zeros(N)

    ev = [hip.bh_event_create() for _ in range(3 * steps)]

    def step(i=None):
        if i is not None:
            hip.check(hip.bh_event_record(ev[3 * i]))
        hip.check(hip.bh_gemm(0, 1, M, K, N, dY.ptr, N, W.ptr, N, dX.ptr, K, None, 0, 1), "dX = dY.W^T")
        if i is not None:
            hip.check(hip.bh_event_record(ev[3 * i + 1]))
        hip.check(hip.bh_gemm(1, 0, K, N, M, X.ptr, K, dY.ptr, N, dW.ptr, N, None, 1, 1), "dW += X^T.dY")
        if i is not None:
            hip.check(hip.bh_event_record(ev[3 * i + 2]))
        hip.check(hip.bh_colsum(dY.ptr, dB.ptr, M, N, 1), "db += colsum(dY)")

    for _ in range(warmup):
        step()
    hip.synchronize()
    t0 = time.perf_counter()
    timer = hip.Timer()
    with timer:
        for i in range(steps):
            step(i)
    hip.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms_per_step = timer.ms / steps
    gemm_ms = 0.0
    for i in range(steps):
        gemm_ms += hip.bh_event_elapsed_ms(ev[3 * i], ev[3 * i + 1]) + hip.bh_event_elapsed_ms(ev[3 * i + 1], ev[3 * i + 2])
    for e in ev:
        hip.bh_event_destroy(e)
    gemm_launch_ms = gemm_ms / (2 * steps)
    flops_per_launch = 2.0 * M * K * N
    achieved = flops_per_launch / (gemm_launch_ms * 1e-3) / 1e12
    # quick correctness guard on the timed buffers (one tile against float64)
    got = dX.numpy()[:32, :32]
    want = dY.numpy()[:32].astype(np.float64) @ W.numpy()[:32].astype(np.float64).T
    assert np.linalg.norm(got - want) <= 1e-3 * np.linalg.norm(want), "dense backward result check failed"
    return {
        "ms_per_step": ms_per_step,
        "wall_ms_per_step": wall_ms,
        "roofline": {
            "bound": "mfma", "kernel": "gemm_mfma_kernel (fp32 v_mfma_f32_32x32x2_f32, tile chosen by the cost model, operands direct to LDS)",
            "achieved": round(achieved, 2), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
            "avg_launch_ms": round(gemm_launch_ms, 4), "flops_per_launch": flops_per_launch,
            "traffic": GEMM_TRAFFIC_BYTES_CONFIG2, "algorithmic_bytes": GEMM_ALGORITHMIC_BYTES_CONFIG2,
            "traffic_source": "profile constant (profiles/pmc_hbm_traffic_and_mfma.md), not measured in this run",
        },
        "step_tflops": round(2 * flops_per_launch / (ms_per_step * 1e-3) / 1e12, 2),
    }


def bench_dense_forward(hip, steps, warmup):
    """Dense forward at the config-2 shape: Y = X.W + b, one GEMM with the bias in its epilogue."""
    M, K, N = 8192, 4096, 4096
    rng = np.random.default_rng(20250108)
    X = hip.to_device(rng.standard_normal((M, K), dtype=np.float32))
    W = hip.to_device((0.02 * rng.standard_normal((K, N), dtype=np.float32)).astype(np.float32))
    b = hip.to_device(rng.standard_normal(N, dtype=np.float32))
    Y = hip.empty((M, N))
    ms = time_steps(hip, lambda: hip.check(hip.bh_gemm(0, 0, M, N, K, X.ptr, K, W.ptr, N, Y.ptr, N, b.ptr, 0, 1)), steps, warmup)
    flops = 2.0 * M * K * N
    tf = flops / (ms * 1e-3) / 1e12
    return {"dense_fwd_8192x4096x4096": {"ms": round(ms, 4), "bound": "mfma", "achieved_TFLOPs": round(tf, 2),
                                         "frac": round(tf / PEAK_FP32_MFMA_TFLOPS, 4), "flops": flops}}


def bench_adam(hip, steps, warmup):
    """Config 5b: flat fused Adam over 268,435,456 parameters (28 B/param)."""
    out = {}
    rng = np.random.default_rng(20250103)
    n = 268435456
    p, g, m, v = (hip.empty(n) for _ in range(4))
    chunk = 1 << 24
    noise_p = (0.02 * rng.standard_normal(chunk, dtype=np.float32)).astype(np.float32)
    noise_g = (1e-3 * rng.standard_normal(chunk, dtype=np.float32)).astype(np.float32)
    for off in range(0, n, chunk):   # N(0,.02) params, N(0,1e-3) grads, tiled from one 16M-element draw
        hip.check(hip.bh_memcpy_h2d(p.ptr + 4 * off, noise_p.ctypes.data, 4 * chunk))
        hip.check(hip.bh_memcpy_h2d(g.ptr + 4 * off, noise_g.ctypes.data, 4 * chunk))
    hip.check(hip.bh_memset_zero(m.ptr, 4 * n))
    hip.check(hip.bh_memset_zero(v.ptr, 4 * n))
    step = [0]

    def adam():
        hip.check(hip.bh_adam_update(p.ptr, g.ptr, m.ptr, v.ptr, n, 1e-3, 0.9, 0.999, 1e-8, step[0]))
        step[0] += 1

    ms = time_steps(hip, adam, steps, warmup)
    gbs = 28.0 * n / (ms * 1e-3) / 1e9
    out["adam_flat_268M"] = {"ms": round(ms, 4), "bound": "hbm", "achieved_GBps": round(gbs, 1), "frac": round(gbs / PEAK_HBM_GBS, 4),
                             "bytes": 28 * n}
    # the same four read and three written streams with one add each instead of Adam's arithmetic: this memory
    # pattern's own ceiling on this part (a read-write mix pays for turning the bus around; a plain copy reaches more)
    ms_probe = time_steps(hip, lambda: hip.check(hip.bh_stream_probe_4r3w(p.ptr, g.ptr, m.ptr, v.ptr, n)), steps, warmup)
    gbs_probe = 28.0 * n / (ms_probe * 1e-3) / 1e9
    out["adam_flat_268M"].update(same_pattern_ceiling_ms=round(ms_probe, 4), same_pattern_ceiling_frac=round(gbs_probe / PEAK_HBM_GBS, 4),
                                 frac_of_same_pattern_ceiling=round(ms_probe / ms, 4))
    hip.check(hip.bh_memset_zero(m.ptr, 4 * n))
    hip.check(hip.bh_memset_zero(v.ptr, 4 * n))
    # RMSprop and Adagrad over the same flat arrays (one state tensor: read p, g, state; write p, state = 20 B/param)
    for name, fn in (("rmsprop_flat_268M", lambda: hip.bh_rmsprop_update(p.ptr, g.ptr, m.ptr, n, 1e-3, 0.99, 1e-8)),
                     ("adagrad_flat_268M", lambda: hip.bh_adagrad_update(p.ptr, g.ptr, v.ptr, n, 1e-3, 1e-10))):
        ms = time_steps(hip, lambda: hip.check(fn()), steps, warmup)
        gbs = 20.0 * n / (ms * 1e-3) / 1e9
        out[name] = {"ms": round(ms, 4), "bound": "hbm", "achieved_GBps": round(gbs, 1), "frac": round(gbs / PEAK_HBM_GBS, 4),
                     "bytes": 20 * n}
    del p, g, m, v
    return out


def bench_ln_gelu(hip, steps, warmup):
    """Config 3: LayerNorm backward and GELU backward, 16384 x 4096, plus a streaming copy of known size."""
    out = {}
    rng = np.random.default_rng(20250104)
    R, H = 16384, 4096
    x = hip.to_device(rng.standard_normal((R, H), dtype=np.float32))
    dy = hip.to_device(rng.standard_normal((R, H), dtype=np.float32))
    gamma = hip.to_device((1 + 0.1 * rng.standard_normal(H)).astype(np.float32))
    beta = hip.to_device((0.1 * rng.standard_normal(H)).astype(np.float32))
    y, mean, rstd = hip.empty((R, H)), hip.empty(R), hip.empty(R)
    hip.check(hip.bh_layernorm_forward(x.ptr, gamma.ptr, beta.ptr, y.ptr, mean.ptr, rstd.ptr, R, H, 1e-5))
    dx, dg, db = hip.empty((R, H)), hip.zeros(H), hip.zeros(H)
    ms = time_steps(hip, lambda: hip.check(hip.bh_layernorm_backward(x.ptr, gamma.ptr, dy.ptr, mean.ptr, rstd.ptr, dx.ptr, dg.ptr,
                                                                      db.ptr, R, H, 0)), steps, warmup)
    nbytes = 3 * 4 * R * H + 4 * (3 * H + 2 * R)
    gbs = nbytes / (ms * 1e-3) / 1e9
    out["layernorm_bwd_16384x4096"] = {"ms": round(ms, 4), "bound": "hbm", "achieved_GBps": round(gbs, 1),
                                       "frac": round(gbs / PEAK_HBM_GBS, 4), "bytes": nbytes}
    # LayerNorm backward's three streams (x and dy read, dx written) without its row structure and arithmetic: an
    # elementwise add over the same buffers is this pattern's own ceiling
    ms_probe = time_steps(hip, lambda: hip.check(hip.bh_binary(0, x.ptr, dy.ptr, dx.ptr, R * H)), steps, warmup)
    out["layernorm_bwd_16384x4096"].update(same_pattern_ceiling_ms=round(ms_probe, 4),
                                           same_pattern_ceiling_frac=round(3 * 4 * R * H / (ms_probe * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                                           frac_of_same_pattern_ceiling=round(ms_probe / ms, 4))
    ms = time_steps(hip, lambda: hip.check(hip.bh_activation_backward(hip.ACT_GELU, x.ptr, dy.ptr, dx.ptr, R * H, 0)), steps, warmup)
    nbytes = 3 * 4 * R * H
    gbs = nbytes / (ms * 1e-3) / 1e9
    out["gelu_bwd_16384x4096"] = {"ms": round(ms, 4), "bound": "hbm", "achieved_GBps": round(gbs, 1),
                                  "frac": round(gbs / PEAK_HBM_GBS, 4), "bytes": nbytes}
    # forward kernels of the same layers: LayerNorm forward emitting mean / rstd (read x, write y) and GELU forward
    ms = time_steps(hip, lambda: hip.check(hip.bh_layernorm_forward(x.ptr, gamma.ptr, beta.ptr, y.ptr, mean.ptr, rstd.ptr, R, H, 1e-5)),
                    steps, warmup)
    nbytes = 2 * 4 * R * H + 4 * (2 * H + 2 * R)
    gbs = nbytes / (ms * 1e-3) / 1e9
    out["layernorm_fwd_16384x4096"] = {"ms": round(ms, 4), "bound": "hbm", "achieved_GBps": round(gbs, 1),
                                       "frac": round(gbs / PEAK_HBM_GBS, 4), "bytes": nbytes}
    ms = time_steps(hip, lambda: hip.check(hip.bh_activation_forward(hip.ACT_GELU, x.ptr, dx.ptr, R * H)), steps, warmup)
    nbytes = 2 * 4 * R * H
    gbs = nbytes / (ms * 1e-3) / 1e9
    out["gelu_fwd_16384x4096"] = {"ms": round(ms, 4), "bound": "hbm", "achieved_GBps": round(gbs, 1),
                                  "frac": round(gbs / PEAK_HBM_GBS, 4), "bytes": nbytes}
    # streaming copy of known size (read 256 MiB, write 256 MiB): the practical HBM ceiling on this part and the
    # calibration kernel for the FETCH_SIZE / WRITE_SIZE counters
    ms = time_steps(hip, lambda: hip.check(hip.bh_scalar_op(2, x.ptr, 1.0, dx.ptr, R * H)), steps, warmup)
    nbytes = 2 * 4 * R * H
    gbs = nbytes / (ms * 1e-3) / 1e9
    out["stream_copy_256MiB"] = {"ms": round(ms, 4), "bound": "hbm", "achieved_GBps": round(gbs, 1),
                                 "frac": round(gbs / PEAK_HBM_GBS, 4), "bytes": nbytes}
    del x, dy, y, dx
    return out


def bench_sdpa(hip, steps, warmup):
    """Config 4: attention core backward, B8 h16 S1024 D64 (credited flops: dV, dP, dQ, dK contractions)."""
    out = {}
    rng = np.random.default_rng(20250106)
    bh_, S, D = 8 * 16, 1024, 64
    q, k, vv, go = (hip.to_device(rng.standard_normal((bh_, S, D), dtype=np.float32)) for _ in range(4))
    o, lse = hip.empty((bh_, S, D)), hip.empty((bh_, S))
    scale = 1.0 / 8.0
    hip.check(hip.bh_sdpa_forward(q.ptr, k.ptr, vv.ptr, scale, 0, o.ptr, lse.ptr, None, bh_, S, D))
    ms = time_steps(hip, lambda: hip.check(hip.bh_sdpa_forward(q.ptr, k.ptr, vv.ptr, scale, 0, o.ptr, lse.ptr, None, bh_, S, D)),
                    steps, warmup)
    flops = 2 * 2.0 * bh_ * S * S * D
    tf = flops / (ms * 1e-3) / 1e12
    out["sdpa_fwd_B8h16S1024D64"] = {"ms": round(ms, 4), "bound": "mfma", "achieved_TFLOPs": round(tf, 2),
                                     "frac": round(tf / PEAK_FP32_MFMA_TFLOPS, 4), "flops": flops}
    dq, dk, dv = hip.empty((bh_, S, D)), hip.empty((bh_, S, D)), hip.empty((bh_, S, D))
    ms = time_steps(hip, lambda: hip.check(hip.bh_sdpa_backward(q.ptr, k.ptr, vv.ptr, o.ptr, lse.ptr, go.ptr, scale, 0, dq.ptr, dk.ptr,
                                                                dv.ptr, bh_, S, D)), steps, warmup)
    flops = 4 * 2.0 * bh_ * S * S * D
    tf = flops / (ms * 1e-3) / 1e12
    out["sdpa_bwd_B8h16S1024D64"] = {"ms": round(ms, 4), "bound": "mfma", "achieved_TFLOPs": round(tf, 2),
                                     "frac": round(tf / PEAK_FP32_MFMA_TFLOPS, 4), "credited_flops": flops,
                                     "note": "recomputes Q.K^T (a fifth contraction that is not credited); no [S, S] matrix in memory"}
    # the pair an attention layer uses when the scores fit its cache limit: the forward pass also leaves the scaled
    # scores (bh*S*S*4 bytes, what the reference keeps as attention weights), the backward pass reads them
    cache = hip.empty((bh_, S, S))
    ms_f = time_steps(hip, lambda: hip.check(hip.bh_sdpa_forward_cached(q.ptr, k.ptr, vv.ptr, scale, 0, o.ptr, lse.ptr, cache.ptr,
                                                                        bh_, S, D)), steps, warmup)
    ms_b = time_steps(hip, lambda: hip.check(hip.bh_sdpa_backward_cached(q.ptr, k.ptr, vv.ptr, o.ptr, lse.ptr, cache.ptr, go.ptr, scale,
                                                                         0, dq.ptr, dk.ptr, dv.ptr, bh_, S, D)), steps, warmup)
    tf_f, tf_b = flops / 2 / (ms_f * 1e-3) / 1e12, flops / (ms_b * 1e-3) / 1e12
    out["sdpa_with_score_cache_B8h16S1024D64"] = {
        "fwd_ms": round(ms_f, 4), "fwd_frac": round(tf_f / PEAK_FP32_MFMA_TFLOPS, 4),
        "bwd_ms": round(ms_b, 4), "bwd_achieved_TFLOPs": round(tf_b, 2), "bwd_frac": round(tf_b / PEAK_FP32_MFMA_TFLOPS, 4),
        "bound": "mfma", "cache_bytes": int(bh_) * S * S * 4,
        "fwd_plus_bwd_ms": round(ms_f + ms_b, 4),
        "fwd_plus_bwd_ms_without_cache": round(out["sdpa_fwd_B8h16S1024D64"]["ms"] + out["sdpa_bwd_B8h16S1024D64"]["ms"], 4)}
    del cache, q, k, vv, go, o, lse, dq, dk, dv
    # the other head sizes of the matrix-core kernels at the same sequence length and 8192 floats per token
    for heads, D in ((64, 128), (256, 32)):
        q, k, vv, go = (hip.to_device(rng.standard_normal((heads, S, D), dtype=np.float32)) for _ in range(4))
        o, lse = hip.empty((heads, S, D)), hip.empty((heads, S))
        dq, dk, dv = hip.empty((heads, S, D)), hip.empty((heads, S, D)), hip.empty((heads, S, D))
        scale = float(1.0 / np.sqrt(D))
        ms_f = time_steps(hip, lambda: hip.check(hip.bh_sdpa_forward(q.ptr, k.ptr, vv.ptr, scale, 0, o.ptr, lse.ptr, None, heads, S, D)),
                          steps, warmup)
        ms_b = time_steps(hip, lambda: hip.check(hip.bh_sdpa_backward(q.ptr, k.ptr, vv.ptr, o.ptr, lse.ptr, go.ptr, scale, 0, dq.ptr,
                                                                      dk.ptr, dv.ptr, heads, S, D)), steps, warmup)
        f_fwd = 2 * 2.0 * heads * S * S * D
        tf_f, tf_b = f_fwd / (ms_f * 1e-3) / 1e12, 2 * f_fwd / (ms_b * 1e-3) / 1e12
        out[f"sdpa_heads{heads}_S{S}_D{D}"] = {
            "fwd_ms": round(ms_f, 4), "fwd_achieved_TFLOPs": round(tf_f, 2), "fwd_frac": round(tf_f / PEAK_FP32_MFMA_TFLOPS, 4),
            "bwd_ms": round(ms_b, 4), "bwd_achieved_TFLOPs": round(tf_b, 2), "bwd_frac": round(tf_b / PEAK_FP32_MFMA_TFLOPS, 4),
            "bound": "mfma", "fwd_flops": f_fwd, "bwd_credited_flops": 2 * f_fwd}
    return out


def bench_gemm_choice(hip):
    """The tile / split choice of bh_gemm away from the headline block's shapes: the nine GEMMs of a pre-LN block with
    8192 rows at d_model 512 and at d_model 2048 (projection and both FFN layers: forward, dX, dW), each timed as the
    library chooses and with every tile shape forced at 1, 2, 4, 8 and 16 cuts of the contraction; `ratio` is chosen / best
    forced (1.0 = the cost model found the fastest tile)."""
    rng = np.random.default_rng(20250110)
    rows = 8192
    nmax = rows * 4 * 2048
    A = hip.to_device(rng.standard_normal((nmax,), dtype=np.float32))
    B = hip.to_device(rng.standard_normal((nmax,), dtype=np.float32))
    Cc = hip.empty((nmax,))

    def timed(fn, n=10):
        warm_clocks(hip.synchronize, fn, 3)
        t = hip.Timer()
        with t:
            for _ in range(n):
                fn()
        hip.synchronize()
        return t.ms / n

    out = {}
    worst = 0.0
    for d in (512, 2048):
        cases = [("proj_fwd", 0, 0, rows, d, d), ("proj_dx", 0, 1, rows, d, d), ("proj_dw", 1, 0, d, d, rows),
                 ("ffn1_fwd", 0, 0, rows, 4 * d, d), ("ffn1_dx", 0, 1, rows, d, 4 * d), ("ffn1_dw", 1, 0, d, 4 * d, rows),
                 ("ffn2_fwd", 0, 0, rows, d, 4 * d), ("ffn2_dx", 0, 1, rows, 4 * d, d), ("ffn2_dw", 1, 0, 4 * d, d, rows)]
        for name, ta, tb, m, n, k in cases:
            def run():
                hip.check(hip.bh_gemm(ta, tb, m, n, k, A.ptr, m if ta else k, B.ptr, k if tb else n, Cc.ptr, n, None, 0, 1))
            chosen = timed(run)
            best, best_cfg = 1e9, None
            try:
                for cfg in (1, 2, 3, 4, 7):                 # 128x128, 256x256, 256x128, 128x256 and 64x64 tiles
                    hip.bh_gemm_force_config(cfg)
                    bm, bn = {1: (128, 128), 2: (256, 256), 3: (256, 128), 4: (128, 256), 7: (64, 64)}[cfg]
                    tiles = -(-m // bm) * -(-n // bn)
                    for sp in (1, 2, 4, 8, 16):
                        if sp > 1 and (tiles * sp > 2048 or k // sp < 128):
                            continue
                        hip.bh_gemm_force_splits(sp)
                        t = timed(run, 6)
                        if t < best:
                            best, best_cfg = t, f"tile{cfg}x{sp}"
            finally:
                hip.bh_gemm_force_config(-1)
                hip.bh_gemm_force_splits(0)
            chosen = min(chosen, timed(run))
            tf = 2.0 * m * n * k / (chosen * 1e-3) / 1e12
            ratio = chosen / best
            worst = max(worst, ratio)
            out[f"d{d}_{name}"] = {"m": m, "n": n, "k": k, "ms": round(chosen, 4), "TFLOPs": round(tf, 1),
                                   "frac": round(tf / PEAK_FP32_MFMA_TFLOPS, 4), "best_forced": best_cfg, "best_forced_ms": round(best, 4),
                                   "ratio": round(ratio, 3)}
    out["worst_ratio"] = round(worst, 3)
    return {"gemm_choice_blocks_d512_d2048": out}


def bench_mlp_step(steps, warmup):
    """Config 1 through Boat's C API from a C program (boat_amd/examples/mlp_train_step.c, built beside the library):
    forward + boat_variable_backward_full + boat_optimizer_step + zero_grad per step, wall ms measured inside it.
    Three runs: the op-by-op loss chain with parameters resident (BOAT_HIP_COHERENT_POINTERS=0), the same with the
    four-op loss chain replaced by the fused softmax + cross-entropy kernel, and the chain in the library's default
    configuration (every tensor whose pointer the program once held is kept coherent with the host on every call)."""
    import subprocess
    exe = ROOT / "boat_amd" / "lib" / "mlp_train_step"
    if not exe.exists():
        raise FileNotFoundError(f"{exe} not found: build it first (python -m boat_amd.build)")

    def run(coherent, *extra):
        env = dict(os.environ, BOAT_HIP_COHERENT_POINTERS=coherent)
        out = subprocess.run([str(exe), str(steps), str(warmup), *extra], check=True, capture_output=True, text=True, env=env).stdout
        rec = json.loads(out.strip().splitlines()[-1])
        assert rec["loss_last"] < rec["loss_first"], f"MLP training does not reduce the loss: {rec}"
        return rec

    chain, fused, default = run("0"), run("0", "fused"), run("1")
    return {"ms": round(chain["ms_per_step"], 4), "bound": "launch latency", "steps": chain["steps"],
            "ms_fused_softmax_cross_entropy": round(fused["ms_per_step"], 4),
            "ms_default_coherent_pointers": round(default["ms_per_step"], 4),
            "loss_first_last": [chain["loss_first"], chain["loss_last"]],
            "loss_first_last_fused": [fused["loss_first"], fused["loss_last"]],
            "note": "MLP 784-128-10 B64 fwd+bwd+Adam+zero_grad through boat_var_* / boat_variable_backward_full / "
                    "boat_optimizer_step, a C caller linked against libboat_amd.so, wall clock; 'fused' replaces log_softmax, "
                    "mul(onehot), sum, mul(-1/B) and their backward by boat_hip_softmax_cross_entropy"}


def bench_block_step_c_caller(steps, warmup):
    """Config 5a from a C program (boat_amd/examples/block_train_step.c, built beside the library): the same block step as
    the headline's, written against Boat's C API only, wall ms measured inside the program between two device
    synchronisations; once with pointers not kept and once in the library's default configuration (the program took the
    data pointers of its weights, input and target during set-up, so the default keeps those coherent with the host on
    every call)."""
    import subprocess
    exe = ROOT / "boat_amd" / "lib" / "block_train_step"
    if not exe.exists():
        raise FileNotFoundError(f"{exe} not found: build it first (python -m boat_amd.build)")
    out = {}
    for key, coherent in (("ms", "0"), ("ms_default_coherent_pointers", "1")):
        env = dict(os.environ, BOAT_HIP_COHERENT_POINTERS=coherent)
        text = subprocess.run([str(exe), str(steps), str(warmup)], check=True, capture_output=True, text=True, env=env).stdout
        rec = json.loads(text.strip().splitlines()[-1])
        assert rec["loss_last"] < rec["loss_first"], f"block training does not reduce the loss: {rec}"
        out[key] = round(rec["ms_per_step"], 4)
        out["loss_first_last"] = [rec["loss_first"], rec["loss_last"]]
    out["note"] = ("the block step (d_model 1024, 16 heads, FFN 4096, seq 512, batch 16: forward, boat_variable_backward, Adam, "
                   "zero_grad) from a C caller linked against libboat_amd.so, wall clock, flat Adam not included")
    return out


def bench_cnn_step(steps, warmup):
    """The MNIST CNN of examples/mnist/mnist_autodiff.c:536-557 through Boat's C API, batch 64: conv(1->32, 3x3, pad 1),
    relu, maxpool 2, conv(32->64), relu, maxpool 2, flatten, dense 3136->128, relu, dense 128->10, cross-entropy chain;
    forward + boat_variable_backward_full + Adam + zero_grad, wall ms."""
    from boat_amd.capi import default_api
    api = default_api()
    api.boat_hip_set_coherent_pointers(0)       # weights written below stay resident in HBM afterwards
    rng = np.random.default_rng(20250107)
    B, classes = 64, 10
    x = rng.random((B, 1, 28, 28), dtype=np.float32)
    labels = rng.integers(0, classes, B)
    onehot = np.zeros((B, classes), np.float32)
    onehot[np.arange(B), labels] = 1
    c1 = api.boat_conv_layer_create(1, 32, 3, 1, 1)
    c2 = api.boat_conv_layer_create(32, 64, 3, 1, 1)
    p1, p2 = api.boat_pool_layer_create(2, 2, 0), api.boat_pool_layer_create(2, 2, 0)
    d1 = api.boat_dense_layer_create(64 * 7 * 7, 128, True)
    d2 = api.boat_dense_layer_create(128, classes, True)
    for layer, shape in ((c1, (32, 1, 3, 3)), (c2, (64, 32, 3, 3))):
        s = np.sqrt(2.0 / (shape[1] * 9))
        api.write(api.boat_conv_layer_get_weight(layer), rng.uniform(-s, s, shape).astype(np.float32))
    for layer, (fi, fo) in ((d1, (3136, 128)), (d2, (128, classes))):
        s = np.sqrt(2.0 / (fi + fo))
        api.write(api.boat_dense_layer_get_weight(layer), rng.uniform(-s, s, (fi, fo)).astype(np.float32))
    opt = api.boat_adam_optimizer_create(1e-3, 0.9, 0.999, 1e-8)
    api.boat_hip_optimizer_add_conv(opt, c1)
    api.boat_hip_optimizer_add_conv(opt, c2)
    api.boat_hip_optimizer_add_dense(opt, d1)
    api.boat_hip_optimizer_add_dense(opt, d2)
    tx, toh = api.tensor(x), api.tensor(onehot)
    tf = api.tensor(np.array([-1.0 / B], np.float32))
    losses = []

    def step(keep_loss=False):
        vx = api.boat_variable_create(tx, True)
        voh = api.boat_variable_create(toh, False)
        vf = api.boat_variable_create(tf, False)
        a1 = api.boat_var_conv(vx, c1)
        r1 = api.boat_var_relu(a1)
        q1 = api.boat_var_pool(r1, p1)
        a2 = api.boat_var_conv(q1, c2)
        r2 = api.boat_var_relu(a2)
        q2 = api.boat_var_pool(r2, p2)
        fl = api.boat_var_flatten(q2)
        h = api.boat_var_dense(fl, d1)
        rh = api.boat_var_relu(h)
        z = api.boat_var_dense(rh, d2)
        ls = api.boat_var_log_softmax(z, 1)
        mm = api.boat_var_mul(voh, ls)
        sm = api.boat_var_sum(mm, None, 0, False)
        loss = api.boat_var_mul(vf, sm)
        assert loss, "CNN forward failed"
        api.boat_variable_backward_full(loss)
        api.boat_optimizer_step(opt)
        api.boat_optimizer_zero_grad(opt)
        if keep_loss:
            losses.append(float(api.numpy(api.boat_variable_data(loss))[0]))
        for var in (loss, sm, mm, ls, z, rh, h, fl, q2, r2, a2, q1, r1, a1, vf, voh, vx):
            api.boat_variable_free(var)

    step(keep_loss=True)
    warm_clocks(api.sync, step, warmup)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    api.sync()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    step(keep_loss=True)
    assert np.isfinite(losses).all() and losses[1] < losses[0], f"CNN training does not reduce the loss: {losses}"
    # the same loop with the 32->64 layer's forward on the matrix cores (opt-in: not bit-identical to the reference)
    api.boat_hip_conv_forward_matrix_cores(1)
    warm_clocks(api.sync, step, warmup)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    api.sync()
    ms_mfma = (time.perf_counter() - t0) * 1e3 / steps
    api.boat_hip_conv_forward_matrix_cores(0)
    conv_flops = 2.0 * B * (32 * 1 * 9 * 28 * 28 + 64 * 32 * 9 * 14 * 14) * 3       # forward + dX + dW of both conv layers
    return {"ms": round(ms, 4), "bound": "launch latency / small kernels", "conv_flops": conv_flops,
            "ms_conv_forward_on_matrix_cores": round(ms_mfma, 4),
            "loss_first_last": [round(l, 6) for l in losses],
            "note": "MNIST CNN B64 (conv 1->32, conv 32->64, dense 3136->128->10): fwd + bwd + Adam + zero_grad through the "
                    "C API from Python, wall clock"}


def bench_conv_forward_kernels():
    """bh_conv2d_forward (direct, the reference's operation order) against bh_conv2d_forward_mfma (one contraction on the
    fp32 matrix cores) on the MNIST network's 32->64 layer at batch 64, on a layer with many channels and on two 5x5 layers (one
    with stride 2); HIP events."""
    from boat_amd import hip
    rng = np.random.default_rng(20250108)
    out = {}
    cases = (("64x32x14x14_to_64", (64, 32, 14, 14, 64, 3, 1, 1)), ("32x128x28x28_to_256", (32, 128, 28, 28, 256, 3, 1, 1)),
             ("64x32x28x28_to_64_k5", (64, 32, 28, 28, 64, 5, 1, 2)), ("32x64x56x56_to_128_k5_stride2", (32, 64, 56, 56, 128, 5, 2, 2)))
    for name, (B, ic, h, w, oc, k, stride, pad) in cases:
        ho, wo = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
        x = hip.to_device(rng.standard_normal((B, ic, h, w), dtype=np.float32))
        wt = hip.to_device((0.1 * rng.standard_normal((oc, ic, k, k), dtype=np.float32)).astype(np.float32))
        b = hip.to_device(rng.standard_normal(oc, dtype=np.float32))
        y = hip.empty((B, oc, ho, wo))
        flops = 2.0 * B * oc * ho * wo * ic * k * k
        res = {}
        for label, fn in (("direct", hip.bh_conv2d_forward), ("matrix_cores", hip.bh_conv2d_forward_mfma)):
            call = lambda: hip.check(fn(x.ptr, wt.ptr, b.ptr, y.ptr, B, ic, h, w, oc, k, stride, pad))
            warm_clocks(hip.synchronize, call, 10)
            timer = hip.Timer()
            with timer:
                for _ in range(50):
                    call()
            ms = timer.ms / 50
            res[label] = {"us": round(ms * 1e3, 1), "TFLOPs": round(flops / (ms * 1e-3) / 1e12, 1)}
        res["speedup"] = round(res["direct"]["us"] / res["matrix_cores"]["us"], 2)
        out[name] = res
    return out


class Block:
    """Config 5a through Boat's C API: pre-LN encoder block d_model 1024, 16 heads, FFN 4096 (GELU), seq 512, batch 16;
    step() = forward + boat_variable_backward + fused Adam over the block's 12,596,224 parameters (16 tensors) + zero_grad."""
    B, S, H, heads, ffn = 16, 512, 1024, 16, 4096

    def __init__(self):
        from boat_amd.capi import AttentionConfig, LayerNormConfig, default_api
        self.api = api = default_api()
        api.boat_hip_set_coherent_pointers(0)       # parameters written below stay resident in HBM afterwards
        rng = np.random.default_rng(20250105)
        B, S, H, heads, ffn = self.B, self.S, self.H, self.heads, self.ffn

        def normal(shape, std):
            return (std * rng.standard_normal(shape, dtype=np.float32)).astype(np.float32)

        self.ln = []
        for _ in range(2):
            cfg = LayerNormConfig(H, 1e-5, True, True)
            self.ln.append(api.boat_layernorm_create(C.byref(cfg)))          # gamma = 1, beta = 0
        cfg = AttentionConfig(H, heads, H // heads, 0.0, False, True, False, 10000.0)
        self.att = api.boat_attention_create(C.byref(cfg))
        for n in "qkvo":
            api.write(getattr(api, f"boat_attention_get_weight_{n}")(self.att), normal((H, H), 0.02))
        self.d1 = api.boat_dense_layer_create(H, ffn, True)
        self.d2 = api.boat_dense_layer_create(ffn, H, True)
        api.write(api.boat_dense_layer_get_weight(self.d1), normal((H, ffn), 0.02))
        api.write(api.boat_dense_layer_get_weight(self.d2), normal((ffn, H), 0.02))
        self.opt = api.boat_adam_optimizer_create(1e-3, 0.9, 0.999, 1e-8)
        api.boat_hip_optimizer_add_layernorm(self.opt, self.ln[0])
        api.boat_hip_optimizer_add_attention(self.opt, self.att)
        api.boat_hip_optimizer_add_layernorm(self.opt, self.ln[1])
        api.boat_hip_optimizer_add_dense(self.opt, self.d1)
        api.boat_hip_optimizer_add_dense(self.opt, self.d2)
        self.tx = api.tensor(normal((B, S, H), 1.0))
        self.tt = api.tensor(normal((B, S, H), 1.0))
        self.shape2 = (C.c_int64 * 2)(B * S, H)
        self.shape3 = (C.c_int64 * 3)(B, S, H)
        self.losses = []
        T = B * S
        # linear layers forward + dX + dW, attention core forward (2 contractions) + backward (4 credited)
        self.flops = 2.0 * T * (4 * H * H + 2 * H * ffn) * 3 + 3 * 2 * 2.0 * (B * heads) * S * S * (H // heads)
        self.n_params = 4 * (H * H + H) + 4 * H + 2 * H * ffn + ffn + H

    def step(self, keep_loss=False):
        api, ln = self.api, self.ln
        vx = api.boat_variable_create(self.tx, True)
        h1 = api.boat_hip_var_layernorm(vx, ln[0])
        a = api.boat_var_attention(h1, h1, h1, self.att, None)
        x1 = api.boat_var_add(vx, a)
        h2 = api.boat_hip_var_layernorm(x1, ln[1])
        h2f = api.boat_hip_var_reshape(h2, self.shape2, 2)
        f1 = api.boat_var_dense(h2f, self.d1)
        g1 = api.boat_hip_var_gelu(f1)
        f2 = api.boat_var_dense(g1, self.d2)
        f2r = api.boat_hip_var_reshape(f2, self.shape3, 3)
        y = api.boat_var_add(x1, f2r)
        grad = C.c_void_p()
        tloss = api.boat_hip_mse_loss(api.boat_variable_data(y), self.tt, C.byref(grad))
        assert tloss and grad, "block forward failed"
        api.boat_variable_backward(y, grad)
        api.boat_optimizer_step(self.opt)
        api.boat_optimizer_zero_grad(self.opt)
        if keep_loss:
            self.losses.append(float(api.numpy(tloss)[0]))
        api.boat_tensor_unref(tloss)
        api.boat_tensor_unref(grad)
        for v in (y, f2r, f2, g1, f1, h2f, h2, x1, a, h1, vx):
            api.boat_variable_free(v)


class FlatAdam:
    """Config 5b: fused Adam over 268,435,456 flat fp32 parameters (p ~N(0,0.02), g ~N(0,1e-3), m = v = 0): 28 B/param."""
    n = 268435456

    def __init__(self, hip):
        self.hip = hip
        rng = np.random.default_rng(20250103)
        n = self.n
        self.p, self.g, self.m, self.v = (hip.empty(n) for _ in range(4))
        chunk = 1 << 24
        noise_p = (0.02 * rng.standard_normal(chunk, dtype=np.float32)).astype(np.float32)
        noise_g = (1e-3 * rng.standard_normal(chunk, dtype=np.float32)).astype(np.float32)
        for off in range(0, n, chunk):   # tiled from one 16M-element draw
            hip.check(hip.bh_memcpy_h2d(self.p.ptr + 4 * off, noise_p.ctypes.data, 4 * chunk))
            hip.check(hip.bh_memcpy_h2d(self.g.ptr + 4 * off, noise_g.ctypes.data, 4 * chunk))
        hip.check(hip.bh_memset_zero(self.m.ptr, 4 * n))
        hip.check(hip.bh_memset_zero(self.v.ptr, 4 * n))
        self.t = 0

    def step(self):
        hip = self.hip
        hip.check(hip.bh_adam_update(self.p.ptr, self.g.ptr, self.m.ptr, self.v.ptr, self.n, 1e-3, 0.9, 0.999, 1e-8, self.t))
        self.t += 1


def bench_training_step(hip, steps, warmup):
    """The headline: config 5 = block step + flat Adam, K steps between two HIP events on the library stream.  Every
    GEMM, attention, LayerNorm, column-sum and optimizer launch inside the timed region is bracketed by its own event
    pair (bh_profile_enable), which gives the dominant kernel family's duration live."""
    block, flat = Block(), FlatAdam(hip)
    block_probe = hip.zeros(64)
    block.step(keep_loss=True)
    for _ in range(warmup):
        block.step()
        flat.step()
    hip.synchronize()
    mid = [hip.bh_event_create() for _ in range(2 * steps)]
    t0 = time.perf_counter()
    timer = hip.Timer()
    with timer:
        for i in range(steps):
            block.step()
            hip.check(hip.bh_event_record(mid[2 * i]))
            flat.step()
            hip.check(hip.bh_event_record(mid[2 * i + 1]))
    hip.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms_per_step = timer.ms / steps
    flat_ms = sum(hip.bh_event_elapsed_ms(mid[2 * i], mid[2 * i + 1]) for i in range(steps)) / steps
    for e in mid:
        hip.bh_event_destroy(e)
    # The same K steps once more, now with an event pair around every instrumented launch.  An event costs the stream
    # about 5 us (the kernel after it waits for the marker), some 0.25 ms per step with 35 instrumented calls, so this
    # pass is kept out of the timed region above; the durations it yields are those of the same kernels on the same data.
    hip.check(hip.bh_profile_enable(128 * steps), "bh_profile_enable")
    profiled = hip.Timer()
    with profiled:
        for i in range(steps):
            block.step()
            flat.step()
    hip.synchronize()
    profiled_ms = profiled.ms / steps
    # what an event pair reads with nothing between its two events: that much of every recorded call is the measurement
    empty = [hip.bh_event_create() for _ in range(40)]
    for i in range(0, 40, 2):
        hip.check(hip.bh_fill(block_probe.ptr, 0.0, 64))          # something before the pair, as in the step
        hip.check(hip.bh_event_record(empty[i]))
        hip.check(hip.bh_event_record(empty[i + 1]))
    hip.synchronize()
    pair_ms = float(np.median([hip.bh_event_elapsed_ms(empty[i], empty[i + 1]) for i in range(0, 40, 2)]))
    for e in empty:
        hip.bh_event_destroy(e)
    classes = {}
    for name, cls in (("gemm", hip.PROF_GEMM), ("attention_core_fwd", hip.PROF_SDPA_FWD), ("attention_core_bwd", hip.PROF_SDPA_BWD),
                      ("layernorm", hip.PROF_NORM), ("adam", hip.PROF_OPTIMIZER), ("colsum", hip.PROF_COLSUM)):
        ms, work, calls = hip.profile_read(cls)
        if name != "gemm":          # short kernels: the pair's own reading is a visible share; the headline family keeps the raw sum
            ms = max(ms - calls * pair_ms, 0.0)
        classes[name] = (ms / steps, work / steps, calls // steps)
    hip.check(hip.bh_profile_enable(0))
    block.step(keep_loss=True)
    losses = block.losses
    assert np.isfinite(losses).all() and losses[1] < losses[0], f"block training does not reduce the loss: {losses}"
    block_ms = ms_per_step - flat_ms
    g_ms, g_flops, g_calls = classes["gemm"]
    achieved = g_flops / (g_ms * 1e-3) / 1e12
    breakdown = {"block_step_ms": round(block_ms, 4), "flat_adam_268M_ms": round(flat_ms, 4)}
    for name, (ms, work, calls) in classes.items():
        entry = {"ms_per_step": round(ms, 4), "launches_per_step": calls}
        if name in ("gemm", "attention_core_fwd", "attention_core_bwd"):
            entry.update(TFLOPs=round(work / (ms * 1e-3) / 1e12, 2), frac=round(work / (ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                         flops_per_step=work)
        else:
            entry.update(GBps=round(work / (ms * 1e-3) / 1e9, 1), frac=round(work / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), bytes_per_step=work)
        breakdown[name] = entry
    accounted = sum(ms for ms, _, _ in classes.values())
    breakdown["other_kernels_and_gaps_ms"] = round(ms_per_step - accounted, 4)
    breakdown["ms_per_step_with_launch_events"] = round(profiled_ms, 4)
    breakdown["empty_event_pair_ms"] = round(pair_ms, 5)
    breakdown["note"] = ("per-class times are sums over HIP event pairs around each call, minus the reading of an empty pair per call for every "
                         "class but gemm; profiles/kernel_trace_block.md has the per-kernel medians of a kernel trace")
    flat_gbs = 28.0 * flat.n / (flat_ms * 1e-3) / 1e9
    return {
        "ms_per_step": ms_per_step, "wall_ms_per_step": wall_ms,
        "roofline": {
            "bound": "mfma", "kernel": "gemm_mfma_kernel family (fp32 v_mfma_f32_32x32x2_f32 tiles, operands direct to LDS): the "
                                       f"{g_calls} bh_gemm launches of one step (projections, FFN, their dX and dW)",
            "achieved": round(achieved, 2), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
            "avg_launch_ms": round(g_ms / max(g_calls, 1), 4), "flops_per_launch": g_flops / max(g_calls, 1),
            "launches_per_step": g_calls, "traffic": GEMM_TRAFFIC_BYTES_STEP, "algorithmic_bytes": GEMM_ALGORITHMIC_BYTES_STEP,
            "traffic_source": "profile constant (profiles/pmc_hbm_traffic_and_mfma.md: 2.0 x FETCH_SIZE + WRITE_SIZE per launch, averaged "
                              "over the step's launches), not measured in this run",
            "measured": "HIP event pairs around each bh_gemm launch of K further steps run right after the timed K (the events "
                        "themselves cost about 5 us each on the stream, so they stay out of the timed region)",
        },
        "breakdown": breakdown,
        "block": {"ms": round(block_ms, 4), "flops": block.flops, "achieved_TFLOPs": round(block.flops / (block_ms * 1e-3) / 1e12, 2),
                  "frac_of_fp32_mfma_peak": round(block.flops / (block_ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                  "adam_params": block.n_params, "loss_first_last": [round(l, 6) for l in losses]},
        "flat_adam": {"ms": round(flat_ms, 4), "bound": "hbm", "achieved_GBps": round(flat_gbs, 1), "frac": round(flat_gbs / PEAK_HBM_GBS, 4),
                      "bytes": 28 * flat.n},
    }


def cpu_baseline():
    """Configuration 5 on ONE host core of this box, on a bounded sample: the reference's routines for the two things
    that make up the step's time -- dense-layer backward (its matmul, where 92 % of the block's flops go) at
    M=K=N=1024, scaled by flops to the block's 670 GFLOP, and boat_optimizer_step (Adam) on 2^24 parameters, scaled by
    element count to the 268,435,456 + 12,596,224 parameters of the step.  (The block itself cannot run on the
    reference: its LayerNorm backward and GELU are stubs.)"""
    sys.path.insert(0, str(ROOT / "tests"))
    import oracle_lib
    m = k = n = 1024
    rng = np.random.default_rng(3)
    x = rng.standard_normal((m, k), dtype=np.float32)
    w = (0.02 * rng.standard_normal((k, n), dtype=np.float32)).astype(np.float32)
    dy = rng.standard_normal((m, n), dtype=np.float32)
    B, S, H, heads, ffn = Block.B, Block.S, Block.H, Block.heads, Block.ffn
    block_flops = 2.0 * B * S * (4 * H * H + 2 * H * ffn) * 3 + 3 * 2 * 2.0 * (B * heads) * S * S * (H // heads)
    adam_params = FlatAdam.n + 4 * (H * H + H) + 4 * H + 2 * H * ffn + ffn + H
    sample_flops = 2 * 2.0 * m * k * n
    n_adam = 1 << 24
    p, g = (rng.standard_normal(n_adam, dtype=np.float32) for _ in range(2))
    ref = oracle_lib.load_reference()
    if ref is not None:
        layer = ref.boat_dense_layer_create(k, n, True)
        ref.write(ref.boat_dense_layer_get_weight(layer), w)
        tx, tdy = ref.tensor(x), ref.tensor(dy)
        ty = ref.boat_dense_layer_forward(layer, tx)          # caches the input; not timed
        t0 = time.perf_counter()
        tdx = ref.boat_dense_layer_backward(layer, tdy)
        sec = time.perf_counter() - t0
        assert ty and tdx, "reference backward failed"
        tp, tg = ref.tensor(p), ref.tensor(g)
        opt = ref.boat_adam_optimizer_create(1e-3, 0.9, 0.999, 1e-8)
        ref.boat_optimizer_add_parameter(opt, tp, tg)
        t0 = time.perf_counter()
        ref.boat_optimizer_step(opt)
        sec_adam = time.perf_counter() - t0
        kind, what = "reference", "boat_dense_layer_backward and boat_optimizer_step (Adam) of the compiled reference (oracle/_ref)"
    else:
        oracle = oracle_lib.load()
        t0 = time.perf_counter()
        oracle.dense_backward(x, w, dy)
        sec = time.perf_counter() - t0
        mm, vv = np.zeros(n_adam, np.float32), np.zeros(n_adam, np.float32)
        t0 = time.perf_counter()
        oracle.adam_update(p, g, mm, vv, 1e-3, 0.9, 0.999, 1e-8, 0)
        sec_adam = time.perf_counter() - t0
        kind, what = "port", "oracle dense_backward and adam_update (loop-order restatements of src/layers/dense.c:190-295, src/optimizers/adam.c:203-222)"
    block_ms = sec * 1e3 * block_flops / sample_flops
    adam_ms = sec_adam * 1e3 * adam_params / n_adam
    return {
        "value": round(block_ms + adam_ms, 1), "unit": "ms", "cores": 1, "kind": kind,
        "host_cores_total": os.cpu_count(),
        "sample": f"{what}: dense backward at M=K=N={m} ({sample_flops / 1e9:.2f} GFLOP) took {sec:.2f} s = "
                  f"{sample_flops / sec / 1e9:.2f} GFLOP/s, Adam on {n_adam} parameters took {sec_adam * 1e3:.1f} ms; value = the "
                  f"block's {block_flops / 1e9:.1f} GFLOP at that rate ({block_ms / 1e3:.0f} s) + Adam over {adam_params} parameters "
                  f"({adam_ms:.0f} ms), both extrapolated",
    }


def cpu_beside_other_configs():
    """The CPU path timed beside the other configurations, each on a bounded sample on ONE host core (a few seconds in
    total): the compiled reference where it has the routine, the oracle's restatement where the reference has a stub."""
    sys.path.insert(0, str(ROOT / "tests"))
    import oracle_lib
    import boat_cases as bc
    out = {}
    rng = np.random.default_rng(5)
    oracle = oracle_lib.load()
    ref = oracle_lib.load_reference()

    def timed(fn):
        t0 = time.perf_counter()
        fn()
        return time.perf_counter() - t0

    # config 5b, flat Adam: 2^24 parameters, scaled by element count
    n = 1 << 24
    p, g = (rng.standard_normal(n, dtype=np.float32) for _ in range(2))
    if ref is not None:
        tp, tg = ref.tensor(p), ref.tensor(g)
        opt = ref.boat_adam_optimizer_create(1e-3, 0.9, 0.999, 1e-8)
        ref.boat_optimizer_add_parameter(opt, tp, tg)
        sec = timed(lambda: ref.boat_optimizer_step(opt))
        ref.boat_optimizer_free(opt)
        ref.boat_tensor_unref(tp)
        ref.boat_tensor_unref(tg)
        what = "boat_optimizer_step (Adam) of the compiled reference"
    else:
        m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
        sec = timed(lambda: oracle.adam_update(p.copy(), g, m, v, 1e-3, 0.9, 0.999, 1e-8, 0))
        what = "oracle adam_update"
    out["adam_flat_268M"] = {"ms_extrapolated": round(sec * 1e3 * 268435456 / n, 1), "sample": f"{what} on {n} parameters: {sec * 1e3:.1f} ms"}
    # config 3: the reference has stubs for both kernels; float64 restatements of the oracle on 512 x 4096
    rows, hidden = 512, 4096
    x, dy = (rng.standard_normal((rows, hidden), dtype=np.float32) for _ in range(2))
    gamma = rng.standard_normal(hidden, dtype=np.float32)
    mean = x.mean(1).astype(np.float32)
    rstd = (1.0 / np.sqrt(x.var(1) + 1e-5)).astype(np.float32)
    sec = timed(lambda: oracle.layernorm_backward_f64(x, gamma, dy, mean, rstd))
    out["layernorm_bwd_16384x4096"] = {"ms_extrapolated": round(sec * 1e3 * 16384 / rows, 1),
                                       "sample": f"oracle layernorm_backward_f64 on {rows} x {hidden}: {sec * 1e3:.1f} ms (the reference's routine is a stub)"}
    sec = timed(lambda: oracle.gelu_backward_f64(x, dy))
    out["gelu_bwd_16384x4096"] = {"ms_extrapolated": round(sec * 1e3 * 16384 / rows, 1),
                                  "sample": f"oracle gelu_backward_f64 on {rows} x {hidden}: {sec * 1e3:.1f} ms (the reference's routine is a stub)"}
    # config 4: attention core backward, 4 blocks of S=256, D=64, scaled by flops (bh * S^2)
    bh_, S, D = 4, 256, 64
    q, k, v, go = (rng.standard_normal((bh_, S, D), dtype=np.float32) for _ in range(4))
    _, _, attn = oracle.sdpa_forward(q, k, v, 0.125)
    sec = timed(lambda: oracle.sdpa_backward(q, k, v, attn, go, 0.125))
    out["sdpa_bwd_B8h16S1024D64"] = {"ms_extrapolated": round(sec * 1e3 * (128 * 1024 * 1024) / (bh_ * S * S), 1),
                                     "sample": f"oracle sdpa_backward (loop-order restatement of src/layers/attention.c:1417-1520) on {bh_} blocks of S={S}: {sec * 1e3:.1f} ms"}
    # config 1: the MLP step at full size
    xb = rng.random((64, 784), dtype=np.float32)
    labels = rng.integers(0, 10, 64)
    w1 = (0.05 * rng.standard_normal((784, 128), dtype=np.float32)).astype(np.float32)
    w2 = (0.05 * rng.standard_normal((128, 10), dtype=np.float32)).astype(np.float32)
    b1, b2 = np.zeros(128, np.float32), np.zeros(10, np.float32)
    if ref is not None:
        steps = 5
        sec = timed(lambda: bc.mlp_ce_adam(ref, xb, labels, w1, b1, w2, b2, steps=steps)) / steps
        out["mlp_784_128_10_step"] = {"ms": round(sec * 1e3, 3), "sample": f"compiled reference, {steps} steps of the same tape chain through its C API (full size)"}
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported in this build (the path has no inter-GPU work)",
              file=sys.stderr)
        sys.exit(2)
    all_legs = ["step", "dense", "adam", "ln_gelu", "sdpa", "gemm", "mlp", "cnn", "conv"]
    legs = all_legs if args.legs == "all" else [l.strip() for l in args.legs.split(",") if l.strip()]
    unknown = [l for l in legs if l not in all_legs]
    if unknown:
        sys.exit(f"unknown leg(s) {unknown}; choose from {all_legs}")
    if args.no_extra:
        legs = [l for l in legs if l == "step"]
    from boat_amd import hip
    hip.check(hip.bh_init(), "bh_init")

    line = {
        "metric": METRIC, "value": None, "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None, "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "benchmark configuration 5: pre-LN transformer encoder block training step (d_model 1024, 16 heads, FFN 4096 "
                               "GELU, seq 512, batch 16; forward + boat_variable_backward + fused Adam over 12,596,224 parameters + zero_grad, "
                               "about 670 GFLOP) followed by fused Adam over 268,435,456 flat fp32 parameters (7.516 GB)",
                   "d_model": 1024, "heads": 16, "ffn": 4096, "seq": 512, "batch": 16, "flat_adam_params": 268435456,
                   "device": hip.bh_device_name().decode().strip(), "compute_units": hip.bh_device_cu_count()},
    }
    extra = {}
    if "step" in legs:
        res = bench_training_step(hip, args.steps, args.warmup)
        line.update({"value": round(res["ms_per_step"], 4), "ms_per_step": round(res["ms_per_step"], 4), "roofline": res["roofline"],
                     "wall_ms_per_step": round(res["wall_ms_per_step"], 4)})
        extra["step_breakdown"] = res["breakdown"]
        extra["transformer_block_step"] = res["block"]
        extra["adam_flat_268M_in_step"] = res["flat_adam"]
        if not args.no_extra:
            extra["transformer_block_step"]["c_caller"] = bench_block_step_c_caller(args.steps, args.warmup)
    if "dense" in legs:
        d = bench_dense_backward(hip, args.steps, args.warmup)
        extra["dense_backward_config2"] = {"ms": round(d["ms_per_step"], 4), "bound": "mfma", "step_TFLOPs": d["step_tflops"],
                                           "frac": round(d["step_tflops"] / PEAK_FP32_MFMA_TFLOPS, 4), "flops": 2 * d["roofline"]["flops_per_launch"],
                                           "gemm_launch": d["roofline"]}
        extra.update(bench_dense_forward(hip, args.steps, args.warmup))
    if "adam" in legs:
        extra.update(bench_adam(hip, args.steps, args.warmup))
    if "ln_gelu" in legs:
        extra.update(bench_ln_gelu(hip, args.steps, args.warmup))
    if "sdpa" in legs:
        extra.update(bench_sdpa(hip, args.steps, args.warmup))
    if "gemm" in legs:
        extra.update(bench_gemm_choice(hip))
    if "mlp" in legs:
        extra["mlp_784_128_10_step"] = bench_mlp_step(max(args.steps, 20) * 25, max(args.warmup, 1) * 100)
    if "conv" in legs:
        extra["conv_forward_kernels"] = bench_conv_forward_kernels()
    if "cnn" in legs:
        extra["mnist_cnn_step"] = bench_cnn_step(max(args.steps, 20), max(args.warmup, 3))
    if extra:
        line["extra"] = extra
    if not args.no_cpu and "step" in legs:
        line["cpu_baseline"] = cpu_baseline()
        if not args.no_extra:
            line["cpu_beside_other_configs"] = cpu_beside_other_configs()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
