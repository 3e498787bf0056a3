#!/usr/bin/env python3
"""Writes tests/golden/*.npz: inputs and expected outputs of the training hot path.

Reference-derived vectors come from the COMPILED REFERENCE (oracle/_ref/libboat_ref.so, built by
oracle/Makefile from the reference's own C sources) driven through its public C API by
tests/boat_cases.py -- the reference is C, so nothing of it is imported.  Two fixtures have no
reference counterpart (the reference ships stubs): LayerNorm backward and GELU; their vectors
come from an independent library, torch autograd in float64 on the CPU.

Run from the repository root in a container that has the reference tree:
    make -C oracle ref && python tests/golden/make_golden.py
Fixtures are plain numpy archives (np.load with allow_pickle=False reads them).

One fixture is text: scheduler_usage_lines.txt holds the learning-rate lines that examples/scheduler_usage.c of the
reference printed when built against the compiled reference:
    gcc -O2 -std=c11 -Dthread_local=_Thread_local -I$REF/include $REF/examples/scheduler_usage.c \
        -Loracle/_ref -lboat_ref -Wl,-rpath,$PWD/oracle/_ref -lm -o /tmp/scheduler_usage && /tmp/scheduler_usage \
        | grep -i "learning rate\|LR" | grep -v "create called\|create:" > tests/golden/scheduler_usage_lines.txt
"""
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

import boat_cases as bc  # noqa: E402
import oracle_lib  # noqa: E402
from test_oracle_vs_reference import ATT_CASES, CONV_CASES, POOL_CASES, cnn_params, conv_inputs, make_attention_inputs  # noqa: E402


ONLY = set(sys.argv[1:])   # fixture names to (re)write; none given = all


def save(name, **arrays):
    if ONLY and name not in ONLY:
        return
    path = HERE / f"{name}.npz"
    np.savez_compressed(path, **{k: np.asarray(v) for k, v in arrays.items() if v is not None})
    print(f"{path.name}: {path.stat().st_size / 1024:.1f} KiB, {len(arrays)} arrays")


def main():
    ref = oracle_lib.load_reference()
    if ref is None:
        sys.exit("oracle/_ref/libboat_ref.so is missing: run `make -C oracle ref` where the reference tree is present")
    rng = np.random.default_rng(20250611)

    # elementwise and activation gradients, [5,7], relu input contains exact zeros
    el = {}
    a = rng.standard_normal((5, 7)).astype(np.float32)
    b = (rng.standard_normal((5, 7)) + 3).astype(np.float32)
    dy = rng.standard_normal((5, 7)).astype(np.float32)
    el.update(a=a, b=b, dy=dy)
    for op in ("add", "sub", "mul", "div"):
        c, da, db = bc.binary_grads(ref, op, a, b, dy)
        el.update({f"{op}_out": c, f"{op}_da": da, f"{op}_db": db})
    x = rng.standard_normal((5, 7)).astype(np.float32)
    x[0, :3] = [0.0, -0.0, 1e-30]
    el["x"] = x
    for op in ("relu", "sigmoid", "tanh"):
        y, dx = bc.unary_grads(ref, op, x, dy)
        el.update({f"{op}_y": y, f"{op}_dx": dx})
    s, ds = bc.unary_grads(ref, "sum", x)
    el.update(sum_y=s, sum_dx=ds)
    save("elementwise", **el)

    sm = {}
    for tag, shape in (("a", (6, 10)), ("b", (3, 33))):
        x = (3 * rng.standard_normal(shape)).astype(np.float32)
        dy = rng.standard_normal(shape).astype(np.float32)
        sm.update({f"{tag}_x": x, f"{tag}_dy": dy})
        for op in ("softmax", "log_softmax"):
            y, dx = bc.unary_grads(ref, op, x, dy)
            sm.update({f"{tag}_{op}_y": y, f"{tag}_{op}_dx": dx})
    save("softmax", **sm)

    a4 = rng.standard_normal((2, 3, 5, 4)).astype(np.float32)
    b4 = rng.standard_normal((2, 3, 4, 6)).astype(np.float32)
    a2 = rng.standard_normal((7, 5)).astype(np.float32)
    b2 = rng.standard_normal((5, 9)).astype(np.float32)
    dy2 = rng.standard_normal((7, 9)).astype(np.float32)
    c2, da2, db2 = bc.matmul_grads(ref, a2, b2, dy2)
    save("matmul", a4=a4, b4=b4, c4=bc.matmul(ref, a4, b4), a4_t23=bc.transpose(ref, a4, 2, 3),
         a2=a2, b2=b2, dy2=dy2, c2=c2, da2=da2, db2=db2, a2_t01=bc.transpose(ref, a2, 0, 1))

    m, k, n = 9, 13, 6
    w = rng.standard_normal((k, n)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    x1, x2 = (rng.standard_normal((m, k)).astype(np.float32) for _ in range(2))
    dy1, dy2 = (rng.standard_normal((m, n)).astype(np.float32) for _ in range(2))
    (dx1, gw1, gb1), (dx2, gw2, gb2) = bc.dense_backward_twice(ref, w, bias, x1, dy1, x2, dy2)
    save("dense_bwd_accum", w=w, b=bias, x1=x1, x2=x2, dy1=dy1, dy2=dy2, y1=bc.dense_forward(ref, x1, w, bias),
         dx1=dx1, gw1=gw1, gb1=gb1, dx2=dx2, gw2=gw2, gb2=gb2)

    # config-1 chain: small MLP with full tensors over 3 Adam steps
    d_in, d_h, d_out, batch = 20, 16, 10, 8
    x = rng.random((batch, d_in), dtype=np.float32)
    labels = rng.integers(0, d_out, batch)
    w1 = rng.uniform(-0.4, 0.4, (d_in, d_h)).astype(np.float32)
    w2 = rng.uniform(-0.4, 0.4, (d_h, d_out)).astype(np.float32)
    b1, b2 = np.zeros(d_h, np.float32), np.zeros(d_out, np.float32)
    hist = bc.mlp_ce_adam(ref, x, labels, w1, b1, w2, b2, steps=3)
    arrays = dict(x=x, labels=labels, w1=w1, b1=b1, w2=w2, b2=b2)
    for t, rec in enumerate(hist):
        for key, val in rec.items():
            arrays[f"s{t}_{key}"] = np.float32(val) if key == "loss" else val
    save("mlp_small_3steps", **arrays)

    # config 1 at its real size (784-128-10, batch 64, one step): inputs are regenerated from the seed,
    # the large tensors are pinned by a few rows plus float64 checksums
    seed = 20250101
    r1 = np.random.default_rng(seed)
    d_in, d_h, d_out, batch = 784, 128, 10, 64
    x = r1.random((batch, d_in), dtype=np.float32)
    labels = r1.integers(0, d_out, batch)
    lim1, lim2 = np.sqrt(6.0 / (d_in + d_h)), np.sqrt(6.0 / (d_h + d_out))
    w1 = r1.uniform(-lim1, lim1, (d_in, d_h)).astype(np.float32)
    w2 = r1.uniform(-lim2, lim2, (d_h, d_out)).astype(np.float32)
    b1, b2 = np.zeros(d_h, np.float32), np.zeros(d_out, np.float32)
    rec = bc.mlp_ce_adam(ref, x, labels, w1, b1, w2, b2, steps=1)[0]

    def chk(arr):
        arr = np.asarray(arr, np.float64)
        return np.array([arr.sum(), np.abs(arr).sum(), (arr * arr).sum()])

    save("mlp_config1_step", seed=seed, labels=labels, input_checksums=np.stack([chk(x), chk(w1), chk(w2)]),
         loss=np.float32(rec["loss"]), gb1=rec["gb1"], gb2=rec["gb2"], gw2=rec["gw2"], b1=rec["b1"], b2=rec["b2"], w2=rec["w2"],
         gw1_rows=rec["gw1"][:4], w1_rows=rec["w1"][:4], gw1_chk=chk(rec["gw1"]), w1_chk=chk(rec["w1"]))

    for i, case in enumerate(ATT_CASES):
        xs, w, b, dys = make_attention_inputs(case, 99)
        out, results = bc.attention(ref, *xs, w, b, case["heads"], case["causal"], dys)
        arrays = dict(xq=xs[0], xk=xs[1], xv=xs[2], dy0=dys[0], dy1=dys[1], out=out,
                      meta=np.array([case["B"], case["S"], case["H"], case["heads"], int(case["causal"]), int(case["bias"])]))
        for nme in "qkvo":
            arrays["w" + nme] = w[nme]
            if b is not None:
                arrays["b" + nme] = b[nme]
        for t, rec in enumerate(results):
            for key, val in rec.items():
                if val is not None:
                    arrays[f"c{t}_{key}"] = val
        save(f"attention_case{i}", **arrays)

    # bare SDPA through identity projections (head split = plain reshape, scale on the scores, double row-dot)
    B, S, H, heads = 1, 8, 16, 2
    xs = [rng.standard_normal((B, S, H)).astype(np.float32) for _ in range(3)]
    eye = {nme: np.eye(H, dtype=np.float32) for nme in "qkvo"}
    dy = rng.standard_normal((B, S, H)).astype(np.float32)
    out, (rec,) = bc.attention(ref, *xs, eye, None, heads, False, [dy])
    save("sdpa_core", xq=xs[0], xk=xs[1], xv=xs[2], dy=dy, out=out, dq=rec["dq"], dk=rec["dk"], dv=rec["dv"],
         meta=np.array([B, S, H, heads]))

    ln = {}
    for tag, shape in (("a", (2, 5, 48)), ("b", (7, 64))):
        x = rng.standard_normal(shape).astype(np.float32)
        gamma = (1 + 0.1 * rng.standard_normal(shape[-1])).astype(np.float32)
        beta = (0.1 * rng.standard_normal(shape[-1])).astype(np.float32)
        ln.update({f"{tag}_x": x, f"{tag}_gamma": gamma, f"{tag}_beta": beta,
                   f"{tag}_y": bc.layernorm_forward(ref, x, gamma, beta, 1e-5)})
    save("layernorm_fwd", **ln)

    shapes = [(4, 3), (7,), (1,)]
    params = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    grads = [[(rng.standard_normal(s) * 10 ** rng.uniform(-4, 1)).astype(np.float32) for s in shapes] for _ in range(10)]
    traj, _ = bc.adam_trajectory(ref, params, grads, lr=1e-2, lr_change=(5, 3e-3))
    arrays = {}
    for i in range(3):
        arrays[f"p{i}"] = params[i]
        arrays[f"g{i}"] = np.stack([g[i] for g in grads])
        arrays[f"traj{i}"] = np.stack([t[i] for t in traj])
    save("adam_traj", **arrays)

    r2 = np.random.default_rng(20250612)   # its own stream, so the fixtures above never change
    for kind in ("rmsprop", "adagrad"):
        params = [r2.standard_normal(s).astype(np.float32) for s in shapes]
        grads = [[(r2.standard_normal(s) * 10 ** r2.uniform(-4, 1)).astype(np.float32) for s in shapes] for _ in range(10)]
        traj, _ = bc.adam_trajectory(ref, params, grads, lr=1e-2, beta1=0.99, eps=1e-8, lr_change=(5, 3e-3), kind=kind)
        arrays = {}
        for i in range(3):
            arrays[f"p{i}"] = params[i]
            arrays[f"g{i}"] = np.stack([g[i] for g in grads])
            arrays[f"traj{i}"] = np.stack([t[i] for t in traj])
        save(f"{kind}_traj", **arrays)

    a, b = np.array([1.5, -2.0], np.float32), np.array([3.0, 0.5], np.float32)
    da, db = bc.fanout(ref, a, b)
    save("fanout_divergence", a=a, b=b, ref_da=da, ref_db=db)

    # convolution (two backward calls: parameter gradients are overwritten), max pooling, the MNIST CNN chain
    conv = {}
    for i, case in enumerate(CONV_CASES[:3]):
        d = conv_inputs(case, 500 + i)
        y, calls = bc.conv_layer(ref, d["x"], d["w"], d["b"], case[6], case[7], [d["dy1"], d["dy2"]])
        conv.update({f"c{i}_{k}": v for k, v in d.items()})
        conv.update({f"c{i}_meta": np.array(case), f"c{i}_y": y})
        for j, (dx, gw, gb) in enumerate(calls):
            conv.update({f"c{i}_dx{j}": dx, f"c{i}_gw{j}": gw, f"c{i}_gb{j}": gb})
    save("conv_layer", **conv)
    r3 = np.random.default_rng(20250613)
    pool = {}
    for i, (B, ch, h, w, k, stride, pad) in enumerate(POOL_CASES):
        x = r3.standard_normal((B, ch, h, w)).astype(np.float32)
        x[0, 0, :2, :2] = 1.5
        ho, wo = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
        dy = r3.standard_normal((B, ch, ho, wo)).astype(np.float32)
        y, dx = bc.pool_layer(ref, x, k, stride, pad, dy)
        pool.update({f"p{i}_meta": np.array([k, stride, pad]), f"p{i}_x": x, f"p{i}_dy": dy, f"p{i}_y": y, f"p{i}_dx": dx})
    save("pool_layer", **pool)
    x = r3.random((3, 2, 8, 8), dtype=np.float32)
    labels = r3.integers(0, 5, 3)
    p = cnn_params(r3, 2, 4, 6, 8, 12, 5)
    rec = bc.cnn_ce_grads(ref, x, labels, p)
    save("cnn_chain", x=x, labels=labels, **{"p_" + k: v for k, v in p.items()},
         **{k: (np.float32(v) if k == "loss" else v) for k, v in rec.items()})
    # the example's weight checkpoint: written by the reference from a model holding p, read back into a model
    # created with other weights; logits of the loaded model (layer hooks, no tape)
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        path = str(Path(tmp) / "model.bin")
        holder = bc.CnnLayers(ref, p)
        holder.save(path)
        other = bc.CnnLayers(ref, {k: np.full_like(v, 0.01) for k, v in p.items()})
        assert other.load(path)
        save("cnn_checkpoint", content=np.frombuffer(Path(path).read_bytes(), np.uint8), x=x, logits=other.logits(x))

    # ---- the reference's layer-based MNIST example on a small synthetic set: what it prints on the reference ----
    if not ONLY or "mnist_synthetic" in ONLY:
        import re
        import subprocess
        import tempfile
        r4 = np.random.default_rng(4)
        sets = {}
        for name, count in (("train", 80), ("test", 16)):
            labels = r4.integers(0, 10, count).astype(np.uint8)
            images = r4.integers(0, 40, (count, 28, 28)).astype(np.uint8)
            for i, c in enumerate(labels):                      # a bright patch whose place tells the class
                row, col = divmod(int(c), 4)
                images[i, 4 + 7 * row: 11 + 7 * row, 2 + 6 * col: 8 + 6 * col] += 200
            sets[name] = (images, labels)
        with tempfile.TemporaryDirectory() as tmp:
            bc.write_mnist_example_files(Path(tmp), *sets["train"], *sets["test"])
            exe = Path(tmp) / "mnist"
            ref_root = Path("/root/reference")
            subprocess.run(["gcc", "-O2", "-std=c11", "-w", "-Dthread_local=_Thread_local", "-D_POSIX_C_SOURCE=200809L",
                            f"-I{ref_root / 'include'}", f"-I{ref_root / 'src'}", str(ref_root / "examples/mnist/mnist.c"),
                            "-o", str(exe), f"-L{ROOT / 'oracle/_ref'}", "-lboat_ref", f"-Wl,-rpath,{ROOT / 'oracle/_ref'}", "-lm"],
                           check=True)
            out = subprocess.run([str(exe)], cwd=tmp, capture_output=True, text=True, errors="replace", check=True).stdout
        lines = [re.sub(r"time=[0-9.]+s, ", "", line) for line in out.splitlines() if re.match(r"Epoch \d|Test accuracy", line)]
        print("\n".join(lines))
        save("mnist_synthetic", train_images=sets["train"][0], train_labels=sets["train"][1], test_images=sets["test"][0],
             test_labels=sets["test"][1], reference_lines=np.array(lines))

    # ---- RMSNorm forward, the public attention core and the non-float32 elementwise ops (own generator: fixtures
    # above keep their values when this block changes) ----
    r5 = np.random.default_rng(20251125)
    rn = {}
    for tag, shape in (("a", (2, 5, 48)), ("b", (7, 64)), ("c", (32,)), ("d", (2, 3, 2, 8))):   # d: only 2*3 rows are visited
        x = (r5.standard_normal(shape) * 10 ** r5.uniform(-2, 1)).astype(np.float32)
        rn.update({f"{tag}_x": x, f"{tag}_y": bc.rmsnorm_forward(ref, x, 1e-6), f"{tag}_y_plain": bc.rmsnorm_forward(ref, x, 1e-3, affine=False)})
    rn["zero_x"] = np.zeros((3, 8), np.float32)
    rn["zero_y"] = bc.rmsnorm_forward(ref, rn["zero_x"], 1e-6)
    save("rmsnorm_fwd", **rn)

    sd = {}
    for tag, (shape, causal) in (("a", ((2, 3, 16, 8), False)), ("b", ((1, 2, 40, 16), True)), ("c", ((2, 2, 64, 64), False))):
        q, k, v = (r5.standard_normal(shape).astype(np.float32) for _ in range(3))
        scale = float(1.0 / np.sqrt(np.float32(shape[-1])))
        sd.update({f"{tag}_q": q, f"{tag}_k": k, f"{tag}_v": v, f"{tag}_scale": np.float32(scale), f"{tag}_causal": np.array(causal),
                   f"{tag}_out": bc.sdpa_public(ref, q, k, v, scale, causal)})
    sd["three_d_q"] = r5.standard_normal((2, 5, 8)).astype(np.float32)          # not 4-D: the reference hands back a copy of value
    sd["three_d_v"] = r5.standard_normal((2, 5, 8)).astype(np.float32)
    sd["three_d_out"] = bc.sdpa_public(ref, sd["three_d_q"], sd["three_d_q"], sd["three_d_v"], 0.5, False)
    save("sdpa_public", **sd)

    ty = {}
    for tag, dt in (("f64", np.float64), ("i32", np.int32), ("i64", np.int64), ("f32", np.float32)):
        if dt in (np.float64, np.float32):
            a = (r5.standard_normal((4, 3, 5)) * 3).astype(dt)
            b = (r5.standard_normal((3, 1)) + 2.5).astype(dt)
            a2 = np.abs(a) + dt(0.25)
        else:
            a = r5.integers(-1000, 1000, (4, 3, 5)).astype(dt)
            b = r5.integers(1, 37, (3, 1)).astype(dt) * np.where(r5.random((3, 1)) < 0.5, -1, 1).astype(dt)
            a2 = a
        same_shape_b = np.broadcast_to(b, a.shape).copy()
        ty.update({f"{tag}_a": a, f"{tag}_b": b})
        for key, val in bc.typed_arithmetic(ref, a, b, 2.75).items():
            ty[f"{tag}_bc_{key}"] = val
        for key, val in bc.typed_arithmetic(ref, a2, same_shape_b, -1.5 if dt in (np.float64, np.float32) else 3.0).items():
            ty[f"{tag}_eq_{key}"] = val
    save("typed_ops", **ty)

    # ---- not the reference: float64 autograd of an independent library ----
    import torch
    torch.manual_seed(0)
    x = torch.randn(9, 64, dtype=torch.float64, requires_grad=True)
    gamma = (1 + 0.1 * torch.randn(64, dtype=torch.float64)).requires_grad_()
    beta = (0.1 * torch.randn(64, dtype=torch.float64)).requires_grad_()
    dy = torch.randn(9, 64, dtype=torch.float64)
    y = torch.nn.functional.layer_norm(x, (64,), gamma, beta, 1e-5)
    y.backward(dy)
    save("ln_bwd_ref64", x=x.detach().numpy(), gamma=gamma.detach().numpy(), beta=beta.detach().numpy(), dy=dy.numpy(),
         y=y.detach().numpy(), dx=x.grad.numpy(), dgamma=gamma.grad.numpy(), dbeta=beta.grad.numpy())
    x = (2 * torch.randn(9, 64, dtype=torch.float64)).requires_grad_()
    y = torch.nn.functional.gelu(x, approximate="none")
    y.backward(dy)
    save("gelu_ref64", x=x.detach().numpy(), dy=dy.numpy(), y=y.detach().numpy(), dx=x.grad.numpy())
    # RMSNorm as the reference defines it (eps outside the root), backward is a stub there
    torch.manual_seed(1)
    for tag, eps in (("a", 1e-6), ("b", 1e-2)):
        x = (torch.randn(11, 96, dtype=torch.float64) * (0.05 if tag == "b" else 1.0)).requires_grad_()
        w = (1 + 0.2 * torch.randn(96, dtype=torch.float64)).requires_grad_()
        dy = torch.randn(11, 96, dtype=torch.float64)
        y = x / (torch.sqrt((x * x).mean(-1, keepdim=True)) + eps) * w
        y.backward(dy)
        rm = {"x": x.detach().numpy(), "w": w.detach().numpy(), "dy": dy.numpy(), "y": y.detach().numpy(), "dx": x.grad.numpy(),
              "dw": w.grad.numpy(), "eps": np.float64(eps)}
        save(f"rmsnorm_bwd_ref64_{tag}", **rm)

    # One batch element of benchmark configuration 5's block at its real sizes (d_model 1024, 16 heads, seq 512, FFN 4096)
    # in float64 autograd: sampled rows of y and dx, sampled entries of every parameter gradient, the loss.  The inputs
    # are regenerated from the seed by tests/test_block.py::make_block, the sample positions by block_ref64_sample().
    if not ONLY or "block_config5_ref64" in ONLY:
        from test_block import BLOCK_REF64, block_ref64_sample, make_block, torch_block_grads
        c = BLOCK_REF64
        x, target, params = make_block(c["seed"], 1, c["S"], c["H"], c["ffn"])
        want = torch_block_grads(x, target, params, c["heads"])
        rows, picks = block_ref64_sample(params)
        blk = {"loss": np.float64(want["loss"]), "y_rows": want["y"][0][rows].astype(np.float32),
               "dx_rows": want["dx"][0][rows].astype(np.float32)}
        for name in bc.BLOCK_PARAM_ORDER:
            blk["g_" + name] = want["g_" + name].reshape(-1)[picks[name]].astype(np.float32)
        save("block_config5_ref64", **blk)


if __name__ == "__main__":
    main()
