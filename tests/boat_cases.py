"""Training-path scenarios written once against Boat's C API and run against any library that
exports it: the compiled reference (to pin the oracle and to write golden vectors) and
libboat_amd.so (the GPU path under test).  Each function takes a BoatAPI and numpy inputs and
returns numpy outputs, so results from two libraries can be compared directly.

The call sequences follow the reference's own callers and tests:
  tests/unit/test_autodiff.c:116-456, tests/test_dense_forward.c, tests/unit/test_optimizer_adam.c,
  tests/unit/test_attention_gradient_check.c, tests/test_attention_training.c:115-179,
  examples/mnist/mnist_autodiff.c:397-522,2437-2488.
"""
import contextlib
import ctypes as C
import os
import tempfile

import numpy as np

from boat_amd.capi import AttentionConfig, LayerNormConfig


@contextlib.contextmanager
def scratch_cwd():
    """The reference's attention backward appends to a debug file in the current directory
    (src/layers/attention.c:478); run it from a throw-away directory."""
    old = os.getcwd()
    with tempfile.TemporaryDirectory() as tmp:
        os.chdir(tmp)
        try:
            yield
        finally:
            os.chdir(old)


def _var(api, arr, requires_grad):
    t = api.tensor(np.asarray(arr, np.float32))
    v = api.boat_variable_create(t, requires_grad)
    api.boat_tensor_unref(t)
    return v


def _grad(api, v):
    g = api.boat_variable_grad(v)
    return None if not g else api.numpy(g)


BINARY = {"add": "boat_var_add", "sub": "boat_var_sub", "mul": "boat_var_mul", "div": "boat_var_div"}
UNARY = {"relu": "boat_var_relu", "sigmoid": "boat_var_sigmoid", "tanh": "boat_var_tanh"}


def binary_grads(api, op, a, b, dy=None):
    """c = a (op) b; backward with dy (or ones).  Returns c, da, db."""
    va, vb = _var(api, a, True), _var(api, b, True)
    vc = getattr(api, BINARY[op])(va, vb)
    c = api.numpy(api.boat_variable_data(vc))
    if dy is None:
        api.boat_variable_backward_full(vc)
    else:
        tdy = api.tensor(np.asarray(dy, np.float32))
        api.boat_variable_backward(vc, tdy)
        api.boat_tensor_unref(tdy)
    out = c, _grad(api, va), _grad(api, vb)
    return out


def unary_grads(api, op, x, dy=None, axis=-1):
    """y = f(x); backward with dy (or ones).  Returns y, dx."""
    vx = _var(api, x, True)
    if op in UNARY:
        vy = getattr(api, UNARY[op])(vx)
    elif op == "softmax":
        vy = api.boat_var_softmax(vx, axis)
    elif op == "log_softmax":
        vy = api.boat_var_log_softmax(vx, axis)
    elif op == "sum":
        vy = api.boat_var_sum(vx, None, 0, False)
    else:
        raise ValueError(op)
    y = api.numpy(api.boat_variable_data(vy))
    if dy is None:
        api.boat_variable_backward_full(vy)
    else:
        tdy = api.tensor(np.asarray(dy, np.float32))
        api.boat_variable_backward(vy, tdy)
        api.boat_tensor_unref(tdy)
    return y, _grad(api, vx)


def dot_grads(api, a, b):
    va, vb = _var(api, a, True), _var(api, b, True)
    vc = api.boat_var_dot(va, vb)
    c = api.numpy(api.boat_variable_data(vc))
    api.boat_variable_backward_full(vc)
    return c, _grad(api, va), _grad(api, vb)


def matmul_grads(api, a, b, dy):
    va, vb = _var(api, a, True), _var(api, b, True)
    vc = api.boat_var_matmul(va, vb)
    c = api.numpy(api.boat_variable_data(vc))
    tdy = api.tensor(np.asarray(dy, np.float32))
    api.boat_variable_backward(vc, tdy)
    api.boat_tensor_unref(tdy)
    return c, _grad(api, va), _grad(api, vb)


def matmul(api, a, b):
    ta, tb = api.tensor(np.asarray(a, np.float32)), api.tensor(np.asarray(b, np.float32))
    tc = api.boat_matmul(ta, tb)
    out = api.numpy(tc)
    for t in (ta, tb, tc):
        api.boat_tensor_unref(t)
    return out


def transpose(api, a, d0, d1):
    ta = api.tensor(np.asarray(a, np.float32))
    tt = api.boat_transpose(ta, d0, d1)
    out = api.numpy(tt)
    api.boat_tensor_unref(ta)
    api.boat_tensor_unref(tt)
    return out


def fanout(api, a, b):
    """z = y + y with y = a*b: the reference's recursive backward double-counts (returns da, db)."""
    va, vb = _var(api, a, True), _var(api, b, True)
    vy = api.boat_var_mul(va, vb)
    vz = api.boat_var_add(vy, vy)
    api.boat_variable_backward_full(vz)
    return _grad(api, va), _grad(api, vb)


def backward_twice(api, a, b, c, d, g1, g2):
    """w = (a*b + c) * d, then boat_variable_backward(w, g1) and boat_variable_backward(w, g2) over the same kept graph.
    Non-leaf gradients are not cleared between the two walks (src/autodiff.c:373-450 adds into what is there), so the
    second walk hands on u.grad = (g1 + g2)*d: a chain, on which the reference and a walk that visits each op once agree.
    Returns the gradients of a, b, c, d."""
    va, vb, vc, vd = (_var(api, t, True) for t in (a, b, c, d))
    vt = api.boat_var_mul(va, vb)
    vu = api.boat_var_add(vt, vc)
    vw = api.boat_var_mul(vu, vd)
    for g in (g1, g2):
        tg = api.tensor(np.asarray(g, np.float32))
        api.boat_variable_backward(vw, tg)
        api.boat_tensor_unref(tg)
    return tuple(_grad(api, v) for v in (va, vb, vc, vd))


def backward_twice_expected(a, b, c, d, g1, g2):
    """Closed form of backward_twice in float64."""
    a, b, c, d, g1, g2 = (np.asarray(t, np.float64) for t in (a, b, c, d, g1, g2))
    u = a * b + c
    gu1 = g1 * d                     # after the first walk
    gu2 = gu1 + g2 * d               # u.grad after the second contribution
    gt = gu1 + gu2                   # t.grad: first walk's, plus the accumulated u.grad handed on by the add
    gc = gu1 + gu2
    return gt * b + gu1 * b, gt * a + gu1 * a, gc, g1 * u + g2 * u


def grad_under_disabled_context(api, a, b):
    """y = a*b recorded while the current context has gradients switched off, then backward: the gradient of a, or None
    when the op left no tape entry."""
    ctx = api.boat_autodiff_context_create()
    before = api.boat_autodiff_get_current_context()
    api.boat_autodiff_set_current_context(ctx)
    api.boat_autodiff_context_disable_grad(ctx)
    va, vb = _var(api, a, True), _var(api, b, True)
    vy = api.boat_var_mul(va, vb)
    api.boat_variable_backward_full(vy)
    g = api.boat_variable_grad(va)
    out = api.numpy(g) if g else None
    api.boat_autodiff_set_current_context(before)
    api.boat_autodiff_context_free(ctx)
    return out


def _make_dense(api, w, b):
    layer = api.boat_dense_layer_create(w.shape[0], w.shape[1], b is not None)
    api.write(api.boat_dense_layer_get_weight(layer), w)      # in place, never set_weight (dangling optimizer pointers)
    if b is not None:
        api.write(api.boat_dense_layer_get_bias(layer), b)
    return layer


def dense_forward(api, x, w, b):
    layer = _make_dense(api, np.asarray(w, np.float32), None if b is None else np.asarray(b, np.float32))
    tx = api.tensor(np.asarray(x, np.float32))
    ty = api.boat_dense_layer_forward(layer, tx)
    y = api.numpy(ty)
    api.boat_tensor_unref(ty)
    api.boat_tensor_unref(tx)
    api.boat_dense_layer_free(layer)
    return y


def dense_backward_twice(api, w, b, x1, dy1, x2, dy2):
    """forward/backward called twice on one layer: grads accumulate (dense.c:255-291).
    Returns [(dx, grad_weight, grad_bias) after call 1, after call 2]."""
    layer = _make_dense(api, np.asarray(w, np.float32), None if b is None else np.asarray(b, np.float32))
    out = []
    for x, dy in ((x1, dy1), (x2, dy2)):
        tx, tdy = api.tensor(np.asarray(x, np.float32)), api.tensor(np.asarray(dy, np.float32))
        ty = api.boat_dense_layer_forward(layer, tx)
        tdx = api.boat_dense_layer_backward(layer, tdy)
        gb = api.boat_dense_layer_get_grad_bias(layer)
        out.append((api.numpy(tdx), api.numpy(api.boat_dense_layer_get_grad_weight(layer)),
                    None if not gb else api.numpy(gb)))
        for t in (ty, tdx, tx, tdy):
            api.boat_tensor_unref(t)
    api.boat_dense_layer_free(layer)
    return out


def mlp_ce_adam(api, x, labels, w1, b1, w2, b2, steps=1, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8):
    """The config-1 training step: dense -> relu -> dense -> log_softmax -> mul(onehot) -> sum -> mul(-1/B),
    boat_variable_backward_full, boat_optimizer_step, boat_optimizer_zero_grad; `steps` times.
    Returns a list per step of dict(loss, gw1, gb1, gw2, gb2, w1, b1, w2, b2)."""
    x = np.asarray(x, np.float32)
    B = x.shape[0]
    classes = w2.shape[1]
    l1 = _make_dense(api, np.asarray(w1, np.float32), np.asarray(b1, np.float32))
    l2 = _make_dense(api, np.asarray(w2, np.float32), np.asarray(b2, np.float32))
    opt = api.boat_adam_optimizer_create(lr, beta1, beta2, eps)
    for layer in (l1, l2):
        api.boat_optimizer_add_parameter(opt, api.boat_dense_layer_get_weight(layer), api.boat_dense_layer_get_grad_weight(layer))
        api.boat_optimizer_add_parameter(opt, api.boat_dense_layer_get_bias(layer), api.boat_dense_layer_get_grad_bias(layer))
    onehot = np.zeros((B, classes), np.float32)
    onehot[np.arange(B), np.asarray(labels)] = 1.0
    history = []
    for _ in range(steps):
        vx = _var(api, x, True)                       # requires_grad so the dense ops record (autodiff.c:2287)
        h = api.boat_var_dense(vx, l1)
        r = api.boat_var_relu(h)
        z = api.boat_var_dense(r, l2)
        ls = api.boat_var_log_softmax(z, 1)
        voh = _var(api, onehot, False)
        m = api.boat_var_mul(voh, ls)
        s = api.boat_var_sum(m, None, 0, False)
        vf = _var(api, np.array([-1.0 / B], np.float32), False)
        loss = api.boat_var_mul(vf, s)
        loss_value = float(api.numpy(api.boat_variable_data(loss))[0])
        api.boat_variable_backward_full(loss)
        rec = {"loss": loss_value}
        for name, layer in (("1", l1), ("2", l2)):
            rec["gw" + name] = api.numpy(api.boat_dense_layer_get_grad_weight(layer))
            rec["gb" + name] = api.numpy(api.boat_dense_layer_get_grad_bias(layer))
        api.boat_optimizer_step(opt)
        api.boat_optimizer_zero_grad(opt)
        for name, layer in (("1", l1), ("2", l2)):
            rec["w" + name] = api.numpy(api.boat_dense_layer_get_weight(layer))
            rec["b" + name] = api.numpy(api.boat_dense_layer_get_bias(layer))
        history.append(rec)
        # variables are left to the library that owns them: the reference cannot release a recorded tape
        if api.is_amd:
            for v in (loss, vf, s, m, voh, ls, z, r, h, vx):
                api.boat_variable_free(v)
    api.boat_optimizer_free(opt)
    if api.is_amd:
        api.boat_dense_layer_free(l1)
        api.boat_dense_layer_free(l2)
    return history


def adam_trajectory(api, params, grads_per_step, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, lr_change=None, kind="adam"):
    """Several tensors registered with one optimizer; grads rewritten in place before each step.
    lr_change = (step_index, new_lr).  kind: "adam", "rmsprop" (beta1 is its alpha) or "adagrad".
    Returns params after every step: list of lists of arrays."""
    tp = [api.tensor(np.asarray(p, np.float32)) for p in params]
    tg = [api.zeros(np.asarray(p).shape) for p in params]
    if kind == "adam":
        opt = api.boat_adam_optimizer_create(lr, beta1, beta2, eps)
    elif kind == "rmsprop":
        opt = api.boat_rmsprop_optimizer_create(lr, beta1, eps)
    else:
        opt = api.boat_adagrad_optimizer_create(lr, eps)
    assert opt, f"{kind} optimizer creation failed"
    for p, g in zip(tp, tg):
        api.boat_optimizer_add_parameter(opt, p, g)
    out = []
    for step, grads in enumerate(grads_per_step):
        if lr_change and lr_change[0] == step:
            api.boat_optimizer_set_learning_rate(opt, lr_change[1])
        for g, arr in zip(tg, grads):
            api.write(g, arr)
        api.boat_optimizer_step(opt)
        out.append([api.numpy(p) for p in tp])
    api.boat_optimizer_zero_grad(opt)
    zeroed = [api.numpy(g) for g in tg]
    api.boat_optimizer_free(opt)
    for t in tp + tg:
        api.boat_tensor_unref(t)
    return out, zeroed


def layernorm_forward(api, x, gamma, beta, eps):
    x = np.asarray(x, np.float32)
    cfg = LayerNormConfig(x.shape[-1], eps, gamma is not None, beta is not None)
    norm = api.boat_layernorm_create(C.byref(cfg))
    if gamma is not None:
        tg = api.tensor(np.asarray(gamma, np.float32))
        api.boat_layernorm_set_weight(norm, tg)
        api.boat_tensor_unref(tg)
    if beta is not None:
        tb = api.tensor(np.asarray(beta, np.float32))
        api.boat_layernorm_set_bias(norm, tb)
        api.boat_tensor_unref(tb)
    tx = api.tensor(x)
    ty = api.boat_layernorm_forward(norm, tx)
    y = api.numpy(ty)
    api.boat_tensor_unref(ty)
    api.boat_tensor_unref(tx)
    api.boat_layernorm_free(norm)
    return y


def rmsnorm_forward(api, x, eps, affine=True):
    """boat_rmsnorm_forward through the layer object (the reference offers no way to set the weight: it stays ones)."""
    from boat_amd.capi import RmsNormConfig
    x = np.asarray(x, np.float32)
    cfg = RmsNormConfig(x.shape[-1], eps, affine)
    norm = api.boat_rmsnorm_create(C.byref(cfg))
    tx = api.tensor(x)
    ty = api.boat_rmsnorm_forward(norm, tx)
    y = api.numpy(ty)
    api.boat_tensor_unref(ty)
    api.boat_tensor_unref(tx)
    api.boat_rmsnorm_free(norm)
    return y


def sdpa_public(api, q, k, v, scale, causal):
    """boat_scaled_dot_product_attention on [batch, heads, seq, head_size] operands."""
    ts = [api.tensor(np.asarray(a, np.float32)) for a in (q, k, v)]
    to = api.boat_scaled_dot_product_attention(ts[0], ts[1], ts[2], scale, None, causal, 0.0)
    out = api.numpy(to) if to else None
    if to:
        api.boat_tensor_unref(to)
    for t in ts:
        api.boat_tensor_unref(t)
    return out


def typed_arithmetic(api, a, b, scalar):
    """The eager elementwise ops on tensors of a's dtype (float64 / int32 / int64 / float32): a dict of results.
    b broadcasts against a; scalar is a Python float."""
    out = {}
    ta, tb = api.tensor(a), api.tensor(b)
    for name in ("add", "sub", "mul", "div", "mod"):
        t = getattr(api, f"boat_{name}")(ta, tb)
        out[name] = api.numpy(t)
        api.boat_tensor_unref(t)
    for name in ("add", "sub", "mul", "div"):
        t = getattr(api, f"boat_{name}_scalar")(ta, scalar)
        out[f"{name}_scalar"] = api.numpy(t)
        api.boat_tensor_unref(t)
        tc = api.tensor(a)
        getattr(api, f"boat_{name}_scalar_")(tc, scalar)
        out[f"{name}_scalar_inplace"] = api.numpy(tc)
        api.boat_tensor_unref(tc)
    if a.shape == b.shape:
        for name in ("add", "sub", "mul", "div"):
            tc = api.tensor(a)
            getattr(api, f"boat_{name}_")(tc, tb)
            out[f"{name}_inplace"] = api.numpy(tc)
            api.boat_tensor_unref(tc)
    if a.dtype.kind == "f":
        t = api.boat_pow_scalar(ta, scalar)
        out["pow_scalar"] = api.numpy(t)
        api.boat_tensor_unref(t)
    else:
        out["pow_scalar_is_null"] = np.array(not api.boat_pow_scalar(ta, scalar))
    api.boat_tensor_unref(ta)
    api.boat_tensor_unref(tb)
    return out


def attention(api, xq, xk, xv, weights, biases, heads, causal, d_out_list):
    """boat_attention_forward once, then boat_attention_backward for each dY in d_out_list
    (parameter grads are overwritten per call).  weights/biases: dicts q,k,v,o (biases None = no bias).
    Returns out and, per backward call, dict(dq, dk, dv, gw{q,k,v,o}, gb{q,k,v,o})."""
    xq = np.asarray(xq, np.float32)
    hidden = xq.shape[-1]
    cfg = AttentionConfig(hidden, heads, hidden // heads, 0.0, bool(causal), biases is not None, False, 10000.0)
    att = api.boat_attention_create(C.byref(cfg))
    for n in "qkvo":
        api.write(getattr(api, f"boat_attention_get_weight_{n}")(att), weights[n])
        if biases is not None:
            api.write(getattr(api, f"boat_attention_get_bias_{n}")(att), biases[n])
    tq, tk, tv = (api.tensor(np.asarray(a, np.float32)) for a in (xq, xk, xv))
    results = []
    with scratch_cwd():
        tout = api.boat_attention_forward(att, tq, tk, tv, None)
        out = api.numpy(tout)
        for d_out in d_out_list:
            tdy = api.tensor(np.asarray(d_out, np.float32))
            gq, gk, gv = C.c_void_p(), C.c_void_p(), C.c_void_p()
            ok = api.boat_attention_backward(att, tdy, C.byref(gq), C.byref(gk), C.byref(gv))
            assert ok, "boat_attention_backward failed"
            rec = {"dq": api.numpy(gq), "dk": api.numpy(gk), "dv": api.numpy(gv)}
            for n in "qkvo":
                rec["gw" + n] = api.numpy(getattr(api, f"boat_attention_get_grad_weight_{n}")(att))
                gb = getattr(api, f"boat_attention_get_grad_bias_{n}")(att)
                rec["gb" + n] = api.numpy(gb) if (biases is not None and gb) else None
            results.append(rec)
            for t in (gq, gk, gv, tdy):
                api.boat_tensor_unref(t)
    api.boat_tensor_unref(tout)
    if api.is_amd:
        api.boat_attention_free(att)
        for t in (tq, tk, tv):
            api.boat_tensor_unref(t)
    return out, results


BLOCK_PARAM_ORDER = ("ln1_g", "ln1_b", "wq", "wk", "wv", "wo", "bq", "bk", "bv", "bo", "ln2_g", "ln2_b", "w1", "b1", "w2", "b2")


def transformer_block_steps(api, x, target, params, heads, steps=1, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8):
    """Pre-LN encoder block training steps through the tape (libboat_amd only: LayerNorm backward and GELU are
    stubs in the reference):
        x1 = x + Attention(LN1(x)) ; y = x1 + Dense2(GELU(Dense1(LN2(x1)))) ; loss = MSE(y, target)
    then boat_variable_backward(y, dLoss/dy), boat_optimizer_step over the 16 parameter tensors, zero_grad.
    x, target: [B, S, H]; params: dict keyed by BLOCK_PARAM_ORDER ([in, out] weights).
    Returns per step dict(loss, y, dx, g_<name>..., p_<name>...)."""
    x = np.asarray(x, np.float32)
    B, S, H = x.shape
    ffn = params["w1"].shape[1]
    ln = []
    for tag in ("ln1", "ln2"):
        cfg = LayerNormConfig(H, 1e-5, True, True)
        norm = api.boat_layernorm_create(C.byref(cfg))
        api.write(api.boat_hip_layernorm_get_weight(norm), params[tag + "_g"])
        api.write(api.boat_hip_layernorm_get_bias(norm), params[tag + "_b"])
        ln.append(norm)
    cfg = AttentionConfig(H, heads, H // heads, 0.0, False, True, False, 10000.0)
    att = api.boat_attention_create(C.byref(cfg))
    for n in "qkvo":
        api.write(getattr(api, f"boat_attention_get_weight_{n}")(att), params["w" + n])
        api.write(getattr(api, f"boat_attention_get_bias_{n}")(att), params["b" + n])
    d1 = _make_dense(api, np.asarray(params["w1"], np.float32), np.asarray(params["b1"], np.float32))
    d2 = _make_dense(api, np.asarray(params["w2"], np.float32), np.asarray(params["b2"], np.float32))
    opt = api.boat_adam_optimizer_create(lr, beta1, beta2, eps)
    api.boat_hip_optimizer_add_layernorm(opt, ln[0])
    api.boat_hip_optimizer_add_attention(opt, att)
    api.boat_hip_optimizer_add_layernorm(opt, ln[1])
    api.boat_hip_optimizer_add_dense(opt, d1)
    api.boat_hip_optimizer_add_dense(opt, d2)

    def tensors():
        out = {"ln1_g": (api.boat_hip_layernorm_get_weight(ln[0]), api.boat_hip_layernorm_get_grad_weight(ln[0])),
               "ln1_b": (api.boat_hip_layernorm_get_bias(ln[0]), api.boat_hip_layernorm_get_grad_bias(ln[0])),
               "ln2_g": (api.boat_hip_layernorm_get_weight(ln[1]), api.boat_hip_layernorm_get_grad_weight(ln[1])),
               "ln2_b": (api.boat_hip_layernorm_get_bias(ln[1]), api.boat_hip_layernorm_get_grad_bias(ln[1])),
               "w1": (api.boat_dense_layer_get_weight(d1), api.boat_dense_layer_get_grad_weight(d1)),
               "b1": (api.boat_dense_layer_get_bias(d1), api.boat_dense_layer_get_grad_bias(d1)),
               "w2": (api.boat_dense_layer_get_weight(d2), api.boat_dense_layer_get_grad_weight(d2)),
               "b2": (api.boat_dense_layer_get_bias(d2), api.boat_dense_layer_get_grad_bias(d2))}
        for n in "qkvo":
            out["w" + n] = (getattr(api, f"boat_attention_get_weight_{n}")(att), getattr(api, f"boat_attention_get_grad_weight_{n}")(att))
            out["b" + n] = (getattr(api, f"boat_attention_get_bias_{n}")(att), getattr(api, f"boat_attention_get_grad_bias_{n}")(att))
        return out

    tt = api.tensor(np.asarray(target, np.float32))
    shape2 = (C.c_int64 * 2)(B * S, H)
    shape3 = (C.c_int64 * 3)(B, S, H)
    history = []
    for _ in range(steps):
        vx = _var(api, x, True)
        h1 = api.boat_hip_var_layernorm(vx, ln[0])
        a = api.boat_var_attention(h1, h1, h1, att, None)
        x1 = api.boat_var_add(vx, a)
        h2 = api.boat_hip_var_layernorm(x1, ln[1])
        h2f = api.boat_hip_var_reshape(h2, shape2, 2)
        f1 = api.boat_var_dense(h2f, d1)
        g1 = api.boat_hip_var_gelu(f1)
        f2 = api.boat_var_dense(g1, d2)
        f2r = api.boat_hip_var_reshape(f2, shape3, 3)
        y = api.boat_var_add(x1, f2r)
        grad = C.c_void_p()
        tloss = api.boat_hip_mse_loss(api.boat_variable_data(y), tt, C.byref(grad))
        rec = {"loss": float(api.numpy(tloss)[0]), "y": api.numpy(api.boat_variable_data(y))}
        api.boat_variable_backward(y, grad)
        rec["dx"] = _grad(api, vx)
        for name, (p, g) in tensors().items():
            rec["g_" + name] = api.numpy(g)
        api.boat_optimizer_step(opt)
        api.boat_optimizer_zero_grad(opt)
        for name, (p, g) in tensors().items():
            rec["p_" + name] = api.numpy(p)
        history.append(rec)
        api.boat_tensor_unref(tloss)
        api.boat_tensor_unref(grad)
        for v in (y, f2r, f2, g1, f1, h2f, h2, x1, a, h1, vx):
            api.boat_variable_free(v)
    api.boat_optimizer_free(opt)
    api.boat_tensor_unref(tt)
    api.boat_dense_layer_free(d1)
    api.boat_dense_layer_free(d2)
    api.boat_attention_free(att)
    for norm in ln:
        api.boat_layernorm_free(norm)
    return history


def _make_conv(api, w, b, stride, pad):
    oc, ic, k, _ = w.shape
    layer = api.boat_conv_layer_create(ic, oc, k, stride, pad)
    api.write(api.boat_conv_layer_get_weight(layer), w)        # in place (set_weight would swap tensors)
    api.write(api.boat_conv_layer_get_bias(layer), b)
    return layer


def conv_layer(api, x, w, b, stride, pad, d_out_list):
    """boat_conv_layer_forward once, then boat_conv_layer_backward per dY (parameter grads are overwritten per call).
    Returns y and per call (dx, grad_weight, grad_bias)."""
    layer = _make_conv(api, np.asarray(w, np.float32), np.asarray(b, np.float32), stride, pad)
    tx = api.tensor(np.asarray(x, np.float32))
    ty = api.boat_conv_layer_forward(layer, tx)
    y = api.numpy(ty)
    out = []
    for dy in d_out_list:
        tdy = api.tensor(np.asarray(dy, np.float32))
        tdx = api.boat_conv_layer_backward(layer, tdy)
        assert tdx, "boat_conv_layer_backward failed"
        out.append((api.numpy(tdx), api.numpy(api.boat_conv_layer_get_grad_weight(layer)),
                    api.numpy(api.boat_conv_layer_get_grad_bias(layer))))
        api.boat_tensor_unref(tdx)
        api.boat_tensor_unref(tdy)
    api.boat_tensor_unref(ty)
    api.boat_tensor_unref(tx)
    api.boat_conv_layer_free(layer)
    return y, out


def pool_layer(api, x, pool, stride, pad, dy):
    """boat_pool_layer_forward / backward.  Returns y, dx."""
    layer = api.boat_pool_layer_create(pool, stride, pad)
    tx = api.tensor(np.asarray(x, np.float32))
    ty = api.boat_pool_layer_forward(layer, tx)
    y = api.numpy(ty)
    tdy = api.tensor(np.asarray(dy, np.float32))
    tdx = api.boat_pool_layer_backward(layer, tdy)
    assert tdx, "boat_pool_layer_backward failed"
    dx = api.numpy(tdx)
    for t in (tdx, tdy, ty, tx):
        api.boat_tensor_unref(t)
    api.boat_pool_layer_free(layer)
    return y, dx


def cnn_ce_grads(api, x, labels, p, pool=2):
    """The MNIST network of examples/mnist/mnist_autodiff.c:536-557 on the tape, one forward + backward:
    conv(3x3, pad 1) -> relu -> maxpool(2) -> conv -> relu -> maxpool -> flatten -> dense -> relu -> dense
    -> log_softmax -> mul(onehot) -> sum -> mul(-1/B); boat_variable_backward_full.
    p: dict cw1, cb1, cw2, cb2, w1, b1, w2, b2.  Returns dict(loss, logits, dx, g_<name>...)."""
    x = np.asarray(x, np.float32)
    B = x.shape[0]
    classes = p["w2"].shape[1]
    c1 = _make_conv(api, p["cw1"], p["cb1"], 1, 1)
    c2 = _make_conv(api, p["cw2"], p["cb2"], 1, 1)
    p1, p2 = api.boat_pool_layer_create(pool, pool, 0), api.boat_pool_layer_create(pool, pool, 0)
    d1 = _make_dense(api, p["w1"], p["b1"])
    d2 = _make_dense(api, p["w2"], p["b2"])
    onehot = np.zeros((B, classes), np.float32)
    onehot[np.arange(B), np.asarray(labels)] = 1.0
    vx = _var(api, x, True)
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
    voh = _var(api, onehot, False)
    m = api.boat_var_mul(voh, ls)
    s = api.boat_var_sum(m, None, 0, False)
    vf = _var(api, np.array([-1.0 / B], np.float32), False)
    loss = api.boat_var_mul(vf, s)
    rec = {"loss": float(api.numpy(api.boat_variable_data(loss))[0]), "logits": api.numpy(api.boat_variable_data(z))}
    with scratch_cwd():
        api.boat_variable_backward_full(loss)
    rec["dx"] = _grad(api, vx)
    rec["g_cw1"] = api.numpy(api.boat_conv_layer_get_grad_weight(c1))
    rec["g_cb1"] = api.numpy(api.boat_conv_layer_get_grad_bias(c1))
    rec["g_cw2"] = api.numpy(api.boat_conv_layer_get_grad_weight(c2))
    rec["g_cb2"] = api.numpy(api.boat_conv_layer_get_grad_bias(c2))
    for name, layer in (("1", d1), ("2", d2)):
        rec["g_w" + name] = api.numpy(api.boat_dense_layer_get_grad_weight(layer))
        rec["g_b" + name] = api.numpy(api.boat_dense_layer_get_grad_bias(layer))
    if api.is_amd:   # the reference cannot release a recorded tape
        for v in (loss, vf, s, m, voh, ls, z, rh, h, fl, q2, r2, a2, q1, r1, a1, vx):
            api.boat_variable_free(v)
        api.boat_conv_layer_free(c1)
        api.boat_conv_layer_free(c2)
        api.boat_pool_layer_free(p1)
        api.boat_pool_layer_free(p2)
        api.boat_dense_layer_free(d1)
        api.boat_dense_layer_free(d2)
    return rec


def scheduler_trajectory(api, kind, base_lr, steps, **kw):
    """Learning rates of a scheduler over `steps` calls of boat_scheduler_step: per step (next_lr before the call,
    last_lr after it), then the pair after boat_scheduler_reset.  kind: "step" (step_size, gamma), "cosine" (T_max,
    eta_min) or "lambda" (fn(step, base_lr) -> float)."""
    from boat_amd.capi import LAMBDA_LR_FN
    keep = None
    if kind == "step":
        s = api.boat_step_lr_scheduler_create(base_lr, kw["step_size"], kw["gamma"])
    elif kind == "cosine":
        s = api.boat_cosine_annealing_scheduler_create(base_lr, kw["T_max"], kw["eta_min"])
    else:
        keep = LAMBDA_LR_FN(kw["fn"])
        s = api.boat_lambda_lr_scheduler_create(base_lr, keep)
    if not s:
        return None
    out = [(np.float32(api.boat_scheduler_get_next_lr(s)), np.float32(api.boat_scheduler_get_last_lr(s)))]
    for _ in range(steps):
        nxt = api.boat_scheduler_get_next_lr(s)
        api.boat_scheduler_step(s)
        out.append((np.float32(nxt), np.float32(api.boat_scheduler_get_last_lr(s))))
    api.boat_scheduler_reset(s)
    out.append((np.float32(api.boat_scheduler_get_next_lr(s)), np.float32(api.boat_scheduler_get_last_lr(s))))
    api.boat_scheduler_free(s)
    return np.array(out, np.float32)


def loss_values(api, kind, pred, target, delta=1.0):
    """boat_loss_compute of a fresh loss object, called twice (the object keeps running totals; the value must not
    depend on them).  kind: "mse", "ce" or "huber".  Returns the two values, or None when creation is refused."""
    if kind == "mse":
        loss = api.boat_mse_loss_create()
    elif kind == "ce":
        loss = api.boat_cross_entropy_loss_create()
    else:
        loss = api.boat_huber_loss_create(delta)
    if not loss:
        return None
    tp, tt = api.tensor(np.asarray(pred, np.float32)), api.tensor(np.asarray(target, np.float32))
    vals = (api.boat_loss_compute(loss, tp, tt), api.boat_loss_compute(loss, tp, tt))
    api.boat_tensor_unref(tp)
    api.boat_tensor_unref(tt)
    api.boat_loss_free(loss)
    return vals


# ---- the example's weight checkpoint (examples/mnist/mnist_autodiff.c:775-995) over the C API ----
CKPT_MAGIC, CKPT_VERSION = 0x4D4E4953, 1


def _ckpt_write_tensor(api, f, t):
    """save_tensor_to_file, mnist_autodiff.c:775-811: u32 null marker, u32 ndim, u32 dims, u32 dtype, raw payload."""
    import struct
    if not t:
        f.write(struct.pack("<I", 1))
        return
    ndim = api.boat_tensor_ndim(t)
    shape = api.boat_tensor_shape(t)
    f.write(struct.pack("<II", 0, ndim))
    f.write(struct.pack("<%dI" % ndim, *[shape[i] for i in range(ndim)]))
    f.write(struct.pack("<I", api.boat_tensor_dtype(t)))
    f.write(C.string_at(api.boat_tensor_const_data(t), api.boat_tensor_nbytes(t)))


def _ckpt_read_tensor(api, f):
    """load_tensor_from_file, mnist_autodiff.c:814-882: the payload goes through boat_tensor_from_data."""
    import struct
    (is_null,) = struct.unpack("<I", f.read(4))
    if is_null:
        return None
    (ndim,) = struct.unpack("<I", f.read(4))
    dims = struct.unpack("<%dI" % ndim, f.read(4 * ndim))
    (dtype,) = struct.unpack("<I", f.read(4))
    nbytes = int(np.prod(dims, dtype=np.int64)) * api.boat_dtype_size(dtype)
    payload = f.read(nbytes)
    assert len(payload) == nbytes
    shape = (C.c_int64 * ndim)(*dims)
    buf = C.create_string_buffer(payload, nbytes)
    return api.boat_tensor_from_data(shape, ndim, dtype, C.cast(buf, C.c_void_p))


class CnnLayers:
    """conv1, pool, conv2, pool, flatten, fc1, fc2 of the MNIST example (mnist_autodiff.c:536-557), as layer objects."""

    def __init__(self, api, p, pool=2):
        self.api = api
        self.c1 = _make_conv(api, p["cw1"], p["cb1"], 1, 1)
        self.c2 = _make_conv(api, p["cw2"], p["cb2"], 1, 1)
        self.p1, self.p2 = api.boat_pool_layer_create(pool, pool, 0), api.boat_pool_layer_create(pool, pool, 0)
        self.fl = api.boat_flatten_layer_create()
        self.d1 = _make_dense(api, p["w1"], p["b1"])
        self.d2 = _make_dense(api, p["w2"], p["b2"])

    def parameters(self):
        a = self.api
        return [(self.c1, "conv", a.boat_conv_layer_get_weight(self.c1), a.boat_conv_layer_get_bias(self.c1)),
                (self.c2, "conv", a.boat_conv_layer_get_weight(self.c2), a.boat_conv_layer_get_bias(self.c2)),
                (self.d1, "dense", a.boat_dense_layer_get_weight(self.d1), a.boat_dense_layer_get_bias(self.d1)),
                (self.d2, "dense", a.boat_dense_layer_get_weight(self.d2), a.boat_dense_layer_get_bias(self.d2))]

    def logits(self, x):
        """Forward through the layer hooks (the chain of mnist_autodiff.c:2345-2412 without the tape)."""
        a = self.api
        t = [a.tensor(np.asarray(x, np.float32))]
        for step in (lambda v: a.boat_conv_layer_forward(self.c1, v), a.boat_relu,
                     lambda v: a.boat_pool_layer_forward(self.p1, v),
                     lambda v: a.boat_conv_layer_forward(self.c2, v), a.boat_relu,
                     lambda v: a.boat_pool_layer_forward(self.p2, v),
                     lambda v: a.boat_flatten_layer_forward(self.fl, v),
                     lambda v: a.boat_dense_layer_forward(self.d1, v), a.boat_relu,
                     lambda v: a.boat_dense_layer_forward(self.d2, v)):
            nxt = step(t[-1])
            assert nxt, "a layer's forward failed"
            t.append(nxt)
        out = a.numpy(t[-1])
        for h in t:
            a.boat_tensor_unref(h)
        return out

    def save(self, path):
        """save_mnist_model, mnist_autodiff.c:885-927."""
        import struct
        with open(path, "wb") as f:
            f.write(struct.pack("<II", CKPT_MAGIC, CKPT_VERSION))
            for _layer, _kind, w, b in self.parameters():
                _ckpt_write_tensor(self.api, f, w)
                _ckpt_write_tensor(self.api, f, b)

    def load(self, path):
        """load_mnist_model, mnist_autodiff.c:930-995: set_weight / set_bias swap the layer's tensors for the loaded ones."""
        import struct
        a = self.api
        with open(path, "rb") as f:
            magic, version = struct.unpack("<II", f.read(8))
            if magic != CKPT_MAGIC or version != CKPT_VERSION:
                return False
            for layer, kind, _w, _b in self.parameters():
                set_w = a.boat_conv_layer_set_weight if kind == "conv" else a.boat_dense_layer_set_weight
                set_b = a.boat_conv_layer_set_bias if kind == "conv" else a.boat_dense_layer_set_bias
                w, b = _ckpt_read_tensor(a, f), _ckpt_read_tensor(a, f)
                if w:
                    set_w(layer, w)
                    a.boat_tensor_unref(w)
                if b:
                    set_b(layer, b)
                    a.boat_tensor_unref(b)
        return True

    def free(self):
        a = self.api
        a.boat_conv_layer_free(self.c1)
        a.boat_conv_layer_free(self.c2)
        a.boat_pool_layer_free(self.p1)
        a.boat_pool_layer_free(self.p2)
        a.boat_flatten_layer_free(self.fl)
        a.boat_dense_layer_free(self.d1)
        a.boat_dense_layer_free(self.d2)


def checkpoint_bytes(p):
    """The checkpoint file of parameters p built without any library: what save_mnist_model must write."""
    import struct
    out = [struct.pack("<II", CKPT_MAGIC, CKPT_VERSION)]
    for name in ("cw1", "cb1", "cw2", "cb2", "w1", "b1", "w2", "b2"):
        arr = np.ascontiguousarray(p[name], np.float32)
        out.append(struct.pack("<II", 0, arr.ndim) + struct.pack("<%dI" % arr.ndim, *arr.shape) + struct.pack("<I", 1))
        out.append(arr.tobytes())
    return b"".join(out)


# ---- the rest of the API on the path: tensor-level ops, variable helpers, contexts, error reporting ----
def tensor_ops(api, a, b, row, col, v1, v2):
    """Tensor-level arithmetic and activations (src/ops/arithmetic.c:157-484, src/ops/linear.c:173-236,
    src/ops/activation.c): a, b same shape [m, n]; row [n], col [m, 1] broadcast against a; v1, v2 vectors."""
    out = {}
    ta, tb, trow, tcol = (api.tensor(np.asarray(t, np.float32)) for t in (a, b, row, col))
    t1, t2 = api.tensor(np.asarray(v1, np.float32)), api.tensor(np.asarray(v2, np.float32))

    def take(name, t):
        out[name] = None if not t else api.numpy(t)
        if t:
            api.boat_tensor_unref(t)

    for name in ("add", "sub", "mul", "div"):
        fn = getattr(api, "boat_" + name)
        take(name, fn(ta, tb))
        take(name + "_row", fn(ta, trow))
        take(name + "_col", fn(tcol, ta))
        take(name + "_scalar", getattr(api, f"boat_{name}_scalar")(ta, 1.75))
    for name in ("add_", "sub_", "mul_", "div_"):
        work = api.tensor(np.asarray(a, np.float32))
        getattr(api, "boat_" + name)(work, tb)
        out[name] = api.numpy(work)
        getattr(api, "boat_" + name)(work, t1)                 # element counts differ: left as it is
        out[name + "_mismatch_unchanged"] = bool(np.array_equal(api.numpy(work), out[name]))
        api.boat_tensor_unref(work)
    take("dot", api.boat_dot(t1, t2))
    out["dot_of_matrices_is_null"] = not api.boat_dot(ta, tb)
    for name in ("relu", "sigmoid", "tanh"):
        take(name, getattr(api, "boat_" + name)(ta))
    take("softmax", api.boat_softmax(ta, -1))
    take("log_softmax", api.boat_log_softmax(ta, -1))
    # arithmetic.c:575-608: the shape rule, and boat_broadcast_to (a dense copy under a new shape of equal element count)
    m, n = np.asarray(a).shape
    tm = api.tensor(np.zeros(m, np.float32))            # [m] against [m, n]: the last dimensions differ
    out["can_broadcast"] = [bool(api.boat_can_broadcast(ta, trow)), bool(api.boat_can_broadcast(tcol, ta)), bool(api.boat_can_broadcast(ta, tm))]
    api.boat_tensor_unref(tm)
    take("broadcast_to_same_count", api.boat_broadcast_to(ta, (C.c_int64 * 3)(1, n, m), 3))
    out["broadcast_to_other_count_is_null"] = not api.boat_broadcast_to(trow, (C.c_int64 * 2)(m, n), 2)
    out["is_contiguous"] = bool(api.boat_tensor_is_contiguous(ta))
    out["dtype_names"] = [api.boat_dtype_name(d).decode() for d in (0, 1, 5, 6, 10, 77)]
    out["dtype_sizes"] = [int(api.boat_dtype_size(d)) for d in (0, 1, 5, 6)]
    for t in (ta, tb, trow, tcol, t1, t2):
        api.boat_tensor_unref(t)
    return out


def variable_helpers(api):
    """boat_variable_create_with_shape / set_requires_grad / reset_data / retain_grad (src/autodiff.c:208-298)."""
    out = {}
    shape = (C.c_int64 * 2)(2, 3)
    v = api.boat_variable_create_with_shape(shape, 2, 1, False)
    out["with_shape_data"] = api.numpy(api.boat_variable_data(v))
    out["requires_grad_before"] = bool(api.boat_variable_requires_grad(v))
    api.boat_variable_set_requires_grad(v, True)
    out["requires_grad_after"] = bool(api.boat_variable_requires_grad(v))
    api.boat_variable_retain_grad(v, True)                                    # accepted, no observable effect
    api.boat_variable_backward_full(v)
    out["grad_after_backward"] = api.numpy(api.boat_variable_grad(v))
    fresh = api.tensor(np.arange(6, dtype=np.float32).reshape(2, 3))
    out["reset_leaf"] = bool(api.boat_variable_reset_data(v, fresh))
    out["data_after_reset"] = api.numpy(api.boat_variable_data(v))
    out["grad_dropped_by_reset"] = not api.boat_variable_grad(v)
    out["reset_null"] = bool(api.boat_variable_reset_data(v, None))
    api.boat_tensor_unref(fresh)
    out["data_survives_callers_unref"] = api.numpy(api.boat_variable_data(v))  # the variable holds its own reference
    if api.is_amd:
        api.boat_variable_free(v)
    return out


def context_and_errors(api):
    """Context objects (src/autodiff.c:606-649) and the error state (src/core/error.c:21-62)."""
    out = {}
    ctx = api.boat_autodiff_context_create()
    out["enabled_at_creation"] = bool(api.boat_autodiff_context_grad_enabled(ctx))
    api.boat_autodiff_context_disable_grad(ctx)
    out["enabled_after_disable"] = bool(api.boat_autodiff_context_grad_enabled(ctx))
    api.boat_autodiff_context_enable_grad(ctx)
    out["enabled_after_enable"] = bool(api.boat_autodiff_context_grad_enabled(ctx))
    out["enabled_of_null"] = bool(api.boat_autodiff_context_grad_enabled(None))
    before = api.boat_autodiff_get_current_context()
    api.boat_autodiff_set_current_context(ctx)
    out["current_is_the_one_set"] = api.boat_autodiff_get_current_context() == ctx
    api.boat_autodiff_set_current_context(before)
    api.boat_autodiff_context_free(ctx)
    api.boat_clear_error()
    out["error_after_clear"] = (int(api.boat_get_last_error()), api.boat_get_last_error_message().decode(), bool(api.boat_has_error()))
    api.boat_set_error(3, b"the operation is not valid here")
    out["error_after_set"] = (int(api.boat_get_last_error()), api.boat_get_last_error_message().decode(), bool(api.boat_has_error()))
    api.boat_set_error(5, b"x" * 400)                                          # longer than the 256-byte message buffer
    out["long_message_length"] = len(api.boat_get_last_error_message())
    api.boat_set_error(2, None)
    out["error_with_null_message"] = (int(api.boat_get_last_error()), api.boat_get_last_error_message().decode())
    api.boat_clear_error()
    out["error_strings"] = [api.boat_error_string(e).decode() for e in range(0, 10)] + [api.boat_error_string(-1).decode()]
    # host memory helpers
    p = api.boat_memory_allocate(64, 0, b"boat_cases.py", 1)
    api.boat_memory_set(p, 0x5A, 64, 0)
    q = api.boat_memory_allocate(64, 0, b"boat_cases.py", 2)
    api.boat_memory_copy(q, p, 64, 0, 0)
    out["memory_set_then_copy"] = C.string_at(q, 64) == b"\x5a" * 64
    api.boat_memory_free(p)
    api.boat_memory_free(q)
    return out


def sgd_hooks(api, x, w, b, dy, lr):
    """boat_dense_layer_update (src/layers/dense.c:297-329): p -= lr * g, gradients cleared; then a second backward
    accumulates from zero.  Returns ((gw, gb) of the first backward, w1, b1, gw_after_update, w2)."""
    layer = _make_dense(api, w, b)
    tx, tdy = api.tensor(np.asarray(x, np.float32)), api.tensor(np.asarray(dy, np.float32))
    ty = api.boat_dense_layer_forward(layer, tx)
    tdx = api.boat_dense_layer_backward(layer, tdy)
    g0 = api.numpy(api.boat_dense_layer_get_grad_weight(layer)), api.numpy(api.boat_dense_layer_get_grad_bias(layer))
    api.boat_dense_layer_update(layer, lr)
    w1, b1 = api.numpy(api.boat_dense_layer_get_weight(layer)), api.numpy(api.boat_dense_layer_get_bias(layer))
    gw = api.numpy(api.boat_dense_layer_get_grad_weight(layer))
    api.boat_tensor_unref(tdx)
    tdx = api.boat_dense_layer_backward(layer, tdy)
    api.boat_dense_layer_update(layer, lr)
    w2 = api.numpy(api.boat_dense_layer_get_weight(layer))
    for t in (tdx, ty, tdy, tx):
        api.boat_tensor_unref(t)
    api.boat_dense_layer_free(layer)
    return g0, w1, b1, gw, w2


def conv_sgd_hook(api, x, w, b, dy, lr):
    """boat_conv_layer_update (src/layers/conv.c:539-562): p -= lr * g through boat_mul_scalar + boat_sub_, gradients kept."""
    layer = _make_conv(api, np.asarray(w, np.float32), np.asarray(b, np.float32), 1, 1)
    tx, tdy = api.tensor(np.asarray(x, np.float32)), api.tensor(np.asarray(dy, np.float32))
    ty = api.boat_conv_layer_forward(layer, tx)
    tdx = api.boat_conv_layer_backward(layer, tdy)
    gw, gb = api.numpy(api.boat_conv_layer_get_grad_weight(layer)), api.numpy(api.boat_conv_layer_get_grad_bias(layer))
    api.boat_conv_layer_update(layer, lr)
    w1, b1 = api.numpy(api.boat_conv_layer_get_weight(layer)), api.numpy(api.boat_conv_layer_get_bias(layer))
    gw_after = api.numpy(api.boat_conv_layer_get_grad_weight(layer))
    for t in (tdx, ty, tdy, tx):
        api.boat_tensor_unref(t)
    api.boat_conv_layer_free(layer)
    return w1, b1, gw, gb, gw_after


def tensor_facts(api):
    """Observable facts of tensor creation, views and argument checks (src/core/tensor.c:65-300,
    src/ops/arithmetic.c:136-156, src/ops/linear.c:12-60,238-262)."""
    out = {}

    def shp(*dims):
        return (C.c_int64 * max(len(dims), 1))(*dims)

    def facts(t):
        if not t:
            return None
        f = (int(api.boat_tensor_ndim(t)), int(api.boat_tensor_nelements(t)), int(api.boat_tensor_nbytes(t)),
             int(api.boat_tensor_dtype(t)), int(api.boat_tensor_device(t)), bool(api.boat_tensor_is_contiguous(t)))
        return f

    def take(name, t):
        out[name] = facts(t)
        if t:
            api.boat_tensor_unref(t)

    if api.is_amd:   # the reference aborts here: zero bytes fail to allocate and the clean-up frees the wrong pointers (tensor.c:118-124)
        take("scalar_null_shape", api.boat_tensor_create(None, 0, 1, 0))
    take("null_shape_with_dims", api.boat_tensor_create(None, 2, 1, 0))
    take("f32_2x3", api.boat_tensor_create(shp(2, 3), 2, 1, 0))
    take("f64_2x3", api.boat_tensor_create(shp(2, 3), 2, 0, 0))
    take("i32_5", api.boat_tensor_create(shp(5), 1, 6, 0))
    take("i64_5", api.boat_tensor_create(shp(5), 1, 5, 0))
    take("f4_5", api.boat_tensor_create(shp(5), 1, 4, 0))
    take("bits1_9", api.boat_tensor_create(shp(9), 1, 9, 0))
    take("eight_dims", api.boat_tensor_create(shp(1, 2, 1, 2, 1, 2, 1, 2), 8, 1, 0))
    base = api.tensor(np.arange(12, dtype=np.float32).reshape(3, 4))
    view = api.boat_tensor_reshape(base, shp(2, 6), 2)
    out["view"] = facts(view)
    out["view_shape"] = api.shape(view)
    out["view_shares_data"] = api.boat_tensor_data(view) == api.boat_tensor_data(base)
    api.boat_tensor_unref(base)                                  # the view keeps its parent alive
    out["view_after_parent_unref"] = api.numpy(view).tolist()
    api.boat_tensor_unref(view)
    base = api.tensor(np.arange(12, dtype=np.float32).reshape(3, 4))
    out["reshape_wrong_count"] = facts(api.boat_tensor_reshape(base, shp(5, 2), 2))
    out["reshape_null_shape"] = facts(api.boat_tensor_reshape(base, None, 2))
    like = api.boat_tensor_create_like(base)
    out["like"] = facts(like)
    out["like_is_zero"] = not api.numpy(like).any()
    api.boat_tensor_unref(like)
    f64 = api.tensor(np.ones((3, 4), np.float64))
    vec3, vec4 = api.tensor(np.ones(3, np.float32)), api.tensor(np.ones(4, np.float32))
    take("add_mixed_dtypes", api.boat_add(base, f64))
    take("add_3x4_and_3", api.boat_add(base, vec3))
    take("add_3x4_and_4", api.boat_add(base, vec4))
    take("matmul_inner_mismatch", api.boat_matmul(base, base))
    take("matmul_3x4_4", api.boat_matmul(base, vec4))
    take("transpose_bad_dim", api.boat_transpose(base, 0, 2))
    take("transpose_same_dim", api.boat_transpose(base, 1, 1))
    take("transpose_negative", api.boat_transpose(base, -1, -2))
    take("sum_all", api.boat_sum(base, None, 0, False))
    take("softmax_vector", api.boat_softmax(vec4, -1))
    take("relu_f64", api.boat_relu(f64))
    take("mul_scalar_f64", api.boat_mul_scalar(f64, 2.0))
    for t in (base, f64, vec3, vec4):
        api.boat_tensor_unref(t)
    return out


def layer_facts(api, only=None):
    """Argument checks and object life cycle of layers, optimizers and the model container: a dict of small facts
    (shapes, NULL or not, scalars).  `only` limits the probes to the named groups."""
    from boat_amd.capi import AttentionConfig, LayerNormConfig
    out = {}
    rng = np.random.default_rng(9)

    def T(*shape):
        return api.tensor(rng.standard_normal(shape).astype(np.float32))

    def shape_of(t, free=True):
        if not t:
            return None
        s = api.shape(t)
        if free:
            api.boat_tensor_unref(t)
        return s

    def group(name):
        return only is None or name in only

    if group("matmul"):
        a2, b2, a3, b3, a4, b4, b3x, v = T(3, 4), T(4, 5), T(2, 3, 4), T(2, 4, 5), T(2, 2, 3, 4), T(2, 2, 4, 5), T(3, 4, 5), T(4)
        out["matmul_2d"] = shape_of(api.boat_matmul(a2, b2))
        out["matmul_3d"] = shape_of(api.boat_matmul(a3, b3))
        out["matmul_4d"] = shape_of(api.boat_matmul(a4, b4))
        out["matmul_batch_mismatch"] = shape_of(api.boat_matmul(a3, b3x))
        out["matmul_3d_with_2d"] = shape_of(api.boat_matmul(a3, b2))
        out["matmul_with_vector"] = shape_of(api.boat_matmul(a2, v))
        t3 = api.boat_matmul(a3, b3)
        out["matmul_3d_value_ok"] = bool(np.allclose(api.numpy(t3), api.numpy(a3) @ api.numpy(b3), rtol=1e-5, atol=1e-5))
        api.boat_tensor_unref(t3)
        for t in (a2, b2, a3, b3, a4, b4, b3x, v):
            api.boat_tensor_unref(t)

    if group("dense"):
        nb = api.boat_dense_layer_create(4, 3, False)
        out["dense_no_bias_has_bias"] = bool(api.boat_dense_layer_get_bias(nb))
        out["dense_no_bias_has_grad_bias"] = bool(api.boat_dense_layer_get_grad_bias(nb))
        out["dense_weight_shape"] = shape_of(api.boat_dense_layer_get_weight(nb), free=False)
        out["dense_grad_weight_zero_at_creation"] = not api.numpy(api.boat_dense_layer_get_grad_weight(nb)).any()
        x2, x3, xbad, dy = T(2, 4), T(2, 5, 4), T(2, 3), T(2, 3)
        out["dense_forward_2d"] = shape_of(api.boat_dense_layer_forward(nb, x2))
        tdx = api.boat_dense_layer_backward(nb, dy)
        out["dense_backward_no_bias"] = shape_of(tdx)
        out["dense_forward_3d"] = shape_of(api.boat_dense_layer_forward(nb, x3))
        out["dense_forward_wrong_features"] = shape_of(api.boat_dense_layer_forward(nb, xbad))
        api.boat_dense_layer_set_bias(nb, dy)                      # refused: the layer has no bias
        out["dense_set_bias_on_no_bias_layer"] = bool(api.boat_dense_layer_get_bias(nb))
        wbad = T(3, 4)
        api.boat_dense_layer_set_weight(nb, wbad)                  # refused: wrong shape
        out["dense_set_weight_wrong_shape_kept"] = shape_of(api.boat_dense_layer_get_weight(nb), free=False)
        for t in (x2, x3, xbad, dy, wbad):
            api.boat_tensor_unref(t)
        api.boat_dense_layer_free(nb)

    if group("optimizer"):
        p, g = T(3, 2), T(3, 2)
        before = api.numpy(p)
        for kind, make, bad in (
                ("adam", lambda: api.boat_adam_optimizer_create(0.1, 0.9, 0.999, 1e-8),
                 [lambda: api.boat_adam_optimizer_create(-1.0, 0.9, 0.999, 1e-8), lambda: api.boat_adam_optimizer_create(0.1, 0.9, 1.5, 1e-8),
                  lambda: api.boat_adam_optimizer_create(0.1, 0.9, 0.999, 0.0), lambda: api.boat_adam_optimizer_create(0.1, 0.9, 0.999, -1.0)]),
                ("rmsprop", lambda: api.boat_rmsprop_optimizer_create(0.1, 0.99, 1e-8),
                 [lambda: api.boat_rmsprop_optimizer_create(0.0, 0.99, 1e-8), lambda: api.boat_rmsprop_optimizer_create(0.1, 1.0, 1e-8),
                  lambda: api.boat_rmsprop_optimizer_create(0.1, 0.99, 0.0)]),
                ("adagrad", lambda: api.boat_adagrad_optimizer_create(0.1, 1e-8),
                 [lambda: api.boat_adagrad_optimizer_create(0.0, 1e-8), lambda: api.boat_adagrad_optimizer_create(0.1, 0.0)])):
            out[kind + "_bad_arguments_refused"] = [not f() for f in bad]
            opt = make()
            out[kind + "_lr"] = round(float(api.boat_optimizer_get_learning_rate(opt)), 6)
            api.boat_optimizer_set_learning_rate(opt, 0.25)
            out[kind + "_lr_after_set"] = round(float(api.boat_optimizer_get_learning_rate(opt)), 6)
            api.boat_optimizer_step(opt)                            # no parameters: nothing to do
            api.boat_optimizer_add_parameter(opt, p, None)          # refused without a gradient tensor
            api.boat_optimizer_step(opt)
            out[kind + "_null_grad_ignored"] = bool(np.array_equal(api.numpy(p), before))
            api.boat_optimizer_add_parameter(opt, p, g)
            api.boat_optimizer_zero_grad(opt)
            out[kind + "_zero_grad_clears"] = not api.numpy(g).any()
            api.boat_optimizer_step(opt)                            # zero gradient: parameters stay
            out[kind + "_zero_grad_step_keeps_params"] = bool(np.array_equal(api.numpy(p), before))
            api.boat_optimizer_free(opt)
            api.write(g, rng.standard_normal((3, 2)).astype(np.float32))
        api.boat_tensor_unref(p)
        api.boat_tensor_unref(g)

    if group("attention"):
        def cfg(hidden, heads, bias=True):
            return AttentionConfig(hidden, heads, 0, 0.0, False, bias, False, 10000.0)
        out["attention_heads_do_not_divide"] = not api.boat_attention_create(C.byref(cfg(10, 3)))
        out["attention_zero_heads"] = not api.boat_attention_create(C.byref(cfg(8, 0)))
        out["attention_null_config"] = not api.boat_attention_create(None)
        att = api.boat_attention_create(C.byref(cfg(8, 2, bias=False)))
        out["attention_no_bias_has_bias_q"] = bool(api.boat_attention_get_bias_q(att))
        out["attention_weight_shape"] = shape_of(api.boat_attention_get_weight_q(att), free=False)
        out["attention_grad_before_backward"] = bool(api.boat_attention_get_grad_weight_q(att))
        x = T(2, 3, 8)
        ty = api.boat_attention_forward(att, x, x, x, None)
        out["attention_forward"] = shape_of(ty)
        api.boat_tensor_unref(x)
        api.boat_attention_free(att)

    if group("layernorm"):
        plain = api.boat_layernorm_create(C.byref(LayerNormConfig(6, 1e-5, False, False)))
        x, xbad = T(4, 6), T(4, 5)
        out["layernorm_plain_forward"] = shape_of(api.boat_layernorm_forward(plain, x))
        out["layernorm_wrong_width"] = shape_of(api.boat_layernorm_forward(plain, xbad))
        out["layernorm_zero_width"] = not api.boat_layernorm_create(C.byref(LayerNormConfig(0, 1e-5, True, True)))
        api.boat_tensor_unref(x)
        api.boat_tensor_unref(xbad)
        api.boat_layernorm_free(plain)

    if group("conv"):
        conv = api.boat_conv_layer_create(2, 3, 3, 1, 1)
        x, xbad, x3 = T(2, 2, 5, 5), T(2, 4, 5, 5), T(2, 5, 5)
        out["conv_forward"] = shape_of(api.boat_conv_layer_forward(conv, x))
        out["conv_wrong_channels"] = shape_of(api.boat_conv_layer_forward(conv, xbad))
        out["conv_3d_input"] = shape_of(api.boat_conv_layer_forward(conv, x3))
        out["conv_weight_shape"] = shape_of(api.boat_conv_layer_get_weight(conv), free=False)
        out["conv_bias_shape"] = shape_of(api.boat_conv_layer_get_bias(conv), free=False)
        pool = api.boat_pool_layer_create(2, 2, 0)
        out["pool_forward"] = shape_of(api.boat_pool_layer_forward(pool, x))
        out["pool_3d_input"] = shape_of(api.boat_pool_layer_forward(pool, x3))
        flat = api.boat_flatten_layer_create()
        out["flatten_forward"] = shape_of(api.boat_flatten_layer_forward(flat, x))
        for t in (x, xbad, x3):
            api.boat_tensor_unref(t)
        api.boat_conv_layer_free(conv)
        api.boat_pool_layer_free(pool)
        api.boat_flatten_layer_free(flat)
    return out


def autodiff_facts(api):
    """How the tape propagates requires_grad and shapes (src/autodiff.c:138-206,2070-2347,2155,2221,2287,530-548)."""
    out = {}
    rng = np.random.default_rng(10)

    def V(shape, rg):
        return _var(api, rng.standard_normal(shape).astype(np.float32), rg)

    def rg(v):
        return None if not v else bool(api.boat_variable_requires_grad(v))

    def shape_of(v):
        return None if not v else api.shape(api.boat_variable_data(v))

    a, b, c, d = V((3, 4), False), V((3, 4), True), V((3, 4), False), V((4, 2), True)
    out["add_false_true"] = rg(api.boat_var_add(a, b))
    out["add_false_false"] = rg(api.boat_var_add(a, c))
    out["mul_true_false"] = rg(api.boat_var_mul(b, a))
    out["matmul_false_true"] = rg(api.boat_var_matmul(a, d))
    out["relu_false"] = rg(api.boat_var_relu(a))
    out["relu_true"] = rg(api.boat_var_relu(b))
    out["add_shape_mismatch"] = shape_of(api.boat_var_add(a, d))
    out["matmul_shape"] = shape_of(api.boat_var_matmul(a, d))
    out["matmul_inner_mismatch"] = shape_of(api.boat_var_matmul(a, b))
    out["sum_all_shape"] = shape_of(api.boat_var_sum(b, None, 0, False))
    x = rng.standard_normal((3, 4)).astype(np.float32)
    vx = _var(api, x, True)
    s_last, s_axis0 = api.boat_var_softmax(vx, -1), api.boat_var_softmax(vx, 0)
    out["softmax_axis_is_ignored"] = bool(np.array_equal(api.numpy(api.boat_variable_data(s_last)), api.numpy(api.boat_variable_data(s_axis0))))
    out["softmax_rows_sum_to_one"] = bool(np.allclose(api.numpy(api.boat_variable_data(s_axis0)).sum(1), 1, atol=1e-6))
    out["flatten_shape"] = shape_of(api.boat_var_flatten(_var(api, rng.standard_normal((2, 3, 4, 5)).astype(np.float32), True)))
    # a dense layer on the tape: the output needs a gradient only if the INPUT does, whatever the layer's parameters
    layer = _make_dense(api, rng.standard_normal((4, 2)).astype(np.float32), np.zeros(2, np.float32))
    y_off = api.boat_var_dense(a, layer)
    out["dense_of_input_without_grad"] = rg(y_off)
    with scratch_cwd():
        api.boat_variable_backward_full(y_off)                        # silently nothing
    out["dense_grads_untouched_without_input_grad"] = not api.numpy(api.boat_dense_layer_get_grad_weight(layer)).any()
    y_on = api.boat_var_dense(b, layer)
    out["dense_of_input_with_grad"] = rg(y_on)
    with scratch_cwd():
        api.boat_variable_backward_full(y_on)
    out["dense_grads_filled_with_input_grad"] = bool(api.numpy(api.boat_dense_layer_get_grad_weight(layer)).any())
    out["input_grad_shape"] = None if not api.boat_variable_grad(b) else api.shape(api.boat_variable_grad(b))
    return out


# ---- the model container with vtables written by the caller (tests/test_model_graph_integration.c:8-77) ----
_FWD = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.c_void_p)
_UPD = C.CFUNCTYPE(None, C.c_void_p, C.c_float)
_FREE = C.CFUNCTYPE(None, C.c_void_p)


class _LayerOps(C.Structure):      # include/boat/model.h:29-34
    _fields_ = [("forward", _FWD), ("backward", _FWD), ("update", _UPD), ("free", _FREE)]


class _Layer(C.Structure):         # include/boat/model.h:23-27
    _fields_ = [("data", C.c_void_p), ("ops", C.POINTER(_LayerOps))]


def model_over_callers_vtables(api, x, weights, biases, dy=None, lr=None):
    """A boat_model_t of dense layers, each behind a boat_layer_ops_t table the CALLER wrote (here: Python callbacks
    that forward to boat_dense_layer_*), as tests/test_model_graph_integration.c:8-41 does in C.  Returns
    dict(count, y, dx or None when boat_model_backward returns NULL, freed = how many free hooks ran, weights after
    boat_model_update when lr is given)."""
    dense = [_make_dense(api, w, b) for w, b in zip(weights, biases)]
    freed = []
    keep = []

    def data_of(layer_ptr):
        return C.cast(layer_ptr, C.POINTER(_Layer)).contents.data

    ops = _LayerOps(_FWD(lambda l, t: api.boat_dense_layer_forward(data_of(l), t)),
                    _FWD(lambda l, g: api.boat_dense_layer_backward(data_of(l), g)),
                    _UPD(lambda l, r: api.boat_dense_layer_update(data_of(l), r)),
                    _FREE(lambda l: freed.append(data_of(l))))
    model = api.boat_model_create()
    for d in dense:
        wrapper = _Layer(d, C.pointer(ops))
        keep.append(wrapper)
        api.boat_model_add_layer(model, C.addressof(wrapper))
    rec = {"count": int(api.boat_model_layer_count(model))}
    tx = api.tensor(np.asarray(x, np.float32))
    ty = api.boat_model_forward(model, tx)
    rec["y"] = None if not ty else api.numpy(ty)
    rec["dx"] = None
    if dy is not None:
        tdy = api.tensor(np.asarray(dy, np.float32))
        tdx = api.boat_model_backward(model, tdy)
        if tdx:
            rec["dx"] = api.numpy(tdx)
            api.boat_tensor_unref(tdx)
        rec["gw"] = [api.numpy(api.boat_dense_layer_get_grad_weight(d)) for d in dense]
        api.boat_tensor_unref(tdy)
    if lr is not None:
        api.boat_model_update(model, lr)
        rec["w_after"] = [api.numpy(api.boat_dense_layer_get_weight(d)) for d in dense]
    if ty:
        api.boat_tensor_unref(ty)
    api.boat_tensor_unref(tx)
    api.boat_model_free(model)
    rec["freed"] = len(freed)
    for d in dense:
        api.boat_dense_layer_free(d)
    return rec


def slice_facts(api):
    """boat_tensor_slice (src/core/tensor.c:302-456): views on ranges of the leading dimension, as the MNIST example
    batches its samples (examples/mnist/mnist_autodiff.c:2387-2392)."""
    out = {}

    def idx(*v):
        return (C.c_size_t * len(v))(*v)

    base_np = np.arange(24, dtype=np.float32).reshape(6, 4)
    base = api.tensor(base_np)
    rows = api.boat_tensor_slice(base, idx(2, 0), idx(5, 4), None)
    out["shape"] = api.shape(rows)
    out["values"] = api.numpy(rows).tolist()
    out["is_contiguous"] = bool(api.boat_tensor_is_contiguous(rows))
    out["pointer_offset"] = api.boat_tensor_data(rows) - api.boat_tensor_data(base)
    out["nbytes"] = int(api.boat_tensor_nbytes(rows))
    out["step_two_refused"] = not api.boat_tensor_slice(base, idx(0, 0), idx(6, 4), idx(2, 1))
    out["step_zero_refused"] = not api.boat_tensor_slice(base, idx(0, 0), idx(6, 4), idx(0, 1))
    out["start_past_end_refused"] = not api.boat_tensor_slice(base, idx(6, 0), idx(6, 4), None)
    out["reversed_range_refused"] = not api.boat_tensor_slice(base, idx(3, 0), idx(2, 4), None)
    out["empty_range_refused"] = not api.boat_tensor_slice(base, idx(3, 0), idx(3, 4), None)
    view = api.boat_tensor_reshape(base, (C.c_int64 * 2)(4, 6), 2)
    out["slice_of_a_view_refused"] = not api.boat_tensor_slice(view, idx(0, 0), idx(2, 6), None)
    api.boat_tensor_unref(view)
    # the slice is a window on its parent: an in-place operation on it changes those rows of the parent and no others
    ones = api.tensor(np.ones((3, 4), np.float32))
    api.boat_add_(rows, ones)
    out["parent_after_add_on_slice"] = api.numpy(base).tolist()
    # arithmetic on a slice that does not start on 16 bytes
    odd = api.tensor(np.arange(18, dtype=np.float32).reshape(6, 3))
    win = api.boat_tensor_slice(odd, idx(1, 0), idx(4, 3), None)
    w = api.tensor(np.array([[1, 0], [0, 1], [1, 1]], np.float32))
    prod = api.boat_matmul(win, w)
    out["matmul_on_slice"] = api.numpy(prod).tolist()
    api.boat_tensor_unref(base)                                    # the slice keeps its parent's payload alive
    out["values_after_parent_unref"] = api.numpy(rows).tolist()
    for t in (prod, w, win, odd, ones, rows):
        api.boat_tensor_unref(t)
    return out


def write_mnist_example_files(folder, train_images, train_labels, test_images, test_labels):
    """The four files examples/mnist/mnist.c reads from ./data (its loader, mnist.c:29-95: u32 ndim, u32 extents, raw
    payload; images as float32 [n, 28, 28], labels as bytes [n])."""
    import struct
    data = folder / "data"
    data.mkdir(parents=True, exist_ok=True)
    for name, arr in (("train_images_small.bin", np.asarray(train_images, np.float32)), ("train_labels_small.bin", np.asarray(train_labels, np.uint8)),
                      ("test_images_small.bin", np.asarray(test_images, np.float32)), ("test_labels_small.bin", np.asarray(test_labels, np.uint8))):
        with open(data / name, "wb") as f:
            f.write(struct.pack("<I", arr.ndim) + struct.pack("<%dI" % arr.ndim, *arr.shape) + arr.tobytes())


def host_allocator_facts(api):
    """Pool, arena and reallocate of the memory header (src/core/memory.c:85-120,283-520) and the model's chain view."""
    out = {}
    pool = api.boat_memory_pool_create(1024, 4)
    blocks = [api.boat_memory_pool_alloc(pool, n) for n in (512, 768, 1024)]
    out["pool_three_taken"] = (int(api.boat_memory_pool_allocated_blocks(pool)), int(api.boat_memory_pool_free_blocks(pool)))
    out["pool_total_memory"] = int(api.boat_memory_pool_total_memory(pool))
    out["pool_refuses_larger_than_a_block"] = not api.boat_memory_pool_alloc(pool, 1025)
    last = api.boat_memory_pool_alloc(pool, 1)
    out["pool_refuses_when_empty"] = bool(last) and not api.boat_memory_pool_alloc(pool, 1)
    api.boat_memory_pool_free_block(pool, blocks[1])
    api.boat_memory_pool_free_block(pool, blocks[1])            # a second time: ignored
    out["pool_after_one_back"] = (int(api.boat_memory_pool_allocated_blocks(pool)), int(api.boat_memory_pool_free_blocks(pool)))
    api.boat_memory_pool_clear(pool)
    out["pool_after_clear"] = (int(api.boat_memory_pool_allocated_blocks(pool)), int(api.boat_memory_pool_free_blocks(pool)))
    api.boat_memory_pool_free(pool)
    out["pool_of_nothing_refused"] = not api.boat_memory_pool_create(0, 4) and not api.boat_memory_pool_create(16, 0)
    arena = api.boat_memory_arena_create(4096)
    a = api.boat_memory_arena_alloc(arena, 10)
    b = api.boat_memory_arena_alloc(arena, 1)
    out["arena_rounds_to_eight"] = (b - a, int(api.boat_memory_arena_used(arena)))
    out["arena_refuses_zero"] = not api.boat_memory_arena_alloc(arena, 0)
    api.boat_memory_arena_alloc(arena, 9000)                    # does not fit: the capacity doubles until it does
    out["arena_grows"] = (int(api.boat_memory_arena_used(arena)), int(api.boat_memory_arena_capacity(arena)))
    api.boat_memory_arena_reset(arena)
    out["arena_after_reset"] = (int(api.boat_memory_arena_used(arena)), int(api.boat_memory_arena_capacity(arena)))
    api.boat_memory_arena_free(arena)
    p = api.boat_memory_allocate(16, 0, b"boat_cases.py", 1)
    C.memmove(p, b"0123456789abcdef", 16)
    q = api.boat_memory_reallocate(p, 64, 0, b"boat_cases.py", 2)
    out["reallocate_keeps_contents"] = C.string_at(q, 16)
    out["reallocate_to_zero_frees"] = not api.boat_memory_reallocate(q, 0, 0, b"boat_cases.py", 3)
    r = api.boat_memory_reallocate(None, 8, 0, b"boat_cases.py", 4)
    out["reallocate_of_null_allocates"] = bool(r)
    api.boat_memory_free(r)
    graph = api.boat_graph_create_with_device(0)
    ctx = api.boat_autodiff_context_create()
    api.boat_autodiff_context_set_graph(ctx, graph)
    out["context_carries_the_graph"] = api.boat_autodiff_context_get_graph(ctx) == graph
    out["fresh_graph_is_empty"] = (int(api.boat_graph_node_count(graph)), int(api.boat_graph_edge_count(graph)))
    api.boat_autodiff_context_free(ctx)
    api.boat_graph_free(graph)
    out["node_type_names"] = [api.boat_node_type_name(t).decode() for t in range(6)]
    return out


def loss_and_scheduler_facts(api):
    """Argument checks of the loss objects (src/loss/*.c) and the schedulers (src/schedulers/*.c)."""
    out = {}
    rng = np.random.default_rng(11)
    pred, target = api.tensor(rng.random((4, 5)).astype(np.float32)), api.tensor(rng.random((4, 5)).astype(np.float32))
    other = api.tensor(rng.random((4, 6)).astype(np.float32))
    for kind, make in (("mse", api.boat_mse_loss_create), ("ce", api.boat_cross_entropy_loss_create), ("huber", lambda: api.boat_huber_loss_create(1.0))):
        loss = make()
        out[kind + "_created"] = bool(loss)
        v = float(api.boat_loss_compute(loss, pred, target))
        out[kind + "_finite_and_positive"] = bool(np.isfinite(v) and v > 0)
        out[kind + "_shape_mismatch"] = round(float(api.boat_loss_compute(loss, pred, other)), 6)
        out[kind + "_null_prediction"] = round(float(api.boat_loss_compute(loss, None, target)), 6)
        api.boat_loss_free(loss)
    out["loss_compute_on_null_loss"] = round(float(api.boat_loss_compute(None, pred, target)), 6)
    out["step_bad"] = [not api.boat_step_lr_scheduler_create(0.0, 10, 0.5), not api.boat_step_lr_scheduler_create(0.1, 0, 0.5),
                       not api.boat_step_lr_scheduler_create(0.1, 10, 0.0), not api.boat_step_lr_scheduler_create(0.1, 10, 1.5)]
    out["cosine_bad"] = [not api.boat_cosine_annealing_scheduler_create(0.0, 10, 0.0), not api.boat_cosine_annealing_scheduler_create(0.1, 0, 0.0),
                         not api.boat_cosine_annealing_scheduler_create(0.1, 10, -1.0), not api.boat_cosine_annealing_scheduler_create(0.1, 10, 0.2)]
    out["null_scheduler_lr"] = (round(float(api.boat_scheduler_get_last_lr(None)), 6), round(float(api.boat_scheduler_get_next_lr(None)), 6))
    sch = api.boat_step_lr_scheduler_create(0.1, 2, 0.5)
    opt = api.boat_adam_optimizer_create(0.3, 0.9, 0.999, 1e-8)
    api.boat_scheduler_update_optimizer(sch, opt)
    out["update_optimizer_sets_last_lr"] = round(float(api.boat_optimizer_get_learning_rate(opt)), 6)
    api.boat_scheduler_update_optimizer(None, opt)
    api.boat_scheduler_update_optimizer(sch, None)
    api.boat_scheduler_free(sch)
    api.boat_optimizer_free(opt)
    for t in (pred, target, other):
        api.boat_tensor_unref(t)
    return out


def attention_facts(api):
    """What boat_attention_forward / backward accept and ignore (src/layers/attention.c:247-466,468-560,1012-1025,1061-1062)."""
    from boat_amd.capi import AttentionConfig
    out = {}
    rng = np.random.default_rng(12)

    def T(*shape):
        return api.tensor(rng.standard_normal(shape).astype(np.float32))

    att = api.boat_attention_create(C.byref(AttentionConfig(8, 2, 0, 0.5, True, True, False, 10000.0)))   # dropout 0.5, causal
    x, mask = T(2, 3, 8), api.tensor(np.zeros((2, 3, 3), np.float32))
    with scratch_cwd():
        out["backward_before_forward"] = bool(api.boat_attention_backward(att, x, None, None, None))
        y1 = api.boat_attention_forward(att, x, x, x, None)
        y2 = api.boat_attention_forward(att, x, x, x, mask)
        y3 = api.boat_attention_forward(att, x, x, x, None)
        out["mask_is_ignored"] = bool(np.array_equal(api.numpy(y1), api.numpy(y2)))
        out["dropout_is_ignored"] = bool(np.array_equal(api.numpy(y1), api.numpy(y3)))
        out["forward_null_query"] = not api.boat_attention_forward(att, None, x, x, None)
        wrong = T(2, 3, 6)
        out["forward_wrong_hidden"] = not api.boat_attention_forward(att, wrong, wrong, wrong, None)
        flat = T(6, 8)
        y2d = api.boat_attention_forward(att, flat, flat, flat, None)
        out["forward_2d_input"] = None if not y2d else api.shape(y2d)
        api.boat_attention_forward(att, x, x, x, None)
        dq, dk, dv = C.c_void_p(), C.c_void_p(), C.c_void_p()
        ok = api.boat_attention_backward(att, x, C.byref(dq), C.byref(dk), C.byref(dv))
        out["backward_ok"] = bool(ok)
        out["backward_grad_shapes"] = tuple(api.shape(g.value) for g in (dq, dk, dv))
        out["grads_exist_after_backward"] = bool(api.boat_attention_get_grad_weight_q(att)) and bool(api.boat_attention_get_grad_bias_o(att))
        out["backward_wrong_shape"] = bool(api.boat_attention_backward(att, wrong, None, None, None))
    return out


def conv_pool_facts(api):
    """Argument checks of the convolution, pooling and flatten hooks (src/layers/conv.c:240-330,475-537,
    src/layers/pool.c:30-62,173-218, src/layers/flatten.c)."""
    out = {}
    rng = np.random.default_rng(13)

    def T(*shape):
        return api.tensor(rng.standard_normal(shape).astype(np.float32))

    def shape_of(t):
        if not t:
            return None
        s = api.shape(t)
        api.boat_tensor_unref(t)
        return s

    conv = api.boat_conv_layer_create(2, 3, 3, 1, 0)
    x, small, dy_bad = T(2, 2, 6, 6), T(2, 2, 2, 2), T(2, 3, 5, 5)
    out["conv_backward_before_forward"] = shape_of(api.boat_conv_layer_backward(conv, dy_bad))
    out["conv_forward_no_padding"] = shape_of(api.boat_conv_layer_forward(conv, x))
    out["conv_backward_wrong_shape"] = shape_of(api.boat_conv_layer_backward(conv, dy_bad))
    out["conv_input_smaller_than_kernel"] = shape_of(api.boat_conv_layer_forward(conv, small))
    out["conv_null_input"] = shape_of(api.boat_conv_layer_forward(conv, None))
    strided = api.boat_conv_layer_create(2, 3, 3, 2, 1)
    out["conv_stride_two_pad_one"] = shape_of(api.boat_conv_layer_forward(strided, x))
    pool = api.boat_pool_layer_create(2, 2, 0)
    out["pool_backward_before_forward"] = shape_of(api.boat_pool_layer_backward(pool, x))
    out["pool_forward_odd_side"] = shape_of(api.boat_pool_layer_forward(pool, T(1, 1, 5, 5)))
    out["pool_backward_wrong_shape"] = shape_of(api.boat_pool_layer_backward(pool, T(1, 1, 3, 3)))
    out["pool_backward"] = shape_of(api.boat_pool_layer_backward(pool, T(1, 1, 2, 2)))
    flat = api.boat_flatten_layer_create()
    out["flatten_backward_before_forward"] = shape_of(api.boat_flatten_layer_backward(flat, x))
    out["flatten_2d_input"] = shape_of(api.boat_flatten_layer_forward(flat, T(3, 4)))
    out["flatten_4d_input"] = shape_of(api.boat_flatten_layer_forward(flat, x))
    out["flatten_backward"] = shape_of(api.boat_flatten_layer_backward(flat, T(2, 72)))
    return out
