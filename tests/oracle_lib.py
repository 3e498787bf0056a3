"""ctypes access to the CPU checker: oracle/libboat_oracle.so and the compiled reference.

Test infrastructure only -- never imported by the boat_amd package.
"""
import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
ORACLE_SO = ROOT / "oracle" / "libboat_oracle.so"
REF_SO = ROOT / "oracle" / "_ref" / "libboat_ref.so"

F = C.POINTER(C.c_float)
D = C.POINTER(C.c_double)
L = C.c_int64


def fp(a):
    return None if a is None else a.ctypes.data_as(F)


def dp(a):
    return None if a is None else a.ctypes.data_as(D)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class Oracle:
    """numpy-in / numpy-out wrappers over the C restatement (one method per oracle routine)."""

    def __init__(self, lib):
        self.lib = lib
        lib.bo_sum.restype = C.c_float
        lib.bo_ce_chain.restype = C.c_float
        lib.bo_mse_loss.restype = C.c_float

    def matmul(self, a, b):
        a, b = f32(a), f32(b)
        batch = int(np.prod(a.shape[:-2])) if a.ndim > 2 else 1
        m, k, n = a.shape[-2], a.shape[-1], b.shape[-1]
        c = np.empty(a.shape[:-2] + (m, n), np.float32)
        self.lib.bo_matmul(fp(a), fp(b), fp(c), L(batch), L(m), L(k), L(n))
        return c

    def transpose_last2(self, a):
        a = f32(a)
        batch = int(np.prod(a.shape[:-2])) if a.ndim > 2 else 1
        out = np.empty(a.shape[:-2] + (a.shape[-1], a.shape[-2]), np.float32)
        self.lib.bo_transpose_last2(fp(a), fp(out), L(batch), L(a.shape[-2]), L(a.shape[-1]))
        return out

    def sum(self, a):
        a = f32(a)
        return float(self.lib.bo_sum(fp(a), L(a.size)))

    def mul_scalar(self, a, s):
        a = f32(a)
        out = np.empty_like(a)
        self.lib.bo_mul_scalar(fp(a), C.c_double(s), fp(out), L(a.size))
        return out

    def _unary(self, fn, x):
        x = f32(x)
        y = np.empty_like(x)
        fn(fp(x), fp(y), L(x.size))
        return y

    def _saved_bwd(self, fn, saved, dy):
        saved, dy = f32(saved), f32(dy)
        dx = np.empty_like(saved)
        fn(fp(saved), fp(dy), fp(dx), L(saved.size))
        return dx

    def relu_forward(self, x): return self._unary(self.lib.bo_relu_forward, x)
    def sigmoid_forward(self, x): return self._unary(self.lib.bo_sigmoid_forward, x)
    def tanh_forward(self, x): return self._unary(self.lib.bo_tanh_forward, x)
    def relu_backward(self, x, dy): return self._saved_bwd(self.lib.bo_relu_backward, x, dy)
    def sigmoid_backward(self, c, dy): return self._saved_bwd(self.lib.bo_sigmoid_backward, c, dy)
    def tanh_backward(self, c, dy): return self._saved_bwd(self.lib.bo_tanh_backward, c, dy)

    def mul_backward(self, a, b, dy):
        a, b, dy = f32(a), f32(b), f32(dy)
        da, db = np.empty_like(a), np.empty_like(a)
        self.lib.bo_mul_backward(fp(a), fp(b), fp(dy), fp(da), fp(db), L(a.size))
        return da, db

    def div_backward(self, a, b, dy):
        a, b, dy = f32(a), f32(b), f32(dy)
        da, db = np.empty_like(a), np.empty_like(a)
        self.lib.bo_div_backward(fp(a), fp(b), fp(dy), fp(da), fp(db), L(a.size))
        return da, db

    def _rows(self, fn, *arrs):
        arrs = [f32(a) for a in arrs]
        cols = arrs[0].shape[-1]
        rows = arrs[0].size // cols
        out = np.empty_like(arrs[0])
        fn(*[fp(a) for a in arrs], fp(out), L(rows), L(cols))
        return out

    def softmax_forward(self, x): return self._rows(self.lib.bo_softmax_forward, x)
    def softmax_backward(self, y, dy): return self._rows(self.lib.bo_softmax_backward, y, dy)
    def log_softmax_forward(self, x): return self._rows(self.lib.bo_log_softmax_forward, x)
    def log_softmax_backward(self, y, dy): return self._rows(self.lib.bo_log_softmax_backward, y, dy)

    def ce_chain(self, logits, onehot):
        logits, onehot = f32(logits), f32(onehot)
        dz = np.empty_like(logits)
        loss = self.lib.bo_ce_chain(fp(logits), fp(onehot), fp(dz), L(logits.shape[0]), L(logits.shape[1]))
        return float(loss), dz

    def dense_forward(self, x, w, b=None):
        x, w = f32(x), f32(w)
        b = None if b is None else f32(b)
        m, k = x.shape
        n = w.shape[1]
        y = np.empty((m, n), np.float32)
        self.lib.bo_dense_forward(fp(x), fp(w), fp(b), fp(y), L(m), L(k), L(n))
        return y

    def dense_backward(self, x, w, dy, gw=None, gb=None, with_bias=True):
        """Returns dx and the accumulated gw, gb (start from the given arrays or zeros)."""
        x, w, dy = f32(x), f32(w), f32(dy)
        m, k = x.shape
        n = w.shape[1]
        gw = np.zeros((k, n), np.float32) if gw is None else f32(gw).copy()
        gb = (np.zeros(n, np.float32) if gb is None else f32(gb).copy()) if with_bias else None
        dx = np.empty((m, k), np.float32)
        self.lib.bo_dense_backward(fp(x), fp(w), fp(dy), fp(dx), fp(gw), fp(gb), L(m), L(k), L(n))
        return dx, gw, gb

    def sdpa_forward(self, q, k, v, scale, causal=False):
        q, k, v = f32(q), f32(k), f32(v)
        s, d = q.shape[-2:]
        bh = q.size // (s * d)
        attn = np.empty((bh, s, s), np.float32)
        out = np.empty_like(q)
        lse = np.empty((bh, s), np.float32)
        self.lib.bo_sdpa_forward(fp(q), fp(k), fp(v), C.c_float(scale), C.c_int(int(causal)), fp(attn), fp(out), fp(lse),
                                 L(bh), L(s), L(d))
        return out, lse, attn

    def sdpa_backward(self, q, k, v, attn, d_out, scale):
        q, k, v, attn, d_out = f32(q), f32(k), f32(v), f32(attn), f32(d_out)
        s, d = q.shape[-2:]
        bh = q.size // (s * d)
        dq, dk, dv = np.empty_like(q), np.empty_like(q), np.empty_like(q)
        self.lib.bo_sdpa_backward(fp(q), fp(k), fp(v), fp(attn), fp(d_out), C.c_float(scale), fp(dq), fp(dk), fp(dv),
                                  L(bh), L(s), L(d))
        return dq, dk, dv

    def attention_forward(self, x_q, x_k, x_v, w, b, heads, causal=False):
        """w, b: dicts with keys q,k,v,o (b may be None). Returns out and the cache dict."""
        x_q, x_k, x_v = f32(x_q), f32(x_k), f32(x_v)
        B, S, H = x_q.shape
        w = {n: f32(w[n]) for n in "qkvo"}
        bb = {n: (None if b is None else f32(b[n])) for n in "qkvo"}
        cache = {n: np.empty((B, S, H), np.float32) for n in ("q_proj", "k_proj", "v_proj", "attn_out")}
        cache["attn"] = np.empty((B * heads, S, S), np.float32)
        out = np.empty((B, S, H), np.float32)
        self.lib.bo_attention_forward(fp(x_q), fp(x_k), fp(x_v), fp(w["q"]), fp(w["k"]), fp(w["v"]), fp(w["o"]),
                                      fp(bb["q"]), fp(bb["k"]), fp(bb["v"]), fp(bb["o"]), C.c_int(int(causal)),
                                      L(B), L(S), L(H), L(heads), fp(cache["q_proj"]), fp(cache["k_proj"]),
                                      fp(cache["v_proj"]), fp(cache["attn"]), fp(cache["attn_out"]), fp(out))
        return out, cache

    def attention_backward(self, x_q, x_k, x_v, w, has_bias, cache, d_out, heads):
        x_q, x_k, x_v, d_out = f32(x_q), f32(x_k), f32(x_v), f32(d_out)
        B, S, H = x_q.shape
        w = {n: f32(w[n]) for n in "qkvo"}
        g = {f"d_{n}": np.empty((B, S, H), np.float32) for n in ("query", "key", "value")}
        for n in "qkvo":
            g[f"gw{n}"] = np.empty((H, H), np.float32)
            g[f"gb{n}"] = np.empty(H, np.float32) if has_bias else None
        self.lib.bo_attention_backward(fp(x_q), fp(x_k), fp(x_v), fp(w["q"]), fp(w["k"]), fp(w["v"]), fp(w["o"]),
                                       C.c_int(int(has_bias)), fp(cache["q_proj"]), fp(cache["k_proj"]), fp(cache["v_proj"]),
                                       fp(cache["attn"]), fp(cache["attn_out"]), fp(d_out), L(B), L(S), L(H), L(heads),
                                       fp(g["d_query"]), fp(g["d_key"]), fp(g["d_value"]),
                                       fp(g["gwq"]), fp(g["gwk"]), fp(g["gwv"]), fp(g["gwo"]),
                                       fp(g["gbq"]), fp(g["gbk"]), fp(g["gbv"]), fp(g["gbo"]))
        return g

    def layernorm_forward(self, x, gamma, beta, eps):
        x = f32(x)
        h = x.shape[-1]
        rows = x.size // h
        gamma = None if gamma is None else f32(gamma)
        beta = None if beta is None else f32(beta)
        y = np.empty_like(x)
        mean, rstd = np.empty(rows, np.float32), np.empty(rows, np.float32)
        self.lib.bo_layernorm_forward(fp(x), fp(gamma), fp(beta), fp(y), fp(mean), fp(rstd), L(rows), L(h), C.c_float(eps))
        return y, mean, rstd

    def layernorm_backward_f64(self, x, gamma, dy, mean, rstd):
        x, dy, mean, rstd = f32(x), f32(dy), f32(mean), f32(rstd)
        h = x.shape[-1]
        rows = x.size // h
        gamma = None if gamma is None else f32(gamma)
        dx = np.empty(x.shape, np.float64)
        dg, db = np.empty(h, np.float64), np.empty(h, np.float64)
        self.lib.bo_layernorm_backward_f64(fp(x), fp(gamma), fp(dy), fp(mean), fp(rstd), dp(dx), dp(dg), dp(db), L(rows), L(h))
        return dx, dg, db

    def rmsnorm_forward(self, x, weight, eps):
        x = f32(x)
        h = x.shape[-1]
        rows = x.size // h
        weight = None if weight is None else f32(weight)
        y = np.empty_like(x)
        inv = np.empty(rows, np.float32)
        self.lib.bo_rmsnorm_forward(fp(x), fp(weight), fp(y), fp(inv), L(rows), L(h), C.c_float(eps))
        return y, inv

    def rmsnorm_backward_f64(self, x, weight, dy, eps):
        x, dy = f32(x), f32(dy)
        h = x.shape[-1]
        rows = x.size // h
        weight = None if weight is None else f32(weight)
        dx = np.empty(x.shape, np.float64)
        dw = np.empty(h, np.float64)
        self.lib.bo_rmsnorm_backward_f64(fp(x), fp(weight), fp(dy), dp(dx), dp(dw), L(rows), L(h), C.c_double(eps))
        return dx, dw

    def gelu_forward_f64(self, x):
        x = f32(x)
        y = np.empty(x.shape, np.float64)
        self.lib.bo_gelu_forward_f64(fp(x), dp(y), L(x.size))
        return y

    def gelu_backward_f64(self, x, dy):
        x, dy = f32(x), f32(dy)
        dx = np.empty(x.shape, np.float64)
        self.lib.bo_gelu_backward_f64(fp(x), fp(dy), dp(dx), L(x.size))
        return dx

    def adam_update(self, p, g, m, v, lr, b1, b2, eps, t):
        """In place on copies; returns (p, m, v)."""
        p, m, v = f32(p).copy(), f32(m).copy(), f32(v).copy()
        g = f32(g)
        self.lib.bo_adam_update(fp(p), fp(g), fp(m), fp(v), L(p.size), C.c_float(lr), C.c_float(b1), C.c_float(b2),
                                C.c_float(eps), L(t))
        return p, m, v

    def conv2d_forward(self, x, w, bias, stride=1, pad=0):
        x, w = f32(x), f32(w)
        bias = None if bias is None else f32(bias)
        B, ic, h, wd = x.shape
        oc, _, k, _ = w.shape
        ho, wo = (h + 2 * pad - k) // stride + 1, (wd + 2 * pad - k) // stride + 1
        y = np.empty((B, oc, ho, wo), np.float32)
        self.lib.bo_conv2d_forward(fp(x), fp(w), fp(bias), fp(y), L(B), L(ic), L(h), L(wd), L(oc), L(k), L(stride), L(pad))
        return y

    def conv2d_backward(self, x, w, dy, stride=1, pad=0, flip_taps=False):
        """Returns dx, gw, gb (all overwritten).  flip_taps=True is the reference's input gradient."""
        x, w, dy = f32(x), f32(w), f32(dy)
        B, ic, h, wd = x.shape
        oc, _, k, _ = w.shape
        dx, gw, gb = np.empty_like(x), np.empty_like(w), np.empty(oc, np.float32)
        self.lib.bo_conv2d_backward(fp(x), fp(w), fp(dy), fp(dx), fp(gw), fp(gb), L(B), L(ic), L(h), L(wd), L(oc), L(k),
                                    L(stride), L(pad), C.c_int(int(flip_taps)))
        return dx, gw, gb

    def maxpool2d_forward(self, x, pool, stride, pad=0):
        x = f32(x)
        B, ch, h, wd = x.shape
        ho, wo = (h + 2 * pad - pool) // stride + 1, (wd + 2 * pad - pool) // stride + 1
        y = np.empty((B, ch, ho, wo), np.float32)
        arg = np.empty((B, ch, ho, wo), np.int64)
        self.lib.bo_maxpool2d_forward(fp(x), fp(y), arg.ctypes.data_as(C.POINTER(C.c_int64)), L(B * ch), L(h), L(wd), L(pool),
                                      L(stride), L(pad))
        return y, arg

    def maxpool2d_backward(self, dy, argmax, in_shape):
        dy = f32(dy)
        argmax = np.ascontiguousarray(argmax, np.int64)
        dx = np.empty(in_shape, np.float32)
        self.lib.bo_maxpool2d_backward(fp(dy), argmax.ctypes.data_as(C.POINTER(C.c_int64)), fp(dx), L(dx.size), L(dy.size))
        return dx

    def loss_value(self, kind, p, t, delta=1.0):
        """kind: "mse", "ce" (p are probabilities) or "huber"."""
        p, t = f32(p), f32(t)
        self.lib.bo_loss_value.restype = C.c_float
        return float(self.lib.bo_loss_value(C.c_int({"mse": 0, "ce": 1, "huber": 2}[kind]), fp(p), fp(t), L(p.size), C.c_float(delta)))

    def rmsprop_update(self, p, g, sq, lr, alpha, eps):
        """In place on copies; returns (p, sq)."""
        p, sq, g = f32(p).copy(), f32(sq).copy(), f32(g)
        self.lib.bo_rmsprop_update(fp(p), fp(g), fp(sq), L(p.size), C.c_float(lr), C.c_float(alpha), C.c_float(eps))
        return p, sq

    def adagrad_update(self, p, g, acc, lr, eps):
        p, acc, g = f32(p).copy(), f32(acc).copy(), f32(g)
        self.lib.bo_adagrad_update(fp(p), fp(g), fp(acc), L(p.size), C.c_float(lr), C.c_float(eps))
        return p, acc

    def mse_loss(self, pred, target):
        pred, target = f32(pred), f32(target)
        return float(self.lib.bo_mse_loss(fp(pred), fp(target), L(pred.size)))

    def mse_grad(self, pred, target):
        pred, target = f32(pred), f32(target)
        g = np.empty_like(pred)
        self.lib.bo_mse_grad(fp(pred), fp(target), fp(g), L(pred.size))
        return g


def load() -> Oracle:
    if not ORACLE_SO.exists():
        subprocess.run(["make", "-C", str(ROOT / "oracle"), "oracle"], check=True, capture_output=True)
    return Oracle(C.CDLL(str(ORACLE_SO)))


def load_reference():
    """BoatAPI over the compiled reference, or None if it has not been built."""
    if not REF_SO.exists():
        return None
    from boat_amd.capi import BoatAPI
    return BoatAPI(REF_SO)


def rel_fro(a, b):
    """||a-b||_F / ||b||_F"""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    den = np.linalg.norm(b.ravel())
    return float(np.linalg.norm((a - b).ravel()) / (den if den > 0 else 1.0))


def max_rel(a, b, floor=1e-30):
    """max |a-b| / max(|b|, floor)"""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.max(np.abs(a - b) / np.maximum(np.abs(b), floor))) if a.size else 0.0


def fp32_gemm_bound(k):
    """Relative Frobenius error that a contraction of length k keeps when products and sums are carried in full fp32
    (about 6e-8 * sqrt(k) / 3 for a sequential sum, less for blocked ones); an operand or accumulator narrowed to 10 or 7
    mantissa bits (tf32, bf16) lands near 3e-4 and 2e-3 and fails it."""
    return max(2e-6, 1.5e-7 * float(np.sqrt(k)))


FP32_ATTENTION_BOUND = 2e-5    # attention outputs and gradients against the fp32 oracle: two rounding paths of about 1e-6 each


def narrow_mantissa(a, bits):
    """float32 values truncated to `bits` explicit mantissa bits (7 = bf16, 10 = tf32 / fp16)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    return (u & np.uint32(0xFFFFFFFF << (23 - bits) & 0xFFFFFFFF)).view(np.float32)
