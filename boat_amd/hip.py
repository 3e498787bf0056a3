"""ctypes binding of the device layer's C-ABI (include/boat_hip.h) plus a tiny device-array helper.

Everything here runs on the GPU through libboat_amd.so; importing the module loads the
library and fails loudly if it has not been built.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from .capi import LIB_PATH

P = C.c_void_p
F = C.c_float
I = C.c_int
L = C.c_int64
Z = C.c_size_t

if not LIB_PATH.exists():
    raise FileNotFoundError(f"{LIB_PATH} not found: build it first (python -m boat_amd.build); there is no host fallback")
lib = C.CDLL(str(LIB_PATH), mode=C.RTLD_LOCAL)

_SIGS = {
    "bh_init": (I, []), "bh_shutdown": (I, []), "bh_synchronize": (I, []),
    "bh_last_error": (C.c_char_p, []), "bh_device_name": (C.c_char_p, []), "bh_device_cu_count": (I, []),
    "bh_stream": (P, []),
    "bh_malloc": (P, [Z]), "bh_free": (None, [P]), "bh_cache_release": (I, []),
    "bh_bytes_in_use": (Z, []), "bh_bytes_cached": (Z, []),
    "bh_buffer_create": (P, [Z, I]), "bh_buffer_ref": (None, [P]), "bh_buffer_unref": (None, [P]),
    "bh_buffer_ptr": (P, [P]), "bh_buffer_nbytes": (Z, [P]), "bh_buffer_refcount": (I, [P]),
    "bh_host_alloc": (P, [Z]), "bh_host_free": (None, [P]), "bh_memcpy_h2d_async": (I, [P, P, Z]), "bh_memcpy_d2h_async": (I, [P, P, Z]),
    "bh_memcpy_h2d": (I, [P, P, Z]), "bh_memcpy_d2h": (I, [P, P, Z]), "bh_memcpy_d2d": (I, [P, P, Z]),
    "bh_memset_zero": (I, [P, Z]),
    "bh_event_create": (P, []), "bh_event_destroy": (None, [P]), "bh_event_record": (I, [P]), "bh_event_wait": (I, [P]),
    "bh_event_elapsed_ms": (F, [P, P]),
    "bh_profile_enable": (I, [I]),
    "bh_profile_read": (I, [I, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(L)]),
    "bh_fill": (I, [P, F, L]),
    "bh_add_inplace": (I, [P, P, L]),
    "bh_binary": (I, [I, P, P, P, L]),
    "bh_binary_broadcast": (I, [I, P, C.POINTER(L), P, C.POINTER(L), P, C.POINTER(L), I]),
    "bh_scalar_op": (I, [I, P, F, P, L]), "bh_copy_f32": (I, [P, P, L]), "bh_scale_by_device_scalar": (I, [P, P, P, L]),
    "bh_div_backward_b": (I, [P, P, P, P, L]),
    "bh_activation_forward": (I, [I, P, P, L]),
    "bh_activation_backward": (I, [I, P, P, P, L, I]),
    "bh_activation_backward_colsum": (I, [I, P, P, P, P, L, L, I]),
    "bh_bias_add_rows": (I, [P, P, L, L]),
    "bh_mse_grad": (I, [P, P, P, L]), "bh_mse_loss": (I, [P, P, P, L]), "bh_mse_loss_grad": (I, [P, P, P, P, L]),
    "bh_sgd_update": (I, [P, P, F, L, I]),
    "bh_sum_all": (I, [P, P, L]),
    "bh_colsum": (I, [P, P, L, L, I]), "bh_colsum_grouped": (I, [C.POINTER(P), C.POINTER(P), I, L, L, I]),
    "bh_softmax_forward": (I, [P, P, L, L]), "bh_softmax_backward": (I, [P, P, P, L, L]),
    "bh_log_softmax_forward": (I, [P, P, L, L]), "bh_log_softmax_backward": (I, [P, P, P, L, L]),
    "bh_softmax_ce_grad": (I, [P, P, P, P, L, L]),
    "bh_log_softmax_weighted_backward": (I, [P, P, P, P, P, L, L]),
    "bh_log_softmax_weighted_backward_colsum": (I, [P, P, P, P, P, P, L, L, I]),
    "bh_layernorm_forward": (I, [P, P, P, P, P, P, L, L, F]),
    "bh_layernorm_backward": (I, [P, P, P, P, P, P, P, P, L, L, I]),
    "bh_layernorm_backward_add": (I, [P, P, P, P, P, P, P, P, P, L, L, I]),
    "bh_rmsnorm_forward": (I, [P, P, P, P, L, L, F]),
    "bh_rmsnorm_backward": (I, [P, P, P, P, P, P, L, L, F, I]),
    "bh_binary_typed": (I, [I, I, P, C.POINTER(L), P, C.POINTER(L), P, C.POINTER(L), I]),
    "bh_scalar_op_typed": (I, [I, I, P, C.c_double, P, L]),
    "bh_layernorm_backward_noalloc": (I, [P, P, P, P, P, P, P, P, L, L, I]),
    "bh_gemm": (I, [I, I, L, L, L, P, L, P, L, P, L, P, I, L]),
    "bh_gemm_grouped": (I, [I, I, L, L, L, I, C.POINTER(P), L, C.POINTER(P), L, C.POINTER(P), L, C.POINTER(P), I]),
    "bh_gemm_ksegments": (I, [I, I, L, L, L, I, C.POINTER(P), L, C.POINTER(P), L, P, L, P, I]),
    "bh_gemm_no_tables": (I, [I]),
    "bh_gemm_force_config": (I, [I]), "bh_gemm_force_direct": (I, [I]), "bh_gemm_force_splits": (I, [I]),
    "bh_transpose_last2": (I, [P, P, L, L, L]),
    "bh_dense_backward": (I, [P, P, P, P, P, P, L, L, L, I]),
    "bh_dense_backward_into": (I, [P, P, P, P, P, P, L, L, L, I, I]),
    "bh_sdpa_forward": (I, [P, P, P, F, I, P, P, P, L, L, L]),
    "bh_sdpa_backward": (I, [P, P, P, P, P, P, F, I, P, P, P, L, L, L]),
    "bh_sdpa_force_general": (I, [I]), "bh_sdpa_force_wide": (I, [I]),
    "bh_sdpa_score_cache_bytes": (C.c_size_t, [L, L, L]),
    "bh_sdpa_forward_cached": (I, [P, P, P, F, I, P, P, P, L, L, L]),
    "bh_sdpa_backward_cached": (I, [P, P, P, P, P, P, P, F, I, P, P, P, L, L, L]),
    "bh_adam_update": (I, [P, P, P, P, L, F, F, F, F, L]),
    "bh_stream_probe_4r3w": (I, [P, P, P, P, L]),
    "bh_conv2d_forward": (I, [P, P, P, P] + [L] * 8),
    "bh_conv2d_forward_mfma": (I, [P, P, P, P] + [L] * 8),
    "bh_conv2d_backward": (I, [P, P, P, P, P, P] + [L] * 8 + [I, I]),
    "bh_maxpool2d_forward": (I, [P, P, P] + [L] * 6),
    "bh_maxpool2d_backward": (I, [P, P, P] + [L] * 6),
    "bh_zero_multi": (I, [C.POINTER(P), C.POINTER(L), I]),
    "bh_loss_terms_sum": (I, [I, P, P, P, L, F]),
    "bh_rmsprop_update": (I, [P, P, P, L, F, F, F]),
    "bh_adagrad_update": (I, [P, P, P, L, F, F]),
    "bh_adam_update_multi": (I, [C.POINTER(P), C.POINTER(P), C.POINTER(P), C.POINTER(P), C.POINTER(L), I, F, F, F, F, L]),
}
for _name, (_res, _args) in _SIGS.items():
    _fn = getattr(lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args
    globals()[_name] = _fn

ACT_RELU, ACT_SIGMOID, ACT_TANH, ACT_GELU = 0, 1, 2, 3
PROF_GEMM, PROF_SDPA_FWD, PROF_SDPA_BWD, PROF_NORM, PROF_OPTIMIZER, PROF_COLSUM = range(6)


def profile_read(cls):
    """(total ms, total declared work, calls) of one class of launches since bh_profile_enable."""
    ms, work, calls = C.c_double(), C.c_double(), L()
    check(lib.bh_profile_read(cls, C.byref(ms), C.byref(work), C.byref(calls)), "bh_profile_read")
    return ms.value, work.value, calls.value


class HipError(RuntimeError):
    pass


def check(rc: int, what: str = "") -> None:
    if rc != 0:
        raise HipError(f"{what or 'device call'} failed ({rc}): {lib.bh_last_error().decode()}")


class DeviceArray:
    """A dense row-major array in HBM (fp32 unless told otherwise); freed when collected."""

    def __init__(self, shape, dtype=np.float32, zero: bool = False):
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.size = int(np.prod(self.shape)) if self.shape else 1
        self.nbytes = self.size * self.dtype.itemsize
        self.ptr = lib.bh_malloc(max(self.nbytes, 4))
        if not self.ptr:
            raise HipError(f"bh_malloc({self.nbytes}) failed: {lib.bh_last_error().decode()}")
        if zero:
            check(lib.bh_memset_zero(self.ptr, self.nbytes), "memset")

    @classmethod
    def from_numpy(cls, a) -> "DeviceArray":
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        if a.nbytes:
            check(lib.bh_memcpy_h2d(d.ptr, a.ctypes.data, a.nbytes), "h2d")
        return d

    def numpy(self) -> np.ndarray:
        out = np.empty(self.shape, dtype=self.dtype)
        if self.nbytes:
            check(lib.bh_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes), "d2h")
        return out

    def __del__(self):
        try:
            if getattr(self, "ptr", None):
                lib.bh_free(self.ptr)
                self.ptr = None
        except Exception:
            pass


def to_device(a) -> DeviceArray:
    return DeviceArray.from_numpy(a)


def empty(shape, dtype=np.float32) -> DeviceArray:
    return DeviceArray(shape, dtype)


def zeros(shape, dtype=np.float32) -> DeviceArray:
    return DeviceArray(shape, dtype, zero=True)


def synchronize() -> None:
    check(lib.bh_synchronize(), "synchronize")


class Timer:
    """Times work enqueued on the library stream with HIP events."""

    def __init__(self):
        self.start = lib.bh_event_create()
        self.stop = lib.bh_event_create()
        if not self.start or not self.stop:
            raise HipError("event creation failed")

    def __enter__(self):
        check(lib.bh_event_record(self.start), "event record")
        return self

    def __exit__(self, *exc):
        check(lib.bh_event_record(self.stop), "event record")
        self.ms = float(lib.bh_event_elapsed_ms(self.start, self.stop))
        return False

    def __del__(self):
        try:
            lib.bh_event_destroy(self.start)
            lib.bh_event_destroy(self.stop)
        except Exception:
            pass

lib.bh_layernorm_tune.restype = I
lib.bh_layernorm_tune.argtypes = [I, I]
bh_layernorm_tune = lib.bh_layernorm_tune
