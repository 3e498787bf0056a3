"""ctypes binding of Boat's C API (the subset on the training hot path).

`BoatAPI(path)` loads any shared library that exports Boat's symbols with Boat's
signatures -- libboat_amd.so (the default, GPU) or a build of the reference itself
-- so the same test code can drive both and compare results.

The binding is deliberately thin: tensors, variables, layers and optimizers are
opaque pointers exactly as in the C headers; only numpy <-> tensor copies are added.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import numpy as np

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libboat_amd.so"

# include/boat/tensor.h:22-55
DTYPE_FLOAT64, DTYPE_FLOAT32 = 0, 1
DTYPE_INT64, DTYPE_INT32, DTYPE_UINT8 = 5, 6, 7
DEVICE_CPU, DEVICE_HIP = 0, 1

_NP = {DTYPE_FLOAT64: np.float64, DTYPE_FLOAT32: np.float32, DTYPE_INT64: np.int64,
       DTYPE_INT32: np.int32, DTYPE_UINT8: np.uint8}
_DT = {np.dtype(v): k for k, v in _NP.items()}

P = C.c_void_p


class MemoryStats(C.Structure):
    """boat_memory_stats_t (returned by value)."""
    _fields_ = [("allocated_bytes", C.c_size_t), ("allocated_blocks", C.c_size_t), ("peak_allocated_bytes", C.c_size_t),
                ("freed_bytes", C.c_size_t), ("freed_blocks", C.c_size_t)]


class AttentionConfig(C.Structure):  # include/boat/layers/attention.h:21-30
    _fields_ = [("hidden_size", C.c_size_t), ("num_heads", C.c_size_t), ("head_size", C.c_size_t),
                ("dropout_prob", C.c_float), ("causal_mask", C.c_bool), ("use_bias", C.c_bool),
                ("use_rotary", C.c_bool), ("rotary_theta", C.c_float)]


class LayerNormConfig(C.Structure):  # include/boat/layers/norm.h:21-26
    _fields_ = [("normalized_shape", C.c_size_t), ("eps", C.c_float),
                ("elementwise_affine", C.c_bool), ("use_bias", C.c_bool)]


class RmsNormConfig(C.Structure):  # include/boat/layers/norm.h:28-32
    _fields_ = [("normalized_shape", C.c_size_t), ("eps", C.c_float), ("elementwise_affine", C.c_bool)]


FREE_FN = C.CFUNCTYPE(None, C.c_void_p)                     # include/boat/model.h: user-data destructor
LAMBDA_LR_FN = C.CFUNCTYPE(C.c_float, C.c_int, C.c_float)   # include/boat/schedulers.h:35-36

_SIGS = {
    # tensor
    "boat_tensor_create": (P, [C.POINTER(C.c_int64), C.c_size_t, C.c_int, C.c_int]),
    "boat_tensor_create_like": (P, [P]),
    "boat_tensor_from_data": (P, [C.POINTER(C.c_int64), C.c_size_t, C.c_int, P]),
    "boat_dtype_size": (C.c_size_t, [C.c_int]),
    "boat_tensor_free": (None, [P]),
    "boat_tensor_ref": (None, [P]),
    "boat_tensor_unref": (None, [P]),
    "boat_tensor_shape": (C.POINTER(C.c_int64), [P]),
    "boat_tensor_ndim": (C.c_size_t, [P]),
    "boat_tensor_dtype": (C.c_int, [P]),
    "boat_tensor_device": (C.c_int, [P]),
    "boat_tensor_nbytes": (C.c_size_t, [P]),
    "boat_tensor_nelements": (C.c_size_t, [P]),
    "boat_tensor_data": (P, [P]),
    "boat_tensor_const_data": (P, [P]),
    "boat_tensor_reshape": (P, [P, C.POINTER(C.c_int64), C.c_size_t]),
    "boat_tensor_slice": (P, [P, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "boat_tensor_is_contiguous": (C.c_bool, [P]),
    "boat_dtype_name": (C.c_char_p, [C.c_int]),
    # memory and error reporting
    "boat_memory_allocate": (P, [C.c_size_t, C.c_int, C.c_char_p, C.c_int]), "boat_memory_free": (None, [P]),
    "boat_memory_allocate_device": (P, [C.c_size_t, C.c_int, C.c_char_p, C.c_int]), "boat_memory_free_device": (None, [P, C.c_int]),
    "boat_memory_copy": (None, [P, P, C.c_size_t, C.c_int, C.c_int]),
    "boat_memory_reallocate": (P, [P, C.c_size_t, C.c_int, C.c_char_p, C.c_int]),
    "boat_memory_pool_create": (P, [C.c_size_t, C.c_size_t]), "boat_memory_pool_free": (None, [P]),
    "boat_memory_pool_alloc": (P, [P, C.c_size_t]), "boat_memory_pool_free_block": (None, [P, P]),
    "boat_memory_pool_clear": (None, [P]), "boat_memory_pool_allocated_blocks": (C.c_size_t, [P]),
    "boat_memory_pool_free_blocks": (C.c_size_t, [P]), "boat_memory_pool_total_memory": (C.c_size_t, [P]),
    "boat_memory_arena_create": (P, [C.c_size_t]), "boat_memory_arena_free": (None, [P]),
    "boat_memory_arena_alloc": (P, [P, C.c_size_t]), "boat_memory_arena_reset": (None, [P]),
    "boat_memory_arena_used": (C.c_size_t, [P]), "boat_memory_arena_capacity": (C.c_size_t, [P]),
    # graph handle and the model's chain view
    "boat_graph_create": (P, []), "boat_graph_create_with_device": (P, [C.c_int]), "boat_graph_free": (None, [P]),
    "boat_autodiff_context_set_graph": (None, [P, P]), "boat_autodiff_context_get_graph": (P, [P]),
    "boat_model_graph": (P, [P]), "boat_graph_node_count": (C.c_size_t, [P]), "boat_graph_edge_count": (C.c_size_t, [P]),
    "boat_graph_get_node_at_index": (P, [P, C.c_size_t]), "boat_node_data": (P, [P]), "boat_node_type": (C.c_int, [P]),
    "boat_node_type_name": (C.c_char_p, [C.c_int]),
    "boat_memory_set": (None, [P, C.c_int, C.c_size_t, C.c_int]), "boat_memory_reset_stats": (None, []),
    "boat_error_string": (C.c_char_p, [C.c_int]), "boat_get_last_error": (C.c_int, []),
    "boat_get_last_error_message": (C.c_char_p, []),
    "boat_set_error": (None, [C.c_int, C.c_char_p]), "boat_clear_error": (None, []), "boat_has_error": (C.c_bool, []),
    # ops
    "boat_add_scalar": (P, [P, C.c_double]), "boat_sub_scalar": (P, [P, C.c_double]), "boat_div_scalar": (P, [P, C.c_double]),
    "boat_sub_": (None, [P, P]), "boat_mul_": (None, [P, P]), "boat_div_": (None, [P, P]),
    "boat_dot": (P, [P, P]), "boat_sigmoid": (P, [P]), "boat_tanh": (P, [P]),
    "boat_add": (P, [P, P]), "boat_sub": (P, [P, P]), "boat_mul": (P, [P, P]), "boat_div": (P, [P, P]),
    "boat_add_": (None, [P, P]),
    "boat_mul_scalar": (P, [P, C.c_double]),
    "boat_matmul": (P, [P, P]),
    "boat_transpose": (P, [P, C.c_int, C.c_int]),
    "boat_relu": (P, [P]),
    "boat_softmax": (P, [P, C.c_int]), "boat_log_softmax": (P, [P, C.c_int]),
    "boat_sum": (P, [P, C.POINTER(C.c_int64), C.c_size_t, C.c_bool]),
    "boat_can_broadcast": (C.c_bool, [P, P]), "boat_broadcast_to": (P, [P, C.POINTER(C.c_int64), C.c_size_t]),
    "boat_mod": (P, [P, P]), "boat_pow_scalar": (P, [P, C.c_double]),
    "boat_add_scalar_": (None, [P, C.c_double]), "boat_sub_scalar_": (None, [P, C.c_double]),
    "boat_mul_scalar_": (None, [P, C.c_double]), "boat_div_scalar_": (None, [P, C.c_double]),
    "boat_inverse": (P, [P]), "boat_selu": (P, [P]),
    "boat_reset_error": (None, []), "boat_memory_free_safe": (None, [C.POINTER(P)]),
    "boat_memory_allocate_aligned": (P, [C.c_size_t, C.c_size_t, C.c_int, C.c_char_p, C.c_int]),
    "boat_memory_free_aligned": (None, [P]),
    # autodiff
    "boat_var_max": (P, [P, C.POINTER(C.c_int64), C.c_size_t, C.c_bool]),
    "boat_var_min": (P, [P, C.POINTER(C.c_int64), C.c_size_t, C.c_bool]),
    "boat_variable_create": (P, [P, C.c_bool]),
    "boat_variable_free": (None, [P]),
    "boat_variable_data": (P, [P]),
    "boat_variable_grad": (P, [P]),
    "boat_variable_requires_grad": (C.c_bool, [P]),
    "boat_variable_zero_grad": (None, [P]),
    "boat_variable_create_with_shape": (P, [C.POINTER(C.c_int64), C.c_size_t, C.c_int, C.c_bool]),
    "boat_variable_set_requires_grad": (None, [P, C.c_bool]), "boat_variable_retain_grad": (None, [P, C.c_bool]),
    "boat_variable_reset_data": (C.c_bool, [P, P]),
    "boat_autodiff_context_create": (P, []), "boat_autodiff_context_free": (None, [P]),
    "boat_autodiff_context_enable_grad": (None, [P]), "boat_autodiff_context_disable_grad": (None, [P]),
    "boat_autodiff_context_grad_enabled": (C.c_bool, [P]),
    "boat_autodiff_set_current_context": (None, [P]), "boat_autodiff_get_current_context": (P, []),
    "boat_variable_backward": (None, [P, P]),
    "boat_variable_backward_full": (None, [P]),
    "boat_var_add": (P, [P, P]), "boat_var_sub": (P, [P, P]), "boat_var_mul": (P, [P, P]), "boat_var_div": (P, [P, P]),
    "boat_var_matmul": (P, [P, P]), "boat_var_dot": (P, [P, P]),
    "boat_var_relu": (P, [P]), "boat_var_sigmoid": (P, [P]), "boat_var_tanh": (P, [P]),
    "boat_var_softmax": (P, [P, C.c_int]), "boat_var_log_softmax": (P, [P, C.c_int]),
    "boat_var_sum": (P, [P, C.POINTER(C.c_int64), C.c_size_t, C.c_bool]),
    "boat_var_dense": (P, [P, P]),
    "boat_var_attention": (P, [P, P, P, P, P]),
    "boat_autodiff_clear_computation_graph": (None, []),
    # dense
    "boat_dense_layer_create": (P, [C.c_size_t, C.c_size_t, C.c_bool]),
    "boat_dense_layer_free": (None, [P]),
    "boat_dense_layer_forward": (P, [P, P]),
    "boat_dense_layer_backward": (P, [P, P]),
    "boat_dense_layer_update": (None, [P, C.c_float]),
    "boat_dense_layer_get_weight": (P, [P]), "boat_dense_layer_get_bias": (P, [P]),
    "boat_dense_layer_set_weight": (None, [P, P]), "boat_dense_layer_set_bias": (None, [P, P]),
    "boat_dense_layer_get_grad_weight": (P, [P]), "boat_dense_layer_get_grad_bias": (P, [P]),
    # conv / pool / flatten
    "boat_conv_layer_create": (P, [C.c_size_t] * 5), "boat_conv_layer_free": (None, [P]),
    "boat_conv_layer_forward": (P, [P, P]), "boat_conv_layer_backward": (P, [P, P]),
    "boat_conv_layer_update": (None, [P, C.c_float]),
    "boat_conv_layer_set_weight": (None, [P, P]), "boat_conv_layer_set_bias": (None, [P, P]),
    "boat_pool_layer_update": (None, [P, C.c_float]), "boat_flatten_layer_update": (None, [P, C.c_float]),
    "boat_conv_layer_get_weight": (P, [P]), "boat_conv_layer_get_bias": (P, [P]),
    "boat_conv_layer_get_grad_weight": (P, [P]), "boat_conv_layer_get_grad_bias": (P, [P]),
    "boat_pool_layer_create": (P, [C.c_size_t] * 3), "boat_pool_layer_free": (None, [P]),
    "boat_pool_layer_forward": (P, [P, P]), "boat_pool_layer_backward": (P, [P, P]),
    "boat_flatten_layer_create": (P, []), "boat_flatten_layer_free": (None, [P]),
    "boat_flatten_layer_forward": (P, [P, P]), "boat_flatten_layer_backward": (P, [P, P]),
    "boat_var_conv": (P, [P, P]), "boat_var_pool": (P, [P, P]), "boat_var_flatten": (P, [P]),
    "boat_autodiff_set_grad_checkpointing": (None, [C.c_bool]), "boat_autodiff_print_graph": (None, [P]),
    "boat_autodiff_graph_to_dot": (P, [P]), "boat_attention_set_dropout": (None, [P, C.c_float]),
    # loss objects
    "boat_mse_loss_create": (P, []), "boat_cross_entropy_loss_create": (P, []), "boat_huber_loss_create": (P, [C.c_float]),
    "boat_loss_compute": (C.c_float, [P, P, P]), "boat_loss_free": (None, [P]),
    # learning-rate schedulers
    "boat_step_lr_scheduler_create": (P, [C.c_float, C.c_int, C.c_float]),
    "boat_cosine_annealing_scheduler_create": (P, [C.c_float, C.c_int, C.c_float]),
    "boat_lambda_lr_scheduler_create": (P, [C.c_float, LAMBDA_LR_FN]),
    "boat_scheduler_step": (None, [P]), "boat_scheduler_reset": (None, [P]),
    "boat_scheduler_get_last_lr": (C.c_float, [P]), "boat_scheduler_get_next_lr": (C.c_float, [P]),
    "boat_scheduler_free": (None, [P]), "boat_scheduler_update_optimizer": (None, [P, P]),
    # relu / softmax hooks
    "boat_relu_layer_create": (P, []), "boat_relu_layer_free": (None, [P]),
    "boat_relu_layer_forward": (P, [P, P]), "boat_relu_layer_backward": (P, [P, P]),
    "boat_relu_layer_update": (None, [P, C.c_float]), "boat_softmax_layer_update": (None, [P, C.c_float]),
    "boat_softmax_layer_create": (P, [C.c_int]), "boat_softmax_layer_free": (None, [P]),
    "boat_softmax_layer_forward": (P, [P, P]), "boat_softmax_layer_backward": (P, [P, P]),
    # layernorm
    "boat_layernorm_create": (P, [C.POINTER(LayerNormConfig)]),
    "boat_layernorm_free": (None, [P]),
    "boat_layernorm_forward": (P, [P, P]),
    "boat_layernorm_backward": (P, [P, P]),
    "boat_layernorm_set_weight": (None, [P, P]), "boat_layernorm_set_bias": (None, [P, P]),
    "boat_layer_norm_grad": (P, [P, P, P, C.POINTER(C.c_int64), C.c_size_t, C.c_float]),
    "boat_norm_layer_update": (None, [P, C.c_float]),
    "boat_norm_layer_create": (P, [C.c_size_t, C.c_float, C.c_bool]),
    "boat_norm_layer_free": (None, [P]),
    "boat_norm_layer_forward": (P, [P, P]), "boat_norm_layer_backward": (P, [P, P]),
    # rmsnorm and the stateless forms
    "boat_rmsnorm_create": (P, [C.POINTER(RmsNormConfig)]), "boat_rmsnorm_free": (None, [P]),
    "boat_rmsnorm_forward": (P, [P, P]), "boat_rmsnorm_backward": (P, [P, P]), "boat_rmsnorm_update": (None, [P, C.c_float]),
    "boat_layer_norm": (P, [P, C.POINTER(C.c_int64), C.c_size_t, C.c_float]),
    "boat_rms_norm": (P, [P, C.POINTER(C.c_int64), C.c_size_t, C.c_float]),
    "boat_rms_norm_grad": (P, [P, P, P, C.POINTER(C.c_int64), C.c_size_t, C.c_float]),
    # attention
    "boat_scaled_dot_product_attention": (P, [P, P, P, C.c_float, P, C.c_bool, C.c_float]),
    "boat_multihead_attention": (P, [P, C.c_size_t, C.c_float, C.c_bool, P]),
    "boat_rotary_position_encoding": (P, [P, C.c_size_t, C.c_size_t, C.c_float]),
    "boat_apply_rotary_embedding": (None, [P, P, C.c_size_t, C.c_size_t, C.c_float]),
    "boat_attention_create": (P, [C.POINTER(AttentionConfig)]),
    "boat_attention_free": (None, [P]),
    "boat_attention_forward": (P, [P, P, P, P, P]),
    "boat_attention_backward": (C.c_bool, [P, P, C.POINTER(P), C.POINTER(P), C.POINTER(P)]),
    "boat_attention_update": (None, [P, C.c_float]),
    # optimizer
    "boat_adam_optimizer_create": (P, [C.c_float, C.c_float, C.c_float, C.c_float]),
    "boat_rmsprop_optimizer_create": (P, [C.c_float, C.c_float, C.c_float]),
    "boat_adagrad_optimizer_create": (P, [C.c_float, C.c_float]),
    "boat_optimizer_add_parameter": (None, [P, P, P]),
    "boat_optimizer_step": (None, [P]),
    "boat_optimizer_zero_grad": (None, [P]),
    "boat_optimizer_free": (None, [P]),
    "boat_optimizer_get_learning_rate": (C.c_float, [P]),
    "boat_optimizer_set_learning_rate": (None, [P, C.c_float]),
    # model
    "boat_model_create": (P, []), "boat_model_free": (None, [P]),
    "boat_model_add_layer": (None, [P, P]), "boat_model_layer_count": (C.c_size_t, [P]),
    "boat_model_forward": (P, [P, P]), "boat_model_backward": (P, [P, P]),
    "boat_model_update": (None, [P, C.c_float]),
    "boat_model_create_with_graph": (P, [P]), "boat_model_set_graph": (None, [P, P]),
    "boat_model_get_user_data": (P, [P]), "boat_model_set_user_data": (None, [P, P, FREE_FN]),
    "boat_model_load": (P, [C.c_char_p]), "boat_model_save": (C.c_bool, [P, C.c_char_p]),
}
for _n in "qkvo":
    for _k in ("weight", "bias", "grad_weight", "grad_bias"):
        _SIGS[f"boat_attention_get_{_k}_{_n}"] = (P, [P])

# symbols only libboat_amd.so has
_EXT_SIGS = {
    "boat_gelu": (P, [P]),
    "boat_tensor_to_device": (P, [P, C.c_int]),
    "boat_tensor_clone": (P, [P]),
    "boat_hip_synchronize": (None, []), "boat_hip_set_coherent_pointers": (None, [C.c_int]),
    "boat_hip_set_reference_exact": (None, [C.c_int]),
    "boat_hip_variable_ensure_grad": (P, [P]),
    "boat_hip_var_gelu": (P, [P]),
    "boat_hip_var_layernorm": (P, [P, P]),
    "boat_hip_var_reshape": (P, [P, C.POINTER(C.c_int64), C.c_size_t]),
    "boat_hip_layernorm_get_weight": (P, [P]), "boat_hip_layernorm_get_bias": (P, [P]),
    "boat_hip_layernorm_get_grad_weight": (P, [P]), "boat_hip_layernorm_get_grad_bias": (P, [P]),
    "boat_hip_rmsnorm_get_weight": (P, [P]), "boat_hip_rmsnorm_get_grad_weight": (P, [P]),
    "boat_hip_softmax_cross_entropy": (P, [P, P, C.POINTER(P)]),
    "boat_hip_mse_loss": (P, [P, P, C.POINTER(P)]),
    "boat_hip_layer_from_dense": (P, [P]), "boat_hip_layer_from_norm": (P, [P]),
    "boat_hip_layer_relu": (P, []), "boat_hip_layer_gelu": (P, []),
    "boat_hip_optimizer_add_dense": (None, [P, P]),
    "boat_hip_optimizer_add_conv": (None, [P, P]),
    "boat_hip_conv_reference_input_grad": (None, [C.c_int]),
    "boat_hip_conv_forward_matrix_cores": (None, [C.c_int]),
    "boat_hip_set_attention_score_cache_limit": (None, [C.c_size_t]),
    "boat_hip_optimizer_add_attention": (None, [P, P]),
    "boat_hip_optimizer_add_layernorm": (None, [P, P]),
    "boat_layernorm_update": (None, [P, C.c_float]),
    "boat_memory_get_stats": (MemoryStats, []),
}


class BoatAPI:
    """Loaded Boat library with typed entry points as attributes (api.boat_tensor_create(...))."""

    def __init__(self, path: str | Path | None = None):
        path = Path(path) if path is not None else LIB_PATH
        if not path.exists():
            raise FileNotFoundError(
                f"{path} not found: build it first (python -m boat_amd.build); there is no host fallback")
        self.path = path
        self.lib = C.CDLL(str(path), mode=C.RTLD_LOCAL)
        self.is_amd = hasattr(self.lib, "boat_hip_synchronize")
        for name, (res, args) in _SIGS.items():
            self._bind(name, res, args)
        if self.is_amd:
            for name, (res, args) in _EXT_SIGS.items():
                self._bind(name, res, args)

    def _bind(self, name, res, args):
        fn = getattr(self.lib, name)
        fn.restype = res
        fn.argtypes = args
        setattr(self, name, fn)

    # ---- numpy helpers ----
    def tensor(self, array, device: int = DEVICE_CPU):
        """New tensor holding a copy of `array` (written through boat_tensor_data, as Boat's tests do)."""
        a = np.ascontiguousarray(array)
        shape = (C.c_int64 * max(a.ndim, 1))(*a.shape)
        t = self.boat_tensor_create(shape, a.ndim, _DT[a.dtype], DEVICE_CPU)
        if not t:
            raise RuntimeError("boat_tensor_create failed")
        if a.size:
            C.memmove(self.boat_tensor_data(t), a.ctypes.data, a.nbytes)
        if device != DEVICE_CPU:
            d = self.boat_tensor_to_device(t, device)
            self.boat_tensor_free(t)
            return d
        return t

    def zeros(self, shape, dtype=DTYPE_FLOAT32, device: int = DEVICE_CPU):
        shape = tuple(shape)
        arr = (C.c_int64 * max(len(shape), 1))(*shape)
        t = self.boat_tensor_create(arr, len(shape), dtype, device)
        if not t:
            raise RuntimeError("boat_tensor_create failed")
        return t

    def shape(self, t):
        n = self.boat_tensor_ndim(t)
        s = self.boat_tensor_shape(t)
        return tuple(int(s[i]) for i in range(n))

    def numpy(self, t):
        """Copy of the tensor's current contents (downloads from the GPU when needed)."""
        if not t:
            raise ValueError("NULL tensor")
        if self.is_amd and self.boat_tensor_device(t) == DEVICE_HIP:
            h = self.boat_tensor_to_device(t, DEVICE_CPU)
            try:
                return self.numpy(h)
            finally:
                self.boat_tensor_free(h)
        shape = self.shape(t)
        dt = _NP[self.boat_tensor_dtype(t)]
        n = self.boat_tensor_nelements(t)
        out = np.empty(n, dtype=dt)
        if n:
            C.memmove(out.ctypes.data, self.boat_tensor_const_data(t), out.nbytes)
        return out.reshape(shape)

    def write(self, t, array):
        """Overwrite a tensor in place through its data pointer (how Boat's tests inject weights)."""
        a = np.ascontiguousarray(array, dtype=_NP[self.boat_tensor_dtype(t)])
        if a.size != self.boat_tensor_nelements(t):
            raise ValueError("size mismatch")
        if a.size:
            C.memmove(self.boat_tensor_data(t), a.ctypes.data, a.nbytes)

    def sync(self):
        if self.is_amd:
            self.boat_hip_synchronize()


_default: BoatAPI | None = None


def default_api() -> BoatAPI:
    """The GPU library, loaded once; raises if it has not been built."""
    global _default
    if _default is None:
        _default = BoatAPI()
    return _default
