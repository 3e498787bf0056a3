"""Entry points of Boat's API that the training scenarios do not reach: tensor-level arithmetic, variable helpers,
context objects, the error state, host memory helpers and the layers' own SGD hooks.  Each scenario of
boat_cases.py runs against the compiled reference (CPU) and against libboat_amd.so (GPU) and is held to the same
expectations, which are closed forms: one IEEE operation per element, or literal values read off the reference's
sources (src/core/error.c:21-62, src/autodiff.c:208-298,606-649, src/layers/dense.c:297-329, conv.c:539-562).
"""
import numpy as np
import pytest

import boat_cases as bc

F = np.float32


def inputs():
    rng = np.random.default_rng(77)
    a = rng.standard_normal((5, 8)).astype(F)
    b = (rng.standard_normal((5, 8)) + 3).astype(F)
    a[0, :3] = [0.0, -0.0, 1e-30]
    return a, b, b[1].copy(), b[:, 2:3].copy(), a[2].copy(), b[3].copy()


def check_tensor_ops(out, stubs_return_null):
    a, b, row, col, v1, v2 = inputs()
    np_op = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}
    np.seterr(divide="ignore")                                                # a holds zeros on purpose
    for name, fn in np_op.items():
        assert np.array_equal(out[name], fn(a, b)), name
        assert np.array_equal(out[name + "_row"], fn(a, row)), name           # [5,8] op [8]
        assert np.array_equal(out[name + "_col"], fn(col, a)), name           # [5,1] op [5,8]
        assert np.array_equal(out[name + "_scalar"], fn(a, F(1.75))), name
        assert np.array_equal(out[name + "_"], fn(a, b)), name                # in place
        assert out[name + "__mismatch_unchanged"], name
    acc = F(0)
    for x, y in zip(v1, v2):                                                  # linear.c:206-213: sequential fp32
        acc = F(acc + F(x * y))
    assert out["dot"].shape == (1,) and abs(out["dot"][0] - acc) <= 1e-5 * abs(acc)
    assert out["dot_of_matrices_is_null"]
    assert np.array_equal(out["relu"], np.maximum(a, 0) * (a > 0))
    a64 = a.astype(np.float64)
    if stubs_return_null:                                                     # activation.c:286-296
        assert out["sigmoid"] is None and out["tanh"] is None
    else:
        assert np.max(np.abs(out["sigmoid"] - 1 / (1 + np.exp(-a64)))) <= 1e-6
        assert np.max(np.abs(out["tanh"] - np.tanh(a64))) <= 1e-6
    e = np.exp(a64 - a64.max(1, keepdims=True))
    assert np.max(np.abs(out["softmax"] - e / e.sum(1, keepdims=True))) <= 1e-6
    assert np.max(np.abs(out["log_softmax"] - np.log(e / e.sum(1, keepdims=True)))) <= 1e-5
    assert out["can_broadcast"] == [True, True, False]                      # [5,8] with [8], [5,1] with [5,8], but not [5,8] with [5]
    assert out["broadcast_to_same_count"].shape == (1, 8, 5) and np.array_equal(out["broadcast_to_same_count"].reshape(-1), a.reshape(-1))
    assert out["broadcast_to_other_count_is_null"]
    assert out["is_contiguous"] is True
    assert out["dtype_names"] == ["float64", "float32", "int64", "int32", "bool", "unknown"]
    assert out["dtype_sizes"] == [8, 4, 8, 4]


def check_variable_helpers(out):
    assert np.array_equal(out["with_shape_data"], np.zeros((2, 3), F))
    assert (out["requires_grad_before"], out["requires_grad_after"]) == (False, True)
    assert np.array_equal(out["grad_after_backward"], np.ones((2, 3), F))
    assert out["reset_leaf"] is True and out["grad_dropped_by_reset"] is True and out["reset_null"] is False
    want = np.arange(6, dtype=F).reshape(2, 3)
    assert np.array_equal(out["data_after_reset"], want) and np.array_equal(out["data_survives_callers_unref"], want)


CONTEXT_AND_ERRORS = {
    "enabled_at_creation": True, "enabled_after_disable": False, "enabled_after_enable": True, "enabled_of_null": False,
    "current_is_the_one_set": True,
    "error_after_clear": (0, "", False), "error_after_set": (3, "the operation is not valid here", True),
    "long_message_length": 255, "error_with_null_message": (2, ""),
    "error_strings": ["Success", "Invalid argument", "Out of memory", "Invalid operation", "Device error", "File I/O error",
                      "Format error", "Not implemented", "Unknown error", "Invalid error code", "Invalid error code"],
    "memory_set_then_copy": True,
}


def sgd_inputs():
    rng = np.random.default_rng(78)
    return (rng.standard_normal((6, 5)).astype(F), rng.standard_normal((5, 3)).astype(F), rng.standard_normal(3).astype(F),
            rng.standard_normal((6, 3)).astype(F), 0.05)


def check_sgd(api):
    x, w, b, dy, lr = sgd_inputs()
    (gw, gb), w1, b1, gw_after, w2 = bc.sgd_hooks(api, x, w, b, dy, lr)
    assert np.max(np.abs(gw - x.T.astype(np.float64) @ dy)) <= 1e-5 and np.max(np.abs(gb - dy.sum(0, dtype=np.float64))) <= 1e-5
    assert np.array_equal(w1, w - F(lr) * gw) and np.array_equal(b1, b - F(lr) * gb)     # one multiply, one subtract
    assert not gw_after.any()                                                             # cleared by the update
    assert np.array_equal(w2, w1 - F(lr) * gw)                                            # so the second step is the same size
    rng = np.random.default_rng(79)
    xc, wc = rng.standard_normal((2, 2, 6, 6)).astype(F), rng.standard_normal((3, 2, 3, 3)).astype(F)
    bcv, dyc = rng.standard_normal(3).astype(F), rng.standard_normal((2, 3, 6, 6)).astype(F)
    w1, b1, gw, gb, gw_after = bc.conv_sgd_hook(api, xc, wc, bcv, dyc, lr)
    assert np.array_equal(w1, wc - F(lr) * gw) and np.array_equal(b1, bcv - F(lr) * gb)
    assert np.array_equal(gw_after, gw) and gw.any()                                      # conv.c:561: gradients are kept


def test_reference_tensor_ops(ref):
    check_tensor_ops(bc.tensor_ops(ref, *inputs()), stubs_return_null=True)


def test_reference_variable_helpers_contexts_errors(ref):
    check_variable_helpers(bc.variable_helpers(ref))
    assert bc.context_and_errors(ref) == CONTEXT_AND_ERRORS


def test_reference_sgd_hooks(ref):
    check_sgd(ref)


@pytest.mark.gpu
def test_gpu_tensor_ops(boat):
    check_tensor_ops(bc.tensor_ops(boat, *inputs()), stubs_return_null=False)


@pytest.mark.gpu
def test_gpu_variable_helpers_contexts_errors(boat):
    check_variable_helpers(bc.variable_helpers(boat))
    assert bc.context_and_errors(boat) == CONTEXT_AND_ERRORS


@pytest.mark.gpu
def test_gpu_sgd_hooks(boat):
    check_sgd(boat)


@pytest.mark.gpu
def test_gpu_disabled_context_records_nothing(boat):
    """The reference keeps the flag without reading it; here an operation recorded while the current context has
    gradients off leaves no tape entry, so its result is a leaf."""
    ctx = boat.boat_autodiff_context_create()
    before = boat.boat_autodiff_get_current_context()
    boat.boat_autodiff_set_current_context(ctx)
    a, b = bc._var(boat, [1, 2, 3], True), bc._var(boat, [4, 5, 6], True)
    boat.boat_autodiff_context_disable_grad(ctx)
    off = boat.boat_var_mul(a, b)
    boat.boat_variable_backward_full(off)
    assert not boat.boat_variable_grad(a) and not boat.boat_variable_grad(b)
    assert boat.numpy(boat.boat_variable_data(off)).tolist() == [4, 10, 18]
    boat.boat_autodiff_context_enable_grad(ctx)
    on = boat.boat_var_mul(a, b)
    boat.boat_variable_backward_full(on)
    assert boat.numpy(boat.boat_variable_grad(a)).tolist() == [4, 5, 6]
    boat.boat_autodiff_set_current_context(before)
    for v in (on, off, a, b):
        boat.boat_variable_free(v)
    boat.boat_autodiff_context_free(ctx)


@pytest.mark.gpu
def test_gpu_layer_norm_grad_and_norm_layer_adapters(boat, oracle):
    """boat_layer_norm_grad (a stub in the reference, src/layers/norm.c:450-463) and the boat_norm_layer_* adapters
    (:523-550) against the float64 closed form of the oracle."""
    import ctypes as C
    rng = np.random.default_rng(80)
    x, dy = rng.standard_normal((7, 48)).astype(F), rng.standard_normal((7, 48)).astype(F)
    tx, tdy = boat.tensor(x), boat.tensor(dy)
    shape = (C.c_int64 * 1)(48)
    tdx = boat.boat_layer_norm_grad(tdy, tx, None, shape, 1, 1e-5)
    assert tdx
    _y, mean, rstd = oracle.layernorm_forward(x, None, None, 1e-5)
    want_dx, _, _ = oracle.layernorm_backward_f64(x, None, dy, mean, rstd)
    assert np.max(np.abs(boat.numpy(tdx) - want_dx)) <= 1e-4 * np.abs(want_dx).max()
    assert not boat.boat_layer_norm_grad(tdy, tx, None, shape, 2, 1e-5)       # only the last axis is supported
    layer = boat.boat_norm_layer_create(48, 1e-5, True)
    ty = boat.boat_norm_layer_forward(layer, tx)
    y = boat.numpy(ty)
    assert np.max(np.abs(y.mean(1))) <= 1e-6 and np.max(np.abs(y.var(1) - 1)) <= 1e-3
    tdx2 = boat.boat_norm_layer_backward(layer, tdy)
    assert np.array_equal(boat.numpy(tdx2), boat.numpy(tdx))                  # gamma = 1, beta = 0 at creation
    boat.boat_norm_layer_update(layer, 0.1)
    for t in (tdx2, ty, tdx, tdy, tx):
        boat.boat_tensor_unref(t)
    boat.boat_norm_layer_free(layer)


@pytest.mark.gpu
def test_gpu_small_hooks(boat):
    """What is left: hooks that do nothing in the reference either (relu.c:74-78, softmax.c:60-64, pool.c:220-224,
    flatten.c:91-95), boat_softmax_layer_forward (softmax.c:34-41), the reference count of a tensor
    (tensor.c:164-191), memory statistics, and boat_layernorm_update (a stub in the reference, norm.c:411-415; here
    the same SGD step as the dense layer's)."""
    rng = np.random.default_rng(81)
    x = rng.standard_normal((4, 6)).astype(F)
    tx = boat.tensor(x)
    sm = boat.boat_softmax_layer_create(-1)
    ty = boat.boat_softmax_layer_forward(sm, tx)
    tz = boat.boat_softmax(tx, -1)
    assert np.array_equal(boat.numpy(ty), boat.numpy(tz))
    boat.boat_softmax_layer_update(sm, 0.1)
    relu, pool, flat = boat.boat_relu_layer_create(), boat.boat_pool_layer_create(2, 2, 0), boat.boat_flatten_layer_create()
    boat.boat_relu_layer_update(relu, 0.1)
    boat.boat_pool_layer_update(pool, 0.1)
    boat.boat_flatten_layer_update(flat, 0.1)
    assert np.array_equal(boat.numpy(tx), x)
    boat.boat_tensor_ref(tx)                      # two owners
    boat.boat_tensor_free(tx)                     # free is unref: one owner left, contents intact
    assert np.array_equal(boat.numpy(tx), x)
    for t in (tz, ty, tx):
        boat.boat_tensor_unref(t)
    boat.boat_softmax_layer_free(sm)
    boat.boat_relu_layer_free(relu)
    boat.boat_pool_layer_free(pool)
    boat.boat_flatten_layer_free(flat)

    boat.boat_memory_reset_stats()
    s0 = boat.boat_memory_get_stats()
    assert (s0.allocated_bytes, s0.allocated_blocks, s0.freed_bytes, s0.freed_blocks, s0.peak_allocated_bytes) == (0, 0, 0, 0, 0)
    p = boat.boat_memory_allocate_device(4096, 0, b"test", 1)
    assert p and boat.boat_memory_get_stats().allocated_blocks == 1
    boat.boat_memory_free_device(p, 0)
    s1 = boat.boat_memory_get_stats()               # memory.c:28-43: allocated_bytes counts what is live
    assert (s1.allocated_bytes, s1.allocated_blocks, s1.freed_blocks) == (0, 1, 1) and s1.freed_bytes == s1.peak_allocated_bytes >= 4096
    assert not boat.boat_memory_allocate(0, 0, b"test", 2)         # memory.c:48-50

    from boat_amd.capi import LayerNormConfig
    import ctypes as C
    cfg = LayerNormConfig(6, 1e-5, True, True)
    norm = boat.boat_layernorm_create(C.byref(cfg))
    tx, tdy = boat.tensor(x), boat.tensor(rng.standard_normal((4, 6)).astype(F))
    ty = boat.boat_layernorm_forward(norm, tx)
    tdx = boat.boat_layernorm_backward(norm, tdy)
    gw = boat.numpy(boat.boat_hip_layernorm_get_grad_weight(norm))
    assert gw.any()
    boat.boat_layernorm_update(norm, 0.5)
    assert np.array_equal(boat.numpy(boat.boat_hip_layernorm_get_weight(norm)), np.ones(6, F) - F(0.5) * gw)
    assert not boat.numpy(boat.boat_hip_layernorm_get_grad_weight(norm)).any()
    for t in (tdx, ty, tdy, tx):
        boat.boat_tensor_unref(t)
    boat.boat_layernorm_free(norm)


TENSOR_FACTS = {   # (ndim, nelements, nbytes, dtype, device, is_contiguous) or None for a refused call
    "null_shape_with_dims": None,
    "f32_2x3": (2, 6, 24, 1, 0, True), "f64_2x3": (2, 6, 48, 0, 0, True), "i32_5": (1, 5, 20, 6, 0, True),
    "i64_5": (1, 5, 40, 5, 0, True), "f4_5": (1, 5, 3, 4, 0, True), "bits1_9": (1, 9, 2, 9, 0, True),
    "eight_dims": (8, 16, 64, 1, 0, True),
    "view": (2, 12, 48, 1, 0, False),                           # tensor.c:288: a reshaped view reports non-contiguous
    "view_shape": (2, 6), "view_shares_data": True,
    "view_after_parent_unref": [[0.0, 1.0, 2.0, 3.0, 4.0, 5.0], [6.0, 7.0, 8.0, 9.0, 10.0, 11.0]],
    "reshape_wrong_count": None, "reshape_null_shape": None,
    "like": (2, 12, 48, 1, 0, True), "like_is_zero": True,
    "add_mixed_dtypes": None, "add_3x4_and_3": None, "add_3x4_and_4": (2, 12, 48, 1, 0, True),
    "matmul_inner_mismatch": None, "matmul_3x4_4": None,
    "transpose_bad_dim": None, "transpose_same_dim": (2, 12, 48, 1, 0, True), "transpose_negative": None,
    "sum_all": (1, 1, 4, 1, 0, True), "softmax_vector": (1, 4, 16, 1, 0, True),
    "relu_f64": (2, 12, 96, 0, 0, True), "mul_scalar_f64": (2, 12, 96, 0, 0, True),
}


def test_reference_tensor_facts(ref):
    assert bc.tensor_facts(ref) == TENSOR_FACTS


@pytest.mark.gpu
def test_gpu_tensor_facts(boat):
    got = bc.tensor_facts(boat)
    scalar = got.pop("scalar_null_shape")          # the reference aborts on this call; here a one-element tensor or a refusal
    assert scalar is None or scalar[:2] == (0, 1)
    diff = {k: (got.get(k), v) for k, v in TENSOR_FACTS.items() if k in got and got[k] != v}
    assert not diff and set(got) == set(TENSOR_FACTS), diff


TRANSPOSE_CASES = [((3, 4), 0, 1), ((3, 4), 1, 0), ((2, 3, 4), 0, 1), ((2, 3, 4), 0, 2), ((2, 3, 4), 1, 2),
                   ((2, 3, 4, 5), 1, 2), ((2, 3, 4, 5), 0, 3), ((2, 3, 4, 5), 2, 3), ((2, 1, 4, 3, 2), 1, 4)]


def check_transposes(api, cases):
    rng = np.random.default_rng(82)
    for shape, d0, d1 in cases:
        x = rng.standard_normal(shape).astype(F)
        got = bc.transpose(api, x, d0, d1)
        assert got.shape == np.swapaxes(x, d0, d1).shape and np.array_equal(got, np.swapaxes(x, d0, d1)), (shape, d0, d1)


def test_reference_transposes_any_two_dimensions(ref):
    check_transposes(ref, TRANSPOSE_CASES)


@pytest.mark.gpu
def test_gpu_transposes_any_two_dimensions(boat):
    check_transposes(boat, TRANSPOSE_CASES + [((70, 33, 65), 0, 2), ((5, 130, 3, 70), 1, 3), ((4, 300, 260), 1, 2)])


LAYER_FACTS = {
    "matmul_2d": (3, 5), "matmul_3d": (2, 3, 5), "matmul_4d": (2, 2, 3, 5), "matmul_batch_mismatch": None,
    "matmul_3d_with_2d": None, "matmul_with_vector": None, "matmul_3d_value_ok": True,
    "dense_no_bias_has_bias": False, "dense_no_bias_has_grad_bias": False, "dense_weight_shape": (4, 3),
    "dense_grad_weight_zero_at_creation": True, "dense_forward_2d": (2, 3), "dense_backward_no_bias": (2, 4),
    "dense_forward_3d": None, "dense_forward_wrong_features": None, "dense_set_bias_on_no_bias_layer": False,
    "dense_set_weight_wrong_shape_kept": (4, 3),
    "adam_bad_arguments_refused": [True, True, False, False],           # adam.c:45-53 checks lr and the betas, not epsilon
    "adam_lr": 0.1, "adam_lr_after_set": 0.25, "adam_null_grad_ignored": True, "adam_zero_grad_clears": True,
    "adam_zero_grad_step_keeps_params": True,
    "rmsprop_bad_arguments_refused": [True, True, True], "rmsprop_lr": 0.1, "rmsprop_lr_after_set": 0.25,
    "rmsprop_null_grad_ignored": True, "rmsprop_zero_grad_clears": True, "rmsprop_zero_grad_step_keeps_params": True,
    "adagrad_bad_arguments_refused": [True, True], "adagrad_lr": 0.1, "adagrad_lr_after_set": 0.25,
    "adagrad_null_grad_ignored": True, "adagrad_zero_grad_clears": True, "adagrad_zero_grad_step_keeps_params": True,
    "attention_heads_do_not_divide": True, "attention_zero_heads": True, "attention_null_config": True,
    "attention_no_bias_has_bias_q": False, "attention_weight_shape": (8, 8), "attention_grad_before_backward": False,
    "attention_forward": (2, 3, 8),
    "layernorm_plain_forward": (4, 6), "layernorm_wrong_width": None, "layernorm_zero_width": True,
    "conv_forward": (2, 3, 5, 5), "conv_wrong_channels": None, "conv_3d_input": None, "conv_weight_shape": (3, 2, 3, 3),
    "conv_bias_shape": (3,), "pool_forward": (2, 2, 2, 2), "pool_3d_input": None, "flatten_forward": (2, 50),
}


def test_reference_layer_facts(ref):
    with bc.scratch_cwd():
        assert bc.layer_facts(ref) == LAYER_FACTS


@pytest.mark.gpu
def test_gpu_layer_facts(boat):
    got = bc.layer_facts(boat)
    want = LAYER_FACTS
    diff = {k: (got.get(k), v) for k, v in want.items() if got.get(k) != v}
    assert not diff and set(got) == set(want), diff


AUTODIFF_FACTS = {
    "add_false_true": True, "add_false_false": False, "mul_true_false": True, "matmul_false_true": True,
    "relu_false": False, "relu_true": True, "add_shape_mismatch": None, "matmul_shape": (3, 2),
    "matmul_inner_mismatch": None, "sum_all_shape": (1,),
    "softmax_axis_is_ignored": True, "softmax_rows_sum_to_one": True,        # autodiff.c:530-535: always the last axis
    "flatten_shape": (2, 60),
    "dense_of_input_without_grad": False, "dense_grads_untouched_without_input_grad": True,   # autodiff.c:2287
    "dense_of_input_with_grad": True, "dense_grads_filled_with_input_grad": True, "input_grad_shape": (3, 4),
}


def test_reference_autodiff_facts(ref):
    assert bc.autodiff_facts(ref) == AUTODIFF_FACTS


@pytest.mark.gpu
def test_gpu_autodiff_facts(boat):
    got = bc.autodiff_facts(boat)
    boat.boat_autodiff_clear_computation_graph()
    diff = {k: (got.get(k), v) for k, v in AUTODIFF_FACTS.items() if got.get(k) != v}
    assert not diff and set(got) == set(AUTODIFF_FACTS), diff


def model_case():
    rng = np.random.default_rng(83)
    x = rng.standard_normal((5, 6)).astype(F)
    ws = [rng.standard_normal((6, 4)).astype(F), rng.standard_normal((4, 3)).astype(F)]
    bs = [rng.standard_normal(4).astype(F), rng.standard_normal(3).astype(F)]
    return x, ws, bs, rng.standard_normal((5, 3)).astype(F)


def test_reference_model_over_callers_vtables(ref, oracle):
    x, ws, bs, dy = model_case()
    rec = bc.model_over_callers_vtables(ref, x, ws, bs, dy=dy, lr=0.1)
    assert rec["count"] == 2 and rec["freed"] == 2
    assert np.array_equal(rec["y"], oracle.dense_forward(oracle.dense_forward(x, ws[0], bs[0]), ws[1], bs[1]))
    assert rec["dx"] is None and not any(g.any() for g in rec["gw"])          # model.c:354-359: backward is a stub
    assert all(np.array_equal(a, b) for a, b in zip(rec["w_after"], ws))       # model.c:361-365: so is update


@pytest.mark.gpu
def test_gpu_model_over_callers_vtables(boat, oracle):
    """The same caller-written tables on this library: forward as the reference, and the two stubs do their work
    (layers[n-1..0] through ops->backward, then ops->update)."""
    x, ws, bs, dy = model_case()
    rec = bc.model_over_callers_vtables(boat, x, ws, bs, dy=dy, lr=0.1)
    assert rec["count"] == 2 and rec["freed"] == 2
    h = oracle.dense_forward(x, ws[0], bs[0])
    assert np.max(np.abs(rec["y"] - oracle.dense_forward(h, ws[1], bs[1]))) <= 1e-5
    dh, gw2, _ = oracle.dense_backward(h, ws[1], dy)
    dx, gw1, _ = oracle.dense_backward(x, ws[0], dh)
    assert np.max(np.abs(rec["dx"] - dx)) <= 1e-5 and np.max(np.abs(rec["gw"][0] - gw1)) <= 1e-5
    assert np.max(np.abs(rec["gw"][1] - gw2)) <= 1e-5
    assert all(np.array_equal(a, w - F(0.1) * g) for a, w, g in zip(rec["w_after"], ws, rec["gw"]))


@pytest.mark.gpu
def test_gpu_kept_pointers_in_the_default_configuration(boat):
    """A caller that keeps the float* of boat_tensor_data() across calls, as the reference's own tests do
    (tests/unit/test_optimizer_adam.c:96-108 reads a parameter through it after the step,
    test_attention_gradient_check.c:22-41 writes a weight through it before a forward).  Nothing is switched on here:
    this is how the library behaves by default.  With the mode switched off the pointer is only good until the next
    call that takes the tensor."""
    import ctypes as C
    p, g = boat.tensor(np.array([5.0], F)), boat.tensor(np.array([2.0], F))
    pp = C.cast(boat.boat_tensor_data(p), C.POINTER(C.c_float))
    gp = C.cast(boat.boat_tensor_data(g), C.POINTER(C.c_float))
    opt = boat.boat_adam_optimizer_create(0.01, 0.9, 0.999, 1e-8)
    boat.boat_optimizer_add_parameter(opt, p, g)
    boat.boat_optimizer_step(opt)
    assert abs(pp[0] - 4.99) < 1e-6                         # read through the pointer taken before the step
    gp[0] = -2.0                                            # written through the pointer taken before the step
    boat.boat_optimizer_step(opt)
    assert pp[0] > 4.99                                     # the step saw the new gradient
    boat.boat_optimizer_zero_grad(opt)
    assert gp[0] == 0.0
    # a weight written through a kept pointer, forward, backward, update, parameter read through the kept pointer
    layer = boat.boat_dense_layer_create(3, 2, True)
    wp = C.cast(boat.boat_tensor_data(boat.boat_dense_layer_get_weight(layer)), C.POINTER(C.c_float))
    for i in range(6):
        wp[i] = 1.0
    x = boat.tensor(np.ones((1, 3), F))
    y1 = boat.boat_dense_layer_forward(layer, x)
    wp[0] = 11.0
    y2 = boat.boat_dense_layer_forward(layer, x)
    assert boat.numpy(y1).tolist() == [[3.0, 3.0]] and boat.numpy(y2).tolist() == [[13.0, 3.0]]
    dy = boat.tensor(np.ones((1, 2), F))
    dx = boat.boat_dense_layer_backward(layer, dy)
    boat.boat_dense_layer_update(layer, 0.5)                # w -= 0.5 * x^T.dy = 0.5 everywhere
    assert [wp[i] for i in range(6)] == [10.5, 0.5, 0.5, 0.5, 0.5, 0.5]
    for t in (y1, y2, dx, dy, x, p, g):
        boat.boat_tensor_unref(t)
    boat.boat_dense_layer_free(layer)
    boat.boat_optimizer_free(opt)
    # switched off: a tensor created now is not tracked, results stay on the device until asked for
    boat.boat_hip_set_coherent_pointers(0)
    try:
        p, g = boat.tensor(np.array([5.0], F)), boat.tensor(np.array([2.0], F))
        pp = C.cast(boat.boat_tensor_data(p), C.POINTER(C.c_float))
        opt = boat.boat_adam_optimizer_create(0.01, 0.9, 0.999, 1e-8)
        boat.boat_optimizer_add_parameter(opt, p, g)
        boat.boat_optimizer_step(opt)
        assert pp[0] == 5.0                                 # the old pointer shows the old value ...
        assert abs(boat.numpy(p)[0] - 4.99) < 1e-6          # ... a fresh one the new
        boat.boat_optimizer_free(opt)
        boat.boat_tensor_unref(p)
        boat.boat_tensor_unref(g)
    finally:
        boat.boat_hip_set_coherent_pointers(1)
    boat.boat_tensor_unref(g)


@pytest.mark.gpu
def test_gpu_kept_pointer_batches_are_staged(boat):
    """The input batch lives behind a kept pointer and is overwritten the moment a forward call returns, while the
    device may not have run that call yet: each forward must have used the values the mirror held when it was called
    (uploads are staged through a page-locked copy before the call returns), a mirror that was not touched is not
    uploaded again, and results written by the device are in the mirror when the writing call returns."""
    import ctypes as C
    rng = np.random.default_rng(31)
    rows, d_in, d_out = 512, 784, 128
    layer = boat.boat_dense_layer_create(d_in, d_out, True)
    w = rng.standard_normal((d_in, d_out)).astype(F)
    boat.write(boat.boat_dense_layer_get_weight(layer), w)
    x = boat.tensor(np.zeros((rows, d_in), F))
    xp = np.ctypeslib.as_array(C.cast(boat.boat_tensor_data(x), C.POINTER(C.c_float)), shape=(rows, d_in))
    batches = [rng.standard_normal((rows, d_in)).astype(F) for _ in range(6)]
    outs = []
    for b in batches:
        xp[:] = b                                          # through the pointer taken once
        outs.append(boat.boat_dense_layer_forward(layer, x))
        xp[:] = -7.0                                       # scribbled over before the device has to have run
    outs.append(boat.boat_dense_layer_forward(layer, x))   # the scribble itself
    outs.append(boat.boat_dense_layer_forward(layer, x))   # an untouched mirror
    for b, t in zip(batches, outs):
        want = b.astype(np.float64) @ w.astype(np.float64)
        assert np.linalg.norm(boat.numpy(t) - want) <= 1e-5 * np.linalg.norm(want)
    want = np.full((rows, d_in), -7.0) @ w.astype(np.float64)
    assert np.linalg.norm(boat.numpy(outs[-2]) - want) <= 1e-5 * np.linalg.norm(want)
    assert np.array_equal(boat.numpy(outs[-1]), boat.numpy(outs[-2]))
    # a device write into a tensor behind a kept pointer: in the mirror when boat_add_ returns, and the next read of
    # the mirror's owner sees a host write made after that
    a = boat.tensor(np.ones((rows, d_in), F))
    ap = np.ctypeslib.as_array(C.cast(boat.boat_tensor_data(a), C.POINTER(C.c_float)), shape=(rows, d_in))
    boat.boat_add_(a, x)                                   # a += x on the device (x holds -7)
    assert np.all(ap == -6.0)
    ap[0, 0] = 100.0
    boat.boat_add_(a, x)
    assert ap[0, 0] == 93.0 and np.all(ap[1:] == -13.0)
    for t in outs + [a, x]:
        boat.boat_tensor_unref(t)
    boat.boat_dense_layer_free(layer)


SLICE_FACTS = {
    "shape": (3, 4), "values": [[8.0, 9.0, 10.0, 11.0], [12.0, 13.0, 14.0, 15.0], [16.0, 17.0, 18.0, 19.0]],
    "is_contiguous": False, "pointer_offset": 32, "nbytes": 48,
    "step_two_refused": True, "step_zero_refused": True, "start_past_end_refused": True, "reversed_range_refused": True,
    "empty_range_refused": True, "slice_of_a_view_refused": True,
    "parent_after_add_on_slice": [[0.0, 1.0, 2.0, 3.0], [4.0, 5.0, 6.0, 7.0], [9.0, 10.0, 11.0, 12.0], [13.0, 14.0, 15.0, 16.0],
                                  [17.0, 18.0, 19.0, 20.0], [20.0, 21.0, 22.0, 23.0]],
    "matmul_on_slice": [[8.0, 9.0], [14.0, 15.0], [20.0, 21.0]],
    "values_after_parent_unref": [[9.0, 10.0, 11.0, 12.0], [13.0, 14.0, 15.0, 16.0], [17.0, 18.0, 19.0, 20.0]],
}


def test_reference_slice_facts(ref):
    assert bc.slice_facts(ref) == SLICE_FACTS


@pytest.mark.gpu
def test_gpu_slice_facts(boat):
    got = bc.slice_facts(boat)
    diff = {k: (got.get(k), v) for k, v in SLICE_FACTS.items() if got.get(k) != v}
    assert not diff and set(got) == set(SLICE_FACTS), diff


@pytest.mark.gpu
def test_gpu_slices_feed_the_layers(boat, oracle):
    """Batches cut from one sample tensor with boat_tensor_slice go through a dense layer forward and backward
    (the loop of examples/mnist/mnist_autodiff.c:2380-2440), including a batch that starts off a 16-byte boundary."""
    import ctypes as C
    rng = np.random.default_rng(84)
    data = rng.standard_normal((10, 7)).astype(F)
    w, b = rng.standard_normal((7, 5)).astype(F), rng.standard_normal(5).astype(F)
    samples = boat.tensor(data)
    layer = bc._make_dense(boat, w, b)
    for lo, hi in ((0, 4), (3, 8), (9, 10)):
        batch = boat.boat_tensor_slice(samples, (C.c_size_t * 2)(lo, 0), (C.c_size_t * 2)(hi, 7), None)
        ty = boat.boat_dense_layer_forward(layer, batch)
        assert np.max(np.abs(boat.numpy(ty) - oracle.dense_forward(data[lo:hi], w, b))) <= 1e-5
        tdy = boat.tensor(np.ones((hi - lo, 5), F))
        tdx = boat.boat_dense_layer_backward(layer, tdy)
        want_dx, _, _ = oracle.dense_backward(data[lo:hi], w, np.ones((hi - lo, 5), F))
        assert np.max(np.abs(boat.numpy(tdx) - want_dx)) <= 1e-5
        for t in (tdx, tdy, ty, batch):
            boat.boat_tensor_unref(t)
    assert np.array_equal(boat.numpy(samples), data)
    boat.boat_tensor_unref(samples)
    boat.boat_dense_layer_free(layer)


HOST_ALLOCATOR_FACTS = {
    "pool_three_taken": (3, 1), "pool_total_memory": 4192, "pool_refuses_larger_than_a_block": True,
    "pool_refuses_when_empty": True, "pool_after_one_back": (3, 1), "pool_after_clear": (0, 4), "pool_of_nothing_refused": True,
    "arena_rounds_to_eight": (16, 24), "arena_refuses_zero": True, "arena_grows": (9024, 16384), "arena_after_reset": (0, 16384),
    "reallocate_keeps_contents": b"0123456789abcdef", "reallocate_to_zero_frees": True, "reallocate_of_null_allocates": True,
    "context_carries_the_graph": True, "fresh_graph_is_empty": (0, 0),
    "node_type_names": ["VARIABLE", "OPERATION", "CONSTANT", "PLACEHOLDER", "OUTPUT", "UNKNOWN"],
}


def test_reference_host_allocator_facts(ref):
    assert bc.host_allocator_facts(ref) == HOST_ALLOCATOR_FACTS


@pytest.mark.gpu
def test_gpu_host_allocator_facts(boat):
    assert bc.host_allocator_facts(boat) == HOST_ALLOCATOR_FACTS


LOSS_AND_SCHEDULER_FACTS = {
    "mse_created": True, "mse_finite_and_positive": True, "mse_shape_mismatch": 0.0, "mse_null_prediction": 0.0,
    "ce_created": True, "ce_finite_and_positive": True, "ce_shape_mismatch": 0.0, "ce_null_prediction": 0.0,
    "huber_created": True, "huber_finite_and_positive": True, "huber_shape_mismatch": 0.0, "huber_null_prediction": 0.0,
    "loss_compute_on_null_loss": 0.0,
    "step_bad": [True, True, True, False],          # a decay factor above 1 is accepted (step_lr.c checks gamma <= 0 only)
    "cosine_bad": [True, True, True, True], "null_scheduler_lr": (0.0, 0.0), "update_optimizer_sets_last_lr": 0.1,
}


def test_reference_loss_and_scheduler_facts(ref):
    assert bc.loss_and_scheduler_facts(ref) == LOSS_AND_SCHEDULER_FACTS


@pytest.mark.gpu
def test_gpu_loss_and_scheduler_facts(boat):
    got = bc.loss_and_scheduler_facts(boat)
    diff = {k: (got.get(k), v) for k, v in LOSS_AND_SCHEDULER_FACTS.items() if got.get(k) != v}
    assert not diff and set(got) == set(LOSS_AND_SCHEDULER_FACTS), diff


ATTENTION_FACTS = {
    "backward_before_forward": False, "mask_is_ignored": True, "dropout_is_ignored": True,       # attention.c:1022-1025,1061-1062
    "forward_null_query": True, "forward_wrong_hidden": True, "forward_2d_input": None,
    "backward_ok": True, "backward_grad_shapes": ((2, 3, 8), (2, 3, 8), (2, 3, 8)), "grads_exist_after_backward": True,
    "backward_wrong_shape": False,
}


def test_reference_attention_facts(ref):
    assert bc.attention_facts(ref) == ATTENTION_FACTS


@pytest.mark.gpu
def test_gpu_attention_facts(boat):
    got = bc.attention_facts(boat)
    diff = {k: (got.get(k), v) for k, v in ATTENTION_FACTS.items() if got.get(k) != v}
    assert not diff and set(got) == set(ATTENTION_FACTS), diff


CONV_POOL_FACTS = {
    "conv_backward_before_forward": None, "conv_forward_no_padding": (2, 3, 4, 4), "conv_backward_wrong_shape": None,
    "conv_input_smaller_than_kernel": None, "conv_null_input": None, "conv_stride_two_pad_one": (2, 3, 3, 3),
    "pool_backward_before_forward": None, "pool_forward_odd_side": (1, 1, 2, 2), "pool_backward_wrong_shape": None,
    "pool_backward": (1, 1, 5, 5), "flatten_backward_before_forward": None, "flatten_2d_input": (3, 4),
    "flatten_4d_input": (2, 72), "flatten_backward": (2, 2, 6, 6),
}


def test_reference_conv_pool_facts(ref):
    assert bc.conv_pool_facts(ref) == CONV_POOL_FACTS


@pytest.mark.gpu
def test_gpu_conv_pool_facts(boat):
    got = bc.conv_pool_facts(boat)
    diff = {k: (got.get(k), v) for k, v in CONV_POOL_FACTS.items() if got.get(k) != v}
    assert not diff and set(got) == set(CONV_POOL_FACTS), diff
