/* ops.c - eager tensor operations used by the backward pass, dispatched to HIP kernels.
 *
 * Same contracts as the reference's src/ops/arithmetic.c (broadcasting binary ops :78-285,
 * in-place ops that silently return on a size mismatch :362-419, scalar ops that narrow the
 * double to float first :425-484, full-reduction boat_sum :611-691), src/ops/linear.c
 * (boat_matmul 2-4-D with equal batch dims :12-170, materialising boat_transpose :238-406)
 * and src/ops/activation.c (:31-283).  Mixed-device operands are refused (arithmetic.c:136-143).
 */
#include "boat_internal.h"

#include <stdlib.h>
#include <string.h>

static bool same_device(const boat_tensor_t* a, const boat_tensor_t* b) { return a->device == b->device; }

/* numpy broadcasting of right-aligned shapes (arithmetic.c:78-104) */
static bool broadcast_shape(const boat_tensor_t* a, const boat_tensor_t* b, int64_t* out, size_t* out_ndim) {
    size_t nd = a->ndim > b->ndim ? a->ndim : b->ndim;
    for (size_t i = 0; i < nd; i++) {
        int64_t da = i < nd - a->ndim ? 1 : a->shape[i - (nd - a->ndim)];
        int64_t db = i < nd - b->ndim ? 1 : b->shape[i - (nd - b->ndim)];
        if (da != db && da != 1 && db != 1) return false;
        out[i] = da > db ? da : db;
        if (da == 0 || db == 0) out[i] = 0;
    }
    *out_ndim = nd;
    return true;
}

/* element types the reference's arithmetic switches on (arithmetic.c:197-282): float32, float64, int32, int64 */
static int typed_code(boat_dtype_t dtype) {
    switch (dtype) {
        case BOAT_DTYPE_FLOAT32: return BH_DT_F32;
        case BOAT_DTYPE_FLOAT64: return BH_DT_F64;
        case BOAT_DTYPE_INT32: return BH_DT_I32;
        case BOAT_DTYPE_INT64: return BH_DT_I64;
        default: return -1;
    }
}

/* the same operators on float64 / int32 / int64 tensors, and boat_mod on all four types (arithmetic.c:157-360) */
static boat_tensor_t* binary_op_typed(int op, const boat_tensor_t* a, const boat_tensor_t* b) {
    const int code = typed_code(a->dtype);
    if (a->dtype != b->dtype || code < 0) return NULL;   /* arithmetic.c:166-170, 278-281 */
    if (!same_device(a, b)) {
        boat_fail(BOAT_ERROR_DEVICE, "elementwise op on tensors of different devices");
        return NULL;
    }
    int64_t shape[BOAT_MAX_DIMS], sa[BOAT_MAX_DIMS], sb[BOAT_MAX_DIMS];
    size_t nd = 0;
    if (!broadcast_shape(a, b, shape, &nd)) return NULL;
    boat_tensor_t* out = boat_tensor_create(shape, nd, a->dtype, a->device);
    if (!out || out->nelements == 0) return out;
    for (size_t i = 0; i < nd; i++) {
        sa[i] = i < nd - a->ndim ? 1 : a->shape[i - (nd - a->ndim)];
        sb[i] = i < nd - b->ndim ? 1 : b->shape[i - (nd - b->ndim)];
    }
    const void* pa = bt_dev_read(a);
    const void* pb = bt_dev_read(b);
    void* po = bt_dev_write(out);
    if (!pa || !pb || !po || !boat_hip_ok(bh_binary_typed(code, op, pa, sa, pb, sb, po, shape, (int)nd), "elementwise op")) {
        boat_tensor_free(out);
        return NULL;
    }
    return out;
}

static boat_tensor_t* binary_op(int op, const boat_tensor_t* a, const boat_tensor_t* b) {
    if (!a || !b) return NULL;
    if (!bt_is_f32(a) || !bt_is_f32(b)) return binary_op_typed(op, a, b);
    if (!same_device(a, b)) {
        boat_fail(BOAT_ERROR_DEVICE, "elementwise op on tensors of different devices");
        return NULL;
    }
    int64_t shape[BOAT_MAX_DIMS];
    size_t nd = 0;
    if (!broadcast_shape(a, b, shape, &nd)) return NULL;
    boat_tensor_t* out = bt_new_uninit(shape, nd, a->device);
    if (!out) return NULL;
    if (out->nelements == 0) return out;
    const float* pa = bt_dev_read(a);
    const float* pb = bt_dev_read(b);
    float* po = bt_dev_write(out);
    bool ok = pa && pb && po;
    if (ok) {
        if (a->nelements == out->nelements && b->nelements == out->nelements) {
            ok = boat_hip_ok(bh_binary(op, pa, pb, po, (int64_t)out->nelements), "elementwise op");
        } else {
            int64_t sa[BOAT_MAX_DIMS], sb[BOAT_MAX_DIMS];
            for (size_t i = 0; i < nd; i++) {
                sa[i] = i < nd - a->ndim ? 1 : a->shape[i - (nd - a->ndim)];
                sb[i] = i < nd - b->ndim ? 1 : b->shape[i - (nd - b->ndim)];
            }
            ok = boat_hip_ok(bh_binary_broadcast(op, pa, sa, pb, sb, po, shape, (int)nd), "broadcast op");
        }
    }
    if (!ok) {
        boat_tensor_free(out);
        return NULL;
    }
    return out;
}

boat_tensor_t* boat_add(const boat_tensor_t* a, const boat_tensor_t* b) { return binary_op(0, a, b); }
boat_tensor_t* boat_sub(const boat_tensor_t* a, const boat_tensor_t* b) { return binary_op(1, a, b); }
boat_tensor_t* boat_mul(const boat_tensor_t* a, const boat_tensor_t* b) { return binary_op(2, a, b); }
boat_tensor_t* boat_div(const boat_tensor_t* a, const boat_tensor_t* b) { return binary_op(3, a, b); }
boat_tensor_t* boat_mod(const boat_tensor_t* a, const boat_tensor_t* b) { return (a && b) ? binary_op_typed(4, a, b) : NULL; }   /* arithmetic.c:288-360 */

static void inplace_op(int op, boat_tensor_t* a, const boat_tensor_t* b) {
    if (!a || !b) return;
    if (a->nelements != b->nelements || a->dtype != b->dtype) return;   /* arithmetic.c:372-376: silent */
    if (!same_device(a, b) || a->nelements == 0) return;
    if (!bt_is_f32(a)) {   /* float64 / int32 / int64 (arithmetic.c:388-412): flat, no broadcasting */
        const int code = typed_code(a->dtype);
        const int64_t n = (int64_t)a->nelements;
        if (code < 0) return;
        const void* pb = bt_dev_read(b);
        void* pa = bt_dev_rw(a);
        if (pa && pb) boat_hip_ok(bh_binary_typed(code, op, pa, &n, pb, &n, pa, &n, 1), "in-place op");
        bt_flush_exposed();
        return;
    }
    const float* pb = bt_dev_read(b);
    if (op == 0 && pb && bt_is_zero(a) && a != b && a->st != b->st) {   /* 0 + b: a copy, the zeros are never written */
        float* pz = bt_dev_write(a);
        if (pz) boat_hip_ok(bh_memcpy_d2d(pz, pb, a->nbytes), "boat_add_");
        bt_flush_exposed();
        return;
    }
    float* pa = bt_dev_rw(a);
    if (!pa || !pb) return;
    if (op == 0) boat_hip_ok(bh_add_inplace(pa, pb, (int64_t)a->nelements), "boat_add_");
    else boat_hip_ok(bh_binary(op, pa, pb, pa, (int64_t)a->nelements), "in-place op");
    bt_flush_exposed();
}
void boat_add_(boat_tensor_t* a, const boat_tensor_t* b) { inplace_op(0, a, b); }
void boat_sub_(boat_tensor_t* a, const boat_tensor_t* b) { inplace_op(1, a, b); }
void boat_mul_(boat_tensor_t* a, const boat_tensor_t* b) { inplace_op(2, a, b); }
void boat_div_(boat_tensor_t* a, const boat_tensor_t* b) { inplace_op(3, a, b); }

/* out = a op scalar on float64 / int32 / int64 tensors, and powf/pow (arithmetic.c:425-518); in_place writes into a */
static boat_tensor_t* scalar_op_typed(int op, const boat_tensor_t* a, double scalar, bool in_place) {
    const int code = typed_code(a->dtype);
    if (code < 0 || (op == 5 && code > BH_DT_F64)) return NULL;
    boat_tensor_t* out = in_place ? (boat_tensor_t*)a : boat_tensor_create(a->shape, a->ndim, a->dtype, a->device);
    if (!out || out->nelements == 0) return out;
    const void* pa = in_place ? bt_dev_rw(out) : bt_dev_read(a);
    void* po = in_place ? (void*)pa : bt_dev_write(out);
    if (!pa || !po || !boat_hip_ok(bh_scalar_op_typed(code, op, pa, scalar, po, (int64_t)a->nelements), "scalar op")) {
        if (!in_place) boat_tensor_free(out);
        return NULL;
    }
    return out;
}

static boat_tensor_t* scalar_op(int op, const boat_tensor_t* a, double scalar) {
    if (!a) return NULL;
    if (!bt_is_f32(a)) return scalar_op_typed(op, a, scalar, false);
    boat_tensor_t* out = bt_new_like_uninit(a);
    if (!out || out->nelements == 0) return out;
    const float* pa = bt_dev_read(a);
    float* po = bt_dev_write(out);
    if (!pa || !po || !boat_hip_ok(bh_scalar_op(op, pa, (float)scalar, po, (int64_t)a->nelements), "scalar op")) {
        boat_tensor_free(out);
        return NULL;
    }
    return out;
}
boat_tensor_t* boat_add_scalar(const boat_tensor_t* a, double s) { return scalar_op(0, a, s); }
boat_tensor_t* boat_sub_scalar(const boat_tensor_t* a, double s) { return scalar_op(1, a, s); }
boat_tensor_t* boat_mul_scalar(const boat_tensor_t* a, double s) { return scalar_op(2, a, s); }
boat_tensor_t* boat_div_scalar(const boat_tensor_t* a, double s) { return scalar_op(3, a, s); }
boat_tensor_t* boat_pow_scalar(const boat_tensor_t* a, double s) { return a ? scalar_op_typed(5, a, s, false) : NULL; }   /* arithmetic.c:486-518 */
/* in-place forms (arithmetic.c:521-570) */
static void scalar_op_inplace(int op, boat_tensor_t* a, double scalar) {
    if (!a) return;
    scalar_op_typed(op, a, scalar, true);
    bt_flush_exposed();
}
void boat_add_scalar_(boat_tensor_t* a, double s) { scalar_op_inplace(0, a, s); }
void boat_sub_scalar_(boat_tensor_t* a, double s) { scalar_op_inplace(1, a, s); }
void boat_mul_scalar_(boat_tensor_t* a, double s) { scalar_op_inplace(2, a, s); }
void boat_div_scalar_(boat_tensor_t* a, double s) { scalar_op_inplace(3, a, s); }
/* stubs in the reference as well (src/ops/linear.c:409-413, src/ops/activation.c:304-308) */
boat_tensor_t* boat_inverse(const boat_tensor_t* a) {
    (void)a;
    return NULL;
}
boat_tensor_t* boat_selu(const boat_tensor_t* a) {
    (void)a;
    return NULL;
}

boat_tensor_t* boat_matmul(const boat_tensor_t* a, const boat_tensor_t* b) {
    if (!a || !b) return NULL;
    if (a->ndim < 2 || a->ndim > 4 || b->ndim < 2 || b->ndim > 4) return NULL;
    if (a->ndim != b->ndim) return NULL;                       /* same number of batch dims (linear.c:34-38) */
    if (a->dtype != b->dtype || !bt_is_f32(a)) return NULL;
    if (!same_device(a, b)) return NULL;
    const size_t bd = a->ndim - 2;
    int64_t batch = 1;
    for (size_t i = 0; i < bd; i++) {
        if (a->shape[i] != b->shape[i]) return NULL;
        batch *= a->shape[i];
    }
    const int64_t m = a->shape[bd], ka = a->shape[bd + 1], kb = b->shape[bd], n = b->shape[bd + 1];
    if (ka != kb) return NULL;
    int64_t shape[BOAT_MAX_DIMS];
    for (size_t i = 0; i < bd; i++) shape[i] = a->shape[i];
    shape[bd] = m;
    shape[bd + 1] = n;
    boat_tensor_t* out = bt_new_uninit(shape, a->ndim, a->device);
    if (!out || out->nelements == 0) return out;
    const float* pa = bt_dev_read(a);
    const float* pb = bt_dev_read(b);
    float* po = bt_dev_write(out);
    bool ok = pa && pb && po;
    /* the batch index lives in a 16-bit grid dimension: walk very large batches in slices */
    for (int64_t b0 = 0; ok && b0 < batch; b0 += 32768) {
        const int64_t nb = batch - b0 < 32768 ? batch - b0 : 32768;
        ok = boat_hip_ok(bh_gemm(0, 0, m, n, ka, pa + b0 * m * ka, ka, pb + b0 * ka * n, n, po + b0 * m * n, n, NULL, 0, nb),
                         "boat_matmul");
    }
    if (!ok) {
        boat_tensor_free(out);
        return NULL;
    }
    return out;
}

boat_tensor_t* boat_transpose(const boat_tensor_t* a, int dim0, int dim1) {
    if (!a) return NULL;
    const int nd = (int)a->ndim;
    if (dim0 < 0 || dim1 < 0 || dim0 >= nd || dim1 >= nd) return NULL;   /* linear.c:241-244 (negative ints compare as huge) */
    if (a->dtype != BOAT_DTYPE_FLOAT32 && a->dtype != BOAT_DTYPE_FLOAT64) {
        /* linear.c:399-402: other element types get the swapped shape over an untransposed copy of the payload */
        boat_tensor_t* copy = boat_tensor_clone(a);
        if (copy) {
            const int64_t t = copy->shape[dim0];
            copy->shape[dim0] = copy->shape[dim1];
            copy->shape[dim1] = t;
        }
        return copy;
    }
    if (dim0 == dim1) return boat_tensor_clone(a);
    if (dim0 > dim1) {
        int t = dim0;
        dim0 = dim1;
        dim1 = t;
    }
    int64_t shape[BOAT_MAX_DIMS];
    int64_t before = 1, between = 1, after = 1;
    for (int i = 0; i < nd; i++) {
        shape[i] = a->shape[i];
        if (i < dim0) before *= a->shape[i];
        else if (i > dim0 && i < dim1) between *= a->shape[i];
        else if (i > dim1) after *= a->shape[i];
    }
    shape[dim0] = a->shape[dim1];
    shape[dim1] = a->shape[dim0];
    boat_tensor_t* out = boat_tensor_create(shape, a->ndim, a->dtype, a->device);
    if (!out || out->nelements == 0) return out;
    const float* pa = bt_dev_read(a);
    float* po = bt_dev_write(out);
    bool ok = pa && po;
    const int64_t rows = a->shape[dim0], cols = a->shape[dim1];
    if (ok && a->dtype == BOAT_DTYPE_FLOAT64) {
        ok = boat_hip_ok(bh_swap_dims_f64((const double*)pa, (double*)po, before, rows, between, cols, after), "boat_transpose");
    } else if (ok && between == 1 && after == 1) {
        /* the hot path's case, the last two dimensions: the tiled kernel, in slabs its grid can index */
        for (int64_t b0 = 0; ok && b0 < before; b0 += 32768) {
            const int64_t nb = before - b0 < 32768 ? before - b0 : 32768;
            ok = boat_hip_ok(bh_transpose_last2(pa + b0 * rows * cols, po + b0 * rows * cols, nb, rows, cols), "boat_transpose");
        }
    } else if (ok) {
        ok = boat_hip_ok(bh_swap_dims(pa, po, before, rows, between, cols, after), "boat_transpose");
    }
    if (!ok) {
        boat_tensor_free(out);
        return NULL;
    }
    return out;
}

boat_tensor_t* boat_sum(const boat_tensor_t* a, const int64_t* dims, size_t n_dims, bool keepdim) {
    (void)keepdim;
    if (!a) return NULL;
    if (dims != NULL || n_dims != 0) return NULL;   /* arithmetic.c:614-618: full reduction only */
    if (!bt_is_f32(a)) return NULL;
    const int64_t one = 1;
    boat_tensor_t* out = bt_new_uninit(&one, 1, a->device);
    if (!out) return NULL;
    const float* pa = a->nelements ? bt_dev_read(a) : NULL;
    float* po = bt_dev_write(out);
    if (!po || (a->nelements && !pa) || !boat_hip_ok(bh_sum_all(pa, po, (int64_t)a->nelements), "boat_sum")) {
        boat_tensor_free(out);
        return NULL;
    }
    return out;
}

boat_tensor_t* boat_mean(const boat_tensor_t* a, const int64_t* dims, size_t n_dims, bool keepdim) {
    boat_tensor_t* s = boat_sum(a, dims, n_dims, keepdim);
    if (!s) return NULL;
    boat_tensor_t* out = boat_div_scalar(s, (double)(float)a->nelements);
    boat_tensor_free(s);
    return out;
}

boat_tensor_t* boat_dot(const boat_tensor_t* a, const boat_tensor_t* b) {
    /* vectors of one length only, as linear.c:176-189 */
    if (!a || !b || a->ndim != 1 || b->ndim != 1 || a->shape[0] != b->shape[0] || a->dtype != b->dtype) return NULL;
    boat_tensor_t* prod = boat_mul(a, b);
    if (!prod) return NULL;
    boat_tensor_t* out = boat_sum(prod, NULL, 0, false);
    boat_tensor_free(prod);
    return out;
}

static boat_tensor_t* activation(int act, const boat_tensor_t* a) {
    if (!a || !bt_is_f32(a)) return NULL;
    boat_tensor_t* out = bt_new_like_uninit(a);
    if (!out || out->nelements == 0) return out;
    const float* pa = bt_dev_read(a);
    float* po = bt_dev_write(out);
    if (!pa || !po || !boat_hip_ok(bh_activation_forward(act, pa, po, (int64_t)a->nelements), "activation")) {
        boat_tensor_free(out);
        return NULL;
    }
    return out;
}
boat_tensor_t* boat_relu(const boat_tensor_t* a) {
    /* activation.c:266-282: float32 is rectified, any other element type comes back as a copy */
    if (a && !bt_is_f32(a)) return boat_tensor_clone(a);
    return activation(BH_ACT_RELU, a);
}
boat_tensor_t* boat_sigmoid(const boat_tensor_t* a) { return activation(BH_ACT_SIGMOID, a); }
boat_tensor_t* boat_tanh(const boat_tensor_t* a) { return activation(BH_ACT_TANH, a); }
boat_tensor_t* boat_gelu(const boat_tensor_t* a) { return activation(BH_ACT_GELU, a); }

/* last-axis softmax family; other axes are out of the hot path */
static boat_tensor_t* row_softmax(bool log_form, const boat_tensor_t* a, int axis) {
    if (!a || !bt_is_f32(a)) return NULL;
    const int nd = (int)a->ndim;
    if (axis < 0) axis += nd;
    if (nd > 0 && axis != nd - 1) {
        boat_fail(BOAT_ERROR_NOT_IMPLEMENTED, "softmax: only the last axis is supported");
        return NULL;
    }
    boat_tensor_t* out = bt_new_like_uninit(a);
    if (!out || out->nelements == 0) return out;
    const int64_t cols = nd > 0 ? a->shape[nd - 1] : 1;
    const int64_t rows = (int64_t)a->nelements / cols;
    const float* pa = bt_dev_read(a);
    float* po = bt_dev_write(out);
    int rc = (!pa || !po) ? BH_EDEVICE
                          : log_form ? bh_log_softmax_forward(pa, po, rows, cols) : bh_softmax_forward(pa, po, rows, cols);
    if (!boat_hip_ok(rc, "softmax")) {
        boat_tensor_free(out);
        return NULL;
    }
    return out;
}
boat_tensor_t* boat_softmax(const boat_tensor_t* a, int axis) { return row_softmax(false, a, axis); }
boat_tensor_t* boat_log_softmax(const boat_tensor_t* a, int axis) { return row_softmax(true, a, axis); }

/* ---- fused losses (no counterpart in the reference's library; see the header) ---- */

boat_tensor_t* boat_hip_softmax_cross_entropy(const boat_tensor_t* logits, const boat_tensor_t* labels, boat_tensor_t** dlogits) {
    if (dlogits) *dlogits = NULL;
    if (!logits || !labels || !bt_is_f32(logits) || logits->ndim != 2) return NULL;
    const int64_t rows = logits->shape[0], cols = logits->shape[1];
    if ((int64_t)labels->nelements != rows || rows == 0 || cols == 0) return NULL;
    if (labels->dtype != BOAT_DTYPE_INT32 && labels->dtype != BOAT_DTYPE_UINT8) return NULL;
    const int64_t one = 1;
    boat_tensor_t* loss = bt_new_uninit(&one, 1, logits->device);
    boat_tensor_t* grad = dlogits ? bt_new_like_uninit(logits) : NULL;
    bool ok = loss && (!dlogits || grad);
    int32_t* staged = NULL;   /* device copy of widened UINT8 labels */
    const int32_t* dev_labels = NULL;
    if (ok && labels->dtype == BOAT_DTYPE_INT32) {
        /* INT32 indices are used where they are: the tensor's device copy (uploaded once, like any tensor) */
        dev_labels = (const int32_t*)bt_dev_read(labels);
        ok = dev_labels != NULL;
    } else if (ok) {
        const void* src = labels->device == BOAT_DEVICE_HIP ? NULL : boat_tensor_const_data(labels);
        int32_t* host_labels = src ? (int32_t*)malloc(sizeof(int32_t) * (size_t)rows) : NULL;
        staged = host_labels ? (int32_t*)bh_malloc(sizeof(int32_t) * (size_t)rows) : NULL;
        ok = staged != NULL;
        if (ok) {
            for (int64_t i = 0; i < rows; i++) host_labels[i] = (int32_t)((const uint8_t*)src)[i];
            ok = boat_hip_ok(bh_memcpy_h2d(staged, host_labels, sizeof(int32_t) * (size_t)rows), "labels upload");
        }
        free(host_labels);
        dev_labels = staged;
    }
    if (ok) {
        const float* pz = bt_dev_read(logits);
        float* pl = bt_dev_write(loss);
        float* pg = grad ? bt_dev_write(grad) : NULL;
        ok = pz && pl && boat_hip_ok(bh_softmax_ce_grad(pz, dev_labels, pg, pl, rows, cols), "softmax cross-entropy");
    }
    if (staged) bh_free(staged);
    if (!ok) {
        boat_tensor_free(loss);
        boat_tensor_free(grad);
        return NULL;
    }
    if (dlogits) *dlogits = grad;
    return loss;
}

boat_tensor_t* boat_hip_mse_loss(const boat_tensor_t* pred, const boat_tensor_t* target, boat_tensor_t** grad) {
    if (grad) *grad = NULL;
    if (!pred || !target || !bt_is_f32(pred) || !bt_is_f32(target) || !bt_same_shape(pred, target) || pred->nelements == 0)
        return NULL;
    const int64_t one = 1;
    boat_tensor_t* loss = bt_new_uninit(&one, 1, pred->device);
    boat_tensor_t* g = grad ? bt_new_like_uninit(pred) : NULL;
    const float* pp = bt_dev_read(pred);
    const float* pt = bt_dev_read(target);
    bool ok = loss && pp && pt && (!grad || g);
    if (ok && g) ok = boat_hip_ok(bh_mse_loss_grad(pp, pt, bt_dev_write(loss), bt_dev_write(g), (int64_t)pred->nelements), "mse loss and gradient");
    else if (ok) ok = boat_hip_ok(bh_mse_loss(pp, pt, bt_dev_write(loss), (int64_t)pred->nelements), "mse loss");
    if (!ok) {
        boat_tensor_free(loss);
        boat_tensor_free(g);
        return NULL;
    }
    if (grad) *grad = g;
    return loss;
}

/* arithmetic.c:575-581: whether the two shapes broadcast under the right-aligned rule of :78-104 */
bool boat_can_broadcast(const boat_tensor_t* a, const boat_tensor_t* b) {
    if (!a || !b) return false;
    int64_t shape[BOAT_MAX_DIMS];
    size_t ndim = 0;
    return broadcast_shape(a, b, shape, &ndim);
}

/* arithmetic.c:583-608: the reference does no broadcasting here either -- a new dense tensor of the target shape holding
 * a's values, and NULL unless the element counts agree */
boat_tensor_t* boat_broadcast_to(const boat_tensor_t* a, const int64_t* shape, size_t ndim) {
    if (!a || !shape) return NULL;
    boat_tensor_t* out = boat_tensor_create(shape, ndim, a->dtype, a->device);
    if (!out) return NULL;
    if (out->nelements != a->nelements) {
        boat_tensor_free(out);
        return NULL;
    }
    if (a->nbytes == 0) return out;
    boat_tensor_t* copy = boat_tensor_clone(a);
    if (!copy) {
        boat_tensor_free(out);
        return NULL;
    }
    /* the clone is dense and owns its payload: hand that payload to the tensor of the new shape */
    boat_storage_t* st = out->st;
    out->st = copy->st;
    copy->st = st;
    boat_tensor_free(copy);
    return out;
}

