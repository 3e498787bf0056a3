/* autodiff.c - tape recording and the backward driver.
 *
 * API and per-op gradient arithmetic follow src/autodiff.c of the reference: variables
 * (:138-297), op recording (:2070-2150, :2283-2347, :2388-2456; layer ops record only when
 * their FIRST input requires grad, generic ops when ANY input does), the per-op backward
 * rules (:1002-2068, :2458-2672) and gradient accumulation into input->grad with boat_add_.
 *
 * The driver differs on purpose.  The reference recurses depth-first from every op into each
 * non-leaf input (:431-450), which propagates a non-leaf's gradient once per consumer and so
 * double-counts fan-out (z = y + y, y = a*b gives dz/da = 4b).  Here every op reachable from
 * the root is visited exactly once, in reverse recording order, after all of its consumers:
 * identical to the reference on chains and leaf fan-out, and the true gradient elsewhere.
 *
 * Lifetime: an op is owned by its output variable and holds references on its inputs, so a
 * variable the caller has freed stays alive while a later result still needs it, and the whole
 * tape of a step is released when its last result is freed.
 */
#include "boat_internal.h"

#include <stdlib.h>
#include <string.h>

typedef enum {
    OP_ADD, OP_SUB, OP_MUL, OP_DIV, OP_RELU, OP_SIGMOID, OP_TANH, OP_MATMUL, OP_DOT, OP_SUM, OP_MEAN,
    OP_SOFTMAX, OP_LOG_SOFTMAX, OP_FLATTEN, OP_DENSE, OP_ATTENTION, OP_GELU, OP_LAYERNORM, OP_CONV, OP_POOL
} op_type_t;

typedef struct boat_op {
    op_type_t type;
    boat_variable_t* inputs[3];
    size_t num_inputs;
    boat_variable_t* output;     /* weak: the output owns the op */
    void* layer;                 /* dense / attention / layernorm */
    boat_tensor_t* saved[3];     /* per-op saved tensors (layernorm: input, mean, rstd) */
    uint64_t seq;                /* recording order == a topological order */
    uint64_t mark;               /* visit epoch of the backward that last collected it */
    uint64_t skip;               /* visit epoch of a backward in which a fused rule already covered this op */
    uint64_t bias_done;          /* dense: visit epoch of a backward in which the consumer's rule already added the bias gradient */
} boat_op_t;

struct boat_variable_t {
    boat_tensor_t* data;
    boat_tensor_t* grad;
    bool requires_grad;
    bool persistent_grad;        /* grad buffer survives zero_grad (boat_hip_variable_ensure_grad) */
    bool grad_shared;            /* grad is a tensor other holders read too: replace it, never add into it */
    boat_op_t* producer;
    size_t refs;
    uint64_t uses_epoch;         /* the backward walk that last counted ... */
    unsigned walk_uses;          /* ... how many of its ops read this variable */
    struct boat_variable_t *prev, *next;   /* live-variable list of the library */
};

struct boat_autodiff_context_t {
    bool grad_enabled;
    const boat_graph_t* graph;   /* carried for the caller, never read here */
};

/* The reference hangs its tape on a graph object (the sources under src/graph) and lets callers hand one to a context
 * (tests/unit/test_gradient_check.c:341-348).  The tape here needs none; the handle exists so that such callers link
 * and run: it can be created, attached, fetched back and freed, nothing more. */
boat_graph_t* boat_graph_create_with_device(boat_device_t device) {
    boat_graph_t* g = (boat_graph_t*)calloc(1, sizeof(*g));
    if (g) g->device = device;
    return g;
}
boat_graph_t* boat_graph_create(void) { return boat_graph_create_with_device(BOAT_DEVICE_CPU); }
void boat_graph_free(boat_graph_t* graph) {
    if (!graph) return;
    free(graph->nodes);
    free(graph);
}
void boat_autodiff_context_set_graph(boat_autodiff_context_t* context, const boat_graph_t* graph) {
    if (context) context->graph = graph;
}
boat_graph_t* boat_autodiff_context_get_graph(const boat_autodiff_context_t* context) {
    return context ? (boat_graph_t*)context->graph : NULL;
}

static _Thread_local boat_autodiff_context_t* g_current = NULL;
static boat_variable_t* g_live = NULL;
static uint64_t g_seq = 0, g_epoch = 0;

/* ------------------------------------------------------------- variables */

static void variable_unref(boat_variable_t* v);

static void op_free(boat_op_t* op) {
    if (!op) return;
    for (size_t i = 0; i < 3; i++) boat_tensor_free(op->saved[i]);
    for (size_t i = 0; i < op->num_inputs; i++) variable_unref(op->inputs[i]);
    free(op);
}

static void variable_unref(boat_variable_t* v) {
    if (!v || --v->refs > 0) return;
    if (v->prev) v->prev->next = v->next; else g_live = v->next;
    if (v->next) v->next->prev = v->prev;
    boat_op_t* op = v->producer;
    v->producer = NULL;
    boat_tensor_free(v->grad);
    boat_tensor_free(v->data);
    free(v);
    op_free(op);
}

boat_variable_t* boat_variable_create(boat_tensor_t* tensor, bool requires_grad) {
    if (!tensor) return NULL;
    boat_variable_t* v = (boat_variable_t*)calloc(1, sizeof(*v));
    if (!v) return NULL;
    v->data = tensor;
    boat_tensor_ref(tensor);
    v->requires_grad = requires_grad;
    v->refs = 1;
    v->next = g_live;
    if (g_live) g_live->prev = v;
    g_live = v;
    if (!g_current) g_current = boat_autodiff_context_create();   /* lazily, as autodiff.c:167-190 */
    return v;
}

boat_variable_t* boat_variable_create_with_shape(const int64_t* shape, size_t ndim, boat_dtype_t dtype, bool requires_grad) {
    boat_tensor_t* t = boat_tensor_create(shape, ndim, dtype, BOAT_DEVICE_CPU);
    if (!t) return NULL;
    boat_variable_t* v = boat_variable_create(t, requires_grad);
    boat_tensor_unref(t);
    return v;
}

void boat_variable_free(const boat_variable_t* variable) { variable_unref((boat_variable_t*)variable); }
boat_tensor_t* boat_variable_data(const boat_variable_t* v) { return v ? v->data : NULL; }
boat_tensor_t* boat_variable_grad(const boat_variable_t* v) { return v ? v->grad : NULL; }
bool boat_variable_requires_grad(const boat_variable_t* v) { return v ? v->requires_grad : false; }
void boat_variable_set_requires_grad(boat_variable_t* v, bool requires_grad) {
    if (v) v->requires_grad = requires_grad;
}

bool boat_variable_reset_data(boat_variable_t* v, boat_tensor_t* new_tensor) {
    if (!v || !new_tensor) return false;
    if (v->producer) {
        fprintf(stderr, "Warning: Cannot reset data for variable with computation graph node\n");
        return false;
    }
    boat_tensor_ref(new_tensor);
    boat_tensor_unref(v->data);
    v->data = new_tensor;
    if (v->grad && !v->persistent_grad) {
        boat_tensor_unref(v->grad);
        v->grad = NULL;
    }
    return true;
}

void boat_variable_zero_grad(boat_variable_t* v) {
    if (!v || !v->grad) return;
    if (v->persistent_grad) {
        if (!bt_set_zero(v->grad)) {
            float* g = bt_dev_write(v->grad);
            if (g) boat_hip_ok(bh_memset_zero(g, v->grad->nbytes), "boat_variable_zero_grad");
        }
        bt_flush_exposed();
    } else {
        boat_tensor_unref(v->grad);   /* the reference drops the tensor (autodiff.c:285-292) */
        v->grad = NULL;
    }
}

boat_tensor_t* boat_hip_variable_ensure_grad(boat_variable_t* v) {
    if (!v) return NULL;
    if (v->grad && (v->grad_shared || v->grad->ref_count > 1)) {
        /* a tensor other holders read too cannot become this variable's own, lasting buffer: take a copy */
        boat_tensor_t* own = boat_tensor_clone(v->grad);
        if (!own) return NULL;
        boat_tensor_unref(v->grad);
        v->grad = own;
        v->grad_shared = false;
    }
    if (!v->grad) v->grad = boat_tensor_create_like(v->data);
    v->persistent_grad = v->grad != NULL;
    return v->grad;
}

void boat_variable_retain_grad(const boat_variable_t* v, bool retain) {
    (void)v;
    (void)retain;   /* every variable keeps its gradient, as in the reference */
}

/* --------------------------------------------------------------- context */

boat_autodiff_context_t* boat_autodiff_context_create(void) {
    boat_autodiff_context_t* c = (boat_autodiff_context_t*)calloc(1, sizeof(*c));
    if (c) c->grad_enabled = true;
    return c;
}
void boat_autodiff_context_free(const boat_autodiff_context_t* c) {
    if (c == g_current) g_current = NULL;
    free((void*)c);
}
void boat_autodiff_context_enable_grad(boat_autodiff_context_t* c) { if (c) c->grad_enabled = true; }
void boat_autodiff_context_disable_grad(boat_autodiff_context_t* c) { if (c) c->grad_enabled = false; }
bool boat_autodiff_context_grad_enabled(const boat_autodiff_context_t* c) { return c ? c->grad_enabled : false; }
void boat_autodiff_set_current_context(const boat_autodiff_context_t* c) { g_current = (boat_autodiff_context_t*)c; }
boat_autodiff_context_t* boat_autodiff_get_current_context(void) { return g_current; }

/* Drops every recorded op: all live variables become leaves, intermediates that only the tape
 * kept alive are released; layers and their parameters are never touched. */
void boat_autodiff_clear_computation_graph(void) {
    /* detach first, free afterwards: freeing an op can free variables further down the list */
    size_t n = 0, cap = 64;
    boat_op_t** ops = (boat_op_t**)malloc(cap * sizeof(*ops));
    if (!ops) return;
    for (boat_variable_t* v = g_live; v; v = v->next) {
        if (!v->producer) continue;
        if (n == cap) {
            boat_op_t** grown = (boat_op_t**)realloc(ops, 2 * cap * sizeof(*ops));
            if (!grown) break;
            ops = grown;
            cap *= 2;
        }
        ops[n++] = v->producer;
        v->producer = NULL;
    }
    for (size_t i = 0; i < n; i++) op_free(ops[i]);
    free(ops);
}

/* ------------------------------------------------------------- recording */

/* the reference stores a context's grad flag and never reads it (autodiff.c:625-632): in reference-exact mode every op is recorded */
static bool recording(void) { return !g_current || g_current->grad_enabled || bt_reference_exact(); }

static boat_variable_t* record(op_type_t type, boat_variable_t* const* inputs, size_t n, boat_tensor_t* out_tensor,
                               bool requires_grad, void* layer) {
    if (!out_tensor) return NULL;
    boat_variable_t* out = boat_variable_create(out_tensor, requires_grad);
    boat_tensor_unref(out_tensor);   /* the variable holds the reference now */
    if (!out) return NULL;
    if (requires_grad && recording()) {
        boat_op_t* op = (boat_op_t*)calloc(1, sizeof(*op));
        if (!op) {
            boat_variable_free(out);
            return NULL;
        }
        op->type = type;
        op->num_inputs = n;
        for (size_t i = 0; i < n; i++) {
            op->inputs[i] = inputs[i];
            inputs[i]->refs++;
        }
        op->output = out;
        op->layer = layer;
        op->seq = ++g_seq;
        out->producer = op;
    }
    return out;
}

static boat_variable_t* binary(op_type_t type, const boat_variable_t* a, const boat_variable_t* b,
                               boat_tensor_t* (*fwd)(const boat_tensor_t*, const boat_tensor_t*)) {
    if (!a || !b) return NULL;
    boat_variable_t* in[2] = {(boat_variable_t*)a, (boat_variable_t*)b};
    return record(type, in, 2, fwd(a->data, b->data), a->requires_grad || b->requires_grad, NULL);
}
static boat_variable_t* unary(op_type_t type, const boat_variable_t* a, boat_tensor_t* out) {
    if (!a) {
        boat_tensor_free(out);
        return NULL;
    }
    boat_variable_t* in[1] = {(boat_variable_t*)a};
    return record(type, in, 1, out, a->requires_grad, NULL);
}

boat_variable_t* boat_var_add(const boat_variable_t* a, const boat_variable_t* b) { return binary(OP_ADD, a, b, boat_add); }
boat_variable_t* boat_var_sub(const boat_variable_t* a, const boat_variable_t* b) { return binary(OP_SUB, a, b, boat_sub); }
boat_variable_t* boat_var_mul(const boat_variable_t* a, const boat_variable_t* b) { return binary(OP_MUL, a, b, boat_mul); }
boat_variable_t* boat_var_div(const boat_variable_t* a, const boat_variable_t* b) { return binary(OP_DIV, a, b, boat_div); }
boat_variable_t* boat_var_matmul(const boat_variable_t* a, const boat_variable_t* b) { return binary(OP_MATMUL, a, b, boat_matmul); }
boat_variable_t* boat_var_dot(const boat_variable_t* a, const boat_variable_t* b) { return binary(OP_DOT, a, b, boat_dot); }
boat_variable_t* boat_var_relu(const boat_variable_t* a) { return a ? unary(OP_RELU, a, boat_relu(a->data)) : NULL; }
boat_variable_t* boat_var_sigmoid(const boat_variable_t* a) { return a ? unary(OP_SIGMOID, a, boat_sigmoid(a->data)) : NULL; }
boat_variable_t* boat_var_tanh(const boat_variable_t* a) { return a ? unary(OP_TANH, a, boat_tanh(a->data)) : NULL; }
boat_variable_t* boat_hip_var_gelu(const boat_variable_t* a) { return a ? unary(OP_GELU, a, boat_gelu(a->data)) : NULL; }
/* the axis argument is ignored by the reference, which always works on the last axis (autodiff.c:530-548) */
boat_variable_t* boat_var_softmax(const boat_variable_t* a, int axis) {
    (void)axis;
    return a ? unary(OP_SOFTMAX, a, boat_softmax(a->data, -1)) : NULL;
}
boat_variable_t* boat_var_log_softmax(const boat_variable_t* a, int axis) {
    (void)axis;
    return a ? unary(OP_LOG_SOFTMAX, a, boat_log_softmax(a->data, -1)) : NULL;
}
boat_variable_t* boat_var_sum(const boat_variable_t* a, const int64_t* dims, size_t n_dims, bool keepdim) {
    (void)dims; (void)n_dims; (void)keepdim;   /* full reduction only (autodiff.c:937-940) */
    return a ? unary(OP_SUM, a, boat_sum(a->data, NULL, 0, false)) : NULL;
}
/* mean keeps the input's shape with the mean in element 0 and zeros elsewhere (autodiff.c:947-985) */
boat_variable_t* boat_var_mean(const boat_variable_t* a, int64_t* dims, size_t n_dims, bool keepdim) {
    (void)dims; (void)n_dims; (void)keepdim;
    if (!a || a->data->nelements == 0 || !bt_is_f32(a->data)) return NULL;
    boat_tensor_t* m = boat_mean(a->data, NULL, 0, false);
    boat_tensor_t* out = m ? boat_tensor_create_like(a->data) : NULL;
    float* po = out ? bt_dev_rw(out) : NULL;
    if (!po || !boat_hip_ok(bh_memcpy_d2d(po, bt_dev_read(m), sizeof(float)), "boat_var_mean")) {
        boat_tensor_free(m);
        boat_tensor_free(out);
        return NULL;
    }
    boat_tensor_free(m);
    return unary(OP_MEAN, a, out);
}
/* no reduction along chosen dimensions exists in the reference either: both return NULL (autodiff.c:595-603) */
boat_variable_t* boat_var_max(const boat_variable_t* a, int64_t* dims, size_t n_dims, bool keepdim) {
    (void)a; (void)dims; (void)n_dims; (void)keepdim;
    return NULL;
}
boat_variable_t* boat_var_min(const boat_variable_t* a, int64_t* dims, size_t n_dims, bool keepdim) {
    (void)a; (void)dims; (void)n_dims; (void)keepdim;
    return NULL;
}
boat_variable_t* boat_var_flatten(const boat_variable_t* a) {
    if (!a) return NULL;
    const boat_tensor_t* t = a->data;
    if (t->ndim < 2) {
        fprintf(stderr, "Error: Flatten expects at least 2D input tensor\n");
        return NULL;
    }
    int64_t rest = 1;
    for (size_t i = 1; i < t->ndim; i++) rest *= t->shape[i];
    const int64_t shape[] = {t->shape[0], rest};
    return unary(OP_FLATTEN, a, boat_tensor_reshape(t, shape, 2));
}

/* any shape with the same element count; the gradient is reshaped back (the same rule as flatten) */
boat_variable_t* boat_hip_var_reshape(const boat_variable_t* a, const int64_t* shape, size_t ndim) {
    if (!a || !shape || ndim == 0 || ndim > BOAT_MAX_DIMS) return NULL;
    return unary(OP_FLATTEN, a, boat_tensor_reshape(a->data, shape, ndim));
}

boat_variable_t* boat_var_dense(const boat_variable_t* input, const struct boat_dense_layer_t* layer) {
    if (!input || !layer) return NULL;
    boat_variable_t* in[1] = {(boat_variable_t*)input};
    return record(OP_DENSE, in, 1, boat_dense_layer_forward((boat_dense_layer_t*)layer, input->data), input->requires_grad, (void*)layer);
}

/* like dense, these record only when their input requires grad (autodiff.c:2155, 2221) */
boat_variable_t* boat_var_conv(const boat_variable_t* input, const struct boat_conv_layer_t* layer) {
    if (!input || !layer) return NULL;
    boat_variable_t* in[1] = {(boat_variable_t*)input};
    return record(OP_CONV, in, 1, boat_conv_layer_forward((boat_conv_layer_t*)layer, input->data), input->requires_grad, (void*)layer);
}

boat_variable_t* boat_var_pool(const boat_variable_t* input, const struct boat_pool_layer_t* layer) {
    if (!input || !layer) return NULL;
    boat_variable_t* in[1] = {(boat_variable_t*)input};
    return record(OP_POOL, in, 1, boat_pool_layer_forward((boat_pool_layer_t*)layer, input->data), input->requires_grad, (void*)layer);
}

boat_variable_t* boat_var_attention(const boat_variable_t* q, const boat_variable_t* k, const boat_variable_t* v,
                                    const struct boat_attention_t* attention, const boat_tensor_t* mask) {
    if (!q || !k || !v || !attention) return NULL;
    boat_variable_t* in[3] = {(boat_variable_t*)q, (boat_variable_t*)k, (boat_variable_t*)v};
    return record(OP_ATTENTION, in, 3, boat_attention_forward((boat_attention_t*)attention, q->data, k->data, v->data, mask),
                  q->requires_grad || k->requires_grad || v->requires_grad, (void*)attention);
}

boat_variable_t* boat_hip_var_layernorm(const boat_variable_t* a, boat_layernorm_t* norm) {
    if (!a || !norm) return NULL;
    boat_tensor_t* y = boat_layernorm_forward(norm, a->data);
    if (!y) return NULL;
    boat_variable_t* in[1] = {(boat_variable_t*)a};
    boat_variable_t* out = record(OP_LAYERNORM, in, 1, y, a->requires_grad, norm);
    if (out && out->producer) {
        /* the layer may run again before this op's backward: keep this call's statistics */
        boat_op_t* op = out->producer;
        op->saved[0] = a->data;
        op->saved[1] = norm->cache_mean;
        op->saved[2] = norm->cache_rstd;
        for (int i = 0; i < 3; i++) boat_tensor_ref(op->saved[i]);
    }
    return out;
}

/* -------------------------------------------------------------- backward */

/* v->grad += g ; takes ownership of g when `own` (it may become the gradient tensor itself,
 * as the reference does with freshly computed gradients, autodiff.c:1128-1135) */
static const boat_tensor_t* g_walk_seed = NULL;   /* the caller's grad_output during a backward walk */
static boat_variable_t* g_lender = NULL;          /* the variable whose gradient the current op hands on (its output) */

static void accumulate(boat_variable_t* v, boat_tensor_t* g, bool own) {
    if (!g) return;
    if (!v->grad) {
        v->grad_shared = false;
        if (own && g->ref_count == 1 && !g->is_view && g->nelements == v->data->nelements) {
            v->grad = g;
            return;
        }
        /* The first contribution to a NON-LEAF variable that cannot be taken over (the consumer's own gradient handed
         * on by an add or a reshape) is shared, not copied: in the reverse walk a gradient is complete before it is
         * handed on, so nobody adds into it afterwards, and this variable replaces it (below) instead of adding into it
         * if a second contribution comes.  Leaves keep a buffer of their own, which outlives the walk.  The
         * reference-exact walk hands on gradients that are still growing, so it copies. */
        /* A leaf shares as well when the tensor is one the walk made itself (a non-leaf's finished gradient handed on
         * by an add): whoever holds a tensor with other holders replaces it instead of writing into it (below), so the
         * leaf's gradient stays what it is.  The caller's own grad_output is never a leaf's gradient: the caller may
         * reuse that buffer. */
        const bool lent = g_lender && g_lender->grad && g_lender->grad->st == g->st;
        if ((v->producer || g != g_walk_seed) && !bt_reference_exact() && bt_is_f32(g) && bt_same_shape(g, v->data) &&
            !(lent && g_lender->persistent_grad)) {
            if (!own) boat_tensor_ref(g);
            v->grad = g;
            v->grad_shared = true;
            /* the variable it came from must not add into it later either (a second backward over a kept graph) */
            if (lent) g_lender->grad_shared = true;
            return;
        }
        if (bt_is_f32(g) && bt_is_f32(v->data) && g->nelements == v->data->nelements && g->nelements > 0) {
            /* first contribution: one copy instead of zero-fill + add (0 + g == g bit for bit) */
            boat_tensor_t* fresh = bt_new_like_uninit(v->data);
            const float* src = fresh ? bt_dev_read(g) : NULL;
            float* dst = src ? bt_dev_write(fresh) : NULL;
            if (dst && boat_hip_ok(bh_memcpy_d2d(dst, src, g->nbytes), "gradient copy")) {
                v->grad = fresh;
                if (own) boat_tensor_unref(g);
                return;
            }
            boat_tensor_free(fresh);
        }
        v->grad = boat_tensor_create_like(v->data);
    }
    if (v->grad && v->grad_shared) {
        /* out of place: the shared tensor stays what it is for its other holders (same cost as adding in place) */
        boat_tensor_t* sum = g->nelements == v->grad->nelements && bt_is_f32(g) ? bt_new_like_uninit(v->grad) : NULL;
        const float* pa = sum ? bt_dev_read(v->grad) : NULL;
        const float* pb = pa ? bt_dev_read(g) : NULL;
        float* ps = pb ? bt_dev_write(sum) : NULL;
        if (ps && boat_hip_ok(bh_binary(0, pa, pb, ps, (int64_t)sum->nelements), "gradient sum")) {
            boat_tensor_unref(v->grad);
            v->grad = sum;
            v->grad_shared = false;
        } else {
            boat_tensor_free(sum);
            boat_add_(v->grad, g);      /* shapes the out-of-place kernel does not take: the reference's in-place add */
        }
    } else if (v->grad) {
        boat_add_(v->grad, g);
    }
    if (own) boat_tensor_unref(g);
}

static boat_tensor_t* ones_like(const boat_tensor_t* t) {
    boat_tensor_t* o = bt_new_like_uninit(t);
    float* p = o ? bt_dev_write(o) : NULL;
    if (!p || !boat_hip_ok(bh_fill(p, 1.0f, (int64_t)o->nelements), "ones_like")) {
        boat_tensor_free(o);
        return NULL;
    }
    return o;
}

static boat_tensor_t* activation_grad(int act, const boat_tensor_t* saved, const boat_tensor_t* dy) {
    if (saved->nelements != dy->nelements) return NULL;
    boat_tensor_t* dx = bt_new_like_uninit(saved);
    const float* ps = bt_dev_read(saved);
    const float* pg = bt_dev_read(dy);
    float* pd = dx ? bt_dev_write(dx) : NULL;
    if (!ps || !pg || !pd || !boat_hip_ok(bh_activation_backward(act, ps, pg, pd, (int64_t)saved->nelements, 0), "activation backward")) {
        boat_tensor_free(dx);
        return NULL;
    }
    return dx;
}

static boat_tensor_t* row_softmax_grad(bool log_form, const boat_tensor_t* y, const boat_tensor_t* dy) {
    if (y->nelements != dy->nelements || y->nelements == 0) return NULL;
    const int64_t cols = y->ndim > 0 ? y->shape[y->ndim - 1] : 1;
    const int64_t rows = (int64_t)y->nelements / cols;
    boat_tensor_t* dx = bt_new_like_uninit(y);
    const float* py = bt_dev_read(y);
    const float* pg = bt_dev_read(dy);
    float* pd = dx ? bt_dev_write(dx) : NULL;
    int rc = (!py || !pg || !pd) ? BH_EDEVICE
                                 : log_form ? bh_log_softmax_backward(py, pg, pd, rows, cols) : bh_softmax_backward(py, pg, pd, rows, cols);
    if (!boat_hip_ok(rc, "softmax backward")) {
        boat_tensor_free(dx);
        return NULL;
    }
    return dx;
}

/* like * dy[0] (like == NULL: a tensor of shape_of's shape filled with dy[0]).  The reference reads grad_output[0] on
 * the host for sum and dot (autodiff.c:1228, 1536); here the scalar is read by the kernel, so backward never waits for
 * the device. */
static boat_tensor_t* scaled_by_first(const boat_tensor_t* shape_of, const boat_tensor_t* like, const boat_tensor_t* dy) {
    if (!dy || dy->nelements < 1 || !bt_is_f32(dy) || !bt_is_f32(shape_of)) return NULL;
    boat_tensor_t* g = bt_new_like_uninit(shape_of);
    if (!g || g->nelements == 0) return g;
    const float* pin = like ? bt_dev_read(like) : NULL;
    const float* ps = bt_dev_read(dy);
    float* pg = bt_dev_write(g);
    if ((like && !pin) || !ps || !pg ||
        !boat_hip_ok(bh_scale_by_device_scalar(pin, ps, pg, (int64_t)g->nelements), "scale by gradient scalar")) {
        boat_tensor_free(g);
        return NULL;
    }
    return g;
}

/* dx of an activation.  When the activation's input is the output of a dense layer with a bias, read by nothing else in
 * this walk and without a gradient so far, dx is all of that layer's grad_output: its column sums, the layer's bias
 * gradient (dense.c:286-291), are taken in the same pass and the dense rule is told so. */
static boat_tensor_t* activation_grad_of(int act, boat_variable_t* in, const boat_tensor_t* saved, const boat_tensor_t* dy) {
    boat_op_t* p = in->producer;
    if (p && p->type == OP_DENSE && p->mark == g_epoch && in->uses_epoch == g_epoch && in->walk_uses == 1 && !in->grad &&
        !bt_reference_exact()) {
        boat_tensor_t* dx = bt_activation_backward_with_dense_bias(act, saved, dy, (boat_dense_layer_t*)p->layer);
        if (dx) {
            p->bias_done = g_epoch;
            return dx;
        }
    }
    return activation_grad(act, saved, dy);
}

static void backward_op(boat_op_t* op, const boat_tensor_t* dy) {
    boat_variable_t* a = op->inputs[0];
    boat_variable_t* b = op->num_inputs > 1 ? op->inputs[1] : NULL;
    switch (op->type) {
        case OP_ADD:   /* autodiff.c:1002-1061 */
            if (a->requires_grad) accumulate(a, (boat_tensor_t*)dy, false);
            if (b->requires_grad) accumulate(b, (boat_tensor_t*)dy, false);
            break;
        case OP_SUB:   /* :1063-1113 */
            if (a->requires_grad) accumulate(a, (boat_tensor_t*)dy, false);
            if (b->requires_grad) accumulate(b, boat_mul_scalar(dy, -1.0), true);
            break;
        case OP_MUL:   /* :1115-1147 */
            if (a->requires_grad) accumulate(a, boat_mul(dy, b->data), true);
            if (b->requires_grad) accumulate(b, boat_mul(dy, a->data), true);
            break;
        case OP_DIV:   /* :1149-1203 */
            if (a->requires_grad) accumulate(a, boat_div(dy, b->data), true);
            if (b->requires_grad && bt_same_shape(a->data, b->data) && bt_same_shape(a->data, dy)) {
                boat_tensor_t* g = bt_new_like_uninit(b->data);
                float* pg = g ? bt_dev_write(g) : NULL;
                if (pg && boat_hip_ok(bh_div_backward_b(bt_dev_read(a->data), bt_dev_read(b->data), bt_dev_read(dy), pg,
                                                        (int64_t)g->nelements), "div backward"))
                    accumulate(b, g, true);
                else
                    boat_tensor_free(g);
            } else if (b->requires_grad) {   /* broadcast operands: the reference's op-by-op form */
                boat_tensor_t* bsq = boat_mul(b->data, b->data);
                boat_tensor_t* adb = bsq ? boat_div(a->data, bsq) : NULL;
                boat_tensor_t* neg = boat_mul_scalar(dy, -1.0);
                boat_tensor_t* g = (adb && neg) ? boat_mul(neg, adb) : NULL;
                boat_tensor_free(bsq);
                boat_tensor_free(adb);
                boat_tensor_free(neg);
                accumulate(b, g, true);
            }
            break;
        case OP_DOT:     /* :1205-1242: da = b * dy[0], db = a * dy[0] */
            if (a->requires_grad) accumulate(a, scaled_by_first(b->data, b->data, dy), true);
            if (b->requires_grad) accumulate(b, scaled_by_first(a->data, a->data, dy), true);
            break;
        case OP_RELU:      /* :1244-1296, mask from the op input */
            if (a->requires_grad) accumulate(a, activation_grad_of(BH_ACT_RELU, a, a->data, dy), true);
            break;
        case OP_GELU:
            if (a->requires_grad) accumulate(a, activation_grad_of(BH_ACT_GELU, a, a->data, dy), true);
            break;
        case OP_SIGMOID:   /* :1298-1353, from the saved output */
            if (a->requires_grad) accumulate(a, activation_grad_of(BH_ACT_SIGMOID, a, op->output->data, dy), true);
            break;
        case OP_TANH:      /* :1355-1452 */
            if (a->requires_grad) accumulate(a, activation_grad_of(BH_ACT_TANH, a, op->output->data, dy), true);
            break;
        case OP_MATMUL: {  /* :1454-1496, 2-D operands */
            const boat_tensor_t *A = a->data, *B = b->data;
            if (A->ndim != 2 || B->ndim != 2 || dy->ndim != 2) break;
            const int64_t m = A->shape[0], k = A->shape[1], n = B->shape[1];
            if (a->requires_grad) {   /* dA = dY . B^T */
                boat_tensor_t* g = bt_new_like_uninit(A);
                float* pg = g ? bt_dev_write(g) : NULL;
                if (pg && boat_hip_ok(bh_gemm(0, 1, m, k, n, bt_dev_read(dy), n, bt_dev_read(B), n, pg, k, NULL, 0, 1), "matmul backward"))
                    accumulate(a, g, true);
                else
                    boat_tensor_free(g);
            }
            if (b->requires_grad) {   /* dB = A^T . dY */
                boat_tensor_t* g = bt_new_like_uninit(B);
                float* pg = g ? bt_dev_write(g) : NULL;
                if (pg && boat_hip_ok(bh_gemm(1, 0, k, n, m, bt_dev_read(A), k, bt_dev_read(dy), n, pg, n, NULL, 0, 1), "matmul backward"))
                    accumulate(b, g, true);
                else
                    boat_tensor_free(g);
            }
            break;
        }
        case OP_SUM:       /* :1498-1548: ones * (float)dy[0], i.e. dy[0] everywhere */
            if (a->requires_grad) accumulate(a, scaled_by_first(a->data, NULL, dy), true);
            break;
        case OP_MEAN: {    /* :1550-1618: (ones * 1/n) * dy */
            if (!a->requires_grad) break;
            boat_tensor_t* ones = ones_like(a->data);
            boat_tensor_t* scaled = ones ? boat_mul_scalar(ones, 1.0f / a->data->nelements) : NULL;
            boat_tensor_t* g = scaled ? boat_mul(scaled, dy) : NULL;
            boat_tensor_free(ones);
            boat_tensor_free(scaled);
            accumulate(a, g, true);
            break;
        }
        case OP_SOFTMAX:       /* :1885-1973 */
            if (a->requires_grad) accumulate(a, row_softmax_grad(false, op->output->data, dy), true);
            break;
        case OP_LOG_SOFTMAX:   /* :1975-2068 */
            if (a->requires_grad) accumulate(a, row_softmax_grad(true, op->output->data, dy), true);
            break;
        case OP_FLATTEN:       /* :2563-2590 */
            if (a->requires_grad) accumulate(a, boat_tensor_reshape(dy, a->data->shape, a->data->ndim), true);
            break;
        case OP_DENSE: {       /* :2640-2672 */
            boat_tensor_t* dx = (op->bias_done == g_epoch && !bt_reference_exact())
                                    ? bt_dense_layer_backward_bias_done((boat_dense_layer_t*)op->layer, dy)
                                    : boat_dense_layer_backward((boat_dense_layer_t*)op->layer, dy);
            if (dx && a->requires_grad) accumulate(a, dx, true);
            else boat_tensor_free(dx);
            break;
        }
        case OP_CONV: {        /* :2349-2386 */
            boat_tensor_t* dx = boat_conv_layer_backward((boat_conv_layer_t*)op->layer, dy);
            if (dx && a->requires_grad) accumulate(a, dx, true);
            else boat_tensor_free(dx);
            break;
        }
        case OP_POOL: {        /* :2590-2630 */
            boat_tensor_t* dx = boat_pool_layer_backward((boat_pool_layer_t*)op->layer, dy);
            if (dx && a->requires_grad) accumulate(a, dx, true);
            else boat_tensor_free(dx);
            break;
        }
        case OP_LAYERNORM: {
            /* A gradient that reached the input earlier in the walk (the residual connection around a pre-LN branch) is
             * added by the LayerNorm kernel's own store: dx = LN'(dy) + pending replaces the pending tensor. */
            const boat_tensor_t* pending = NULL;
            if (a->requires_grad && a->grad && !a->persistent_grad && !bt_reference_exact() && bt_is_f32(a->grad) &&
                bt_same_shape(a->grad, a->data) && a->data == op->saved[0])
                pending = a->grad;
            boat_tensor_t* dx = boat_layernorm_backward_add_impl((boat_layernorm_t*)op->layer, op->saved[0], op->saved[1], op->saved[2], dy, pending);
            if (dx && pending) {
                boat_tensor_unref(a->grad);
                a->grad = dx;
                a->grad_shared = false;
            } else if (dx && a->requires_grad) {
                accumulate(a, dx, true);
            } else {
                boat_tensor_free(dx);
            }
            break;
        }
        case OP_ATTENTION: {   /* :2458-2532 */
            if (op->inputs[0] == op->inputs[1] && op->inputs[0] == op->inputs[2] && !bt_reference_exact()) {
                /* self-attention: the three input gradients go to one variable; the key and value projections' input
                 * gradients are added into the query projection's by their GEMM epilogues */
                boat_tensor_t* g_in = NULL;
                if (boat_attention_backward_self((boat_attention_t*)op->layer, dy, &g_in) && op->inputs[0]->requires_grad)
                    accumulate(op->inputs[0], g_in, true);
                else
                    boat_tensor_free(g_in);
                break;
            }
            boat_tensor_t *gq = NULL, *gk = NULL, *gv = NULL;
            if (!boat_attention_backward((boat_attention_t*)op->layer, dy, &gq, &gk, &gv)) break;
            boat_variable_t* in[3] = {op->inputs[0], op->inputs[1], op->inputs[2]};
            boat_tensor_t* g[3] = {gq, gk, gv};
            for (int i = 0; i < 3; i++) {
                if (in[i]->requires_grad) accumulate(in[i], g[i], true);
                else boat_tensor_free(g[i]);
            }
            break;
        }
    }
}

/* The loss chain of the MNIST example (examples/mnist/mnist_autodiff.c:397-522), loss = f * sum(onehot o log_softmax(z))
 * with f and onehot constants, recognised at the root of a walk: its four gradient rules (mul :1115-1147, sum :1498-1548,
 * mul, log-softmax :1975-2068) run as one kernel that keeps their operations and order, so z receives the same bits.
 * Only when nothing else in the walk reads the intermediate variables and none of them holds a gradient yet; their own
 * gradients are then not materialised.  Returns true when z's gradient has been accumulated and the four ops are done. */
static bool fuse_log_softmax_loss(boat_variable_t* root, const boat_tensor_t* seed, uint64_t epoch) {
    boat_op_t* r = root->producer;
    if (!r || r->type != OP_MUL || root->data->nelements != 1 || (seed && (!bt_is_f32(seed) || seed->nelements < 1))) return false;
    boat_variable_t* vf = r->inputs[0]->requires_grad ? r->inputs[1] : r->inputs[0];
    boat_variable_t* s = r->inputs[0]->requires_grad ? r->inputs[0] : r->inputs[1];
    if (vf == s || vf->requires_grad || !s->requires_grad || !bt_is_f32(vf->data) || vf->data->nelements != 1) return false;
    boat_op_t* sum = s->producer;
    if (!sum || sum->type != OP_SUM || s->walk_uses != 1 || s->grad || s->data->nelements != 1) return false;
    boat_variable_t* m = sum->inputs[0];
    boat_op_t* mul = m->producer;
    if (!mul || mul->type != OP_MUL || m->walk_uses != 1 || m->grad || !m->requires_grad) return false;
    boat_variable_t* w = mul->inputs[0]->requires_grad ? mul->inputs[1] : mul->inputs[0];
    boat_variable_t* ls = mul->inputs[0]->requires_grad ? mul->inputs[0] : mul->inputs[1];
    if (w == ls || w->requires_grad || !ls->requires_grad || !bt_is_f32(w->data) || !bt_same_shape(w->data, ls->data) ||
        !bt_same_shape(m->data, ls->data))
        return false;
    boat_op_t* lsm = ls->producer;
    if (!lsm || lsm->type != OP_LOG_SOFTMAX || ls->walk_uses != 1 || ls->grad || !bt_is_f32(ls->data) || ls->data->ndim < 1) return false;
    boat_variable_t* z = lsm->inputs[0];
    if (!z->requires_grad || !bt_same_shape(z->data, ls->data) || ls->data->nelements == 0) return false;
    const int64_t cols = ls->data->shape[ls->data->ndim - 1];
    const int64_t rows = (int64_t)ls->data->nelements / cols;
    boat_tensor_t* dz = bt_new_like_uninit(z->data);
    const float* py = dz ? bt_dev_read(ls->data) : NULL;
    const float* pw = py ? bt_dev_read(w->data) : NULL;
    const float* pf = pw ? bt_dev_read(vf->data) : NULL;
    const float* ps = (pf && seed) ? bt_dev_read(seed) : NULL;
    float* pd = pf ? bt_dev_write(dz) : NULL;
    /* z straight out of a dense layer and read by nothing else: dz is that layer's whole grad_output, and its bias gradient
     * (the column sums, dense.c:286-291) comes out of the same launch */
    boat_op_t* zp = z->producer;
    int acc = 1;
    float* pgb = (pd && (!seed || ps) && zp && zp->type == OP_DENSE && zp->mark == epoch && z->uses_epoch == epoch && z->walk_uses == 1 &&
                  !z->grad && z->data->ndim == 2)
                     ? bt_dense_bias_grad_target((boat_dense_layer_t*)zp->layer, cols, &acc)
                     : NULL;
    if (!pd || (seed && !ps) ||
        !boat_hip_ok(pgb ? bh_log_softmax_weighted_backward_colsum(py, pw, ps, pf, pd, pgb, rows, cols, acc)
                         : bh_log_softmax_weighted_backward(py, pw, ps, pf, pd, rows, cols),
                     "loss chain backward")) {
        boat_tensor_free(dz);
        return false;
    }
    if (pgb) zp->bias_done = epoch;
    r->skip = sum->skip = mul->skip = lsm->skip = epoch;
    accumulate(z, dz, true);
    return true;
}

static int by_seq_desc(const void* x, const void* y) {
    const boat_op_t* a = *(boat_op_t* const*)x;
    const boat_op_t* b = *(boat_op_t* const*)y;
    return a->seq < b->seq ? 1 : a->seq > b->seq ? -1 : 0;
}

/* Reference-exact mode: the reference's own walk (autodiff.c:373-450), depth first from the root: run the op's gradient
 * rule, then descend into every non-leaf input with that input's gradient AS ACCUMULATED SO FAR.  A non-leaf variable
 * with several consumers is therefore descended into once per consumer, each time with a larger gradient: z = y + y,
 * y = a*b gives da = 4b where the true gradient is 2b. */
static void backward_depth_first(boat_variable_t* v, const boat_tensor_t* dy) {
    boat_op_t* op = v->producer;
    backward_op(op, dy);
    for (size_t i = 0; i < op->num_inputs; i++) {
        boat_variable_t* in = op->inputs[i];
        if (!in || !in->requires_grad || !in->grad || !in->producer) continue;
        boat_tensor_t* g = in->grad;
        boat_tensor_ref(g);
        backward_depth_first(in, g);
        boat_tensor_unref(g);
    }
}

static void backward_walk(boat_variable_t* variable, boat_tensor_t* grad_output);
static void boat_variable_backward_unflushed(boat_variable_t* variable, boat_tensor_t* grad_output) {
    g_walk_seed = grad_output;
    backward_walk(variable, grad_output);
    g_walk_seed = NULL;
}
static void backward_walk(boat_variable_t* variable, boat_tensor_t* grad_output) {
    if (!variable || !variable->requires_grad) return;
    boat_tensor_t* seed = grad_output;
    if (!seed && !bt_is_f32(variable->data)) return;
    if (!seed && (!variable->producer || bt_reference_exact())) {   /* (the walk below makes its own when it needs one) */
        seed = ones_like(variable->data);   /* autodiff.c:313-338 */
        if (!seed) return;
    }
    if (!variable->producer) {
        accumulate(variable, seed, false);  /* leaf: grad += dY (autodiff.c:346-361) */
        if (!grad_output) boat_tensor_unref(seed);
        return;
    }
    if (bt_reference_exact()) {
        backward_depth_first(variable, seed);
        if (!grad_output) boat_tensor_unref(seed);
        return;
    }
    /* collect the ops reachable from the root, each once */
    const uint64_t epoch = ++g_epoch;
    size_t n = 0, cap = 64, head = 0;
    boat_op_t** ops = (boat_op_t**)malloc(cap * sizeof(*ops));
    if (!ops) return;
    variable->producer->mark = epoch;
    ops[n++] = variable->producer;
    while (head < n) {
        boat_op_t* op = ops[head++];
        for (size_t i = 0; i < op->num_inputs; i++) {
            boat_variable_t* in = op->inputs[i];
            if (in) {
                if (in->uses_epoch != epoch) {
                    in->uses_epoch = epoch;
                    in->walk_uses = 0;
                }
                in->walk_uses++;
            }
            if (!in || !in->requires_grad || !in->producer || in->producer->mark == epoch) continue;
            in->producer->mark = epoch;
            if (n == cap) {
                boat_op_t** grown = (boat_op_t**)realloc(ops, 2 * cap * sizeof(*ops));
                if (!grown) break;
                ops = grown;
                cap *= 2;
            }
            ops[n++] = in->producer;
        }
    }
    qsort(ops, n, sizeof(*ops), by_seq_desc);
    /* the example's loss chain at the root: one kernel, and without a grad_output not even the tensor of ones */
    const bool fused_root = fuse_log_softmax_loss(variable, grad_output, epoch);
    if (!fused_root && !seed) {
        seed = bt_is_f32(variable->data) ? ones_like(variable->data) : NULL;   /* autodiff.c:313-338 */
        if (!seed) {
            free(ops);
            return;
        }
    }
    /* reverse recording order: every consumer of a variable runs before its producer */
    for (size_t i = 0; i < n; i++) {
        boat_op_t* op = ops[i];
        if (op->skip == epoch) continue;
        const boat_tensor_t* dy = op == variable->producer ? seed : op->output->grad;
        g_lender = op == variable->producer ? NULL : op->output;
        if (dy) backward_op(op, dy);
    }
    g_lender = NULL;
    free(ops);
    if (!grad_output && seed) boat_tensor_unref(seed);
}
void boat_variable_backward(boat_variable_t* variable, boat_tensor_t* grad_output) {
    boat_variable_backward_unflushed(variable, grad_output);
    bt_flush_exposed();
}

/* gradient checkpointing is a stub in the reference too (autodiff.c:652-655): every op keeps what its backward needs */
void boat_autodiff_set_grad_checkpointing(bool enabled) { (void)enabled; }

static const char* op_name(op_type_t t) {
    static const char* names[] = {"add", "sub", "mul", "div", "relu", "sigmoid", "tanh", "matmul", "dot", "sum", "mean",
                                  "softmax", "log_softmax", "flatten", "dense", "attention", "gelu", "layernorm", "conv", "pool"};
    return (size_t)t < sizeof(names) / sizeof(names[0]) ? names[t] : "?";
}

/* the ops `variable` depends on, in recording order; caller frees.  (The reference declares graph printing and DOT
 * export, autodiff.h:97-98, and leaves both empty, autodiff.c:727-736.) */
static boat_op_t** tape_of(const boat_variable_t* variable, size_t* count) {
    *count = 0;
    if (!variable || !variable->producer) return NULL;
    const uint64_t epoch = ++g_epoch;
    size_t n = 0, cap = 64, head = 0;
    boat_op_t** ops = (boat_op_t**)malloc(cap * sizeof(*ops));
    if (!ops) return NULL;
    variable->producer->mark = epoch;
    ops[n++] = variable->producer;
    while (head < n) {
        boat_op_t* op = ops[head++];
        for (size_t i = 0; i < op->num_inputs; i++) {
            boat_variable_t* in = op->inputs[i];
            if (!in || !in->producer || in->producer->mark == epoch) continue;
            if (n == cap) {
                boat_op_t** grown = (boat_op_t**)realloc(ops, 2 * cap * sizeof(*ops));
                if (!grown) break;
                ops = grown;
                cap *= 2;
            }
            in->producer->mark = epoch;
            ops[n++] = in->producer;
        }
    }
    qsort(ops, n, sizeof(*ops), by_seq_desc);
    for (size_t i = 0; i < n / 2; i++) {   /* ascending recording order */
        boat_op_t* t = ops[i];
        ops[i] = ops[n - 1 - i];
        ops[n - 1 - i] = t;
    }
    *count = n;
    return ops;
}

static int shape_text(char* buf, size_t cap, const boat_tensor_t* t) {
    int off = snprintf(buf, cap, "[");
    for (size_t i = 0; t && i < t->ndim && (size_t)off < cap; i++)
        off += snprintf(buf + off, cap - (size_t)off, i ? ",%lld" : "%lld", (long long)t->shape[i]);
    if ((size_t)off < cap) off += snprintf(buf + off, cap - (size_t)off, "]");
    return off;
}

void boat_autodiff_print_graph(const boat_variable_t* variable) {
    size_t n = 0;
    boat_op_t** ops = tape_of(variable, &n);
    if (!ops) return;
    for (size_t i = 0; i < n; i++) {
        char shape[128];
        shape_text(shape, sizeof(shape), ops[i]->output ? ops[i]->output->data : NULL);
        printf("%3zu: %-12s -> %s%s\n", i, op_name(ops[i]->type), shape,
               ops[i]->output && ops[i]->output->requires_grad ? " (grad)" : "");
    }
    free(ops);
}

/* Graphviz text of the tape behind `variable` (malloc'ed; the caller frees it), NULL for a leaf */
char* boat_autodiff_graph_to_dot(const boat_variable_t* variable) {
    size_t n = 0;
    boat_op_t** ops = tape_of(variable, &n);
    if (!ops) return NULL;
    size_t cap = 256 + n * 512, off = 0;
    char* out = (char*)malloc(cap);
    if (!out) {
        free(ops);
        return NULL;
    }
    off += (size_t)snprintf(out + off, cap - off, "digraph boat_tape {\n");
    for (size_t i = 0; i < n && off + 400 < cap; i++) {
        char shape[128];
        shape_text(shape, sizeof(shape), ops[i]->output ? ops[i]->output->data : NULL);
        off += (size_t)snprintf(out + off, cap - off, "  v%p [label=\"%s %s\"];\n", (void*)ops[i]->output, op_name(ops[i]->type), shape);
        for (size_t j = 0; j < ops[i]->num_inputs; j++)
            off += (size_t)snprintf(out + off, cap - off, "  v%p -> v%p;\n", (void*)ops[i]->inputs[j], (void*)ops[i]->output);
    }
    snprintf(out + off, cap - off, "}\n");
    free(ops);
    return out;
}

void boat_variable_backward_full(const boat_variable_t* variable) {
    if (!variable || !variable->requires_grad) return;
    boat_variable_backward((boat_variable_t*)variable, NULL);
}
