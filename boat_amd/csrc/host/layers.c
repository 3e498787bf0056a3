/* layers.c - stateful layers whose forward caches what backward needs; all arithmetic on the GPU.
 *
 * Same hooks, ownership and error behaviour as the reference:
 *   dense      src/layers/dense.c:25-395   (weight [in,out]; backward returns a NEW dX tensor and
 *                                           ACCUMULATES grad_weight/grad_bias; update = SGD + clear)
 *   relu/softmax layers  src/layers/relu.c:24-77, src/layers/softmax.c:20-63 (backward passes the
 *                                           incoming gradient through with ref++ -- kept as is)
 *   layernorm  src/layers/norm.c:13-317,397-550 (forward as the reference; backward/update are
 *                                           stubs there and are implemented here)
 *   attention  src/layers/attention.c:49-815,882-1534 (projections [in,out]; head split is a plain
 *                                           reshape [B,S,H]->[B,nh,S,hd]; parameter grads are
 *                                           OVERWRITTEN per backward call, not accumulated)
 */
#include "boat_internal.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* Xavier-style uniform init drawn from libc rand() exactly as dense.c:61-67 / attention.c:92-105 do,
 * so the same srand() seed gives the same weights as the reference. */
static boat_tensor_t* create_linear_weights(size_t in_features, size_t out_features) {
    const int64_t shape[] = {(int64_t)in_features, (int64_t)out_features};
    boat_tensor_t* w = boat_tensor_create(shape, 2, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    if (!w) return NULL;
    float* data = (float*)bt_host_rw(w);
    if (!data) {
        boat_tensor_free(w);
        return NULL;
    }
    const size_t n = w->nelements;
    const float scale = sqrtf(2.0f / (in_features + out_features));
    for (size_t i = 0; i < n; i++) data[i] = ((float)rand() / RAND_MAX) * 2.0f * scale - scale;
    return w;
}

static boat_tensor_t* create_vector(size_t n) {
    const int64_t shape[] = {(int64_t)n};
    return boat_tensor_create(shape, 1, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);   /* zero-filled */
}

static void swap_tensor(boat_tensor_t** slot, boat_tensor_t* fresh) {
    if (*slot) boat_tensor_unref(*slot);
    *slot = fresh;
    if (fresh) boat_tensor_ref(fresh);
}

/* ------------------------------------------------------------------- dense */

boat_dense_layer_t* boat_dense_layer_create(size_t input_features, size_t output_features, bool use_bias) {
    boat_dense_layer_t* layer = (boat_dense_layer_t*)calloc(1, sizeof(*layer));
    if (!layer) return NULL;
    layer->input_features = input_features;
    layer->output_features = output_features;
    layer->use_bias = use_bias;
    layer->weight = create_linear_weights(input_features, output_features);
    const int64_t wshape[] = {(int64_t)input_features, (int64_t)output_features};
    layer->grad_weight = boat_tensor_create(wshape, 2, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    if (use_bias) {
        layer->bias = create_vector(output_features);
        layer->grad_bias = create_vector(output_features);
    }
    if (!layer->weight || !layer->grad_weight || (use_bias && (!layer->bias || !layer->grad_bias))) {
        boat_dense_layer_free(layer);
        return NULL;
    }
    return layer;
}

void boat_dense_layer_free(boat_dense_layer_t* layer) {
    if (!layer) return;
    boat_tensor_free(layer->weight);
    boat_tensor_free(layer->bias);
    boat_tensor_free(layer->grad_weight);
    boat_tensor_free(layer->grad_bias);
    if (layer->cache_input) boat_tensor_unref(layer->cache_input);
    free(layer);
}

boat_tensor_t* boat_dense_layer_forward(boat_dense_layer_t* layer, const boat_tensor_t* input) {
    if (!layer || !input) return NULL;
    swap_tensor(&layer->cache_input, (boat_tensor_t*)input);
    if (!bt_is_f32(input) || input->ndim != 2 || input->shape[1] != (int64_t)layer->input_features) return NULL;
    const int64_t m = input->shape[0], k = input->shape[1], n = (int64_t)layer->output_features;
    const int64_t shape[] = {m, n};
    boat_tensor_t* out = bt_new_uninit(shape, 2, input->device);
    if (!out || out->nelements == 0) return out;
    const float* px = bt_dev_read(input);
    const float* pw = bt_dev_read(layer->weight);
    const float* pb = (layer->use_bias && layer->bias) ? bt_dev_read(layer->bias) : NULL;
    float* py = bt_dev_write(out);
    if (!px || !pw || !py || !boat_hip_ok(bh_gemm(0, 0, m, n, k, px, k, pw, n, py, n, pb, 0, 1), "dense forward")) {
        boat_tensor_free(out);
        return NULL;
    }
    return out;
}

static boat_tensor_t* dense_backward_impl(boat_dense_layer_t* layer, const boat_tensor_t* grad_output, bool bias_done) {
    if (!layer || !grad_output || !layer->cache_input) return NULL;
    const boat_tensor_t* input = layer->cache_input;
    if (input->ndim != 2 || grad_output->ndim != 2) {
        fprintf(stderr, "Error: Dense layer backward expects 2D tensors\n");
        return NULL;
    }
    const int64_t m = input->shape[0], k = input->shape[1], n = grad_output->shape[1];
    if (k != (int64_t)layer->input_features || n != (int64_t)layer->output_features || grad_output->shape[0] != m) {
        fprintf(stderr, "Error: Dense layer backward shape mismatch\n");
        return NULL;
    }
    if (!bt_is_f32(grad_output) || !bt_is_f32(input)) return NULL;
    const int64_t shape[] = {m, k};
    boat_tensor_t* dx = bt_new_uninit(shape, 2, grad_output->device);
    if (!dx) return NULL;
    if (!layer->grad_weight) layer->grad_weight = boat_tensor_create_like(layer->weight);
    const bool with_bias = layer->use_bias && layer->bias && !bias_done;   /* (done: the caller has already added this call's column sums) */
    if (with_bias && !layer->grad_bias) layer->grad_bias = boat_tensor_create_like(layer->bias);
    const float* px = bt_dev_read(input);
    const float* pw = bt_dev_read(layer->weight);
    const float* pg = bt_dev_read(grad_output);
    float* pdx = bt_dev_write(dx);
    /* the parameter gradients accumulate (dense.c:255-291); into gradients that are still the zeros of a zero_grad
     * nobody has looked at since, the kernels write instead of adding */
    boat_tensor_t* gb = (with_bias && layer->grad_bias) ? layer->grad_bias : NULL;
    const bool fresh = bt_is_zero(layer->grad_weight) && (!gb || bt_is_zero(gb));
    float* pgw = !layer->grad_weight ? NULL : fresh ? bt_dev_write(layer->grad_weight) : bt_dev_rw(layer->grad_weight);
    float* pgb = !gb ? NULL : fresh ? bt_dev_write(gb) : bt_dev_rw(gb);
    if (!px || !pw || !pg || !pdx || !pgw ||
        !boat_hip_ok(bh_dense_backward(px, pw, pg, pdx, pgw, pgb, m, k, n, fresh ? 0 : 1), "dense backward")) {
        boat_tensor_free(dx);
        return NULL;
    }
    return dx;
}
boat_tensor_t* bt_dense_layer_backward_bias_done(boat_dense_layer_t* layer, const boat_tensor_t* grad_output) {
    boat_tensor_t* result = dense_backward_impl(layer, grad_output, true);
    bt_flush_exposed();
    return result;
}
float* bt_dense_bias_grad_target(boat_dense_layer_t* layer, int64_t cols, int* accumulate) {
    if (!layer || !(layer->use_bias && layer->bias) || cols != (int64_t)layer->output_features) return NULL;
    if (!layer->grad_bias) layer->grad_bias = boat_tensor_create_like(layer->bias);
    return layer->grad_bias ? bt_dev_accumulate(layer->grad_bias, accumulate) : NULL;
}
boat_tensor_t* bt_activation_backward_with_dense_bias(int act, const boat_tensor_t* saved, const boat_tensor_t* dy,
                                                      boat_dense_layer_t* layer) {
    if (!layer || !saved || !dy || !(layer->use_bias && layer->bias) || !bt_is_f32(saved) || !bt_is_f32(dy) || dy->ndim != 2 ||
        !bt_same_shape(saved, dy) || dy->shape[1] != (int64_t)layer->output_features || dy->nelements == 0)
        return NULL;
    if (!layer->grad_bias) layer->grad_bias = boat_tensor_create_like(layer->bias);
    boat_tensor_t* dx = layer->grad_bias ? bt_new_like_uninit(saved) : NULL;
    if (!dx) return NULL;
    const float* ps = bt_dev_read(saved);
    const float* pg = bt_dev_read(dy);
    float* pd = bt_dev_write(dx);
    int acc = 1;
    float* pgb = (ps && pg && pd) ? bt_dev_accumulate(layer->grad_bias, &acc) : NULL;
    if (!pgb || !boat_hip_ok(bh_activation_backward_colsum(act, ps, pg, pd, pgb, dy->shape[0], dy->shape[1], acc),
                             "activation backward with the bias gradient")) {
        boat_tensor_free(dx);
        return NULL;
    }
    return dx;
}
boat_tensor_t* boat_dense_layer_backward(boat_dense_layer_t* layer, const boat_tensor_t* grad_output) {
    boat_tensor_t* result = dense_backward_impl(layer, grad_output, false);
    bt_flush_exposed();
    return result;
}

static void sgd_step(boat_tensor_t* p, boat_tensor_t* g, float lr, bool clear) {
    if (!p || !g || p->nelements != g->nelements || p->nelements == 0) return;
    float* pp = bt_dev_rw(p);
    float* pg = bt_dev_rw(g);
    if (pp && pg) boat_hip_ok(bh_sgd_update(pp, pg, lr, (int64_t)p->nelements, clear), "sgd update");
}

void boat_dense_layer_update(boat_dense_layer_t* layer, float learning_rate) {
    if (!layer) return;
    sgd_step(layer->weight, layer->grad_weight, learning_rate, true);
    if (layer->use_bias) sgd_step(layer->bias, layer->grad_bias, learning_rate, true);
    bt_flush_exposed();
}

void boat_dense_layer_set_weight(boat_dense_layer_t* layer, boat_tensor_t* weight) {
    if (!layer || !weight) return;
    if (weight->ndim != 2 || weight->shape[0] != (int64_t)layer->input_features || weight->shape[1] != (int64_t)layer->output_features) {
        fprintf(stderr, "Error: Weight shape does not match layer dimensions [%zu, %zu]\n", layer->input_features, layer->output_features);
        return;
    }
    swap_tensor(&layer->weight, weight);
}
void boat_dense_layer_set_bias(boat_dense_layer_t* layer, boat_tensor_t* bias) {
    if (!layer || !bias) return;
    if (!layer->use_bias) {
        fprintf(stderr, "Warning: Layer was created without bias, ignoring bias tensor\n");
        return;
    }
    if (bias->ndim < 1 || bias->shape[0] != (int64_t)layer->output_features) {
        fprintf(stderr, "Error: Bias shape does not match output features %zu\n", layer->output_features);
        return;
    }
    swap_tensor(&layer->bias, bias);
}
boat_tensor_t* boat_dense_layer_get_weight(const boat_dense_layer_t* l) { return l ? l->weight : NULL; }
boat_tensor_t* boat_dense_layer_get_bias(const boat_dense_layer_t* l) { return l ? l->bias : NULL; }
boat_tensor_t* boat_dense_layer_get_grad_weight(const boat_dense_layer_t* l) { return l ? l->grad_weight : NULL; }
boat_tensor_t* boat_dense_layer_get_grad_bias(const boat_dense_layer_t* l) { return l ? l->grad_bias : NULL; }

/* ------------------------------------------------- relu / softmax layer hooks */

struct boat_relu_layer_t { char dummy; };
boat_relu_layer_t* boat_relu_layer_create(void) { return (boat_relu_layer_t*)calloc(1, sizeof(boat_relu_layer_t)); }
void boat_relu_layer_free(boat_relu_layer_t* layer) { free(layer); }
boat_tensor_t* boat_relu_layer_forward(const boat_relu_layer_t* layer, const boat_tensor_t* input) {
    if (!layer || !input) return NULL;
    return boat_relu(input);
}
boat_tensor_t* boat_relu_layer_backward(boat_relu_layer_t* layer, const boat_tensor_t* grad_output) {
    (void)layer;
    if (!grad_output) return NULL;
    boat_tensor_ref((boat_tensor_t*)grad_output);   /* pass-through, as relu.c:58-72 */
    return (boat_tensor_t*)grad_output;
}
void boat_relu_layer_update(boat_relu_layer_t* layer, float learning_rate) {
    (void)layer;
    (void)learning_rate;
}

struct boat_softmax_layer_t { int axis; };
boat_softmax_layer_t* boat_softmax_layer_create(int axis) {
    boat_softmax_layer_t* l = (boat_softmax_layer_t*)calloc(1, sizeof(*l));
    if (l) l->axis = axis;
    return l;
}
void boat_softmax_layer_free(boat_softmax_layer_t* layer) { free(layer); }
boat_tensor_t* boat_softmax_layer_forward(const boat_softmax_layer_t* layer, const boat_tensor_t* input) {
    if (!layer || !input) return NULL;
    return boat_softmax(input, layer->axis);
}
boat_tensor_t* boat_softmax_layer_backward(boat_softmax_layer_t* layer, const boat_tensor_t* grad_output) {
    (void)layer;
    if (!grad_output) return NULL;
    boat_tensor_ref((boat_tensor_t*)grad_output);   /* caller passes p - onehot (softmax.c:43-58) */
    return (boat_tensor_t*)grad_output;
}
void boat_softmax_layer_update(boat_softmax_layer_t* layer, float learning_rate) {
    (void)layer;
    (void)learning_rate;
}

/* --------------------------------------------------------------- layernorm */

boat_layernorm_t* boat_layernorm_create(const boat_layernorm_config_t* config) {
    if (!config || config->normalized_shape == 0) return NULL;
    boat_layernorm_t* norm = (boat_layernorm_t*)calloc(1, sizeof(*norm));
    if (!norm) return NULL;
    norm->config = *config;
    if (config->elementwise_affine) {
        norm->weight = create_vector(config->normalized_shape);
        norm->grad_weight = create_vector(config->normalized_shape);
        float* g = norm->weight ? (float*)bt_host_rw(norm->weight) : NULL;
        if (!g || !norm->grad_weight) {
            boat_layernorm_free(norm);
            return NULL;
        }
        for (size_t i = 0; i < config->normalized_shape; i++) g[i] = 1.0f;
        if (config->use_bias) {
            norm->bias = create_vector(config->normalized_shape);
            norm->grad_bias = create_vector(config->normalized_shape);
            if (!norm->bias || !norm->grad_bias) {
                boat_layernorm_free(norm);
                return NULL;
            }
        }
    }
    return norm;
}

void boat_layernorm_free(boat_layernorm_t* norm) {
    if (!norm) return;
    boat_tensor_free(norm->weight);
    boat_tensor_free(norm->bias);
    boat_tensor_free(norm->grad_weight);
    boat_tensor_free(norm->grad_bias);
    boat_tensor_free(norm->cache_input);
    boat_tensor_free(norm->cache_mean);
    boat_tensor_free(norm->cache_rstd);
    free(norm);
}

/* rows the reference's loop nest visits (norm.c:279-281): the product of the first two dims for
 * ndim >= 3, the first dim for 2-D, one row for 1-D; any further rows stay zero. */
static int64_t layernorm_rows(const boat_tensor_t* t) {
    if (t->ndim >= 3) return t->shape[0] * t->shape[1];
    if (t->ndim == 2) return t->shape[0];
    return 1;
}

boat_tensor_t* boat_layernorm_forward(boat_layernorm_t* norm, const boat_tensor_t* input) {
    if (!norm || !input || input->ndim < 1 || !bt_is_f32(input)) return NULL;
    const int64_t hidden = (int64_t)norm->config.normalized_shape;
    if (input->shape[input->ndim - 1] != hidden) return NULL;
    const int64_t rows = layernorm_rows(input);
    const bool covers_all = rows * hidden == (int64_t)input->nelements;
    boat_tensor_t* out = covers_all ? bt_new_like_uninit(input) : boat_tensor_create_like(input);
    const int64_t rshape[] = {rows};
    boat_tensor_t* mean = bt_new_uninit(rshape, 1, input->device);
    boat_tensor_t* rstd = bt_new_uninit(rshape, 1, input->device);
    bool ok = out && mean && rstd;
    if (ok && rows > 0) {
        const float* px = bt_dev_read(input);
        const float* pg = norm->weight ? bt_dev_read(norm->weight) : NULL;
        const float* pb = norm->bias ? bt_dev_read(norm->bias) : NULL;
        float* py = covers_all ? bt_dev_write(out) : bt_dev_rw(out);
        ok = px && py &&
             boat_hip_ok(bh_layernorm_forward(px, pg, pb, py, bt_dev_write(mean), bt_dev_write(rstd), rows, hidden, norm->config.eps),
                         "layernorm forward");
    }
    if (!ok) {
        boat_tensor_free(out);
        boat_tensor_free(mean);
        boat_tensor_free(rstd);
        return NULL;
    }
    swap_tensor(&norm->cache_input, (boat_tensor_t*)input);
    boat_tensor_free(norm->cache_mean);
    boat_tensor_free(norm->cache_rstd);
    norm->cache_mean = mean;
    norm->cache_rstd = rstd;
    return out;
}

boat_tensor_t* boat_layernorm_backward_impl(boat_layernorm_t* norm, const boat_tensor_t* x, const boat_tensor_t* mean,
                                            const boat_tensor_t* rstd, const boat_tensor_t* grad_output) {
    return boat_layernorm_backward_add_impl(norm, x, mean, rstd, grad_output, NULL);
}
boat_tensor_t* boat_layernorm_backward_add_impl(boat_layernorm_t* norm, const boat_tensor_t* x, const boat_tensor_t* mean,
                                                const boat_tensor_t* rstd, const boat_tensor_t* grad_output, const boat_tensor_t* add) {
    if (!norm || !x || !mean || !rstd || !grad_output) return NULL;
    if (add && (!bt_is_f32(add) || add->nelements != x->nelements)) return NULL;
    if (!bt_is_f32(grad_output) || grad_output->nelements != x->nelements) {
        fprintf(stderr, "Error: LayerNorm backward shape mismatch\n");
        return NULL;
    }
    const int64_t hidden = (int64_t)norm->config.normalized_shape;
    const int64_t rows = (int64_t)mean->nelements;
    const bool covers_all = rows * hidden == (int64_t)x->nelements;
    if (add && (!covers_all || rows == 0)) {
        /* rows the kernel does not visit keep the other gradient alone: start from a copy of it */
        boat_tensor_t* base = boat_tensor_clone(add);
        boat_tensor_t* part = base ? boat_layernorm_backward_add_impl(norm, x, mean, rstd, grad_output, NULL) : NULL;
        if (part) boat_add_(base, part);
        else {
            boat_tensor_free(base);
            base = NULL;
        }
        boat_tensor_free(part);
        return base;
    }
    boat_tensor_t* dx = covers_all ? bt_new_like_uninit(x) : boat_tensor_create_like(x);
    if (!dx) return NULL;
    if (rows == 0) return dx;
    const float* px = bt_dev_read(x);
    const float* pdy = bt_dev_read(grad_output);
    const float* pg = norm->weight ? bt_dev_read(norm->weight) : NULL;
    const float* padd = add ? bt_dev_read(add) : NULL;
    float* pdx = covers_all ? bt_dev_write(dx) : bt_dev_rw(dx);
    /* parameter gradients accumulate across calls like the dense layer's (dense.c:255-291), or are written when they
     * are still the untouched zeros of a zero_grad */
    const bool fresh = (!norm->grad_weight || bt_is_zero(norm->grad_weight)) && (!norm->grad_bias || bt_is_zero(norm->grad_bias));
    float* pgw = !norm->grad_weight ? NULL : fresh ? bt_dev_write(norm->grad_weight) : bt_dev_rw(norm->grad_weight);
    float* pgb = !norm->grad_bias ? NULL : fresh ? bt_dev_write(norm->grad_bias) : bt_dev_rw(norm->grad_bias);
    const int acc = fresh ? 0 : 1;
    bool ok = px && pdy && pdx && (padd || !add);
    if (ok && add) ok = boat_hip_ok(bh_layernorm_backward_add(px, pg, pdy, bt_dev_read(mean), bt_dev_read(rstd), padd, pdx, pgw, pgb, rows, hidden, acc),
                                    "layernorm backward");
    else if (ok) ok = boat_hip_ok(bh_layernorm_backward(px, pg, pdy, bt_dev_read(mean), bt_dev_read(rstd), pdx, pgw, pgb, rows, hidden, acc),
                                  "layernorm backward");
    if (!ok) {
        boat_tensor_free(dx);
        return NULL;
    }
    return dx;
}

static boat_tensor_t* boat_layernorm_backward_unflushed(boat_layernorm_t* norm, const boat_tensor_t* grad_output) {
    if (!norm || !grad_output) return NULL;
    if (!norm->cache_input || !norm->cache_mean || !norm->cache_rstd) {
        fprintf(stderr, "Error: LayerNorm backward called before forward\n");
        return NULL;
    }
    return boat_layernorm_backward_impl(norm, norm->cache_input, norm->cache_mean, norm->cache_rstd, grad_output);
}
boat_tensor_t* boat_layernorm_backward(boat_layernorm_t* norm, const boat_tensor_t* grad_output) {
    boat_tensor_t* result = boat_layernorm_backward_unflushed(norm, grad_output);
    bt_flush_exposed();
    return result;
}

void boat_layernorm_update(boat_layernorm_t* norm, float learning_rate) {
    if (!norm) return;
    sgd_step(norm->weight, norm->grad_weight, learning_rate, true);
    sgd_step(norm->bias, norm->grad_bias, learning_rate, true);
    bt_flush_exposed();
}

void boat_layernorm_set_weight(boat_layernorm_t* norm, boat_tensor_t* weight) {
    if (!norm || !weight || weight->nelements != norm->config.normalized_shape) return;
    swap_tensor(&norm->weight, weight);
    if (!norm->grad_weight) norm->grad_weight = create_vector(norm->config.normalized_shape);
}
void boat_layernorm_set_bias(boat_layernorm_t* norm, boat_tensor_t* bias) {
    if (!norm || !bias || bias->nelements != norm->config.normalized_shape) return;
    swap_tensor(&norm->bias, bias);
    if (!norm->grad_bias) norm->grad_bias = create_vector(norm->config.normalized_shape);
}
boat_tensor_t* boat_hip_layernorm_get_weight(const boat_layernorm_t* n) { return n ? n->weight : NULL; }
boat_tensor_t* boat_hip_layernorm_get_bias(const boat_layernorm_t* n) { return n ? n->bias : NULL; }
boat_tensor_t* boat_hip_layernorm_get_grad_weight(const boat_layernorm_t* n) { return n ? n->grad_weight : NULL; }
boat_tensor_t* boat_hip_layernorm_get_grad_bias(const boat_layernorm_t* n) { return n ? n->grad_bias : NULL; }

/* stateless input gradient (no affine): recomputes the statistics from `input` */
boat_tensor_t* boat_layer_norm_grad(const boat_tensor_t* grad_output, const boat_tensor_t* input, const boat_tensor_t* output,
                                    const int64_t* normalized_shape, size_t normalized_shape_len, float eps) {
    (void)output;
    if (!grad_output || !input || !normalized_shape || normalized_shape_len != 1) return NULL;
    boat_layernorm_config_t cfg = {(size_t)normalized_shape[0], eps, false, false};
    boat_layernorm_t* tmp = boat_layernorm_create(&cfg);
    if (!tmp) return NULL;
    boat_tensor_t* y = boat_layernorm_forward(tmp, input);
    boat_tensor_t* dx = y ? boat_layernorm_backward(tmp, grad_output) : NULL;
    boat_tensor_free(y);
    boat_layernorm_free(tmp);
    return dx;
}

/* stateless forms (stubs in the reference, norm.c:424-448): normalisation over the last dimension, no affine */
boat_tensor_t* boat_layer_norm(const boat_tensor_t* input, const int64_t* normalized_shape, size_t normalized_shape_len, float eps) {
    if (!input || !normalized_shape || normalized_shape_len != 1) return NULL;
    boat_layernorm_config_t cfg = {(size_t)normalized_shape[0], eps, false, false};
    boat_layernorm_t* tmp = boat_layernorm_create(&cfg);
    if (!tmp) return NULL;
    boat_tensor_t* y = boat_layernorm_forward(tmp, input);
    boat_layernorm_free(tmp);
    return y;
}

/* ----------------------------------------------------------------- rmsnorm
 * src/layers/norm.c:136-181 (create/free), :319-395 (forward: rms = sqrtf(mean(x^2)), y = x/(rms+eps)*weight, eps OUTSIDE
 * the root); backward and update are stubs in the reference (:404-421) and are implemented here like LayerNorm's. */
boat_rmsnorm_t* boat_rmsnorm_create(const boat_rmsnorm_config_t* config) {
    if (!config || config->normalized_shape == 0) return NULL;
    boat_rmsnorm_t* norm = (boat_rmsnorm_t*)calloc(1, sizeof(*norm));
    if (!norm) return NULL;
    norm->config = *config;
    if (config->elementwise_affine) {
        norm->weight = create_vector(config->normalized_shape);
        norm->grad_weight = create_vector(config->normalized_shape);
        float* g = norm->weight ? (float*)bt_host_rw(norm->weight) : NULL;
        if (!g || !norm->grad_weight) {
            boat_rmsnorm_free(norm);
            return NULL;
        }
        for (size_t i = 0; i < config->normalized_shape; i++) g[i] = 1.0f;
    }
    return norm;
}

void boat_rmsnorm_free(boat_rmsnorm_t* norm) {
    if (!norm) return;
    boat_tensor_free(norm->weight);
    boat_tensor_free(norm->grad_weight);
    boat_tensor_free(norm->cache_input);
    boat_tensor_free(norm->cache_inv_rms);
    free(norm);
}

boat_tensor_t* boat_rmsnorm_forward(boat_rmsnorm_t* norm, const boat_tensor_t* input) {
    if (!norm || !input || input->ndim < 1 || !bt_is_f32(input)) return NULL;
    const int64_t hidden = (int64_t)norm->config.normalized_shape;
    if (input->shape[input->ndim - 1] != hidden) return NULL;
    const int64_t rows = layernorm_rows(input);   /* the same loop nest as LayerNorm's (norm.c:360-362) */
    const bool covers_all = rows * hidden == (int64_t)input->nelements;
    boat_tensor_t* out = covers_all ? bt_new_like_uninit(input) : boat_tensor_create_like(input);
    const int64_t rshape[] = {rows};
    boat_tensor_t* inv = bt_new_uninit(rshape, 1, input->device);
    bool ok = out && inv;
    if (ok && rows > 0) {
        const float* px = bt_dev_read(input);
        const float* pw = norm->weight ? bt_dev_read(norm->weight) : NULL;
        float* py = covers_all ? bt_dev_write(out) : bt_dev_rw(out);
        ok = px && py && boat_hip_ok(bh_rmsnorm_forward(px, pw, py, bt_dev_write(inv), rows, hidden, norm->config.eps), "rmsnorm forward");
    }
    if (!ok) {
        boat_tensor_free(out);
        boat_tensor_free(inv);
        return NULL;
    }
    swap_tensor(&norm->cache_input, (boat_tensor_t*)input);
    boat_tensor_free(norm->cache_inv_rms);
    norm->cache_inv_rms = inv;
    return out;
}

boat_tensor_t* boat_rmsnorm_backward(boat_rmsnorm_t* norm, const boat_tensor_t* grad_output) {
    if (!norm || !grad_output) return NULL;
    if (!norm->cache_input || !norm->cache_inv_rms) {
        fprintf(stderr, "Error: RMSNorm backward called before forward\n");
        return NULL;
    }
    const boat_tensor_t* x = norm->cache_input;
    if (!bt_is_f32(grad_output) || grad_output->nelements != x->nelements) {
        fprintf(stderr, "Error: RMSNorm backward shape mismatch\n");
        return NULL;
    }
    const int64_t hidden = (int64_t)norm->config.normalized_shape;
    const int64_t rows = (int64_t)norm->cache_inv_rms->nelements;
    const bool covers_all = rows * hidden == (int64_t)x->nelements;
    boat_tensor_t* dx = covers_all ? bt_new_like_uninit(x) : boat_tensor_create_like(x);
    if (!dx || rows == 0) return dx;
    const float* px = bt_dev_read(x);
    const float* pdy = bt_dev_read(grad_output);
    const float* pw = norm->weight ? bt_dev_read(norm->weight) : NULL;
    float* pdx = covers_all ? bt_dev_write(dx) : bt_dev_rw(dx);
    /* the parameter gradient accumulates across calls like the dense layer's (dense.c:255-291) */
    int acc = 1;
    float* pgw = norm->grad_weight ? bt_dev_accumulate(norm->grad_weight, &acc) : NULL;
    if (!px || !pdy || !pdx ||
        !boat_hip_ok(bh_rmsnorm_backward(px, pw, pdy, bt_dev_read(norm->cache_inv_rms), pdx, pgw, rows, hidden, norm->config.eps, acc),
                     "rmsnorm backward")) {
        boat_tensor_free(dx);
        dx = NULL;
    }
    bt_flush_exposed();
    return dx;
}

void boat_rmsnorm_update(boat_rmsnorm_t* norm, float learning_rate) {
    if (!norm) return;
    sgd_step(norm->weight, norm->grad_weight, learning_rate, true);
    bt_flush_exposed();
}
boat_tensor_t* boat_hip_rmsnorm_get_weight(const boat_rmsnorm_t* n) { return n ? n->weight : NULL; }
boat_tensor_t* boat_hip_rmsnorm_get_grad_weight(const boat_rmsnorm_t* n) { return n ? n->grad_weight : NULL; }

boat_tensor_t* boat_rms_norm(const boat_tensor_t* input, const int64_t* normalized_shape, size_t normalized_shape_len, float eps) {
    if (!input || !normalized_shape || normalized_shape_len != 1) return NULL;
    boat_rmsnorm_config_t cfg = {(size_t)normalized_shape[0], eps, false};
    boat_rmsnorm_t* tmp = boat_rmsnorm_create(&cfg);
    if (!tmp) return NULL;
    boat_tensor_t* y = boat_rmsnorm_forward(tmp, input);
    boat_rmsnorm_free(tmp);
    return y;
}
boat_tensor_t* boat_rms_norm_grad(const boat_tensor_t* grad_output, const boat_tensor_t* input, const boat_tensor_t* output,
                                  const int64_t* normalized_shape, size_t normalized_shape_len, float eps) {
    (void)output;
    if (!grad_output || !input || !normalized_shape || normalized_shape_len != 1) return NULL;
    boat_rmsnorm_config_t cfg = {(size_t)normalized_shape[0], eps, false};
    boat_rmsnorm_t* tmp = boat_rmsnorm_create(&cfg);
    if (!tmp) return NULL;
    boat_tensor_t* y = boat_rmsnorm_forward(tmp, input);
    boat_tensor_t* dx = y ? boat_rmsnorm_backward(tmp, grad_output) : NULL;
    boat_tensor_free(y);
    boat_rmsnorm_free(tmp);
    return dx;
}

boat_norm_layer_t* boat_norm_layer_create(size_t normalized_shape, float eps, bool elementwise_affine) {
    boat_layernorm_config_t config = {normalized_shape, eps, elementwise_affine, elementwise_affine};
    return boat_layernorm_create(&config);
}
void boat_norm_layer_free(boat_norm_layer_t* layer) { boat_layernorm_free(layer); }
boat_tensor_t* boat_norm_layer_forward(boat_norm_layer_t* layer, const boat_tensor_t* input) { return boat_layernorm_forward(layer, input); }
boat_tensor_t* boat_norm_layer_backward(boat_norm_layer_t* layer, const boat_tensor_t* g) { return boat_layernorm_backward(layer, g); }
void boat_norm_layer_update(boat_norm_layer_t* layer, float lr) { boat_layernorm_update(layer, lr); }

/* --------------------------------------------------------------- attention */

boat_attention_t* boat_attention_create(const boat_attention_config_t* config) {
    if (!config || config->hidden_size == 0 || config->num_heads == 0) return NULL;
    if (config->hidden_size % config->num_heads != 0) return NULL;
    boat_attention_t* a = (boat_attention_t*)calloc(1, sizeof(*a));
    if (!a) return NULL;
    a->config = *config;
    if (config->head_size == 0) a->config.head_size = config->hidden_size / config->num_heads;
    const size_t h = config->hidden_size;
    /* same creation order as attention.c:152-170, so rand() hands out the same weights */
    a->weight_q = create_linear_weights(h, h);
    a->weight_k = create_linear_weights(h, h);
    a->weight_v = create_linear_weights(h, h);
    a->weight_o = create_linear_weights(h, h);
    bool ok = a->weight_q && a->weight_k && a->weight_v && a->weight_o;
    if (ok && config->use_bias) {
        a->bias_q = create_vector(h);
        a->bias_k = create_vector(h);
        a->bias_v = create_vector(h);
        a->bias_o = create_vector(h);
        ok = a->bias_q && a->bias_k && a->bias_v && a->bias_o;
    }
    if (!ok) {
        boat_attention_free(a);
        return NULL;
    }
    return a;
}

/* largest [B*nh, S, S] score matrix (bytes) an attention layer keeps from its forward pass for its backward pass; 0 = never.
 * BOAT_HIP_ATTENTION_SCORE_CACHE (bytes) in the environment sets the initial value. */
static size_t g_score_cache_limit = (size_t)1 << 30;
static int g_score_cache_env_read = 0;
static void score_cache_env(void) {
    if (g_score_cache_env_read) return;
    g_score_cache_env_read = 1;
    const char* e = getenv("BOAT_HIP_ATTENTION_SCORE_CACHE");
    if (e && *e) g_score_cache_limit = (size_t)strtoull(e, NULL, 10);
}
void boat_hip_set_attention_score_cache_limit(size_t bytes) {
    g_score_cache_env_read = 1;
    g_score_cache_limit = bytes;
}

void boat_attention_free(boat_attention_t* a) {
    if (!a) return;
    boat_tensor_t** all[] = {&a->weight_q, &a->weight_k, &a->weight_v, &a->weight_o, &a->bias_q, &a->bias_k, &a->bias_v,
                             &a->bias_o, &a->grad_weight_q, &a->grad_weight_k, &a->grad_weight_v, &a->grad_weight_o,
                             &a->grad_bias_q, &a->grad_bias_k, &a->grad_bias_v, &a->grad_bias_o, &a->cache_query,
                             &a->cache_key, &a->cache_value, &a->cache_q_proj, &a->cache_k_proj, &a->cache_v_proj,
                             &a->cache_lse, &a->cache_attention_output, &a->cache_scores};
    for (size_t i = 0; i < sizeof(all) / sizeof(all[0]); i++) boat_tensor_free(*all[i]);
    free(a);
}

/* y[rows,h] = x[rows,h] . w[h,h] (+ bias) */
static boat_tensor_t* project(const boat_tensor_t* x, const boat_tensor_t* w, const boat_tensor_t* bias, int64_t rows, int64_t h) {
    boat_tensor_t* y = bt_new_like_uninit(x);
    if (!y) return NULL;
    const float* px = bt_dev_read(x);
    const float* pw = bt_dev_read(w);
    const float* pb = bias ? bt_dev_read(bias) : NULL;
    float* py = bt_dev_write(y);
    if (!px || !pw || !py || !boat_hip_ok(bh_gemm(0, 0, rows, h, h, px, h, pw, h, py, h, pb, 0, 1), "attention projection")) {
        boat_tensor_free(y);
        return NULL;
    }
    return y;
}

boat_tensor_t* boat_attention_forward(boat_attention_t* a, const boat_tensor_t* query, const boat_tensor_t* key,
                                      const boat_tensor_t* value, const boat_tensor_t* attention_mask) {
    (void)attention_mask;   /* ignored by the reference too (attention.c:1022-1025) */
    if (!a || !query || !key || !value) return NULL;
    const int64_t h = (int64_t)a->config.hidden_size, nh = (int64_t)a->config.num_heads, hd = (int64_t)a->config.head_size;
    if (!bt_is_f32(query) || !bt_is_f32(key) || !bt_is_f32(value)) return NULL;
    if (query->ndim != 3 || !bt_same_shape(query, key) || !bt_same_shape(query, value) || query->shape[2] != h || nh * hd != h) {
        boat_fail(BOAT_ERROR_INVALID_ARGUMENT, "attention forward expects query/key/value of shape [batch, seq, %lld]", (long long)h);
        return NULL;
    }
    const int64_t batch = query->shape[0], seq = query->shape[1], rows = batch * seq;

    swap_tensor(&a->cache_query, (boat_tensor_t*)query);
    swap_tensor(&a->cache_key, (boat_tensor_t*)key);
    swap_tensor(&a->cache_value, (boat_tensor_t*)value);
    boat_tensor_t** stale[] = {&a->cache_q_proj, &a->cache_k_proj, &a->cache_v_proj, &a->cache_lse, &a->cache_attention_output,
                               &a->cache_scores};
    for (size_t i = 0; i < 6; i++) {
        boat_tensor_free(*stale[i]);
        *stale[i] = NULL;
    }
    if (rows == 0) return bt_new_like_uninit(query);

    /* the three input projections (attention.c:363-365) as one grouped launch */
    a->cache_q_proj = bt_new_like_uninit(query);
    a->cache_k_proj = bt_new_like_uninit(query);
    a->cache_v_proj = bt_new_like_uninit(query);
    if (!a->cache_q_proj || !a->cache_k_proj || !a->cache_v_proj) return NULL;
    {
        const float* px[3] = {bt_dev_read(query), bt_dev_read(key), bt_dev_read(value)};
        const float* pw[3] = {bt_dev_read(a->weight_q), bt_dev_read(a->weight_k), bt_dev_read(a->weight_v)};
        const float* pb[3] = {a->bias_q ? bt_dev_read(a->bias_q) : NULL, a->bias_k ? bt_dev_read(a->bias_k) : NULL,
                              a->bias_v ? bt_dev_read(a->bias_v) : NULL};
        float* py[3] = {bt_dev_write(a->cache_q_proj), bt_dev_write(a->cache_k_proj), bt_dev_write(a->cache_v_proj)};
        for (int i = 0; i < 3; i++)
            if (!px[i] || !pw[i] || !py[i]) return NULL;
        if (!boat_hip_ok(bh_gemm_grouped(0, 0, rows, h, h, 3, px, h, pw, h, py, h, pb, 0), "attention input projections")) return NULL;
    }

    /* [B,S,H] viewed as [B*nh, S, hd]: block (b,h) is the h-th run of S*hd floats of batch b */
    const int64_t lshape[] = {batch * nh, seq};
    a->cache_lse = bt_new_uninit(lshape, 2, query->device);
    a->cache_attention_output = bt_new_like_uninit(query);
    if (!a->cache_lse || !a->cache_attention_output) return NULL;
    const float scale = 1.0f / sqrtf((float)hd);
    /* The reference keeps the [B, nh, S, S] attention weights for its backward pass (attention.c:424-431, 584-598).  Here
     * the forward kernel can leave the scaled scores instead, which saves the backward kernel one of its five contractions;
     * kept when the shape has that path and the matrix fits the score-cache limit, otherwise the backward pass recomputes. */
    score_cache_env();
    const size_t score_bytes = bh_sdpa_score_cache_bytes(batch * nh, seq, hd);
    if (score_bytes && score_bytes <= g_score_cache_limit) {
        const int64_t sshape[] = {batch * nh, seq, seq};
        a->cache_scores = bt_new_uninit(sshape, 3, query->device);     /* no room: fall back to recomputing */
    }
    const boat_error_t err_before = boat_get_last_error();
    float* scores = a->cache_scores ? bt_dev_write(a->cache_scores) : NULL;
    if (a->cache_scores && !scores) {           /* no HBM for it: the backward pass recomputes */
        boat_tensor_free(a->cache_scores);
        a->cache_scores = NULL;
        if (err_before == BOAT_SUCCESS) boat_reset_error();   /* only the error this attempt raised */
    }
    a->cache_causal = a->config.causal_mask;
    const int rc = scores ? bh_sdpa_forward_cached(bt_dev_read(a->cache_q_proj), bt_dev_read(a->cache_k_proj), bt_dev_read(a->cache_v_proj),
                                                   scale, a->cache_causal ? 1 : 0, bt_dev_write(a->cache_attention_output),
                                                   bt_dev_write(a->cache_lse), scores, batch * nh, seq, hd)
                          : bh_sdpa_forward(bt_dev_read(a->cache_q_proj), bt_dev_read(a->cache_k_proj), bt_dev_read(a->cache_v_proj), scale,
                                            a->cache_causal ? 1 : 0, bt_dev_write(a->cache_attention_output),
                                            bt_dev_write(a->cache_lse), NULL, batch * nh, seq, hd);
    if (!boat_hip_ok(rc, "attention core forward")) return NULL;
    return project(a->cache_attention_output, a->weight_o, a->bias_o, rows, h);
}

/* attention.c:1082-1092 over :882-1079: softmax(scale * Q.K^T) . V on [batch, heads, seq, head_size] tensors of one shape;
 * the mask argument and dropout are ignored there (:1022-1025, 1061-1062) and here.  Operands that are not 4-D get a copy
 * of `value` back, as the reference's compatibility branch does (:905-917). */
boat_tensor_t* boat_scaled_dot_product_attention(const boat_tensor_t* query, const boat_tensor_t* key, const boat_tensor_t* value,
                                                 float scale_factor, const boat_tensor_t* attention_mask, bool causal_mask,
                                                 float dropout_prob) {
    (void)attention_mask;
    (void)dropout_prob;
    if (!query || !key || !value) return NULL;
    if (query->ndim < 3 || key->ndim < 3 || value->ndim < 3) return NULL;
    if (query->ndim != 4 || key->ndim != 4 || value->ndim != 4) return boat_tensor_clone(value);
    if (!bt_same_shape(query, key) || !bt_same_shape(query, value)) return NULL;
    if (!bt_is_f32(query) || !bt_is_f32(key) || !bt_is_f32(value)) return NULL;
    boat_tensor_t* out = bt_new_like_uninit(value);
    if (!out || out->nelements == 0) return out;
    const int64_t heads = query->shape[0] * query->shape[1], seq = query->shape[2], hd = query->shape[3];
    const int64_t lshape[] = {heads, seq};
    boat_tensor_t* lse = bt_new_uninit(lshape, 2, value->device);
    const float* pq = bt_dev_read(query);
    const float* pk = bt_dev_read(key);
    const float* pv = bt_dev_read(value);
    float* po = bt_dev_write(out);
    float* pl = lse ? bt_dev_write(lse) : NULL;
    if (!pq || !pk || !pv || !po || !pl ||
        !boat_hip_ok(bh_sdpa_forward(pq, pk, pv, scale_factor, causal_mask ? 1 : 0, po, pl, NULL, heads, seq, hd),
                     "scaled dot-product attention")) {
        boat_tensor_free(out);
        out = NULL;
    }
    boat_tensor_free(lse);
    return out;
}

/* attention.c:830-880: self-attention through a throw-away layer with fresh random projections (bias on) */
boat_tensor_t* boat_multihead_attention(const boat_tensor_t* input, size_t num_heads, float dropout_prob, bool causal_mask,
                                        const boat_tensor_t* attention_mask) {
    if (!input || input->ndim != 3 || num_heads == 0) return NULL;
    const size_t hidden = (size_t)input->shape[2];
    if (hidden % num_heads != 0) return NULL;
    boat_attention_config_t config = {hidden, num_heads, hidden / num_heads, dropout_prob, causal_mask, true, false, 10000.0f};
    boat_attention_t* attention = boat_attention_create(&config);
    if (!attention) return NULL;
    boat_tensor_t* output = boat_attention_forward(attention, input, input, input, attention_mask);
    boat_attention_free(attention);
    return output;
}

/* not implemented in the reference either (attention.c:1094-1120): NULL and no effect */
boat_tensor_t* boat_rotary_position_encoding(const boat_tensor_t* tensor, size_t seq_len, size_t head_size, float theta) {
    (void)tensor; (void)seq_len; (void)head_size; (void)theta;
    return NULL;
}
void boat_apply_rotary_embedding(boat_tensor_t* query, boat_tensor_t* key, size_t seq_len, size_t head_size, float theta) {
    (void)query; (void)key; (void)seq_len; (void)head_size; (void)theta;
}

/* linear_projection_backward, attention.c:1186-1285, for the four projections: dx = dy.w^T ; *gw = x^T.dy ; *gb = colsum(dy),
 * all overwritten */
/* the backward of the three input projections; sum: *gq = dq.Wq^T + dk.Wk^T + dv.Wv^T and *gk, *gv are further
 * references to it.  The parameter gradients of the output projection (x^T.dy and colsum(dy) of attention output and
 * grad_output) have the same shapes and depend on nothing computed in between, so they ride along as a fourth group. */
static bool project_backward3(boat_attention_t* a, const boat_tensor_t* dqp, const boat_tensor_t* dkp, const boat_tensor_t* dvp,
                              const boat_tensor_t* grad_output, int64_t rows, int64_t h, bool sum, boat_tensor_t** gq,
                              boat_tensor_t** gk, boat_tensor_t** gv) {
    const boat_tensor_t* x[4] = {a->cache_query, a->cache_key, a->cache_value, a->cache_attention_output};
    const boat_tensor_t* w[4] = {a->weight_q, a->weight_k, a->weight_v, a->weight_o};
    const boat_tensor_t* bias[4] = {a->bias_q, a->bias_k, a->bias_v, a->bias_o};
    const boat_tensor_t* dy[4] = {dqp, dkp, dvp, grad_output};
    boat_tensor_t** gw[4] = {&a->grad_weight_q, &a->grad_weight_k, &a->grad_weight_v, &a->grad_weight_o};
    boat_tensor_t** gb[4] = {&a->grad_bias_q, &a->grad_bias_k, &a->grad_bias_v, &a->grad_bias_o};
    boat_tensor_t* dx[3] = {NULL, NULL, NULL};
    const float *px[4], *pw[4], *pdy[4];
    float *pgw[4], *pdx[3];
    bool ok = true;
    for (int i = 0; i < 4 && ok; i++) {
        if (!*gw[i]) *gw[i] = boat_tensor_create_like(w[i]);
        if (bias[i] && !*gb[i]) *gb[i] = boat_tensor_create_like(bias[i]);
        if (i < 3 && (i == 0 || !sum)) dx[i] = bt_new_like_uninit(x[i]);
        ok = *gw[i] && (!bias[i] || *gb[i]) && (i == 3 || dx[i] || (sum && i > 0));
        if (!ok) break;
        px[i] = bt_dev_read(x[i]);
        pw[i] = bt_dev_read(w[i]);
        pdy[i] = bt_dev_read(dy[i]);
        pgw[i] = bt_dev_write(*gw[i]);
        if (i < 3) pdx[i] = dx[i] ? bt_dev_write(dx[i]) : NULL;
        ok = px[i] && pw[i] && pdy[i] && pgw[i] && (i == 3 || pdx[i] || !dx[i]);
    }
    /* dx = dy.w^T */
    if (ok && sum) ok = boat_hip_ok(bh_gemm_ksegments(0, 1, rows, h, h, 3, pdy, h, pw, h, pdx[0], h, NULL, 0), "attention input gradient");
    else if (ok) ok = boat_hip_ok(bh_gemm_grouped(0, 1, rows, h, h, 3, pdy, h, pw, h, pdx, h, NULL, 0), "attention input gradients");
    /* gw = x^T.dy (overwritten per call, attention.c:1262-1279): the four in one launch */
    if (ok) ok = boat_hip_ok(bh_gemm_grouped(1, 0, h, h, rows, 4, px, h, pdy, h, pgw, h, NULL, 0), "attention weight gradients");
    /* gb = colsum(dy): the four in one pair of launches when all projections have a bias */
    if (ok && bias[0] && bias[1] && bias[2] && bias[3]) {
        float* pgb[4] = {bt_dev_write(*gb[0]), bt_dev_write(*gb[1]), bt_dev_write(*gb[2]), bt_dev_write(*gb[3])};
        ok = pgb[0] && pgb[1] && pgb[2] && pgb[3] && boat_hip_ok(bh_colsum_grouped(pdy, pgb, 4, rows, h, 0), "attention bias gradients");
    } else {
        for (int i = 0; i < 4 && ok; i++) {
            float* pgb = bias[i] ? bt_dev_write(*gb[i]) : NULL;
            if (bias[i]) ok = pgb && boat_hip_ok(bh_colsum(pdy[i], pgb, rows, h, 0), "attention bias gradient");
        }
    }
    if (!ok) {
        for (int i = 0; i < 3; i++) boat_tensor_free(dx[i]);
        return false;
    }
    if (sum) {
        boat_tensor_ref(dx[0]);
        boat_tensor_ref(dx[0]);
        dx[1] = dx[2] = dx[0];
    }
    *gq = dx[0];
    *gk = dx[1];
    *gv = dx[2];
    return true;
}

static bool attention_backward_unflushed(boat_attention_t* a, const boat_tensor_t* grad_output, boat_tensor_t** grad_query,
                                         boat_tensor_t** grad_key, boat_tensor_t** grad_value);
static boat_tensor_t* g_sum_into = NULL;   /* set by boat_attention_backward_self for the duration of one call */
bool boat_attention_backward_self(boat_attention_t* a, const boat_tensor_t* grad_output, boat_tensor_t** grad_input) {
    *grad_input = NULL;
    boat_tensor_t *gq = NULL, *gk = NULL, *gv = NULL;
    const bool same = a && a->cache_query && a->cache_query == a->cache_key && a->cache_query == a->cache_value;
    g_sum_into = same ? (boat_tensor_t*)a->cache_query : NULL;   /* non-NULL: sum the three input gradients into the first */
    const bool ok = attention_backward_unflushed(a, grad_output, &gq, &gk, &gv);
    g_sum_into = NULL;
    bt_flush_exposed();
    if (!ok) return false;
    if (same) {          /* gk and gv are further references to gq */
        boat_tensor_unref(gk);
        boat_tensor_unref(gv);
        *grad_input = gq;
        return true;
    }
    /* the inputs were different tensors after all: add on the device */
    boat_add_(gq, gk);
    boat_add_(gq, gv);
    boat_tensor_unref(gk);
    boat_tensor_unref(gv);
    *grad_input = gq;
    return true;
}
bool boat_attention_backward(boat_attention_t* a, const boat_tensor_t* grad_output, boat_tensor_t** grad_query,
                             boat_tensor_t** grad_key, boat_tensor_t** grad_value) {
    const bool ok = attention_backward_unflushed(a, grad_output, grad_query, grad_key, grad_value);
    bt_flush_exposed();
    return ok;
}
static bool attention_backward_unflushed(boat_attention_t* a, const boat_tensor_t* grad_output, boat_tensor_t** grad_query,
                                         boat_tensor_t** grad_key, boat_tensor_t** grad_value) {
    if (!a || !grad_output) {
        fprintf(stderr, "[ERROR] boat_attention_backward: invalid arguments\n");
        return false;
    }
    if (!a->cache_query || !a->cache_key || !a->cache_value || !a->cache_q_proj || !a->cache_k_proj || !a->cache_v_proj ||
        !a->cache_attention_output || !a->cache_lse) {
        fprintf(stderr, "[ERROR] boat_attention_backward: missing cached tensors (forward not run)\n");
        return false;
    }
    const boat_tensor_t* q = a->cache_query;
    const int64_t h = (int64_t)a->config.hidden_size, nh = (int64_t)a->config.num_heads, hd = (int64_t)a->config.head_size;
    const int64_t batch = q->shape[0], seq = q->shape[1], rows = batch * seq;
    if (!bt_is_f32(grad_output) || grad_output->nelements != q->nelements) {
        fprintf(stderr, "[ERROR] boat_attention_backward: grad_output shape mismatch\n");
        return false;
    }
    /* 1. output projection: its input gradient now, its parameter gradients with those of the input projections (step 3) */
    boat_tensor_t* d_ao = bt_new_like_uninit(a->cache_attention_output);
    {
        const float* pdy = bt_dev_read(grad_output);
        const float* pwo = bt_dev_read(a->weight_o);
        float* pd = d_ao ? bt_dev_write(d_ao) : NULL;
        if (!pdy || !pwo || !pd || !boat_hip_ok(bh_gemm(0, 1, rows, h, h, pdy, h, pwo, h, pd, h, NULL, 0, 1), "attention output projection backward")) {
            boat_tensor_free(d_ao);
            return false;
        }
    }
    /* 2. attention core on [B*nh, S, hd] blocks */
    boat_tensor_t* dqp = bt_new_like_uninit(q);
    boat_tensor_t* dkp = bt_new_like_uninit(q);
    boat_tensor_t* dvp = bt_new_like_uninit(q);
    const float scale = 1.0f / sqrtf((float)hd);
    bool ok = dqp && dkp && dvp;
    if (ok) {
        int rc = a->cache_scores
            ? bh_sdpa_backward_cached(bt_dev_read(a->cache_q_proj), bt_dev_read(a->cache_k_proj), bt_dev_read(a->cache_v_proj),
                                      bt_dev_read(a->cache_attention_output), bt_dev_read(a->cache_lse), bt_dev_read(a->cache_scores),
                                      bt_dev_read(d_ao), scale, a->cache_causal ? 1 : 0, bt_dev_write(dqp), bt_dev_write(dkp),
                                      bt_dev_write(dvp), batch * nh, seq, hd)
            : bh_sdpa_backward(bt_dev_read(a->cache_q_proj), bt_dev_read(a->cache_k_proj), bt_dev_read(a->cache_v_proj),
                               bt_dev_read(a->cache_attention_output), bt_dev_read(a->cache_lse), bt_dev_read(d_ao), scale,
                               a->cache_causal ? 1 : 0, bt_dev_write(dqp), bt_dev_write(dkp), bt_dev_write(dvp), batch * nh, seq, hd);
        /* no room for the cached kernel's dQ workspace: the plain entry point can fall back to its bounded GEMM path */
        if (rc == BH_ENOMEM && a->cache_scores)
            rc = bh_sdpa_backward(bt_dev_read(a->cache_q_proj), bt_dev_read(a->cache_k_proj), bt_dev_read(a->cache_v_proj),
                                  bt_dev_read(a->cache_attention_output), bt_dev_read(a->cache_lse), bt_dev_read(d_ao), scale,
                                  a->cache_causal ? 1 : 0, bt_dev_write(dqp), bt_dev_write(dkp), bt_dev_write(dvp), batch * nh, seq, hd);
        ok = boat_hip_ok(rc, "attention core backward");
    }
    boat_tensor_free(d_ao);
    /* the score matrix has served its one backward pass: a repeated backward call recomputes Q.K^T from the projections,
     * and a model of many layers holds no score matrices between steps */
    boat_tensor_free(a->cache_scores);
    a->cache_scores = NULL;
    /* 3. input projections (linear_projection_backward three times, attention.c:1186-1285): the three weight gradients
     * as one grouped launch, the three column sums, and the input gradients either as one grouped launch or, for
     * self-attention through the tape, as ONE product whose contraction runs over the three (dY, W) pairs */
    boat_tensor_t *gq = NULL, *gk = NULL, *gv = NULL;
    const bool sum = g_sum_into != NULL;
    if (ok) ok = project_backward3(a, dqp, dkp, dvp, grad_output, rows, h, sum, &gq, &gk, &gv);
    boat_tensor_free(dqp);
    boat_tensor_free(dkp);
    boat_tensor_free(dvp);
    if (!gq || !gk || !gv) {
        boat_tensor_free(gq);
        boat_tensor_free(gk);
        boat_tensor_free(gv);
        return false;
    }
    if (grad_query) *grad_query = gq; else boat_tensor_free(gq);
    if (grad_key) *grad_key = gk; else boat_tensor_free(gk);
    if (grad_value) *grad_value = gv; else boat_tensor_free(gv);
    return true;
}

void boat_attention_update(boat_attention_t* a, float lr) {
    if (!a) return;
    /* W -= lr*grad (attention.c:734-815); gradients are left in place, the next backward overwrites them */
    sgd_step(a->weight_q, a->grad_weight_q, lr, false);
    sgd_step(a->weight_k, a->grad_weight_k, lr, false);
    sgd_step(a->weight_v, a->grad_weight_v, lr, false);
    sgd_step(a->weight_o, a->grad_weight_o, lr, false);
    sgd_step(a->bias_q, a->grad_bias_q, lr, false);
    sgd_step(a->bias_k, a->grad_bias_k, lr, false);
    sgd_step(a->bias_v, a->grad_bias_v, lr, false);
    sgd_step(a->bias_o, a->grad_bias_o, lr, false);
    bt_flush_exposed();
}

/* stored only: the reference's forward ignores dropout as well (attention.c:1061-1062) */
void boat_attention_set_dropout(boat_attention_t* a, float dropout_prob) {
    if (a) a->config.dropout_prob = dropout_prob;
}

void boat_attention_set_causal(boat_attention_t* a, bool causal) {
    if (a) a->config.causal_mask = causal;
}

#define BOAT_ATT_GET(name, field) \
    boat_tensor_t* boat_attention_get_##name(const boat_attention_t* a) { return a ? a->field : NULL; }
BOAT_ATT_GET(weight_q, weight_q) BOAT_ATT_GET(weight_k, weight_k) BOAT_ATT_GET(weight_v, weight_v) BOAT_ATT_GET(weight_o, weight_o)
BOAT_ATT_GET(bias_q, bias_q) BOAT_ATT_GET(bias_k, bias_k) BOAT_ATT_GET(bias_v, bias_v) BOAT_ATT_GET(bias_o, bias_o)
BOAT_ATT_GET(grad_weight_q, grad_weight_q) BOAT_ATT_GET(grad_weight_k, grad_weight_k)
BOAT_ATT_GET(grad_weight_v, grad_weight_v) BOAT_ATT_GET(grad_weight_o, grad_weight_o)
BOAT_ATT_GET(grad_bias_q, grad_bias_q) BOAT_ATT_GET(grad_bias_k, grad_bias_k)
BOAT_ATT_GET(grad_bias_v, grad_bias_v) BOAT_ATT_GET(grad_bias_o, grad_bias_o)

/* simplified adapter, include/boat/layers.h:82-92: the same object under another name
 * (attention.c:1119-1175); backward hands back the query gradient only, as the reference does */
boat_attention_layer_t* boat_attention_layer_create(size_t hidden_size, size_t num_heads, float dropout_prob, bool causal_mask) {
    if (num_heads == 0) return NULL;
    boat_attention_config_t cfg = {hidden_size, num_heads, hidden_size / num_heads, dropout_prob, causal_mask, true, false, 10000.0f};
    return (boat_attention_layer_t*)boat_attention_create(&cfg);
}
void boat_attention_layer_free(boat_attention_layer_t* l) { boat_attention_free((boat_attention_t*)l); }
boat_tensor_t* boat_attention_layer_forward(boat_attention_layer_t* l, const boat_tensor_t* q, const boat_tensor_t* k,
                                            const boat_tensor_t* v, const boat_tensor_t* mask) {
    return boat_attention_forward((boat_attention_t*)l, q, k, v, mask);
}
boat_tensor_t* boat_attention_layer_backward(boat_attention_layer_t* l, const boat_tensor_t* grad_output) {
    boat_tensor_t *gq = NULL, *gk = NULL, *gv = NULL;
    if (!boat_attention_backward((boat_attention_t*)l, grad_output, &gq, &gk, &gv)) return NULL;
    boat_tensor_free(gk);
    boat_tensor_free(gv);
    return gq;
}
void boat_attention_layer_update(boat_attention_layer_t* l, float lr) { boat_attention_update((boat_attention_t*)l, lr); }
