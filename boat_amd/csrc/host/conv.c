/* conv.c - convolution, max-pooling and flatten layers of the MNIST network, all arithmetic on the GPU.
 *
 * Hooks, shapes, ownership and error behaviour follow the reference:
 *   conv     src/layers/conv.c:17-625  (NCHW, weight [out, in, k, k], bias always present, init
 *            U(-s, s) with s = sqrtf(2/(in*k*k)) drawn from rand(); backward OVERWRITES grad_weight and
 *            grad_bias and returns a new dX tensor)
 *   pool     src/layers/pool.c:17-223  (max pooling, first maximum wins, backward routes dY to it)
 *   flatten  src/layers/flatten.c:17-94 ([B, ...] -> [B, rest] view; backward reshapes back)
 * Two deliberate differences:
 *   - the gradient tensors keep their identity across backward calls (the reference frees and replaces
 *     them, conv.c:523-532, which leaves a registered optimizer holding dangling pointers);
 *   - the input gradient is the true one by default; the reference pairs each tap with the mirrored weight
 *     (conv.c:86-88).  boat_hip_conv_reference_input_grad(1), or reference-exact mode, switches to the reference's
 *     pairing for callers that need its numbers.
 */
#include "boat_internal.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

static int g_reference_input_grad = -1;   /* -1: not set by a call, follow reference-exact mode */

void boat_hip_conv_reference_input_grad(int enable) { g_reference_input_grad = enable < 0 ? -1 : enable != 0; }
/* forward on the matrix cores (3x3 and 5x5 kernels of layers wide enough for it to win, see conv_forward_wants_mfma); off by
 * default because the direct kernel's output is bit-identical to the reference's and the MFMA order is not.
 * BOAT_HIP_CONV_FORWARD_MFMA=1 in the environment sets the initial value. */
static int g_forward_mfma = -1;
void boat_hip_conv_forward_matrix_cores(int enable) { g_forward_mfma = enable != 0; }
/* The matrix-core kernel works on tiles of 64 output channels and pairs of input channels, and a workgroup of it costs
 * a weight staging and a reduction whatever the layer: measured against the direct kernel over batch 16-256, images
 * 14x14 and 28x28, it wins (1.3x to 4x) from 32 output channels on with at least 8 input channels (a tie at 8 -> 32)
 * and from 16 output channels on with at least 32 input channels; narrower layers lose up to 2x. */
static int conv_forward_wants_mfma(size_t in_channels, size_t out_channels) {
    return (in_channels >= 8 && out_channels >= 32) || (in_channels >= 32 && out_channels >= 16);
}
static int forward_mfma(void) {
    if (g_forward_mfma < 0) {
        const char* e = getenv("BOAT_HIP_CONV_FORWARD_MFMA");
        g_forward_mfma = e && *e && *e != '0';
    }
    return g_forward_mfma;
}
static int reference_input_grad(void) { return g_reference_input_grad >= 0 ? g_reference_input_grad : (bt_reference_exact() ? 1 : 0); }

struct boat_conv_layer_t {
    size_t in_channels, out_channels, kernel_size, stride, padding;
    bool use_bias;
    boat_tensor_t *weight, *bias, *grad_weight, *grad_bias;
    boat_tensor_t* cache_input;
    int64_t cache_output_shape[4];
};

boat_conv_layer_t* boat_conv_layer_create(size_t in_channels, size_t out_channels, size_t kernel_size, size_t stride, size_t padding) {
    if (in_channels == 0 || out_channels == 0 || kernel_size == 0 || stride == 0) return NULL;
    boat_conv_layer_t* l = (boat_conv_layer_t*)calloc(1, sizeof(*l));
    if (!l) return NULL;
    l->in_channels = in_channels;
    l->out_channels = out_channels;
    l->kernel_size = kernel_size;
    l->stride = stride;
    l->padding = padding;
    l->use_bias = true;
    const int64_t wshape[] = {(int64_t)out_channels, (int64_t)in_channels, (int64_t)kernel_size, (int64_t)kernel_size};
    const int64_t bshape[] = {(int64_t)out_channels};
    l->weight = boat_tensor_create(wshape, 4, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    l->bias = boat_tensor_create(bshape, 1, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    l->grad_weight = boat_tensor_create(wshape, 4, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    l->grad_bias = boat_tensor_create(bshape, 1, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    float* w = l->weight ? (float*)bt_host_rw(l->weight) : NULL;
    if (!w || !l->bias || !l->grad_weight || !l->grad_bias) {
        boat_conv_layer_free(l);
        return NULL;
    }
    const float scale = sqrtf(2.0f / (in_channels * kernel_size * kernel_size));   /* conv.c:243-246 */
    for (size_t i = 0; i < l->weight->nelements; i++) w[i] = ((float)rand() / RAND_MAX) * 2.0f * scale - scale;
    return l;
}

void boat_conv_layer_free(boat_conv_layer_t* l) {
    if (!l) return;
    boat_tensor_free(l->weight);
    boat_tensor_free(l->bias);
    boat_tensor_free(l->grad_weight);
    boat_tensor_free(l->grad_bias);
    boat_tensor_free(l->cache_input);
    free(l);
}

boat_tensor_t* boat_conv_layer_forward(boat_conv_layer_t* l, const boat_tensor_t* input) {
    if (!l || !input) return NULL;
    if (input->ndim != 4) {
        fprintf(stderr, "Error: Conv2d expects 4D input tensor\n");
        return NULL;
    }
    if ((size_t)input->shape[1] != l->in_channels) {
        fprintf(stderr, "Error: Input channels %lld don't match layer in_channels %zu\n", (long long)input->shape[1], l->in_channels);
        return NULL;
    }
    if (!bt_is_f32(input) || !bt_is_f32(l->weight) || (l->use_bias && l->bias && !bt_is_f32(l->bias))) {
        fprintf(stderr, "Error: Conv2d only supports FLOAT32 tensors\n");
        return NULL;
    }
    const int64_t batch = input->shape[0], h = input->shape[2], w = input->shape[3];
    const int64_t k = (int64_t)l->kernel_size, s = (int64_t)l->stride, p = (int64_t)l->padding;
    const int64_t ho = (h + 2 * p - k) / s + 1, wo = (w + 2 * p - k) / s + 1;
    if (h + 2 * p < k || w + 2 * p < k || ho <= 0 || wo <= 0) {
        fprintf(stderr, "Error: Invalid convolution parameters - output dimensions would be non-positive\n");
        return NULL;
    }
    boat_tensor_ref((boat_tensor_t*)input);
    boat_tensor_free(l->cache_input);
    l->cache_input = (boat_tensor_t*)input;
    const int64_t oshape[] = {batch, (int64_t)l->out_channels, ho, wo};
    memcpy(l->cache_output_shape, oshape, sizeof(oshape));
    boat_tensor_t* out = bt_new_uninit(oshape, 4, input->device);
    if (!out || out->nelements == 0) return out;
    const float* px = bt_dev_read(input);
    const float* pw = bt_dev_read(l->weight);
    const float* pb = (l->use_bias && l->bias) ? bt_dev_read(l->bias) : NULL;
    float* py = bt_dev_write(out);
    const int mfma = forward_mfma() && (k == 3 || k == 5) && conv_forward_wants_mfma(l->in_channels, l->out_channels);
    if (!px || !pw || !py ||
        !boat_hip_ok((mfma ? bh_conv2d_forward_mfma : bh_conv2d_forward)(px, pw, pb, py, batch, (int64_t)l->in_channels, h, w,
                                                                         (int64_t)l->out_channels, k, s, p),
                     "conv forward")) {
        boat_tensor_free(out);
        return NULL;
    }
    return out;
}

static boat_tensor_t* boat_conv_layer_backward_unflushed(boat_conv_layer_t* l, const boat_tensor_t* grad_output) {
    if (!l || !grad_output) {
        fprintf(stderr, "Error: conv backward: NULL input\n");
        return NULL;
    }
    if (!l->cache_input) {
        fprintf(stderr, "Error: conv backward: no cached input (forward not called or cache cleared)\n");
        return NULL;
    }
    const boat_tensor_t* x = l->cache_input;
    if (grad_output->ndim != 4 || memcmp(grad_output->shape, l->cache_output_shape, sizeof(l->cache_output_shape)) != 0 ||
        !bt_is_f32(grad_output)) {
        fprintf(stderr, "Error: conv backward: grad_output shape doesn't match cached output shape\n");
        return NULL;
    }
    boat_tensor_t* dx = bt_new_like_uninit(x);
    if (!dx) return NULL;
    if (dx->nelements == 0) return dx;
    const float* px = bt_dev_read(x);
    const float* pw = bt_dev_read(l->weight);
    const float* pg = bt_dev_read(grad_output);
    float* pdx = bt_dev_write(dx);
    float* pgw = bt_dev_write(l->grad_weight);
    float* pgb = (l->use_bias && l->grad_bias) ? bt_dev_write(l->grad_bias) : NULL;
    if (!px || !pw || !pg || !pdx || !pgw ||
        !boat_hip_ok(bh_conv2d_backward(px, pw, pg, pdx, pgw, pgb, x->shape[0], (int64_t)l->in_channels, x->shape[2], x->shape[3],
                                        (int64_t)l->out_channels, (int64_t)l->kernel_size, (int64_t)l->stride, (int64_t)l->padding,
                                        0, reference_input_grad()),
                     "conv backward")) {
        boat_tensor_free(dx);
        return NULL;
    }
    return dx;
}
boat_tensor_t* boat_conv_layer_backward(boat_conv_layer_t* l, const boat_tensor_t* grad_output) {
    boat_tensor_t* result = boat_conv_layer_backward_unflushed(l, grad_output);
    bt_flush_exposed();
    return result;
}

/* weight -= lr * grad (conv.c:537-560); the gradients are left in place, the next backward overwrites them */
void boat_conv_layer_update(boat_conv_layer_t* l, float learning_rate) {
    if (!l) return;
    boat_tensor_t* pairs[2][2] = {{l->weight, l->grad_weight}, {l->use_bias ? l->bias : NULL, l->grad_bias}};
    for (int i = 0; i < 2; i++) {
        boat_tensor_t *p = pairs[i][0], *g = pairs[i][1];
        if (!p || !g || p->nelements != g->nelements || p->nelements == 0) continue;
        float* pp = bt_dev_rw(p);
        float* pg = bt_dev_rw(g);
        if (pp && pg) boat_hip_ok(bh_sgd_update(pp, pg, learning_rate, (int64_t)p->nelements, 0), "conv update");
    }
    bt_flush_exposed();
}

void boat_conv_layer_set_weight(boat_conv_layer_t* l, boat_tensor_t* weight) {
    if (!l || !weight) return;
    if (weight->ndim != 4 || weight->shape[0] != (int64_t)l->out_channels || weight->shape[1] != (int64_t)l->in_channels ||
        weight->shape[2] != (int64_t)l->kernel_size || weight->shape[3] != (int64_t)l->kernel_size) {
        fprintf(stderr, "Error: Weight shape does not match layer dimensions\n");
        return;
    }
    boat_tensor_ref(weight);
    boat_tensor_free(l->weight);
    l->weight = weight;
}

void boat_conv_layer_set_bias(boat_conv_layer_t* l, boat_tensor_t* bias) {
    if (!l || !bias) return;
    if (!l->use_bias) {
        fprintf(stderr, "Warning: Layer was created without bias, ignoring bias tensor\n");
        return;
    }
    if (bias->ndim < 1 || bias->shape[0] != (int64_t)l->out_channels) {
        fprintf(stderr, "Error: Bias shape does not match output channels %zu\n", l->out_channels);
        return;
    }
    boat_tensor_ref(bias);
    boat_tensor_free(l->bias);
    l->bias = bias;
}

boat_tensor_t* boat_conv_layer_get_weight(const boat_conv_layer_t* l) { return l ? l->weight : NULL; }
boat_tensor_t* boat_conv_layer_get_bias(const boat_conv_layer_t* l) { return l ? l->bias : NULL; }
boat_tensor_t* boat_conv_layer_get_grad_weight(const boat_conv_layer_t* l) { return l ? l->grad_weight : NULL; }
boat_tensor_t* boat_conv_layer_get_grad_bias(const boat_conv_layer_t* l) { return l ? l->grad_bias : NULL; }

/* -------------------------------------------------------------------- pool */

struct boat_pool_layer_t {
    size_t pool_size, stride, padding;
    boat_tensor_t* cache_input;
    bh_buffer_t* argmax;          /* int32 per output element: offset of the window's maximum inside its plane */
    int64_t cache_output_shape[4];
};

boat_pool_layer_t* boat_pool_layer_create(size_t pool_size, size_t stride, size_t padding) {
    boat_pool_layer_t* l = (boat_pool_layer_t*)calloc(1, sizeof(*l));
    if (!l) return NULL;
    l->pool_size = pool_size;
    l->stride = stride;
    l->padding = padding;
    return l;
}

void boat_pool_layer_free(boat_pool_layer_t* l) {
    if (!l) return;
    boat_tensor_free(l->cache_input);
    if (l->argmax) bh_buffer_unref(l->argmax);
    free(l);
}

boat_tensor_t* boat_pool_layer_forward(boat_pool_layer_t* l, const boat_tensor_t* input) {
    if (!l || !input) return NULL;
    if (input->ndim != 4) {
        fprintf(stderr, "Error: MaxPool2d expects 4D input tensor\n");
        return NULL;
    }
    if (!bt_is_f32(input) || l->pool_size == 0 || l->stride == 0) return NULL;
    const int64_t batch = input->shape[0], ch = input->shape[1], h = input->shape[2], w = input->shape[3];
    const int64_t k = (int64_t)l->pool_size, s = (int64_t)l->stride, p = (int64_t)l->padding;
    if (h + 2 * p < k || w + 2 * p < k) return NULL;
    const int64_t ho = (h + 2 * p - k) / s + 1, wo = (w + 2 * p - k) / s + 1;
    const int64_t oshape[] = {batch, ch, ho, wo};
    boat_tensor_t* out = bt_new_uninit(oshape, 4, input->device);
    if (!out) return NULL;
    boat_tensor_ref((boat_tensor_t*)input);
    boat_tensor_free(l->cache_input);
    l->cache_input = (boat_tensor_t*)input;
    if (l->argmax) bh_buffer_unref(l->argmax);
    l->argmax = NULL;
    memcpy(l->cache_output_shape, oshape, sizeof(oshape));
    if (out->nelements == 0) return out;
    l->argmax = bh_buffer_create(out->nelements * sizeof(int32_t), 0);
    const float* px = bt_dev_read(input);
    float* py = bt_dev_write(out);
    if (!l->argmax || !px || !py ||
        !boat_hip_ok(bh_maxpool2d_forward(px, py, (int32_t*)bh_buffer_ptr(l->argmax), batch * ch, h, w, k, s, p), "pool forward")) {
        boat_tensor_free(out);
        return NULL;
    }
    return out;
}

boat_tensor_t* boat_pool_layer_backward(boat_pool_layer_t* l, const boat_tensor_t* grad_output) {
    if (!l || !grad_output || !l->cache_input) return NULL;
    if (grad_output->ndim != 4 || memcmp(grad_output->shape, l->cache_output_shape, sizeof(l->cache_output_shape)) != 0 ||
        !bt_is_f32(grad_output)) {
        fprintf(stderr, "Error: MaxPool2d backward gradient shape mismatch\n");
        return NULL;
    }
    const boat_tensor_t* x = l->cache_input;
    boat_tensor_t* dx = bt_new_like_uninit(x);
    if (!dx || dx->nelements == 0) return dx;
    if (!l->argmax) {
        boat_tensor_free(dx);
        return NULL;
    }
    const float* pg = bt_dev_read(grad_output);
    float* pdx = bt_dev_write(dx);
    if (!pg || !pdx ||
        !boat_hip_ok(bh_maxpool2d_backward(pg, (const int32_t*)bh_buffer_ptr(l->argmax), pdx, x->shape[0] * x->shape[1], x->shape[2],
                                           x->shape[3], (int64_t)l->pool_size, (int64_t)l->stride, (int64_t)l->padding),
                     "pool backward")) {
        boat_tensor_free(dx);
        return NULL;
    }
    return dx;
}

void boat_pool_layer_update(boat_pool_layer_t* l, float learning_rate) {
    (void)l;
    (void)learning_rate;
}

/* ----------------------------------------------------------------- flatten */

struct boat_flatten_layer_t {
    int64_t cached_shape[BOAT_MAX_DIMS];
    size_t cached_ndim;
};

boat_flatten_layer_t* boat_flatten_layer_create(void) { return (boat_flatten_layer_t*)calloc(1, sizeof(boat_flatten_layer_t)); }
void boat_flatten_layer_free(boat_flatten_layer_t* l) { free(l); }

boat_tensor_t* boat_flatten_layer_forward(boat_flatten_layer_t* l, const boat_tensor_t* input) {
    if (!l || !input) return NULL;
    if (input->ndim < 2) {
        fprintf(stderr, "Error: Flatten expects at least 2D input tensor\n");
        return NULL;
    }
    memcpy(l->cached_shape, input->shape, input->ndim * sizeof(int64_t));
    l->cached_ndim = input->ndim;
    int64_t features = 1;
    for (size_t i = 1; i < input->ndim; i++) features *= input->shape[i];
    const int64_t oshape[] = {input->shape[0], features};
    return boat_tensor_reshape(input, oshape, 2);
}

boat_tensor_t* boat_flatten_layer_backward(const boat_flatten_layer_t* l, const boat_tensor_t* grad_output) {
    if (!l || !grad_output) return NULL;
    if (l->cached_ndim == 0) {
        fprintf(stderr, "Error: Flatten backward called without cached shape (forward not called)\n");
        return NULL;
    }
    return boat_tensor_reshape(grad_output, l->cached_shape, l->cached_ndim);
}

void boat_flatten_layer_update(boat_flatten_layer_t* l, float learning_rate) {
    (void)l;
    (void)learning_rate;
}
