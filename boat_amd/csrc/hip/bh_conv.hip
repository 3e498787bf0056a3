// bh_conv.hip - direct 2-D convolution (NCHW, square kernel) and max pooling, forward and backward.
//
// Replaces the loops of the reference's convolution and pooling layers:
//   boat_conv_layer_forward            src/layers/conv.c:326-437
//   compute_weight_gradient            src/layers/conv.c:105-163
//   compute_bias_gradient              src/layers/conv.c:165-201
//   compute_input_gradient             src/layers/conv.c:46-103
//   boat_pool_layer_forward/backward   src/layers/pool.c:63-218
// The shapes on this path are the small ones of the MNIST network (1->32 and 32->64 channels, 3x3, 28x28 and
// 14x14 images, batches of tens), far too small to fill the matrix cores through an im2col GEMM, so every
// kernel is a direct gather: one lane per output element, operands served by the caches, no atomics, and each
// result is written exactly once (deterministic).
//
// Input gradient.  The reference pairs tap (kh, kw) of the scatter ih = oh*stride - pad + kh with the weight
// of the mirrored tap (k-1-kh, k-1-kw) (conv.c:86-88); that is the gradient of a different layer, and its own
// gradient check only looks at weight and bias gradients (tests/unit/test_conv_gradient_check.c:317-332).
// flip_taps == 0 computes the true gradient dx[ih,iw] = sum w[oc,ic,kh,kw]*dy[oh,ow]; flip_taps != 0 reproduces
// the reference's pairing, so that its numbers can be checked against.
//
// Forward keeps the reference's fp32 operation order (per input channel a running sum over the taps, added to
// the output, bias last), so it is bit-identical; the gradient reductions add in wavefront trees and agree to
// rounding.
#include "bh_common.h"

#include <math.h>

namespace bh {

constexpr int kCBlock = 256;

struct ConvShape {
    int batch, ic, h, w, oc, k, stride, pad, ho, wo;
};

__global__ __launch_bounds__(kCBlock) void conv2d_fwd_kernel(const float* __restrict__ x, const float* __restrict__ wt,
                                                             const float* __restrict__ bias, float* __restrict__ y,
                                                             ConvShape c, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * kCBlock + threadIdx.x;
    if (i >= total) return;
    const int ow = (int)(i % c.wo);
    const int oh = (int)((i / c.wo) % c.ho);
    const int oc = (int)((i / ((int64_t)c.wo * c.ho)) % c.oc);
    const int b = (int)(i / ((int64_t)c.wo * c.ho * c.oc));
    const int ih0 = oh * c.stride - c.pad, iw0 = ow * c.stride - c.pad;
    float out = 0.f;
    for (int ci = 0; ci < c.ic; ci++) {
        const float* xp = x + ((int64_t)b * c.ic + ci) * c.h * c.w;
        const float* wp = wt + ((int64_t)oc * c.ic + ci) * c.k * c.k;
        float sum = 0.f;
        for (int kh = 0; kh < c.k; kh++) {
            const int ih = ih0 + kh;
            if (ih < 0 || ih >= c.h) continue;
            for (int kw = 0; kw < c.k; kw++) {
                const int iw = iw0 + kw;
                if (iw < 0 || iw >= c.w) continue;
                sum += xp[ih * c.w + iw] * wp[kh * c.k + kw];
            }
        }
        out += sum;
    }
    if (bias) out += bias[oc];
    y[i] = out;
}

// dx[b,ic,ih,iw] = sum_{oc,kh,kw} w[oc,ic,kh',kw'] * dy[b,oc,oh,ow] with oh*stride - pad + kh == ih
__global__ __launch_bounds__(kCBlock) void conv2d_bwd_input_kernel(const float* __restrict__ wt, const float* __restrict__ dy,
                                                                   float* __restrict__ dx, ConvShape c, int64_t total,
                                                                   int flip_taps) {
    const int64_t i = (int64_t)blockIdx.x * kCBlock + threadIdx.x;
    if (i >= total) return;
    const int iw = (int)(i % c.w);
    const int ih = (int)((i / c.w) % c.h);
    const int ci = (int)((i / ((int64_t)c.w * c.h)) % c.ic);
    const int b = (int)(i / ((int64_t)c.w * c.h * c.ic));
    float acc = 0.f;
    for (int oc = 0; oc < c.oc; oc++) {
        const float* wp = wt + ((int64_t)oc * c.ic + ci) * c.k * c.k;
        const float* gp = dy + ((int64_t)b * c.oc + oc) * c.ho * c.wo;
        for (int kh = 0; kh < c.k; kh++) {
            const int t = ih + c.pad - kh;
            if (t < 0 || t % c.stride) continue;
            const int oh = t / c.stride;
            if (oh >= c.ho) continue;
            for (int kw = 0; kw < c.k; kw++) {
                const int u = iw + c.pad - kw;
                if (u < 0 || u % c.stride) continue;
                const int ow = u / c.stride;
                if (ow >= c.wo) continue;
                const int wk = flip_taps ? (c.k - 1 - kh) * c.k + (c.k - 1 - kw) : kh * c.k + kw;
                acc += wp[wk] * gp[oh * c.wo + ow];
            }
        }
    }
    dx[i] = acc;
}

// gw[oc,ic,kh,kw] (+)= sum_{b,oh,ow} x[b,ic,ih,iw] * dy[b,oc,oh,ow]: one wavefront per weight element
__global__ __launch_bounds__(kCBlock) void conv2d_bwd_weight_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                                    float* __restrict__ gw, ConvShape c, int64_t n_weights,
                                                                    int accumulate) {
    const int lane = threadIdx.x & 63;
    const int64_t wi = (int64_t)blockIdx.x * (kCBlock / 64) + (threadIdx.x >> 6);
    if (wi >= n_weights) return;
    const int kw = (int)(wi % c.k);
    const int kh = (int)((wi / c.k) % c.k);
    const int ci = (int)((wi / ((int64_t)c.k * c.k)) % c.ic);
    const int oc = (int)(wi / ((int64_t)c.k * c.k * c.ic));
    const int per_image = c.ho * c.wo;
    const int64_t terms = (int64_t)c.batch * per_image;
    float acc = 0.f;
    for (int64_t t = lane; t < terms; t += 64) {
        const int b = (int)(t / per_image);
        const int rem = (int)(t % per_image);
        const int oh = rem / c.wo, ow = rem % c.wo;
        const int ih = oh * c.stride - c.pad + kh, iw = ow * c.stride - c.pad + kw;
        if (ih < 0 || ih >= c.h || iw < 0 || iw >= c.w) continue;
        acc += x[(((int64_t)b * c.ic + ci) * c.h + ih) * c.w + iw] * dy[((int64_t)b * c.oc + oc) * per_image + rem];
    }
    acc = wave_sum(acc);
    if (lane == 0) gw[wi] = accumulate ? gw[wi] + acc : acc;
}

// gb[oc] (+)= sum_{b,oh,ow} dy[b,oc,oh,ow]: one workgroup per output channel
__global__ __launch_bounds__(kCBlock) void conv2d_bwd_bias_kernel(const float* __restrict__ dy, float* __restrict__ gb,
                                                                  ConvShape c, int accumulate) {
    __shared__ float red[kCBlock / 64];
    const int oc = blockIdx.x;
    const int per_image = c.ho * c.wo;
    const int64_t terms = (int64_t)c.batch * per_image;
    float acc = 0.f;
    for (int64_t t = threadIdx.x; t < terms; t += kCBlock) {
        const int64_t b = t / per_image, rem = t % per_image;
        acc += dy[(b * c.oc + oc) * per_image + rem];
    }
    const float total = block_sum<kCBlock / 64>(acc, red);
    if (threadIdx.x == 0) gb[oc] = accumulate ? gb[oc] + total : total;
}

struct PoolShape {
    int64_t planes;   // batch * channels
    int h, w, ho, wo, pool, stride, pad;
};

// first maximum in row-major scan order wins (strict >, pool.c:118-123); index is the offset inside the plane, -1 if none
__global__ __launch_bounds__(kCBlock) void maxpool_fwd_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                              int32_t* __restrict__ idx, PoolShape p, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * kCBlock + threadIdx.x;
    if (i >= total) return;
    const int ow = (int)(i % p.wo);
    const int oh = (int)((i / p.wo) % p.ho);
    const int64_t plane = i / ((int64_t)p.wo * p.ho);
    const float* xp = x + plane * p.h * p.w;
    int h0 = oh * p.stride - p.pad, w0 = ow * p.stride - p.pad;
    int h1 = h0 + p.pool, w1 = w0 + p.pool;
    h0 = h0 < 0 ? 0 : h0;
    w0 = w0 < 0 ? 0 : w0;
    h1 = h1 > p.h ? p.h : h1;
    w1 = w1 > p.w ? p.w : w1;
    float best = -INFINITY;
    int where = -1;
    for (int ph = h0; ph < h1; ph++)
        for (int pw = w0; pw < w1; pw++) {
            const float v = xp[ph * p.w + pw];
            if (v > best) {
                best = v;
                where = ph * p.w + pw;
            }
        }
    y[i] = best;
    idx[i] = where;
}

// dx[plane, ih, iw] = sum of dy over the windows whose maximum sits at (ih, iw), visited in increasing output
// index, which is the order in which the reference's scatter loop adds them (pool.c:207-212)
__global__ __launch_bounds__(kCBlock) void maxpool_bwd_kernel(const float* __restrict__ dy, const int32_t* __restrict__ idx,
                                                              float* __restrict__ dx, PoolShape p, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * kCBlock + threadIdx.x;
    if (i >= total) return;
    const int iw = (int)(i % p.w);
    const int ih = (int)((i / p.w) % p.h);
    const int64_t plane = i / ((int64_t)p.w * p.h);
    const int me = ih * p.w + iw;
    // windows covering row ih: oh*stride - pad <= ih < oh*stride - pad + pool
    int oh_lo = ih + p.pad - p.pool + 1;
    oh_lo = oh_lo <= 0 ? 0 : (oh_lo + p.stride - 1) / p.stride;
    int oh_hi = (ih + p.pad) / p.stride;
    if (oh_hi >= p.ho) oh_hi = p.ho - 1;
    int ow_lo = iw + p.pad - p.pool + 1;
    ow_lo = ow_lo <= 0 ? 0 : (ow_lo + p.stride - 1) / p.stride;
    int ow_hi = (iw + p.pad) / p.stride;
    if (ow_hi >= p.wo) ow_hi = p.wo - 1;
    const float* gp = dy + plane * p.ho * p.wo;
    const int32_t* ip = idx + plane * p.ho * p.wo;
    float acc = 0.f;
    for (int oh = oh_lo; oh <= oh_hi; oh++)
        for (int ow = ow_lo; ow <= ow_hi; ow++)
            if (ip[oh * p.wo + ow] == me) acc += gp[oh * p.wo + ow];
    dx[i] = acc;
}

static int make_conv_shape(ConvShape& c, int64_t batch, int64_t ic, int64_t h, int64_t w, int64_t oc, int64_t k, int64_t stride,
                           int64_t pad) {
    if (batch < 0 || ic <= 0 || h <= 0 || w <= 0 || oc <= 0 || k <= 0 || stride <= 0 || pad < 0)
        return set_error(BH_EINVAL, "conv2d: bad shape");
    const int64_t ho = (h + 2 * pad - k) / stride + 1, wo = (w + 2 * pad - k) / stride + 1;
    if (h + 2 * pad < k || w + 2 * pad < k || ho <= 0 || wo <= 0) return set_error(BH_EINVAL, "conv2d: kernel larger than the padded image");
    const int64_t lim = (int64_t)1 << 30;
    if (batch * ic * h * w >= lim || batch * oc * ho * wo >= lim || oc * ic * k * k >= lim)
        return set_error(BH_EINVAL, "conv2d: tensor too large for 32-bit indexing");
    c.batch = (int)batch; c.ic = (int)ic; c.h = (int)h; c.w = (int)w; c.oc = (int)oc; c.k = (int)k;
    c.stride = (int)stride; c.pad = (int)pad; c.ho = (int)ho; c.wo = (int)wo;
    return BH_OK;
}

}  // namespace bh

using namespace bh;

extern "C" {

int bh_conv2d_forward(const float* x, const float* w, const float* bias, float* y, int64_t batch, int64_t in_channels,
                      int64_t height, int64_t width, int64_t out_channels, int64_t kernel, int64_t stride, int64_t pad) {
    BH_REQUIRE_INIT();
    ConvShape c;
    int rc = make_conv_shape(c, batch, in_channels, height, width, out_channels, kernel, stride, pad);
    if (rc) return rc;
    if (batch == 0) return BH_OK;
    BH_CHECK_ARG(x && w && y, "null pointer");
    const int64_t total = (int64_t)c.batch * c.oc * c.ho * c.wo;
    hipLaunchKernelGGL(conv2d_fwd_kernel, dim3((unsigned)ceil_div(total, kCBlock)), dim3(kCBlock), 0, stream(), x, w, bias, y, c, total);
    return BH_LAUNCH_CHECK("conv2d_fwd_kernel");
}

int bh_conv2d_backward(const float* x, const float* w, const float* dy, float* dx, float* gw, float* gb, int64_t batch,
                       int64_t in_channels, int64_t height, int64_t width, int64_t out_channels, int64_t kernel,
                       int64_t stride, int64_t pad, int accumulate, int flip_taps) {
    BH_REQUIRE_INIT();
    ConvShape c;
    int rc = make_conv_shape(c, batch, in_channels, height, width, out_channels, kernel, stride, pad);
    if (rc) return rc;
    BH_CHECK_ARG(dy || batch == 0, "null pointer");
    if (dx && batch > 0) {
        BH_CHECK_ARG(w, "null pointer");
        const int64_t total = (int64_t)c.batch * c.ic * c.h * c.w;
        hipLaunchKernelGGL(conv2d_bwd_input_kernel, dim3((unsigned)ceil_div(total, kCBlock)), dim3(kCBlock), 0, stream(), w, dy, dx,
                           c, total, flip_taps);
        rc = BH_LAUNCH_CHECK("conv2d_bwd_input_kernel");
        if (rc) return rc;
    }
    if (gw) {
        BH_CHECK_ARG(x || batch == 0, "null pointer");
        const int64_t n_weights = (int64_t)c.oc * c.ic * c.k * c.k;
        hipLaunchKernelGGL(conv2d_bwd_weight_kernel, dim3((unsigned)ceil_div(n_weights, kCBlock / 64)), dim3(kCBlock), 0, stream(),
                           x, dy, gw, c, n_weights, accumulate);
        rc = BH_LAUNCH_CHECK("conv2d_bwd_weight_kernel");
        if (rc) return rc;
    }
    if (gb) {
        hipLaunchKernelGGL(conv2d_bwd_bias_kernel, dim3((unsigned)c.oc), dim3(kCBlock), 0, stream(), dy, gb, c, accumulate);
        rc = BH_LAUNCH_CHECK("conv2d_bwd_bias_kernel");
    }
    return rc;
}

static int make_pool_shape(PoolShape& p, int64_t planes, int64_t h, int64_t w, int64_t pool, int64_t stride, int64_t pad) {
    if (planes < 0 || h <= 0 || w <= 0 || pool <= 0 || stride <= 0 || pad < 0) return set_error(BH_EINVAL, "maxpool2d: bad shape");
    const int64_t ho = (h + 2 * pad - pool) / stride + 1, wo = (w + 2 * pad - pool) / stride + 1;
    if (h + 2 * pad < pool || w + 2 * pad < pool || ho <= 0 || wo <= 0) return set_error(BH_EINVAL, "maxpool2d: window larger than the padded image");
    if (h * w >= ((int64_t)1 << 30)) return set_error(BH_EINVAL, "maxpool2d: plane too large for 32-bit indexing");
    p.planes = planes; p.h = (int)h; p.w = (int)w; p.ho = (int)ho; p.wo = (int)wo;
    p.pool = (int)pool; p.stride = (int)stride; p.pad = (int)pad;
    return BH_OK;
}

int bh_maxpool2d_forward(const float* x, float* y, int32_t* argmax, int64_t planes, int64_t height, int64_t width, int64_t pool,
                         int64_t stride, int64_t pad) {
    BH_REQUIRE_INIT();
    PoolShape p;
    int rc = make_pool_shape(p, planes, height, width, pool, stride, pad);
    if (rc) return rc;
    if (planes == 0) return BH_OK;
    BH_CHECK_ARG(x && y && argmax, "null pointer");
    const int64_t total = planes * p.ho * p.wo;
    BH_CHECK_ARG(ceil_div(total, kCBlock) <= 0x7fffffff, "tensor too large");
    hipLaunchKernelGGL(maxpool_fwd_kernel, dim3((unsigned)ceil_div(total, kCBlock)), dim3(kCBlock), 0, stream(), x, y, argmax, p, total);
    return BH_LAUNCH_CHECK("maxpool_fwd_kernel");
}

int bh_maxpool2d_backward(const float* dy, const int32_t* argmax, float* dx, int64_t planes, int64_t height, int64_t width,
                          int64_t pool, int64_t stride, int64_t pad) {
    BH_REQUIRE_INIT();
    PoolShape p;
    int rc = make_pool_shape(p, planes, height, width, pool, stride, pad);
    if (rc) return rc;
    if (planes == 0) return BH_OK;
    BH_CHECK_ARG(dy && argmax && dx, "null pointer");
    const int64_t total = planes * p.h * p.w;
    BH_CHECK_ARG(ceil_div(total, kCBlock) <= 0x7fffffff, "tensor too large");
    hipLaunchKernelGGL(maxpool_bwd_kernel, dim3((unsigned)ceil_div(total, kCBlock)), dim3(kCBlock), 0, stream(), dy, argmax, dx, p, total);
    return BH_LAUNCH_CHECK("maxpool_bwd_kernel");
}

}  // extern "C"
