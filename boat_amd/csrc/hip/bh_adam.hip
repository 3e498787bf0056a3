// bh_adam.hip - fused one-pass Adam step.
//
// Replaces adam_update_parameter / adam_optimizer_step, src/optimizers/adam.c:180-240:
//   m = b1*m + (1-b1)*g ; v = b2*v + (1-b2)*g*g ;
//   p -= lr * (m/(1-b1^t)) / (sqrtf(v/(1-b2^t)) + eps)
// with epsilon outside the square root and the bias corrections formed from
// powf(beta, (float)(timestep+1)) on the host in fp32, exactly as the reference forms
// them.  The kernel keeps the reference's operation order (two roundings per a*b+c,
// true divisions, IEEE sqrt; the file is compiled with -ffp-contract=off), so the
// result is bit-identical to the scalar C loop, not merely within tolerance.
//
// Traffic per element: read p,g,m,v + write p,m,v = 28 bytes, one pass, float4 lanes.
#include "bh_common.h"

#include <math.h>

namespace bh {

constexpr int kAdamBlock = 256;
constexpr int kAdamMaxTensors = 48;

struct AdamScalars {
    float lr, beta1, beta2, eps;
    float one_minus_beta1, one_minus_beta2;
    float corr1, corr2;   // 1 - beta^(t+1)
};

__device__ __forceinline__ void adam_one(float& p, float g, float& m, float& v, const AdamScalars& s) {
    m = s.beta1 * m + s.one_minus_beta1 * g;
    v = s.beta2 * v + s.one_minus_beta2 * g * g;
    float m_hat = m / s.corr1;
    float v_hat = v / s.corr2;
    p -= s.lr * m_hat / (sqrtf(v_hat) + s.eps);
}

__device__ __forceinline__ void adam_span(float* __restrict__ p, const float* __restrict__ g, float* __restrict__ m,
                                          float* __restrict__ v, int64_t n, const AdamScalars& s, int64_t first,
                                          int64_t stride) {
    // n4 float4 groups, then a scalar tail
    const int64_t n4 = n >> 2;
    float4* p4 = reinterpret_cast<float4*>(p);
    const float4* g4 = reinterpret_cast<const float4*>(g);
    float4* m4 = reinterpret_cast<float4*>(m);
    float4* v4 = reinterpret_cast<float4*>(v);
    for (int64_t i = first; i < n4; i += stride) {
        float4 pp = p4[i], gg = g4[i], mm = m4[i], vv = v4[i];
        adam_one(pp.x, gg.x, mm.x, vv.x, s);
        adam_one(pp.y, gg.y, mm.y, vv.y, s);
        adam_one(pp.z, gg.z, mm.z, vv.z, s);
        adam_one(pp.w, gg.w, mm.w, vv.w, s);
        p4[i] = pp;
        m4[i] = mm;
        v4[i] = vv;
    }
    const int64_t tail = n & 3;
    if (first < tail) {
        const int64_t i = (n4 << 2) + first;
        float pp = p[i], mm = m[i], vv = v[i];
        adam_one(pp, g[i], mm, vv, s);
        p[i] = pp;
        m[i] = mm;
        v[i] = vv;
    }
}

__global__ __launch_bounds__(kAdamBlock) void adam_flat_kernel(float* p, const float* g, float* m, float* v,
                                                               int64_t n, AdamScalars s) {
    adam_span(p, g, m, v, n, s, (int64_t)blockIdx.x * blockDim.x + threadIdx.x, (int64_t)gridDim.x * blockDim.x);
}

__global__ __launch_bounds__(kAdamBlock) void adam_flat_scalar_kernel(float* p, const float* g, float* m, float* v,
                                                                      int64_t n, AdamScalars s) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float pp = p[i], mm = m[i], vv = v[i];
        adam_one(pp, g[i], mm, vv, s);
        p[i] = pp;
        m[i] = mm;
        v[i] = vv;
    }
}

// One launch over up to kAdamMaxTensors tensors.  Blocks are dealt to tensors in
// proportion to their size: block b works on tensor t where first_block[t] <= b <
// first_block[t+1], striding over that tensor with the blocks it shares it with.
struct AdamTable {
    float* p[kAdamMaxTensors];
    const float* g[kAdamMaxTensors];
    float* m[kAdamMaxTensors];
    float* v[kAdamMaxTensors];
    int64_t n[kAdamMaxTensors];
    int first_block[kAdamMaxTensors + 1];
    int count;
};

__global__ __launch_bounds__(kAdamBlock) void adam_multi_kernel(AdamTable t, AdamScalars s) {
    int lo = 0, hi = t.count;   // find tensor with first_block[lo] <= blockIdx.x < first_block[lo+1]
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if ((int)blockIdx.x >= t.first_block[mid]) lo = mid; else hi = mid;
    }
    const int nb = t.first_block[lo + 1] - t.first_block[lo];
    const int lb = (int)blockIdx.x - t.first_block[lo];
    float* p = t.p[lo];
    const float* g = t.g[lo];
    float* m = t.m[lo];
    float* v = t.v[lo];
    const int64_t n = t.n[lo];
    const bool vec = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(m) |
                       reinterpret_cast<uintptr_t>(v)) & 15) == 0;
    const int64_t first = (int64_t)lb * blockDim.x + threadIdx.x, stride = (int64_t)nb * blockDim.x;
    if (vec) {
        adam_span(p, g, m, v, n, s, first, stride);
    } else {
        for (int64_t i = first; i < n; i += stride) {
            float pp = p[i], mm = m[i], vv = v[i];
            adam_one(pp, g[i], mm, vv, s);
            p[i] = pp;
            m[i] = mm;
            v[i] = vv;
        }
    }
}

static AdamScalars make_scalars(float lr, float beta1, float beta2, float eps, int64_t timestep) {
    AdamScalars s;
    s.lr = lr;
    s.beta1 = beta1;
    s.beta2 = beta2;
    s.eps = eps;
    s.one_minus_beta1 = 1.0f - beta1;
    s.one_minus_beta2 = 1.0f - beta2;
    // adam.c:203-204: the exponent is converted to float before powf
    s.corr1 = 1.0f - powf(beta1, (float)(timestep + 1));
    s.corr2 = 1.0f - powf(beta2, (float)(timestep + 1));
    return s;
}

static int blocks_for(int64_t n) {
    int64_t b = ceil_div(ceil_div(n, 4), kAdamBlock);
    if (b > 256 * 16) b = 256 * 16;
    if (b < 1) b = 1;
    return (int)b;
}

}  // namespace bh

using namespace bh;

extern "C" {

int bh_adam_update(float* p, const float* g, float* m, float* v, int64_t n, float lr, float beta1, float beta2,
                   float eps, int64_t timestep) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && timestep >= 0, "negative size or timestep");
    if (n == 0) return BH_OK;
    BH_CHECK_ARG(p && g && m && v, "null pointer");
    AdamScalars s = make_scalars(lr, beta1, beta2, eps, timestep);
    const bool vec = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(m) |
                       reinterpret_cast<uintptr_t>(v)) & 15) == 0;
    if (vec)
        hipLaunchKernelGGL(adam_flat_kernel, dim3(blocks_for(n)), dim3(kAdamBlock), 0, stream(), p, g, m, v, n, s);
    else
        hipLaunchKernelGGL(adam_flat_scalar_kernel, dim3(blocks_for(n * 4)), dim3(kAdamBlock), 0, stream(), p, g, m, v,
                           n, s);
    return BH_LAUNCH_CHECK("bh_adam_update");
}

int bh_adam_update_multi(float* const* p, const float* const* g, float* const* m, float* const* v, const int64_t* n,
                         int count, float lr, float beta1, float beta2, float eps, int64_t timestep) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(count >= 0 && timestep >= 0, "negative count or timestep");
    BH_CHECK_ARG(count == 0 || (p && g && m && v && n), "null table");
    AdamScalars s = make_scalars(lr, beta1, beta2, eps, timestep);
    int done = 0;
    while (done < count) {
        AdamTable t;
        t.count = 0;
        int blocks = 0;
        while (done < count && t.count < kAdamMaxTensors) {
            const int i = done++;
            BH_CHECK_ARG(n[i] >= 0, "negative element count");
            if (n[i] == 0) continue;
            BH_CHECK_ARG(p[i] && g[i] && m[i] && v[i], "null tensor pointer");
            const int k = t.count++;
            t.p[k] = p[i];
            t.g[k] = g[i];
            t.m[k] = m[i];
            t.v[k] = v[i];
            t.n[k] = n[i];
            t.first_block[k] = blocks;
            blocks += blocks_for(n[i]);
        }
        if (t.count == 0) continue;
        t.first_block[t.count] = blocks;
        hipLaunchKernelGGL(adam_multi_kernel, dim3(blocks), dim3(kAdamBlock), 0, stream(), t, s);
        int rc = BH_LAUNCH_CHECK("bh_adam_update_multi");
        if (rc) return rc;
    }
    return BH_OK;
}

}  // extern "C"
