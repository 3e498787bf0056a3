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
//
// RMSprop (src/optimizers/rmsprop.c:181-211) and Adagrad (src/optimizers/adagrad.c:167-197) use the same
// launch shapes with one state tensor instead of two (20 bytes per element):
//   RMSprop  s = alpha*s + (1-alpha)*g*g ; p -= lr*g/(sqrtf(s)+eps)
//   Adagrad  s += g*g                    ; p -= lr*g/(sqrtf(s)+eps)
#include "bh_common.h"

#include <math.h>

namespace bh {

constexpr int kAdamBlock = 64;    // one wavefront per workgroup: 6.44 TB/s on the flat step against 6.06 with 256 lanes
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

struct SqScalars {
    float lr, alpha, one_minus_alpha, eps;
    int rule;   // 0 = RMSprop, 1 = Adagrad
};

__device__ __forceinline__ void sq_one(float& p, float g, float& sq, const SqScalars& s) {
    if (s.rule == 0) sq = s.alpha * sq + s.one_minus_alpha * g * g;
    else sq += g * g;
    p -= s.lr * g / (sqrtf(sq) + s.eps);
}

typedef float f32x4 __attribute__((ext_vector_type(4)));

// same lane map as adam_group, one state tensor
__device__ __forceinline__ void sq_group(float* __restrict__ p, const float* __restrict__ g, float* __restrict__ sq,
                                         int64_t n, const SqScalars& s, int64_t idx) {
    const int64_t n4 = n >> 2;
    if (idx < n4) {
        f32x4 pp = __builtin_nontemporal_load(reinterpret_cast<f32x4*>(p) + idx);
        f32x4 gg = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(g) + idx);
        f32x4 ss = __builtin_nontemporal_load(reinterpret_cast<f32x4*>(sq) + idx);
        float px = pp.x, py = pp.y, pz = pp.z, pw = pp.w;
        float sx = ss.x, sy = ss.y, sz = ss.z, sw = ss.w;
        sq_one(px, gg.x, sx, s);
        sq_one(py, gg.y, sy, s);
        sq_one(pz, gg.z, sz, s);
        sq_one(pw, gg.w, sw, s);
        pp = (f32x4){px, py, pz, pw};
        ss = (f32x4){sx, sy, sz, sw};
        __builtin_nontemporal_store(pp, reinterpret_cast<f32x4*>(p) + idx);
        __builtin_nontemporal_store(ss, reinterpret_cast<f32x4*>(sq) + idx);
    }
    if (idx < (n & 3)) {
        const int64_t i = (n4 << 2) + idx;
        float pp = p[i], ss = sq[i];
        sq_one(pp, g[i], ss, s);
        p[i] = pp;
        sq[i] = ss;
    }
}

// One float4 group per lane: lane `idx` of the tensor's own grid updates elements 4*idx..4*idx+3;
// the first (n % 4) lanes also take one tail element.  No loop: the grid covers the tensor, so the
// resident workgroups sweep p, g, m and v as four contiguous moving windows, and every access is
// non-temporal (each byte is touched once per step).
__device__ __forceinline__ void adam_group(float* __restrict__ p, const float* __restrict__ g, float* __restrict__ m,
                                           float* __restrict__ v, int64_t n, const AdamScalars& s, int64_t idx) {
    const int64_t n4 = n >> 2;
    if (idx < n4) {
        f32x4 pp = __builtin_nontemporal_load(reinterpret_cast<f32x4*>(p) + idx);
        f32x4 gg = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(g) + idx);
        f32x4 mm = __builtin_nontemporal_load(reinterpret_cast<f32x4*>(m) + idx);
        f32x4 vv = __builtin_nontemporal_load(reinterpret_cast<f32x4*>(v) + idx);
        float px = pp.x, py = pp.y, pz = pp.z, pw = pp.w;
        float mx = mm.x, my = mm.y, mz = mm.z, mw = mm.w;
        float vx = vv.x, vy = vv.y, vz = vv.z, vw = vv.w;
        adam_one(px, gg.x, mx, vx, s);
        adam_one(py, gg.y, my, vy, s);
        adam_one(pz, gg.z, mz, vz, s);
        adam_one(pw, gg.w, mw, vw, s);
        pp = (f32x4){px, py, pz, pw};
        mm = (f32x4){mx, my, mz, mw};
        vv = (f32x4){vx, vy, vz, vw};
        __builtin_nontemporal_store(pp, reinterpret_cast<f32x4*>(p) + idx);
        __builtin_nontemporal_store(mm, reinterpret_cast<f32x4*>(m) + idx);
        __builtin_nontemporal_store(vv, reinterpret_cast<f32x4*>(v) + idx);
    }
    if (idx < (n & 3)) {
        const int64_t i = (n4 << 2) + idx;
        float pp = p[i], mm = m[i], vv = v[i];
        adam_one(pp, g[i], mm, vv, s);
        p[i] = pp;
        m[i] = mm;
        v[i] = vv;
    }
}

__global__ __launch_bounds__(kAdamBlock) void adam_flat_kernel(float* p, const float* g, float* m, float* v,
                                                               int64_t n, AdamScalars s) {
    adam_group(p, g, m, v, n, s, (int64_t)blockIdx.x * kAdamBlock + threadIdx.x);
}

// Adam's memory pattern without Adam's arithmetic (four streams read, three written, one add each): what the same
// grid of the same workgroups reaches when nothing but the memory system is in the way (benchmark hook)
__global__ __launch_bounds__(kAdamBlock) void stream_4r3w_kernel(float* __restrict__ p, const float* __restrict__ g,
                                                                 float* __restrict__ m, float* __restrict__ v, int64_t n4) {
    const int64_t idx = (int64_t)blockIdx.x * kAdamBlock + threadIdx.x;
    if (idx >= n4) return;
    f32x4 pp = __builtin_nontemporal_load(reinterpret_cast<f32x4*>(p) + idx);
    const f32x4 gg = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(g) + idx);
    f32x4 mm = __builtin_nontemporal_load(reinterpret_cast<f32x4*>(m) + idx);
    f32x4 vv = __builtin_nontemporal_load(reinterpret_cast<f32x4*>(v) + idx);
    pp += gg;
    mm += gg;
    vv += gg;
    __builtin_nontemporal_store(pp, reinterpret_cast<f32x4*>(p) + idx);
    __builtin_nontemporal_store(mm, reinterpret_cast<f32x4*>(m) + idx);
    __builtin_nontemporal_store(vv, reinterpret_cast<f32x4*>(v) + idx);
}

__global__ __launch_bounds__(kAdamBlock) void adam_flat_scalar_kernel(float* p, const float* g, float* m, float* v,
                                                                      int64_t n, AdamScalars s) {
    const int64_t i = (int64_t)blockIdx.x * kAdamBlock + threadIdx.x;
    if (i < n) {
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
    const int64_t idx = (int64_t)((int)blockIdx.x - t.first_block[lo]) * kAdamBlock + threadIdx.x;
    float* p = t.p[lo];
    const float* g = t.g[lo];
    float* m = t.m[lo];
    float* v = t.v[lo];
    const int64_t n = t.n[lo];
    const bool vec = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(m) |
                       reinterpret_cast<uintptr_t>(v)) & 15) == 0;
    if (vec) {
        adam_group(p, g, m, v, n, s, idx);
    } else {
        // unaligned tensor: this block's lanes walk the tensor with the stride of the blocks it was given
        const int64_t stride = (int64_t)(t.first_block[lo + 1] - t.first_block[lo]) * kAdamBlock;
        for (int64_t i = idx; i < n; i += stride) {
            float pp = p[i], mm = m[i], vv = v[i];
            adam_one(pp, g[i], mm, vv, s);
            p[i] = pp;
            m[i] = mm;
            v[i] = vv;
        }
    }
}

__global__ __launch_bounds__(kAdamBlock) void sq_multi_kernel(AdamTable t, SqScalars s) {
    int lo = 0, hi = t.count;
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if ((int)blockIdx.x >= t.first_block[mid]) lo = mid; else hi = mid;
    }
    const int64_t idx = (int64_t)((int)blockIdx.x - t.first_block[lo]) * kAdamBlock + threadIdx.x;
    float* p = t.p[lo];
    const float* g = t.g[lo];
    float* sq = t.m[lo];
    const int64_t n = t.n[lo];
    const bool vec = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(sq)) & 15) == 0;
    if (vec) {
        sq_group(p, g, sq, n, s, idx);
    } else {
        const int64_t stride = (int64_t)(t.first_block[lo + 1] - t.first_block[lo]) * kAdamBlock;
        for (int64_t i = idx; i < n; i += stride) {
            float pp = p[i], ss = sq[i];
            sq_one(pp, g[i], ss, s);
            p[i] = pp;
            sq[i] = ss;
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

// zero up to kAdamMaxTensors tensors in one launch (gradient buffers before the next backward)
struct ZeroTable {
    float* p[kAdamMaxTensors];
    int64_t n[kAdamMaxTensors];
    int first_block[kAdamMaxTensors + 1];
    int count;
};

__global__ __launch_bounds__(kAdamBlock) void zero_multi_kernel(ZeroTable t) {
    int lo = 0, hi = t.count;
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if ((int)blockIdx.x >= t.first_block[mid]) lo = mid; else hi = mid;
    }
    const int64_t idx = (int64_t)((int)blockIdx.x - t.first_block[lo]) * kAdamBlock + threadIdx.x;
    float* p = t.p[lo];
    const int64_t n = t.n[lo];
    if ((reinterpret_cast<uintptr_t>(p) & 15) == 0) {
        const int64_t i = idx * 4;
        if (i + 3 < n) *reinterpret_cast<float4*>(p + i) = make_float4(0.f, 0.f, 0.f, 0.f);
        else for (int64_t j = i; j < n; j++) p[j] = 0.f;
    } else {
        const int64_t stride = (int64_t)(t.first_block[lo + 1] - t.first_block[lo]) * kAdamBlock;
        for (int64_t i = idx; i < n; i += stride) p[i] = 0.f;
    }
}

// workgroups that cover n elements with one float4 group per lane
static int64_t blocks_for(int64_t n) {
    int64_t b = ceil_div(ceil_div(n, 4), kAdamBlock);
    return b < 1 ? 1 : b;
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
    ProfScope prof(BH_PROF_OPTIMIZER, 28.0 * (double)n);
    AdamScalars s = make_scalars(lr, beta1, beta2, eps, timestep);
    const bool vec = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(m) |
                       reinterpret_cast<uintptr_t>(v)) & 15) == 0;
    const int64_t blocks = vec ? blocks_for(n) : blocks_for(n * 4);
    BH_CHECK_ARG(blocks <= 0x7fffffff, "tensor too large");
    if (vec)
        hipLaunchKernelGGL(adam_flat_kernel, dim3((unsigned)blocks), dim3(kAdamBlock), 0, stream(), p, g, m, v, n, s);
    else
        hipLaunchKernelGGL(adam_flat_scalar_kernel, dim3((unsigned)blocks), dim3(kAdamBlock), 0, stream(), p, g, m, v, n, s);
    return BH_LAUNCH_CHECK("bh_adam_update");
}

// benchmark hook: p += g, m += g, v += g over n floats (n % 4 == 0, 16-byte aligned) with Adam's grid and access pattern
int bh_stream_probe_4r3w(float* p, const float* g, float* m, float* v, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && n % 4 == 0, "n must be a multiple of 4");
    if (n == 0) return BH_OK;
    BH_CHECK_ARG(p && g && m && v, "null pointer");
    BH_CHECK_ARG(((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(m) |
                   reinterpret_cast<uintptr_t>(v)) & 15) == 0, "pointers must be 16-byte aligned");
    const int64_t blocks = blocks_for(n);
    BH_CHECK_ARG(blocks <= 0x7fffffff, "tensor too large");
    hipLaunchKernelGGL(stream_4r3w_kernel, dim3((unsigned)blocks), dim3(kAdamBlock), 0, stream(), p, g, m, v, n / 4);
    return BH_LAUNCH_CHECK("bh_stream_probe_4r3w");
}

int bh_adam_update_multi(float* const* p, const float* const* g, float* const* m, float* const* v, const int64_t* n,
                         int count, float lr, float beta1, float beta2, float eps, int64_t timestep) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(count >= 0 && timestep >= 0, "negative count or timestep");
    BH_CHECK_ARG(count == 0 || (p && g && m && v && n), "null table");
    double total = 0.0;
    for (int i = 0; i < count; i++) total += n[i] > 0 ? (double)n[i] : 0.0;
    ProfScope prof(BH_PROF_OPTIMIZER, 28.0 * total);
    AdamScalars s = make_scalars(lr, beta1, beta2, eps, timestep);
    int done = 0;
    while (done < count) {
        AdamTable t;
        t.count = 0;
        int64_t blocks = 0;
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
            t.first_block[k] = (int)blocks;
            blocks += blocks_for(n[i]);
            BH_CHECK_ARG(blocks <= 0x7fffffff, "tensors too large for one launch");
        }
        if (t.count == 0) continue;
        t.first_block[t.count] = (int)blocks;
        hipLaunchKernelGGL(adam_multi_kernel, dim3((unsigned)blocks), dim3(kAdamBlock), 0, stream(), t, s);
        int rc = BH_LAUNCH_CHECK("bh_adam_update_multi");
        if (rc) return rc;
    }
    return BH_OK;
}

int bh_zero_multi(float* const* p, const int64_t* n, int count) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(count >= 0 && (count == 0 || (p && n)), "bad table");
    int done = 0;
    while (done < count) {
        ZeroTable t;
        t.count = 0;
        int64_t blocks = 0;
        while (done < count && t.count < kAdamMaxTensors) {
            const int i = done++;
            BH_CHECK_ARG(n[i] >= 0, "negative element count");
            if (n[i] == 0) continue;
            BH_CHECK_ARG(p[i], "null tensor pointer");
            const int k = t.count++;
            t.p[k] = p[i];
            t.n[k] = n[i];
            t.first_block[k] = (int)blocks;
            blocks += blocks_for(n[i]);
            BH_CHECK_ARG(blocks <= 0x7fffffff, "tensors too large for one launch");
        }
        if (t.count == 0) continue;
        t.first_block[t.count] = (int)blocks;
        hipLaunchKernelGGL(zero_multi_kernel, dim3((unsigned)blocks), dim3(kAdamBlock), 0, stream(), t);
        int rc = BH_LAUNCH_CHECK("bh_zero_multi");
        if (rc) return rc;
    }
    return BH_OK;
}

// rule 0: RMSprop (alpha used), rule 1: Adagrad (alpha ignored)
static int sq_update_multi(int rule, float* const* p, const float* const* g, float* const* sq, const int64_t* n, int count,
                           float lr, float alpha, float eps) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(count >= 0, "negative count");
    BH_CHECK_ARG(count == 0 || (p && g && sq && n), "null table");
    SqScalars s;
    s.lr = lr;
    s.alpha = alpha;
    s.one_minus_alpha = 1.0f - alpha;
    s.eps = eps;
    s.rule = rule;
    int done = 0;
    while (done < count) {
        AdamTable t;
        t.count = 0;
        int64_t blocks = 0;
        while (done < count && t.count < kAdamMaxTensors) {
            const int i = done++;
            BH_CHECK_ARG(n[i] >= 0, "negative element count");
            if (n[i] == 0) continue;
            BH_CHECK_ARG(p[i] && g[i] && sq[i], "null tensor pointer");
            const int k = t.count++;
            t.p[k] = p[i];
            t.g[k] = g[i];
            t.m[k] = sq[i];
            t.v[k] = nullptr;
            t.n[k] = n[i];
            t.first_block[k] = (int)blocks;
            blocks += blocks_for(n[i]);
            BH_CHECK_ARG(blocks <= 0x7fffffff, "tensors too large for one launch");
        }
        if (t.count == 0) continue;
        t.first_block[t.count] = (int)blocks;
        hipLaunchKernelGGL(sq_multi_kernel, dim3((unsigned)blocks), dim3(kAdamBlock), 0, stream(), t, s);
        int rc = BH_LAUNCH_CHECK("bh_sq_update_multi");
        if (rc) return rc;
    }
    return BH_OK;
}

int bh_rmsprop_update_multi(float* const* p, const float* const* g, float* const* sq, const int64_t* n, int count, float lr,
                            float alpha, float eps) {
    return sq_update_multi(0, p, g, sq, n, count, lr, alpha, eps);
}
int bh_adagrad_update_multi(float* const* p, const float* const* g, float* const* sum, const int64_t* n, int count, float lr,
                            float eps) {
    return sq_update_multi(1, p, g, sum, n, count, lr, 0.0f, eps);
}
int bh_rmsprop_update(float* p, const float* g, float* sq, int64_t n, float lr, float alpha, float eps) {
    const float* gg = g;
    return sq_update_multi(0, &p, &gg, &sq, &n, 1, lr, alpha, eps);
}
int bh_adagrad_update(float* p, const float* g, float* sum, int64_t n, float lr, float eps) {
    const float* gg = g;
    return sq_update_multi(1, &p, &gg, &sum, &n, 1, lr, 0.0f, eps);
}

}  // extern "C"
