// bh_layernorm.hip - LayerNorm forward (emits mean, rstd) and single-pass backward.
//
// Forward follows boat_layernorm_forward, src/layers/norm.c:184-209 (per-row mean, then
// two-pass biased variance) and :283-305 (rstd = 1/sqrtf(var+eps); y = (x-mean)*rstd*gamma+beta),
// and additionally writes mean/rstd, which the reference computes and frees (:313-314).
//
// Backward has no counterpart in the reference (boat_layernorm_backward is a stub,
// src/layers/norm.c:397-402).  It implements
//   xhat = (x-mean)*rstd ; g = dy*gamma
//   dx = rstd*(g - mean_h(g) - xhat*mean_h(g*xhat)) ; dgamma = sum_rows dy*xhat ; dbeta = sum_rows dy
// in one read of x and dy: each thread owns fixed columns, keeps its slice of the row in
// registers, reduces the two row sums with wavefront shuffles (+ one LDS exchange when a row
// spans 4 wavefronts), and accumulates dgamma/dbeta for its columns over all rows of its
// block.  Per-block partials are folded by a second small kernel (two-stage reduction, no
// atomics, deterministic).
#include "bh_common.h"

namespace bh {

constexpr int kLnBlock = 256;

// Scratch of bh_layernorm_backward_noalloc: the per-workgroup dgamma/dbeta partials that bh_layernorm_backward
// takes from bh_malloc.  One copy per GPU, held until the process ends.  Host code never uses the array's name
// as an address: ln_scratch_setup() asks the runtime for the device address once per device and keeps it.
constexpr size_t kLnScratchFloats = size_t(4) << 20;   // 16 MiB
static __device__ __align__(256) float ln_scratch[kLnScratchFloats];
constexpr int kMaxDevices = 16;
static float* g_ln_scratch_ptr[kMaxDevices] = {};

__device__ __forceinline__ float4 ld4(const float* p, int64_t i4) { return reinterpret_cast<const float4*>(p)[i4]; }
__device__ __forceinline__ void st4(float* p, int64_t i4, float4 v) { reinterpret_cast<float4*>(p)[i4] = v; }
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 ld4_stream(const float* p, int64_t i4) {
    f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p) + i4);
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st4_stream(float* p, int64_t i4, float4 v) {
    f32x4 o = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(o, reinterpret_cast<f32x4*>(p) + i4);
}


// Sum of two values over the TPR threads that share a row.
template <int TPR>
__device__ __forceinline__ void row_sum2(float& a, float& b, float* lds, int group) {
    a = wave_sum(a);
    b = wave_sum(b);
    if (TPR > 64) {
        constexpr int W = TPR / 64;
        const int lane = threadIdx.x & 63, w = (threadIdx.x >> 6) % W;
        float* slot = lds + group * W * 2;
        __syncthreads();
        if (lane == 0) {
            slot[w * 2] = a;
            slot[w * 2 + 1] = b;
        }
        __syncthreads();
        float ta = 0.f, tb = 0.f;
#pragma unroll
        for (int i = 0; i < W; i++) {
            ta += slot[i * 2];
            tb += slot[i * 2 + 1];
        }
        a = ta;
        b = tb;
    }
}

// ---------------------------------------------------------------- forward
// RMS: the RMSNorm of src/layers/norm.c:212-229,366-389 instead: r = sqrtf(mean(x^2)), y = x * (1/(r+eps)) * weight,
// no mean, no bias; `rstd` then receives 1/(r+eps).
template <int TPR, int VPT, bool RMS>
__global__ __launch_bounds__(kLnBlock) void ln_fwd_kernel(const float* __restrict__ x, const float* __restrict__ gamma,
                                                          const float* __restrict__ beta, float* __restrict__ y,
                                                          float* __restrict__ mean, float* __restrict__ rstd,
                                                          int64_t rows, int hidden, float eps, int64_t rows_per_group) {
    constexpr int GROUPS = kLnBlock / TPR;
    __shared__ float lds[GROUPS * (TPR / 64) * 2 + 2];
    const int group = threadIdx.x / TPR, t = threadIdx.x % TPR;
    const int h4 = hidden >> 2;
    const int64_t g_id = (int64_t)blockIdx.x * GROUPS + group;
    const int64_t total_groups = (int64_t)gridDim.x * GROUPS;

    float4 gm[VPT], bt[VPT];
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int c4 = t + i * TPR;
        gm[i] = (gamma && c4 < h4) ? ld4(gamma, c4) : make_float4(1, 1, 1, 1);
        bt[i] = (beta && c4 < h4) ? ld4(beta, c4) : make_float4(0, 0, 0, 0);
    }
    // Group g takes rows g, g+G, g+2G, ...: the resident workgroups read neighbouring rows (one moving
    // window).  rows_per_group is the same for every group, so the loop trip count (and every barrier
    // inside row_sum2) is uniform across the block; out-of-range rows are masked.
    // The next row of the group is fetched before the current one is reduced, so that its trip to memory runs under the
    // two reductions and the stores instead of in front of them.
    float4 xn[VPT];
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int c4 = t + i * TPR;
        xn[i] = (g_id < rows && c4 < h4 && rows_per_group > 0) ? ld4_stream(x + g_id * hidden, c4) : make_float4(0, 0, 0, 0);
    }
    for (int64_t it = 0; it < rows_per_group; it++) {
        const int64_t r = it * total_groups + g_id;
        const bool live = r < rows;
        float4 xv[VPT];
        float s = 0.f, dummy = 0.f;
        const int64_t rn = r + total_groups;
        const bool live_n = it + 1 < rows_per_group && rn < rows;
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int c4 = t + i * TPR;
            xv[i] = xn[i];
            xn[i] = (live_n && c4 < h4) ? ld4_stream(x + rn * hidden, c4) : make_float4(0, 0, 0, 0);
            s += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);
        }
        float mu = 0.f;
        if (!RMS) {
            row_sum2<TPR>(s, dummy, lds, group);
            mu = s / (float)hidden;
        }
        float q = 0.f;
        dummy = 0.f;
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int c4 = t + i * TPR;
            if (c4 < h4) {
                float dx0 = xv[i].x - mu, dx1 = xv[i].y - mu, dx2 = xv[i].z - mu, dx3 = xv[i].w - mu;
                q += (dx0 * dx0 + dx1 * dx1) + (dx2 * dx2 + dx3 * dx3);
            }
        }
        row_sum2<TPR>(q, dummy, lds, group);
        const float var = q / (float)hidden;
        const float rs = RMS ? 1.0f / (sqrtf(var) + eps) : 1.0f / sqrtf(var + eps);
        if (live) {
#pragma unroll
            for (int i = 0; i < VPT; i++) {
                const int c4 = t + i * TPR;
                if (c4 < h4) {
                    float4 o;
                    o.x = (xv[i].x - mu) * rs;
                    o.y = (xv[i].y - mu) * rs;
                    o.z = (xv[i].z - mu) * rs;
                    o.w = (xv[i].w - mu) * rs;
                    if (gamma) { o.x *= gm[i].x; o.y *= gm[i].y; o.z *= gm[i].z; o.w *= gm[i].w; }
                    if (beta) { o.x += bt[i].x; o.y += bt[i].y; o.z += bt[i].z; o.w += bt[i].w; }
                    st4_stream(y + r * hidden, c4, o);
                }
            }
            if (t == 0) {
                if (mean) mean[r] = mu;
                if (rstd) rstd[r] = rs;
            }
        }
    }
}

// any hidden size: one block per row, three passes over the row (served from cache)
__global__ __launch_bounds__(kLnBlock) void ln_fwd_generic_kernel(const float* __restrict__ x, const float* __restrict__ gamma,
                                                                  const float* __restrict__ beta, float* __restrict__ y,
                                                                  float* __restrict__ mean, float* __restrict__ rstd,
                                                                  int64_t rows, int64_t hidden, float eps, int rms) {
    __shared__ float red[kLnBlock / 64];
    const int64_t r = blockIdx.x;
    const float* xr = x + r * hidden;
    float s = 0.f;
    if (!rms)
        for (int64_t c = threadIdx.x; c < hidden; c += kLnBlock) s += xr[c];
    const float mu = rms ? 0.f : block_sum<kLnBlock / 64>(s, red) / (float)hidden;
    float q = 0.f;
    for (int64_t c = threadIdx.x; c < hidden; c += kLnBlock) {
        float d = xr[c] - mu;
        q += d * d;
    }
    const float var = block_sum<kLnBlock / 64>(q, red) / (float)hidden;
    const float rs = rms ? 1.0f / (sqrtf(var) + eps) : 1.0f / sqrtf(var + eps);
    for (int64_t c = threadIdx.x; c < hidden; c += kLnBlock) {
        float o = (xr[c] - mu) * rs;
        if (gamma) o *= gamma[c];
        if (beta) o += beta[c];
        y[r * hidden + c] = o;
    }
    if (threadIdx.x == 0) {
        if (mean) mean[r] = mu;
        if (rstd) rstd[r] = rs;
    }
}

// --------------------------------------------------------------- backward
// partial layout: [num_blocks][2][hidden]  (dgamma slice, then dbeta slice)
//
// Row -> workgroup map: group g of G takes rows g, g+G, g+2G, ... so that at any moment the resident
// workgroups read neighbouring rows (one contiguous moving window over x and dy) instead of G far-apart
// chunks.  The loop is software-pipelined: the loads of the next row are issued before the current
// row's reduction barrier and dx stores, so memory requests stay in flight across the barrier.
// x, dy and dx are streamed once each and marked non-temporal.
//
// RMS: backward of y = x*s*w with s = 1/(r+eps), r = sqrtf(mean(x^2)) (`rstd` holds s, `mean` is not read).  With
// xhat = x*s and g = dy*w:  dx = s*(g - xhat*mean_h(g*xhat)/c), c = r*s = 1 - eps*s (a row of zeros has c = 0 and
// xhat = 0: the second term is dropped); dweight = sum_rows dy*xhat.  The dbeta half of a partial is then unused.
// ADD: dx = (the gradient above) + add, the residual branch's gradient that a pre-LN block would otherwise add in a
// pass of its own; the row of `add` is fetched at the top of the row's iteration and lands under the row sums.
template <int TPR, int VPT, bool RMS, bool ADD>
__device__ __forceinline__ void ln_bwd_body(const float* __restrict__ x, const float* __restrict__ gamma,
                                            const float* __restrict__ dy, const float* __restrict__ mean,
                                            const float* __restrict__ rstd, const float* __restrict__ add,
                                            float* __restrict__ dx, float* __restrict__ partial, int64_t rows, int hidden,
                                            int64_t iters, float eps) {
    constexpr int GROUPS = kLnBlock / TPR;
    extern __shared__ float dyn_lds[];           // GROUPS>1: [GROUPS][2][hidden] for the cross-group fold
    __shared__ float lds[GROUPS * (TPR / 64) * 2 + 2];
    const int group = threadIdx.x / TPR, t = threadIdx.x % TPR;
    const int h4 = hidden >> 2;
    const int64_t total_groups = (int64_t)gridDim.x * GROUPS;
    const int64_t g_id = (int64_t)blockIdx.x * GROUPS + group;

    float4 gm[VPT], dg[VPT], db[VPT], xv[VPT], gy[VPT];
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int c4 = t + i * TPR;
        gm[i] = (gamma && c4 < h4) ? ld4(gamma, c4) : make_float4(1, 1, 1, 1);
        dg[i] = make_float4(0, 0, 0, 0);
        db[i] = make_float4(0, 0, 0, 0);
    }
    const float inv_h = 1.0f / (float)hidden;
    // prologue: first row of this group
    int64_t row = g_id;
    bool live = row < rows;
    float mu = (live && !RMS) ? mean[row] : 0.f, rs = live ? rstd[row] : 0.f;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int c4 = t + i * TPR;
        const bool on = live && c4 < h4;
        xv[i] = on ? ld4_stream(x + row * hidden, c4) : make_float4(0, 0, 0, 0);
        gy[i] = on ? ld4_stream(dy + row * hidden, c4) : make_float4(0, 0, 0, 0);
    }
    // `iters` is the same for every group, so the barriers below are reached uniformly; rows past the
    // end are masked (they contribute zeros and store nothing).
    for (int64_t it = 0; it < iters; it++) {
        float4 xh[VPT], g[VPT], av[ADD ? VPT : 1];
        float s1 = 0.f, s2 = 0.f;
        if constexpr (ADD) {
#pragma unroll
            for (int i = 0; i < VPT; i++) {
                const int c4 = t + i * TPR;
                av[i] = (live && c4 < h4) ? ld4_stream(add + row * hidden, c4) : make_float4(0, 0, 0, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            xh[i].x = (xv[i].x - mu) * rs; xh[i].y = (xv[i].y - mu) * rs; xh[i].z = (xv[i].z - mu) * rs; xh[i].w = (xv[i].w - mu) * rs;
            g[i].x = gy[i].x * gm[i].x; g[i].y = gy[i].y * gm[i].y; g[i].z = gy[i].z * gm[i].z; g[i].w = gy[i].w * gm[i].w;
            s1 += (g[i].x + g[i].y) + (g[i].z + g[i].w);
            s2 += (g[i].x * xh[i].x + g[i].y * xh[i].y) + (g[i].z * xh[i].z + g[i].w * xh[i].w);
            dg[i].x += gy[i].x * xh[i].x; dg[i].y += gy[i].y * xh[i].y; dg[i].z += gy[i].z * xh[i].z; dg[i].w += gy[i].w * xh[i].w;
            db[i].x += gy[i].x; db[i].y += gy[i].y; db[i].z += gy[i].z; db[i].w += gy[i].w;
        }
        const int64_t cur_row = row;
        const bool cur_live = live;
        const float cur_rs = rs;
        // issue the next row's loads before the barrier
        row = (it + 1) * total_groups + g_id;
        live = (it + 1 < iters) && row < rows;
        mu = (live && !RMS) ? mean[row] : 0.f;
        rs = live ? rstd[row] : 0.f;
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int c4 = t + i * TPR;
            const bool on = live && c4 < h4;
            xv[i] = on ? ld4_stream(x + row * hidden, c4) : make_float4(0, 0, 0, 0);
            gy[i] = on ? ld4_stream(dy + row * hidden, c4) : make_float4(0, 0, 0, 0);
        }
        row_sum2<TPR>(s1, s2, lds, group);
        s1 *= inv_h;
        s2 *= inv_h;
        if (RMS) {
            const float c = 1.0f - eps * cur_rs;
            s1 = 0.f;
            s2 = c > 0.f ? s2 / c : 0.f;
        }
        if (cur_live) {
#pragma unroll
            for (int i = 0; i < VPT; i++) {
                const int c4 = t + i * TPR;
                if (c4 < h4) {
                    float4 o;
                    o.x = cur_rs * (g[i].x - s1 - xh[i].x * s2);
                    o.y = cur_rs * (g[i].y - s1 - xh[i].y * s2);
                    o.z = cur_rs * (g[i].z - s1 - xh[i].z * s2);
                    o.w = cur_rs * (g[i].w - s1 - xh[i].w * s2);
                    if constexpr (ADD) {
                        o.x += av[i].x; o.y += av[i].y; o.z += av[i].z; o.w += av[i].w;
                    }
                    st4_stream(dx + cur_row * hidden, c4, o);
                }
            }
        }
    }
    float* out = partial + (int64_t)blockIdx.x * 2 * hidden;
    if (GROUPS == 1) {
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int c4 = t + i * TPR;
            if (c4 < h4) {
                st4(out, c4, dg[i]);
                st4(out + hidden, c4, db[i]);
            }
        }
    } else {
        // fold the GROUPS row-groups of this block through LDS, then write one partial
        float* mine = dyn_lds + (size_t)group * 2 * hidden;
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int c4 = t + i * TPR;
            if (c4 < h4) {
                st4(mine, c4, dg[i]);
                st4(mine + hidden, c4, db[i]);
            }
        }
        __syncthreads();
        for (int c = threadIdx.x; c < 2 * hidden; c += kLnBlock) {
            float acc = 0.f;
#pragma unroll
            for (int gidx = 0; gidx < GROUPS; gidx++) acc += dyn_lds[(size_t)gidx * 2 * hidden + c];
            out[c] = acc;
        }
    }
}

template <int TPR, int VPT, bool RMS>
__global__ __launch_bounds__(kLnBlock) void ln_bwd_kernel(const float* __restrict__ x, const float* __restrict__ gamma,
                                                          const float* __restrict__ dy, const float* __restrict__ mean,
                                                          const float* __restrict__ rstd, const float* __restrict__ add,
                                                          float* __restrict__ dx, float* __restrict__ partial, int64_t rows,
                                                          int hidden, int64_t iters, float eps) {
    ln_bwd_body<TPR, VPT, RMS, false>(x, gamma, dy, mean, rstd, nullptr, dx, partial, rows, hidden, iters, eps);
}
template <int TPR, int VPT, bool RMS>
__global__ __launch_bounds__(kLnBlock) void ln_bwd_add_kernel(const float* __restrict__ x, const float* __restrict__ gamma,
                                                              const float* __restrict__ dy, const float* __restrict__ mean,
                                                              const float* __restrict__ rstd, const float* __restrict__ add,
                                                              float* __restrict__ dx, float* __restrict__ partial, int64_t rows,
                                                              int hidden, int64_t iters, float eps) {
    ln_bwd_body<TPR, VPT, RMS, true>(x, gamma, dy, mean, rstd, add, dx, partial, rows, hidden, iters, eps);
}

// generic backward: one block per row, partial per row-chunk accumulated by columns
__global__ __launch_bounds__(kLnBlock) void ln_bwd_dx_generic_kernel(const float* __restrict__ x, const float* __restrict__ gamma,
                                                                     const float* __restrict__ dy, const float* __restrict__ mean,
                                                                     const float* __restrict__ rstd, const float* __restrict__ add,
                                                                     float* __restrict__ dx,
                                                                     int64_t rows, int64_t hidden, int rms, float eps) {
    __shared__ float red[kLnBlock / 64];
    const int64_t r = blockIdx.x;
    const float mu = rms ? 0.f : mean[r], rs = rstd[r];
    float s1 = 0.f, s2 = 0.f;
    for (int64_t c = threadIdx.x; c < hidden; c += kLnBlock) {
        float xh = (x[r * hidden + c] - mu) * rs;
        float g = dy[r * hidden + c] * (gamma ? gamma[c] : 1.0f);
        s1 += g;
        s2 += g * xh;
    }
    s1 = block_sum<kLnBlock / 64>(s1, red) / (float)hidden;
    s2 = block_sum<kLnBlock / 64>(s2, red) / (float)hidden;
    if (rms) {
        const float cc = 1.0f - eps * rs;
        s1 = 0.f;
        s2 = cc > 0.f ? s2 / cc : 0.f;
    }
    for (int64_t c = threadIdx.x; c < hidden; c += kLnBlock) {
        float xh = (x[r * hidden + c] - mu) * rs;
        float g = dy[r * hidden + c] * (gamma ? gamma[c] : 1.0f);
        const float o = rs * (g - s1 - xh * s2);
        dx[r * hidden + c] = add ? o + add[r * hidden + c] : o;
    }
}
__global__ __launch_bounds__(kLnBlock) void ln_bwd_param_generic_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                                        const float* __restrict__ mean, const float* __restrict__ rstd,
                                                                        float* __restrict__ partial, int64_t rows, int64_t hidden,
                                                                        int64_t rows_per_block, int rms) {
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= hidden) return;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    int64_t r1 = r0 + rows_per_block;
    if (r1 > rows) r1 = rows;
    float dg = 0.f, db = 0.f;
    for (int64_t r = r0; r < r1; r++) {
        float gy = dy[r * hidden + c];
        dg += gy * ((x[r * hidden + c] - (rms ? 0.f : mean[r])) * rstd[r]);
        db += gy;
    }
    partial[((int64_t)blockIdx.y * 2) * hidden + c] = dg;
    partial[((int64_t)blockIdx.y * 2 + 1) * hidden + c] = db;
}

static int g_ln_bwd_blocks = 512;    // cap on backward workgroups (2 per CU)
static int g_ln_fwd_blocks = 512;    // cap on forward workgroups (2 per CU: 88 us at 16384 x 4096 against 93 with 2048)

struct LnPlan {
    bool vector;     // register-resident float4 path
    int tpr, vpt;
};

static LnPlan plan_for(int64_t hidden, const void* p0, const void* p1, const void* p2) {
    LnPlan p{false, 0, 0};
    const bool al = ((reinterpret_cast<uintptr_t>(p0) | reinterpret_cast<uintptr_t>(p1) | reinterpret_cast<uintptr_t>(p2)) & 15) == 0;
    if (!al || (hidden & 3) || hidden <= 0) return p;
    const int64_t h4 = hidden >> 2;
    if (h4 <= 64 * 8) {
        p.tpr = 64;
    } else if (h4 <= 256 * 8) {
        p.tpr = 256;
    } else {
        return p;
    }
    const int64_t need = ceil_div(h4, p.tpr);
    p.vpt = need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : 8;
    p.vector = true;
    return p;
}

// Called by bh_init with the library's device current: resolves that device's copy of ln_scratch.
int ln_scratch_setup() {
    int dev = -1;
    int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
    if (rc) return rc;
    if (dev < 0 || dev >= kMaxDevices) return set_error(BH_EDEVICE, "ln_scratch_setup: device index %d out of range", dev);
    if (g_ln_scratch_ptr[dev]) return BH_OK;
    float* p = nullptr;
    rc = check_hip(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(ln_scratch)), "hipGetSymbolAddress(ln_scratch)");
    if (rc) return rc;
    if (!p) return set_error(BH_EDEVICE, "ln_scratch_setup: the runtime returned no address for ln_scratch");
    g_ln_scratch_ptr[dev] = p;
    return BH_OK;
}

}  // namespace bh

using namespace bh;

#define BH_LN_DISPATCH_1(KERNEL, RMS, plan, grid, shmem, ...)                                                   \
    do {                                                                                                       \
        if ((plan).tpr == 64) {                                                                                \
            switch ((plan).vpt) {                                                                              \
                case 1: hipLaunchKernelGGL((KERNEL<64, 1, RMS>), grid, dim3(kLnBlock), shmem, stream(), __VA_ARGS__); break; \
                case 2: hipLaunchKernelGGL((KERNEL<64, 2, RMS>), grid, dim3(kLnBlock), shmem, stream(), __VA_ARGS__); break; \
                case 4: hipLaunchKernelGGL((KERNEL<64, 4, RMS>), grid, dim3(kLnBlock), shmem, stream(), __VA_ARGS__); break; \
                default: hipLaunchKernelGGL((KERNEL<64, 8, RMS>), grid, dim3(kLnBlock), shmem, stream(), __VA_ARGS__); break; \
            }                                                                                                  \
        } else {                                                                                               \
            switch ((plan).vpt) {                                                                              \
                case 4: hipLaunchKernelGGL((KERNEL<256, 4, RMS>), grid, dim3(kLnBlock), shmem, stream(), __VA_ARGS__); break; \
                default: hipLaunchKernelGGL((KERNEL<256, 8, RMS>), grid, dim3(kLnBlock), shmem, stream(), __VA_ARGS__); break; \
            }                                                                                                  \
        }                                                                                                      \
    } while (0)
#define BH_LN_DISPATCH(KERNEL, rms, plan, grid, shmem, ...)                         \
    do {                                                                            \
        if (rms) BH_LN_DISPATCH_1(KERNEL, true, plan, grid, shmem, __VA_ARGS__);    \
        else BH_LN_DISPATCH_1(KERNEL, false, plan, grid, shmem, __VA_ARGS__);       \
    } while (0)

extern "C" {

// tuning hook for benchmarks: cap on backward workgroups
int bh_layernorm_tune(int bwd_blocks, int fwd_blocks) {
    if (fwd_blocks > 0) g_ln_fwd_blocks = fwd_blocks;
    if (bwd_blocks > 0) g_ln_bwd_blocks = bwd_blocks;
    return BH_OK;
}

static int norm_forward(bool rms, const char* name, const float* x, const float* gamma, const float* beta, float* y,
                        float* mean, float* rstd, int64_t rows, int64_t hidden, float eps) {
    ProfScope prof(BH_PROF_NORM, 8.0 * (double)rows * (double)hidden);
    LnPlan plan = plan_for(hidden, x, y, gamma ? (const void*)gamma : (const void*)x);
    if (plan.vector && beta && (reinterpret_cast<uintptr_t>(beta) & 15)) plan.vector = false;
    if (!plan.vector) {
        hipLaunchKernelGGL(ln_fwd_generic_kernel, dim3((unsigned)rows), dim3(kLnBlock), 0, stream(), x, gamma, beta, y,
                           mean, rstd, rows, hidden, eps, rms ? 1 : 0);
        return BH_LAUNCH_CHECK(name);
    }
    const int groups = kLnBlock / plan.tpr;
    int64_t blocks = ceil_div(rows, groups);
    const int64_t cap = g_ln_fwd_blocks;
    if (blocks > cap) blocks = cap;
    const int64_t rpg = ceil_div(rows, blocks * groups);
    BH_LN_DISPATCH(ln_fwd_kernel, rms, plan, dim3((unsigned)blocks), 0, x, gamma, beta, y, mean, rstd, rows, (int)hidden, eps, rpg);
    return BH_LAUNCH_CHECK(name);
}

int bh_layernorm_forward(const float* x, const float* gamma, const float* beta, float* y, float* mean, float* rstd,
                         int64_t rows, int64_t hidden, float eps) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(rows >= 0 && hidden > 0, "bad shape");
    if (rows == 0) return BH_OK;
    BH_CHECK_ARG(x && y, "null pointer");
    BH_CHECK_ARG(hidden < (int64_t(1) << 30), "hidden too large");
    return norm_forward(false, "bh_layernorm_forward", x, gamma, beta, y, mean, rstd, rows, hidden, eps);
}

int bh_rmsnorm_forward(const float* x, const float* weight, float* y, float* inv_rms, int64_t rows, int64_t hidden, float eps) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(rows >= 0 && hidden > 0, "bad shape");
    if (rows == 0) return BH_OK;
    BH_CHECK_ARG(x && y, "null pointer");
    BH_CHECK_ARG(hidden < (int64_t(1) << 30), "hidden too large");
    return norm_forward(true, "bh_rmsnorm_forward", x, weight, nullptr, y, nullptr, inv_rms, rows, hidden, eps);
}

// The register-resident path: ln_bwd_kernel writes one dgamma/dbeta partial per workgroup into `partial`
// (blocks x 2 x hidden floats), fold_rows_kernel sums them.
static int ln_backward_vector(bool rms, float eps, const LnPlan& plan, size_t shmem, int64_t blocks, float* partial,
                              const float* x, const float* gamma, const float* dy, const float* mean, const float* rstd,
                              const float* add, float* dx, float* dgamma, float* dbeta, int64_t rows, int64_t hidden,
                              int accumulate) {
    const int groups = kLnBlock / plan.tpr;
    const int64_t iters = ceil_div(rows, blocks * groups);
    if (add)
        BH_LN_DISPATCH(ln_bwd_add_kernel, rms, plan, dim3((unsigned)blocks), shmem, x, gamma, dy, mean, rstd, add, dx, partial,
                       rows, (int)hidden, iters, eps);
    else
        BH_LN_DISPATCH(ln_bwd_kernel, rms, plan, dim3((unsigned)blocks), shmem, x, gamma, dy, mean, rstd, add, dx, partial, rows,
                       (int)hidden, iters, eps);
    if (dgamma || dbeta)
        hipLaunchKernelGGL(fold_rows_kernel, dim3((unsigned)ceil_div(2 * hidden, kFoldCols)), dim3(kFoldCols * kFoldLanes), 0,
                           stream(), partial, blocks, 2 * hidden, dgamma, dbeta, hidden, accumulate);
    return BH_LAUNCH_CHECK("norm backward");
}

// Dynamic LDS of the vector path (the cross-group fold when a workgroup holds several row groups); the path is
// not taken when this plus the kernel's static LDS would pass the 64 KiB a launch gets without an opt-in.
static bool ln_backward_plan(LnPlan& plan, size_t& shmem, const float* x, const float* gamma, const float* dy, float* dx,
                             int64_t hidden) {
    plan = plan_for(hidden, x, dy, dx);
    if (plan.vector && gamma && (reinterpret_cast<uintptr_t>(gamma) & 15)) plan.vector = false;
    const int groups = plan.vector ? kLnBlock / plan.tpr : 1;
    shmem = (plan.vector && groups > 1) ? sizeof(float) * (size_t)groups * 2 * (size_t)hidden : 0;
    if (shmem + 256 > 64 * 1024) {
        // one row group per workgroup needs no fold through LDS
        if (plan.vector && (hidden >> 2) >= 256) {
            plan.tpr = 256;
            const int64_t need = ceil_div(hidden >> 2, 256);
            plan.vpt = need <= 4 ? 4 : 8;
            shmem = 0;
        } else {
            plan.vector = false;
        }
    }
    return plan.vector;
}

static int norm_backward(bool rms, float eps, const float* x, const float* gamma, const float* dy, const float* mean,
                         const float* rstd, const float* add, float* dx, float* dgamma, float* dbeta, int64_t rows,
                         int64_t hidden, int accumulate) {
    ProfScope prof(BH_PROF_NORM, (add ? 16.0 : 12.0) * (double)rows * (double)hidden);
    LnPlan plan;
    size_t shmem;
    ln_backward_plan(plan, shmem, x, gamma, dy, dx, hidden);
    if (plan.vector && add && (reinterpret_cast<uintptr_t>(add) & 15)) plan.vector = false;

    int rc;
    if (plan.vector) {
        const int groups = kLnBlock / plan.tpr;
        int64_t blocks = ceil_div(rows, groups);
        const int64_t cap = g_ln_bwd_blocks;   // per-block dgamma/dbeta partials cost 2*hidden floats each way
        if (blocks > cap) blocks = cap;
        float* partial = (float*)bh_malloc(sizeof(float) * (size_t)(blocks * 2 * hidden));
        if (!partial) return BH_ENOMEM;
        rc = ln_backward_vector(rms, eps, plan, shmem, blocks, partial, x, gamma, dy, mean, rstd, add, dx, dgamma, dbeta, rows,
                                hidden, accumulate);
        bh_free(partial);
    } else {
        hipLaunchKernelGGL(ln_bwd_dx_generic_kernel, dim3((unsigned)rows), dim3(kLnBlock), 0, stream(), x, gamma, dy, mean,
                           rstd, add, dx, rows, hidden, rms ? 1 : 0, eps);
        rc = BH_LAUNCH_CHECK("norm backward dx");
        if (rc == BH_OK && (dgamma || dbeta)) {
            int64_t chunks = ceil_div(rows, 64);
            if (chunks > 256) chunks = 256;
            const int64_t rpb = ceil_div(rows, chunks);
            chunks = ceil_div(rows, rpb);
            float* partial = (float*)bh_malloc(sizeof(float) * (size_t)(chunks * 2 * hidden));
            if (!partial) return BH_ENOMEM;
            hipLaunchKernelGGL(ln_bwd_param_generic_kernel, dim3((unsigned)ceil_div(hidden, kLnBlock), (unsigned)chunks),
                               dim3(kLnBlock), 0, stream(), x, dy, mean, rstd, partial, rows, hidden, rpb, rms ? 1 : 0);
            hipLaunchKernelGGL(fold_rows_kernel, dim3((unsigned)ceil_div(2 * hidden, kFoldCols)), dim3(kFoldCols * kFoldLanes), 0,
                               stream(), partial, chunks, 2 * hidden, dgamma, dbeta, hidden, accumulate);
            bh_free(partial);
            rc = BH_LAUNCH_CHECK("norm backward params");
        }
    }
    return rc;
}

int bh_layernorm_backward(const float* x, const float* gamma, const float* dy, const float* mean, const float* rstd,
                          float* dx, float* dgamma, float* dbeta, int64_t rows, int64_t hidden, int accumulate) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(rows >= 0 && hidden > 0, "bad shape");
    BH_CHECK_ARG(hidden < (int64_t(1) << 30), "hidden too large");
    if (rows == 0) {
        if (!accumulate) {
            if (dgamma) bh_memset_zero(dgamma, sizeof(float) * (size_t)hidden);
            if (dbeta) bh_memset_zero(dbeta, sizeof(float) * (size_t)hidden);
        }
        return BH_OK;
    }
    BH_CHECK_ARG(x && dy && mean && rstd && dx, "null pointer");
    return norm_backward(false, 0.f, x, gamma, dy, mean, rstd, nullptr, dx, dgamma, dbeta, rows, hidden, accumulate);
}

// dx = (LayerNorm input gradient) + add: the same kernel with the other gradient of a variable that feeds both a
// LayerNorm and a residual connection added on the way out (add must not overlap dx)
int bh_layernorm_backward_add(const float* x, const float* gamma, const float* dy, const float* mean, const float* rstd,
                              const float* add, float* dx, float* dgamma, float* dbeta, int64_t rows, int64_t hidden, int accumulate) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(rows >= 0 && hidden > 0, "bad shape");
    BH_CHECK_ARG(hidden < (int64_t(1) << 30), "hidden too large");
    if (rows == 0) return bh_layernorm_backward(x, gamma, dy, mean, rstd, dx, dgamma, dbeta, rows, hidden, accumulate);
    BH_CHECK_ARG(x && dy && mean && rstd && dx && add, "null pointer");
    BH_CHECK_ARG(add + rows * hidden <= dx || dx + rows * hidden <= add, "add overlaps dx");
    return norm_backward(false, 0.f, x, gamma, dy, mean, rstd, add, dx, dgamma, dbeta, rows, hidden, accumulate);
}

int bh_rmsnorm_backward(const float* x, const float* weight, const float* dy, const float* inv_rms, float* dx, float* dweight,
                        int64_t rows, int64_t hidden, float eps, int accumulate) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(rows >= 0 && hidden > 0, "bad shape");
    BH_CHECK_ARG(hidden < (int64_t(1) << 30), "hidden too large");
    if (rows == 0) {
        if (!accumulate && dweight) bh_memset_zero(dweight, sizeof(float) * (size_t)hidden);
        return BH_OK;
    }
    BH_CHECK_ARG(x && dy && inv_rms && dx, "null pointer");
    return norm_backward(true, eps, x, weight, dy, nullptr, inv_rms, nullptr, dx, dweight, nullptr, rows, hidden, accumulate);
}

// bh_layernorm_backward for callers that may not allocate: same kernels, the partials live in ln_scratch.
// No hipMalloc/hipFree, no bh_malloc; the library must already be initialised (bh_init creates the stream and
// resolves the scratch address).  Calls on one GPU share the array: they must not overlap.
int bh_layernorm_backward_noalloc(const float* x, const float* gamma, const float* dy, const float* mean, const float* rstd,
                                  float* dx, float* dgamma, float* dbeta, int64_t rows, int64_t hidden, int accumulate) {
    if (!ready()) return set_error(BH_EINVAL, "bh_layernorm_backward_noalloc: call bh_init() first (this entry point sets nothing up)");
    int dev = -1;
    int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
    if (rc) return rc;
    float* scratch = (dev >= 0 && dev < kMaxDevices) ? g_ln_scratch_ptr[dev] : nullptr;
    if (!scratch) return set_error(BH_EDEVICE, "bh_layernorm_backward_noalloc: no scratch address for device %d", dev);
    BH_CHECK_ARG(rows >= 0 && hidden > 0, "bad shape");
    if (rows == 0) {
        if (!accumulate) {
            if (dgamma) bh_memset_zero(dgamma, sizeof(float) * (size_t)hidden);
            if (dbeta) bh_memset_zero(dbeta, sizeof(float) * (size_t)hidden);
        }
        return BH_OK;
    }
    BH_CHECK_ARG(x && dy && mean && rstd && dx, "null pointer");
    LnPlan plan;
    size_t shmem;
    if (hidden > BH_LN_NOALLOC_MAX_HIDDEN || !ln_backward_plan(plan, shmem, x, gamma, dy, dx, hidden))
        return set_error(BH_EINVAL,
                         "bh_layernorm_backward_noalloc: hidden=%lld is not supported: it must be a multiple of 4, at most %d, "
                         "with 16-byte aligned x, dy, dx and gamma (use bh_layernorm_backward)",
                         (long long)hidden, BH_LN_NOALLOC_MAX_HIDDEN);
    const int groups = kLnBlock / plan.tpr;
    int64_t blocks = ceil_div(rows, groups);
    int64_t cap = g_ln_bwd_blocks;
    const int64_t fit = (int64_t)(kLnScratchFloats / (size_t)(2 * hidden));   // >= 256 for every supported hidden
    if (cap > fit) cap = fit;
    if (blocks > cap) blocks = cap;
    // every partial the fold reads is written by this call's ln_bwd_kernel first: nothing to clear
    return ln_backward_vector(false, 0.f, plan, shmem, blocks, scratch, x, gamma, dy, mean, rstd, nullptr, dx, dgamma, dbeta, rows,
                              hidden, accumulate);
}

}  // extern "C"
