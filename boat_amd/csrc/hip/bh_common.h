// bh_common.h - shared helpers of the gfx950 device layer (internal).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "boat_hip.h"

namespace bh {

constexpr int kWave = 64;          // CDNA4 wavefront width
constexpr int kNumXcd = 8;         // MI355X: 8 XCDs, workgroups are dealt to them round-robin

hipStream_t stream();
int set_error(int code, const char* fmt, ...);
int check_hip(hipError_t e, const char* what);
bool ready();
int ln_scratch_setup();   // bh_layernorm.hip: resolves the current device's copy of the no-alloc scratch array

// Per-class timing of the library's launches with HIP events on the library stream (bh_profile_* in boat_hip.h).
// An entry point opens a scope after its argument checks; when profiling is off this is one branch.
void prof_open(int cls, double work, int* slot);
void prof_close(int slot);
struct ProfScope {
    int slot = -1;   // -1: profiling off; -2: open but not recorded (nested, or no events left); >= 0: record index
    ProfScope(int cls, double work) { prof_open(cls, work, &slot); }
    ~ProfScope() { if (slot != -1) prof_close(slot); }
};

#define BH_REQUIRE_INIT()                                   \
    do {                                                    \
        if (!::bh::ready()) {                               \
            int rc__ = bh_init();                           \
            if (rc__ != BH_OK) return rc__;                 \
        }                                                   \
    } while (0)

#define BH_CHECK_ARG(cond, msg)                                         \
    do {                                                                \
        if (!(cond)) return ::bh::set_error(BH_EINVAL, "%s: %s", __func__, msg); \
    } while (0)

#define BH_LAUNCH_CHECK(name) ::bh::check_hip(hipGetLastError(), name)

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- wavefront reductions (64 lanes) ----
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Block-wide sum for blocks of NWAVES wavefronts; `red` is NWAVES floats of LDS.
template <int NWAVES>
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NWAVES; i++) t += red[i];
    return t;
}

// Column sums of a small row-major matrix of per-workgroup partials: out[c] (+)= sum_r partial[r][c].
// 1024 lanes per workgroup = 64 columns x 16 row-lanes, so a column's rows are summed by 16 lanes in
// parallel (4 loads in flight each) and folded through LDS.  Columns [0, split) go to out_a, the rest
// to out_b (either may be NULL).  Launch with grid = ceil(ncols / 64), block = 1024.
constexpr int kFoldCols = 64;
constexpr int kFoldLanes = 16;
static __global__ __launch_bounds__(kFoldCols * kFoldLanes) void fold_rows_kernel(
    const float* __restrict__ partial, int64_t nrows, int64_t ncols, float* __restrict__ out_a,
    float* __restrict__ out_b, int64_t split, int accumulate) {
    __shared__ float red[kFoldLanes][kFoldCols + 1];
    const int tx = threadIdx.x % kFoldCols, ty = threadIdx.x / kFoldCols;
    const int64_t c = (int64_t)blockIdx.x * kFoldCols + tx;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    if (c < ncols) {
        int64_t r = ty;
        for (; r + 3 * kFoldLanes < nrows; r += 4 * kFoldLanes) {
            a0 += partial[r * ncols + c];
            a1 += partial[(r + kFoldLanes) * ncols + c];
            a2 += partial[(r + 2 * kFoldLanes) * ncols + c];
            a3 += partial[(r + 3 * kFoldLanes) * ncols + c];
        }
        for (; r < nrows; r += kFoldLanes) a0 += partial[r * ncols + c];
    }
    red[ty][tx] = (a0 + a1) + (a2 + a3);
    __syncthreads();
    if (ty == 0 && c < ncols) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < kFoldLanes; i++) acc += red[i][tx];
        float* dst = c < split ? (out_a ? out_a + c : nullptr) : (out_b ? out_b + (c - split) : nullptr);
        if (dst) *dst = accumulate ? *dst + acc : acc;
    }
}

}  // namespace bh
