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

}  // namespace bh
