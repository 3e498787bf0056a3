// bh_elementwise.hip - one-pass, coalesced, HBM-bound elementwise kernels.
//
// Covers the reference's elementwise forward/backward arithmetic:
//   boat_add_/boat_mul/boat_div/boat_*_scalar     src/ops/arithmetic.c:157-285,362-484
//   add/sub/mul/div/relu/sigmoid/tanh gradients    src/autodiff.c:1002-1452
//   bias broadcast of the dense forward            src/layers/dense.c:180-184
//   plain SGD update inside layers                 src/layers/dense.c:297-329
// plus exact-erf GELU forward/backward, which the reference only declares.
//
// Every kernel reads each input once and writes each output once, 16 bytes per lane
// per access (float4) when the pointers allow it.  The file is compiled with
// -ffp-contract=off so a*b+c stays two roundings like the reference's scalar C loops;
// division and sqrt are hipcc's correctly-rounded defaults.
#include "bh_common.h"

namespace bh {

constexpr int kBlock = 256;

static inline int grid_for(int64_t work_items) {
    int64_t blocks = ceil_div(work_items, kBlock);
    const int64_t cap = 256 * 16;   // 16 resident blocks' worth per CU on a 256-CU part
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (int)blocks;
}

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// out[i] = f(in0[i], in1[i], in2[i], out[i]); NIN inputs are read, out is read when RO.
// One float4 per lane per input, one single-wavefront workgroup per 64 float4: the grid is as large as the data, so
// the resident workgroups sweep memory as one contiguous moving window (measured faster on MI355X
// than a persistent grid-stride loop), and the accesses are marked non-temporal (streamed once).
// Workgroups of one wavefront: a compute unit takes a new one whenever any wavefront slot frees (measured on the
// seven-stream Adam step: 6.44 TB/s with 64 lanes per workgroup, 6.06 with 256, 5.85 with 1024).
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int kVecBlock = 64;

template <int NIN, bool RO, typename F>
__global__ __launch_bounds__(kVecBlock) void ew_vec4(F f, float* __restrict__ out, const float* __restrict__ in0,
                                                  const float* __restrict__ in1, const float* __restrict__ in2,
                                                  int64_t n) {
    const int64_t n4 = n >> 2;
    const int64_t i = (int64_t)blockIdx.x * kVecBlock + threadIdx.x;
    if (i < n4) {
        const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
        f32x4 a = NIN > 0 ? __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(in0) + i) : zero;
        f32x4 b = NIN > 1 ? __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(in1) + i) : zero;
        f32x4 c = NIN > 2 ? __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(in2) + i) : zero;
        f32x4 o = RO ? __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(out) + i) : zero;
        f32x4 r;
        r.x = f(a.x, b.x, c.x, o.x);
        r.y = f(a.y, b.y, c.y, o.y);
        r.z = f(a.z, b.z, c.z, o.z);
        r.w = f(a.w, b.w, c.w, o.w);
        __builtin_nontemporal_store(r, reinterpret_cast<f32x4*>(out) + i);
    }
    // tail (n % 4 elements), first lanes of block 0
    const int64_t tail = n & 3;
    if (blockIdx.x == 0 && threadIdx.x < tail) {
        const int64_t j = (n4 << 2) + threadIdx.x;
        out[j] = f(NIN > 0 ? in0[j] : 0.f, NIN > 1 ? in1[j] : 0.f, NIN > 2 ? in2[j] : 0.f, RO ? out[j] : 0.f);
    }
}

template <int NIN, bool RO, typename F>
__global__ __launch_bounds__(kBlock) void ew_scalar(F f, float* out, const float* in0, const float* in1,
                                                    const float* in2, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        out[i] = f(NIN > 0 ? in0[i] : 0.f, NIN > 1 ? in1[i] : 0.f, NIN > 2 ? in2[i] : 0.f, RO ? out[i] : 0.f);
}

template <int NIN, bool RO, typename F>
static int launch_ew(const char* name, F f, float* out, const float* in0, const float* in1, const float* in2,
                     int64_t n) {
    if (n == 0) return BH_OK;
    const bool vec = aligned16(out) && (NIN < 1 || aligned16(in0)) && (NIN < 2 || aligned16(in1)) &&
                     (NIN < 3 || aligned16(in2));
    if (vec) {
        const int64_t blocks = ceil_div((n >> 2) > 0 ? (n >> 2) : 1, kVecBlock);
        if (blocks > 0x7fffffff) return set_error(BH_EINVAL, "%s: tensor too large", name);
        hipLaunchKernelGGL((ew_vec4<NIN, RO, F>), dim3((unsigned)blocks), dim3(kVecBlock), 0, stream(), f, out, in0, in1,
                           in2, n);
    } else {
        hipLaunchKernelGGL((ew_scalar<NIN, RO, F>), dim3(grid_for(n)), dim3(kBlock), 0, stream(), f, out, in0, in1,
                           in2, n);
    }
    return BH_LAUNCH_CHECK(name);
}

// ---- functors (a, b, c = inputs; o = previous output) ----
struct FFill { float v; __device__ float operator()(float, float, float, float) const { return v; } };
// the scalar lives in device memory (a [1] gradient tensor): no readback to the host
struct FFillAt { const float* s; __device__ float operator()(float, float, float, float) const { return s[0]; } };
struct FMulAt { const float* s; __device__ float operator()(float a, float, float, float) const { return a * s[0]; } };
struct FCopy { __device__ float operator()(float a, float, float, float) const { return a; } };
struct FAddInto { __device__ float operator()(float a, float, float, float o) const { return o + a; } };
struct FAdd { __device__ float operator()(float a, float b, float, float) const { return a + b; } };
struct FSub { __device__ float operator()(float a, float b, float, float) const { return a - b; } };
struct FMul { __device__ float operator()(float a, float b, float, float) const { return a * b; } };
struct FDiv { __device__ float operator()(float a, float b, float, float) const { return a / b; } };
struct FAddS { float s; __device__ float operator()(float a, float, float, float) const { return a + s; } };
struct FSubS { float s; __device__ float operator()(float a, float, float, float) const { return a - s; } };
struct FMulS { float s; __device__ float operator()(float a, float, float, float) const { return a * s; } };
struct FDivS { float s; __device__ float operator()(float a, float, float, float) const { return a / s; } };
// (dy * -1) * (a / (b*b)): a=a, b=b, c=dy
struct FDivBwdB {
    __device__ float operator()(float a, float b, float dy, float) const {
        float bsq = b * b;
        float adb = a / bsq;
        float neg = dy * -1.0f;
        return neg * adb;
    }
};

struct FRelu { __device__ float operator()(float x, float, float, float) const { return x > 0 ? x : 0.0f; } };
struct FSigmoid { __device__ float operator()(float x, float, float, float) const { return 1.0f / (1.0f + expf(-x)); } };
struct FTanh {
    __device__ float operator()(float x, float, float, float) const {
        float ex = expf(x), emx = expf(-x);
        return (ex - emx) / (ex + emx);
    }
};
__device__ __forceinline__ float gelu_cdf(float x) { return 0.5f * (1.0f + erff(x * 0.70710678118654752440f)); }
struct FGelu { __device__ float operator()(float x, float, float, float) const { return x * gelu_cdf(x); } };

// backward functors: a = saved tensor, b = dy, o = previous dx (used when ACC)
template <bool ACC> struct FReluBwd {
    __device__ float operator()(float x, float dy, float, float o) const {
        float g = dy * (x > 0 ? 1.0f : 0.0f);
        return ACC ? o + g : g;
    }
};
template <bool ACC> struct FSigmoidBwd {
    __device__ float operator()(float c, float dy, float, float o) const {
        float omc = 1.0f - c;
        float t = c * omc;
        float g = dy * t;
        return ACC ? o + g : g;
    }
};
template <bool ACC> struct FTanhBwd {
    __device__ float operator()(float c, float dy, float, float o) const {
        float csq = c * c;
        float om = 1.0f - csq;
        float g = dy * om;
        return ACC ? o + g : g;
    }
};
template <bool ACC> struct FGeluBwd {
    __device__ float operator()(float x, float dy, float, float o) const {
        float pdf = 0.39894228040143267794f * expf(-0.5f * x * x);
        float g = dy * (gelu_cdf(x) + x * pdf);
        return ACC ? o + g : g;
    }
};

struct FMseGrad {
    float n;
    __device__ float operator()(float p, float t, float, float) const { return 2.0f * (p - t) / n; }
};

// ---- broadcasting binary op (arithmetic.c:78-104 shape rule, :199-203 index rule) ----
struct BcastDims {
    int ndim;
    int64_t out_shape[8];
    int64_t a_stride[8];   // 0 where the operand is broadcast along that axis
    int64_t b_stride[8];
};

template <typename F>
__global__ __launch_bounds__(kBlock) void bcast_kernel(F f, float* out, const float* a, const float* b,
                                                       BcastDims d, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        int64_t rem = i, ia = 0, ib = 0;
#pragma unroll
        for (int ax = 7; ax >= 0; ax--) {
            if (ax < d.ndim) {
                int64_t c = rem % d.out_shape[ax];
                rem /= d.out_shape[ax];
                ia += c * d.a_stride[ax];
                ib += c * d.b_stride[ax];
            }
        }
        out[i] = f(a[ia], b[ib], 0.f, 0.f);
    }
}

// y[r, c] += bias[c]
__global__ __launch_bounds__(kBlock) void bias_rows_kernel(float* y, const float* bias, int64_t rows, int64_t cols) {
    const int64_t n = rows * cols;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) y[i] = y[i] + bias[i % cols];
}

__global__ __launch_bounds__(kBlock) void sgd_kernel(float* p, float* g, float lr, int64_t n, int zero) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        p[i] -= lr * g[i];
        if (zero) g[i] = 0.0f;
    }
}

// rows a wavefront of the kernel below keeps in flight per trip: eight, except where the derivative itself is long
// arithmetic (GELU's erf and exp: 8192x4096 takes 75 us with four rows in flight and 79 with eight, ReLU 88 and 73)
template <typename F> struct ActRowsInFlight { static constexpr int value = 8; };
template <bool ACC> struct ActRowsInFlight<FGeluBwd<ACC>> { static constexpr int value = 4; };

// ---- activation backward that also sums its result over the rows (see launch_act_bwd_colsum) ----
// Row chunk y of Y takes rows y, y+Y, ...; a lane owns one column (VEC: four neighbouring ones); per column four running
// sums, exactly the sums of colsum_partial_kernel on the stored dx.
template <typename F, bool VEC>
__global__ __launch_bounds__(VEC ? 64 : 256) void act_bwd_colsum_partial_kernel(F f, const float* __restrict__ saved,
                                                                                 const float* __restrict__ dy, float* __restrict__ dx,
                                                                                 float* __restrict__ partial, int64_t rows, int64_t cols) {
    const int64_t step = gridDim.y;
    if constexpr (VEC) {
        const int64_t c = ((int64_t)blockIdx.x * 64 + threadIdx.x) * 4;
        if (c >= cols) return;
        f32x4 acc[4];
#pragma unroll
        for (int j = 0; j < 4; j++) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        int64_t r = blockIdx.y;
        // eight rows in flight per trip while they last (a wavefront is one of only two on its SIMD here); row j still goes
        // to running sum j % 4, so the sums and their order are the ones of the four-row trips below
        for (; ActRowsInFlight<F>::value == 8 && r + 7 * step < rows; r += 8 * step) {
            f32x4 a[8], g[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                a[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(saved + (r + j * step) * cols + c));
                g[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(dy + (r + j * step) * cols + c));
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                f32x4 v;
                v.x = f(a[j].x, g[j].x, 0.f, 0.f);
                v.y = f(a[j].y, g[j].y, 0.f, 0.f);
                v.z = f(a[j].z, g[j].z, 0.f, 0.f);
                v.w = f(a[j].w, g[j].w, 0.f, 0.f);
                __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(dx + (r + j * step) * cols + c));
                acc[j & 3].x += v.x; acc[j & 3].y += v.y; acc[j & 3].z += v.z; acc[j & 3].w += v.w;
            }
        }
        for (; r + 3 * step < rows; r += 4 * step) {
            f32x4 a[4], g[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                a[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(saved + (r + j * step) * cols + c));
                g[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(dy + (r + j * step) * cols + c));
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                f32x4 v;
                v.x = f(a[j].x, g[j].x, 0.f, 0.f);
                v.y = f(a[j].y, g[j].y, 0.f, 0.f);
                v.z = f(a[j].z, g[j].z, 0.f, 0.f);
                v.w = f(a[j].w, g[j].w, 0.f, 0.f);
                __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(dx + (r + j * step) * cols + c));
                acc[j].x += v.x; acc[j].y += v.y; acc[j].z += v.z; acc[j].w += v.w;
            }
        }
        for (; r < rows; r += step) {
            const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(saved + r * cols + c));
            const f32x4 g = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(dy + r * cols + c));
            f32x4 v;
            v.x = f(a.x, g.x, 0.f, 0.f);
            v.y = f(a.y, g.y, 0.f, 0.f);
            v.z = f(a.z, g.z, 0.f, 0.f);
            v.w = f(a.w, g.w, 0.f, 0.f);
            __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(dx + r * cols + c));
            acc[0].x += v.x; acc[0].y += v.y; acc[0].z += v.z; acc[0].w += v.w;
        }
        f32x4 t;
        t.x = (acc[0].x + acc[1].x) + (acc[2].x + acc[3].x);
        t.y = (acc[0].y + acc[1].y) + (acc[2].y + acc[3].y);
        t.z = (acc[0].z + acc[1].z) + (acc[2].z + acc[3].z);
        t.w = (acc[0].w + acc[1].w) + (acc[2].w + acc[3].w);
        *reinterpret_cast<f32x4*>(partial + (int64_t)blockIdx.y * cols + c) = t;
    } else {
        const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
        if (c >= cols) return;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        int64_t r = blockIdx.y;
        for (; r + 3 * step < rows; r += 4 * step) {
            const float v0 = f(saved[r * cols + c], dy[r * cols + c], 0.f, 0.f);
            const float v1 = f(saved[(r + step) * cols + c], dy[(r + step) * cols + c], 0.f, 0.f);
            const float v2 = f(saved[(r + 2 * step) * cols + c], dy[(r + 2 * step) * cols + c], 0.f, 0.f);
            const float v3 = f(saved[(r + 3 * step) * cols + c], dy[(r + 3 * step) * cols + c], 0.f, 0.f);
            dx[r * cols + c] = v0;
            dx[(r + step) * cols + c] = v1;
            dx[(r + 2 * step) * cols + c] = v2;
            dx[(r + 3 * step) * cols + c] = v3;
            a0 += v0; a1 += v1; a2 += v2; a3 += v3;
        }
        for (; r < rows; r += step) {
            const float v = f(saved[r * cols + c], dy[r * cols + c], 0.f, 0.f);
            dx[r * cols + c] = v;
            a0 += v;
        }
        partial[(int64_t)blockIdx.y * cols + c] = (a0 + a1) + (a2 + a3);
    }
}
// The same sums from four wavefronts per row chunk, for matrices too small to fill the chip with one wavefront per
// chunk and column group (the chunks are bh_colsum's, so their number is given): wavefront w keeps running sum w, i.e.
// rows w, w+4, ... of the chunk's whole trips of four, two of them in flight; the first wavefront also takes the rows
// after the last whole trip, as the first running sum does above; the four sums meet in LDS and are added in the order
// above.  4096x1024 GELU: 15 us against 26, the same bits.
template <typename F>
__global__ __launch_bounds__(256) void act_bwd_colsum_partial4_kernel(F f, const float* __restrict__ saved, const float* __restrict__ dy,
                                                                      float* __restrict__ dx, float* __restrict__ partial, int64_t rows,
                                                                      int64_t cols) {
    __shared__ f32x4 red[4][64];
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t step = gridDim.y;
    const int64_t c = ((int64_t)blockIdx.x * 64 + lane) * 4;
    const bool live = c < cols;
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    const auto one_row = [&](int64_t r) {
        const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(saved + r * cols + c));
        const f32x4 g = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(dy + r * cols + c));
        f32x4 v;
        v.x = f(a.x, g.x, 0.f, 0.f);
        v.y = f(a.y, g.y, 0.f, 0.f);
        v.z = f(a.z, g.z, 0.f, 0.f);
        v.w = f(a.w, g.w, 0.f, 0.f);
        __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(dx + r * cols + c));
        acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    };
    if (live) {
        const int64_t in_chunk = (rows - blockIdx.y + step - 1) / step;    // rows blockIdx.y, blockIdx.y + step, ... (gridDim.y <= rows)
        const int64_t trips = in_chunk / 4;
        const int64_t first = blockIdx.y + w * step;                       // this wavefront's row of trip 0
        int64_t t = 0;
        for (; t + 2 <= trips; t += 2) {
            const int64_t r0 = first + t * 4 * step, r1 = r0 + 4 * step;
            const f32x4 a0 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(saved + r0 * cols + c));
            const f32x4 g0 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(dy + r0 * cols + c));
            const f32x4 a1 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(saved + r1 * cols + c));
            const f32x4 g1 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(dy + r1 * cols + c));
            f32x4 v;
            v.x = f(a0.x, g0.x, 0.f, 0.f);
            v.y = f(a0.y, g0.y, 0.f, 0.f);
            v.z = f(a0.z, g0.z, 0.f, 0.f);
            v.w = f(a0.w, g0.w, 0.f, 0.f);
            __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(dx + r0 * cols + c));
            acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
            v.x = f(a1.x, g1.x, 0.f, 0.f);
            v.y = f(a1.y, g1.y, 0.f, 0.f);
            v.z = f(a1.z, g1.z, 0.f, 0.f);
            v.w = f(a1.w, g1.w, 0.f, 0.f);
            __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(dx + r1 * cols + c));
            acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
        }
        if (t < trips) one_row(first + t * 4 * step);
        if (w == 0)
            for (int64_t q = trips * 4; q < in_chunk; q++) one_row(blockIdx.y + q * step);
    }
    red[w][lane] = acc;
    __syncthreads();
    if (w == 0 && live) {
        const f32x4 s1 = red[1][lane], s2 = red[2][lane], s3 = red[3][lane];
        f32x4 t;
        t.x = (acc.x + s1.x) + (s2.x + s3.x);
        t.y = (acc.y + s1.y) + (s2.y + s3.y);
        t.z = (acc.z + s1.z) + (s2.z + s3.z);
        t.w = (acc.w + s1.w) + (s2.w + s3.w);
        *reinterpret_cast<f32x4*>(partial + (int64_t)blockIdx.y * cols + c) = t;
    }
}
// few rows: fold_rows_kernel's shape (64 columns x 16 row lanes, folded through LDS in lane order) on values computed here
template <typename F>
__global__ __launch_bounds__(kFoldCols * kFoldLanes) void act_bwd_colsum_small_kernel(F f, const float* __restrict__ saved,
                                                                                      const float* __restrict__ dy, float* __restrict__ dx,
                                                                                      int64_t rows, int64_t cols, float* __restrict__ out,
                                                                                      int accumulate) {
    __shared__ float red[kFoldLanes][kFoldCols + 1];
    const int tx = threadIdx.x % kFoldCols, ty = threadIdx.x / kFoldCols;
    const int64_t c = (int64_t)blockIdx.x * kFoldCols + tx;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    if (c < cols) {
        int64_t r = ty;
        for (; r + 3 * kFoldLanes < rows; r += 4 * kFoldLanes) {
            const float v0 = f(saved[r * cols + c], dy[r * cols + c], 0.f, 0.f);
            const float v1 = f(saved[(r + kFoldLanes) * cols + c], dy[(r + kFoldLanes) * cols + c], 0.f, 0.f);
            const float v2 = f(saved[(r + 2 * kFoldLanes) * cols + c], dy[(r + 2 * kFoldLanes) * cols + c], 0.f, 0.f);
            const float v3 = f(saved[(r + 3 * kFoldLanes) * cols + c], dy[(r + 3 * kFoldLanes) * cols + c], 0.f, 0.f);
            dx[r * cols + c] = v0;
            dx[(r + kFoldLanes) * cols + c] = v1;
            dx[(r + 2 * kFoldLanes) * cols + c] = v2;
            dx[(r + 3 * kFoldLanes) * cols + c] = v3;
            a0 += v0; a1 += v1; a2 += v2; a3 += v3;
        }
        for (; r < rows; r += kFoldLanes) {
            const float v = f(saved[r * cols + c], dy[r * cols + c], 0.f, 0.f);
            dx[r * cols + c] = v;
            a0 += v;
        }
    }
    red[ty][tx] = (a0 + a1) + (a2 + a3);
    __syncthreads();
    if (ty == 0 && c < cols) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < kFoldLanes; i++) acc += red[i][tx];
        out[c] = accumulate ? out[c] + acc : acc;
    }
}

// dx = dy * f'(saved) and, in the same pass, the column sums of dx (the bias gradient of the dense layer whose output the
// activation took): out[c] (+)= sum_r dx[r][c].  The sums are bh_colsum's, in its order: rows <= 256 take the one-launch
// fold (64 columns x 16 row lanes), larger matrices the same row chunks, four running sums per lane and fold_rows_kernel.
// up to this many elements the partial kernel runs four wavefronts per row chunk (measured: faster up to 8M elements, level at 16M, slower at 32M)
constexpr int64_t kActFourWaveMax = (int64_t)1 << 23;

template <typename F>
static int launch_act_bwd_colsum(const char* name, F f, const float* saved, const float* dy, float* dx, float* out, int64_t rows,
                                 int64_t cols, int accumulate) {
    if (rows <= 256) {
        hipLaunchKernelGGL((act_bwd_colsum_small_kernel<F>), dim3((unsigned)ceil_div(cols, kFoldCols)), dim3(kFoldCols * kFoldLanes), 0,
                           stream(), f, saved, dy, dx, rows, cols, out, accumulate);
        return BH_LAUNCH_CHECK(name);
    }
    const int col_blocks = (int)ceil_div(cols, 256);
    int64_t chunks = ceil_div(2048, col_blocks);          // as bh_colsum cuts the rows
    if (chunks > ceil_div(rows, 32)) chunks = ceil_div(rows, 32);
    if (chunks < 1) chunks = 1;
    float* partial = (float*)bh_malloc(sizeof(float) * (size_t)(chunks * cols));
    if (!partial) return BH_ENOMEM;
    const bool vec = cols % 4 == 0 && aligned16(saved) && aligned16(dy) && aligned16(dx);
    if (vec && rows * cols <= kActFourWaveMax)
        hipLaunchKernelGGL((act_bwd_colsum_partial4_kernel<F>), dim3(col_blocks, (unsigned)chunks), dim3(256), 0, stream(), f, saved, dy,
                           dx, partial, rows, cols);
    else if (vec)
        hipLaunchKernelGGL((act_bwd_colsum_partial_kernel<F, true>), dim3(col_blocks, (unsigned)chunks), dim3(64), 0, stream(), f, saved, dy,
                           dx, partial, rows, cols);
    else
        hipLaunchKernelGGL((act_bwd_colsum_partial_kernel<F, false>), dim3(col_blocks, (unsigned)chunks), dim3(256), 0, stream(), f, saved,
                           dy, dx, partial, rows, cols);
    hipLaunchKernelGGL(fold_rows_kernel, dim3((unsigned)ceil_div(cols, kFoldCols)), dim3(kFoldCols * kFoldLanes), 0, stream(), partial,
                       chunks, cols, out, (float*)nullptr, cols, accumulate);
    bh_free(partial);
    return BH_LAUNCH_CHECK(name);
}

}  // namespace bh

using namespace bh;

extern "C" {

int bh_fill(float* x, float value, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && (x || n == 0), "bad argument");
    return launch_ew<0, false>("bh_fill", FFill{value}, x, nullptr, nullptr, nullptr, n);
}

int bh_memset_zero(void* dst, size_t nbytes) {
    BH_REQUIRE_INIT();
    if (nbytes == 0) return BH_OK;
    BH_CHECK_ARG(dst, "null pointer");
    // a fill kernel rather than hipMemsetAsync, so callers may capture it into a HIP graph
    const size_t words = nbytes / 4, tail = nbytes % 4;
    int rc = launch_ew<0, false>("bh_memset_zero", FFill{0.0f}, (float*)dst, nullptr, nullptr, nullptr, (int64_t)words);
    if (rc == BH_OK && tail)
        rc = check_hip(hipMemsetAsync((char*)dst + words * 4, 0, tail, stream()), "hipMemsetAsync");
    return rc;
}

int bh_add_inplace(float* a, const float* b, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && ((a && b) || n == 0), "bad argument");
    return launch_ew<1, true>("bh_add_inplace", FAddInto{}, a, b, nullptr, nullptr, n);
}

int bh_binary(int op, const float* a, const float* b, float* out, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && ((a && b && out) || n == 0), "bad argument");
    switch (op) {
        case 0: return launch_ew<2, false>("bh_binary add", FAdd{}, out, a, b, nullptr, n);
        case 1: return launch_ew<2, false>("bh_binary sub", FSub{}, out, a, b, nullptr, n);
        case 2: return launch_ew<2, false>("bh_binary mul", FMul{}, out, a, b, nullptr, n);
        case 3: return launch_ew<2, false>("bh_binary div", FDiv{}, out, a, b, nullptr, n);
    }
    return set_error(BH_EINVAL, "bh_binary: unknown op %d", op);
}

int bh_binary_broadcast(int op, const float* a, const int64_t* a_shape, const float* b, const int64_t* b_shape,
                        float* out, const int64_t* out_shape, int ndim) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(ndim >= 1 && ndim <= 8 && a && b && out && a_shape && b_shape && out_shape, "bad argument");
    BcastDims d;
    d.ndim = ndim;
    int64_t n = 1, sa = 1, sb = 1;
    for (int ax = ndim - 1; ax >= 0; ax--) {
        BH_CHECK_ARG(out_shape[ax] >= 0, "negative extent");
        BH_CHECK_ARG(a_shape[ax] == out_shape[ax] || a_shape[ax] == 1, "operand a does not broadcast");
        BH_CHECK_ARG(b_shape[ax] == out_shape[ax] || b_shape[ax] == 1, "operand b does not broadcast");
        d.out_shape[ax] = out_shape[ax];
        d.a_stride[ax] = a_shape[ax] == 1 ? 0 : sa;
        d.b_stride[ax] = b_shape[ax] == 1 ? 0 : sb;
        sa *= a_shape[ax];
        sb *= b_shape[ax];
        n *= out_shape[ax];
    }
    for (int ax = ndim; ax < 8; ax++) d.out_shape[ax] = 1, d.a_stride[ax] = 0, d.b_stride[ax] = 0;
    if (n == 0) return BH_OK;
    const int grid = grid_for(n);
    switch (op) {
        case 0: hipLaunchKernelGGL((bcast_kernel<FAdd>), dim3(grid), dim3(kBlock), 0, stream(), FAdd{}, out, a, b, d, n); break;
        case 1: hipLaunchKernelGGL((bcast_kernel<FSub>), dim3(grid), dim3(kBlock), 0, stream(), FSub{}, out, a, b, d, n); break;
        case 2: hipLaunchKernelGGL((bcast_kernel<FMul>), dim3(grid), dim3(kBlock), 0, stream(), FMul{}, out, a, b, d, n); break;
        case 3: hipLaunchKernelGGL((bcast_kernel<FDiv>), dim3(grid), dim3(kBlock), 0, stream(), FDiv{}, out, a, b, d, n); break;
        default: return set_error(BH_EINVAL, "bh_binary_broadcast: unknown op %d", op);
    }
    return BH_LAUNCH_CHECK("bh_binary_broadcast");
}

int bh_scale_by_device_scalar(const float* in, const float* scalar, float* out, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && ((scalar && out) || n == 0), "bad argument");
    if (!in) return launch_ew<0, false>("bh_scale_by_device_scalar", FFillAt{scalar}, out, nullptr, nullptr, nullptr, n);
    return launch_ew<1, false>("bh_scale_by_device_scalar", FMulAt{scalar}, out, in, nullptr, nullptr, n);
}

int bh_copy_f32(float* dst, const float* src, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && ((dst && src) || n == 0), "bad argument");
    return launch_ew<1, false>("bh_copy_f32", FCopy{}, dst, src, nullptr, nullptr, n);
}

int bh_scalar_op(int op, const float* a, float s, float* out, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && ((a && out) || n == 0), "bad argument");
    switch (op) {
        case 0: return launch_ew<1, false>("bh_scalar_op add", FAddS{s}, out, a, nullptr, nullptr, n);
        case 1: return launch_ew<1, false>("bh_scalar_op sub", FSubS{s}, out, a, nullptr, nullptr, n);
        case 2: return launch_ew<1, false>("bh_scalar_op mul", FMulS{s}, out, a, nullptr, nullptr, n);
        case 3: return launch_ew<1, false>("bh_scalar_op div", FDivS{s}, out, a, nullptr, nullptr, n);
    }
    return set_error(BH_EINVAL, "bh_scalar_op: unknown op %d", op);
}

int bh_div_backward_b(const float* a, const float* b, const float* dy, float* db, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && ((a && b && dy && db) || n == 0), "bad argument");
    return launch_ew<3, false>("bh_div_backward_b", FDivBwdB{}, db, a, b, dy, n);
}

int bh_activation_forward(int act, const float* x, float* y, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && ((x && y) || n == 0), "bad argument");
    switch (act) {
        case BH_ACT_RELU: return launch_ew<1, false>("relu fwd", FRelu{}, y, x, nullptr, nullptr, n);
        case BH_ACT_SIGMOID: return launch_ew<1, false>("sigmoid fwd", FSigmoid{}, y, x, nullptr, nullptr, n);
        case BH_ACT_TANH: return launch_ew<1, false>("tanh fwd", FTanh{}, y, x, nullptr, nullptr, n);
        case BH_ACT_GELU: return launch_ew<1, false>("gelu fwd", FGelu{}, y, x, nullptr, nullptr, n);
    }
    return set_error(BH_EINVAL, "bh_activation_forward: unknown activation %d", act);
}

int bh_activation_backward_colsum(int act, const float* saved, const float* dy, float* dx, float* colsum, int64_t rows, int64_t cols,
                                  int accumulate) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(rows >= 0 && cols >= 0 && (colsum || cols == 0) && ((saved && dy && dx) || rows * cols == 0), "bad argument");
    if (cols == 0) return BH_OK;
    if (rows == 0) return accumulate ? BH_OK : bh_memset_zero(colsum, sizeof(float) * (size_t)cols);
    switch (act) {
        case BH_ACT_RELU: return launch_act_bwd_colsum("relu bwd + colsum", FReluBwd<false>{}, saved, dy, dx, colsum, rows, cols, accumulate);
        case BH_ACT_SIGMOID: return launch_act_bwd_colsum("sigmoid bwd + colsum", FSigmoidBwd<false>{}, saved, dy, dx, colsum, rows, cols, accumulate);
        case BH_ACT_TANH: return launch_act_bwd_colsum("tanh bwd + colsum", FTanhBwd<false>{}, saved, dy, dx, colsum, rows, cols, accumulate);
        case BH_ACT_GELU: return launch_act_bwd_colsum("gelu bwd + colsum", FGeluBwd<false>{}, saved, dy, dx, colsum, rows, cols, accumulate);
    }
    return set_error(BH_EINVAL, "bh_activation_backward_colsum: unknown activation %d", act);
}

int bh_activation_backward(int act, const float* saved, const float* dy, float* dx, int64_t n, int accumulate) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && ((saved && dy && dx) || n == 0), "bad argument");
#define BH_BWD(FN, label)                                                                              \
    return accumulate ? launch_ew<2, true>(label, FN<true>{}, dx, saved, dy, nullptr, n)               \
                      : launch_ew<2, false>(label, FN<false>{}, dx, saved, dy, nullptr, n)
    switch (act) {
        case BH_ACT_RELU: BH_BWD(FReluBwd, "relu bwd");
        case BH_ACT_SIGMOID: BH_BWD(FSigmoidBwd, "sigmoid bwd");
        case BH_ACT_TANH: BH_BWD(FTanhBwd, "tanh bwd");
        case BH_ACT_GELU: BH_BWD(FGeluBwd, "gelu bwd");
    }
#undef BH_BWD
    return set_error(BH_EINVAL, "bh_activation_backward: unknown activation %d", act);
}

int bh_bias_add_rows(float* y, const float* bias, int64_t rows, int64_t cols) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(rows >= 0 && cols >= 0 && ((y && bias) || rows * cols == 0), "bad argument");
    if (rows * cols == 0) return BH_OK;
    hipLaunchKernelGGL(bias_rows_kernel, dim3(grid_for(rows * cols)), dim3(kBlock), 0, stream(), y, bias, rows, cols);
    return BH_LAUNCH_CHECK("bh_bias_add_rows");
}

int bh_mse_grad(const float* pred, const float* target, float* grad, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && ((pred && target && grad) || n == 0), "bad argument");
    return launch_ew<2, false>("bh_mse_grad", FMseGrad{(float)(size_t)n}, grad, pred, target, nullptr, n);
}

int bh_sgd_update(float* p, float* g, float lr, int64_t n, int zero_grad) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && ((p && g) || n == 0), "bad argument");
    if (n == 0) return BH_OK;
    hipLaunchKernelGGL(sgd_kernel, dim3(grid_for(n)), dim3(kBlock), 0, stream(), p, g, lr, n, zero_grad);
    return BH_LAUNCH_CHECK("bh_sgd_update");
}

}  // extern "C"
