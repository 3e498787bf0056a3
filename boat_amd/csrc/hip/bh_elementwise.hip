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
