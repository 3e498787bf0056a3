// bh_typed.hip - elementwise arithmetic on the element types the reference's arithmetic handles besides the hot
// path's float32: float64, int32, int64 (src/ops/arithmetic.c:157-360 binary ops with broadcasting and boat_mod,
// :425-560 scalar ops and boat_pow_scalar).  Same operators on the same C types, one element per lane; these are
// off the training path and are not tuned beyond coalesced access.
#include "bh_common.h"

#include <math.h>

namespace bh {

struct BroadcastMap {
    int ndim;
    int64_t out_shape[8];
    int64_t a_stride[8];   // 0 where a is broadcast along the dimension
    int64_t b_stride[8];
};

__device__ __forceinline__ float mod_of(float a, float b) { return fmodf(a, b); }
__device__ __forceinline__ double mod_of(double a, double b) { return fmod(a, b); }
// integer division by zero raises SIGFPE on the host; a GPU lane has nothing to raise, the result is defined as 0
__device__ __forceinline__ int32_t mod_of(int32_t a, int32_t b) { return b == 0 ? 0 : (b == -1 ? 0 : a % b); }
__device__ __forceinline__ int64_t mod_of(int64_t a, int64_t b) { return b == 0 ? 0 : (b == -1 ? 0 : a % b); }
__device__ __forceinline__ float div_of(float a, float b) { return a / b; }
__device__ __forceinline__ double div_of(double a, double b) { return a / b; }
__device__ __forceinline__ int32_t div_of(int32_t a, int32_t b) {
    return b == 0 ? 0 : (b == -1 ? (int32_t)(0u - (uint32_t)a) : a / b);
}
__device__ __forceinline__ int64_t div_of(int64_t a, int64_t b) {
    return b == 0 ? 0 : (b == -1 ? (int64_t)(0ull - (uint64_t)a) : a / b);
}
__device__ __forceinline__ float pow_of(float a, float b) { return powf(a, b); }
__device__ __forceinline__ double pow_of(double a, double b) { return pow(a, b); }
__device__ __forceinline__ int32_t pow_of(int32_t a, int32_t) { return a; }   // never selected for integers
__device__ __forceinline__ int64_t pow_of(int64_t a, int64_t) { return a; }

template <typename T>
__device__ __forceinline__ T apply_op(int op, T a, T b) {
    switch (op) {
        case 0: return a + b;
        case 1: return a - b;
        case 2: return a * b;
        case 3: return div_of(a, b);
        case 4: return mod_of(a, b);
        default: return pow_of(a, b);
    }
}

// no __restrict__: the in-place forms pass the same buffer as input and output (each lane reads its element, then writes it)
template <typename T>
__global__ __launch_bounds__(256) void typed_binary_kernel(int op, const T* a, const T* b,
                                                           T* out, int64_t n, BroadcastMap map, bool flat) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        int64_t ia = i, ib = i;
        if (!flat) {
            ia = 0;
            ib = 0;
            int64_t rest = i;
            for (int d = map.ndim - 1; d >= 0; d--) {
                const int64_t c = rest % map.out_shape[d];
                rest /= map.out_shape[d];
                ia += c * map.a_stride[d];
                ib += c * map.b_stride[d];
            }
        }
        out[i] = apply_op<T>(op, a[ia], b[ib]);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void typed_scalar_kernel(int op, const T* a, T s, T* out, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) out[i] = apply_op<T>(op, a[i], s);
}

static unsigned grid_for(int64_t n) {
    int64_t blocks = ceil_div(n, 256);
    if (blocks > 256 * 32) blocks = 256 * 32;
    return (unsigned)blocks;
}

}  // namespace bh

using namespace bh;

extern "C" {

int bh_binary_typed(int dtype, int op, const void* a, const int64_t* a_shape, const void* b, const int64_t* b_shape, void* out,
                    const int64_t* out_shape, int ndim) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(dtype >= BH_DT_F32 && dtype <= BH_DT_I64, "unknown element type");
    BH_CHECK_ARG(op >= 0 && op <= 4, "unknown op");
    BH_CHECK_ARG(ndim >= 0 && ndim <= 8 && (ndim == 0 || (a_shape && b_shape && out_shape)), "bad rank");
    BroadcastMap map;
    map.ndim = ndim;
    int64_t n = 1, sa = 1, sb = 1;
    bool flat = true;
    for (int d = ndim - 1; d >= 0; d--) {
        BH_CHECK_ARG(out_shape[d] >= 0 && (a_shape[d] == out_shape[d] || a_shape[d] == 1) && (b_shape[d] == out_shape[d] || b_shape[d] == 1),
                     "shapes do not broadcast");
        map.out_shape[d] = out_shape[d];
        map.a_stride[d] = a_shape[d] == 1 ? 0 : sa;
        map.b_stride[d] = b_shape[d] == 1 ? 0 : sb;
        if (a_shape[d] != out_shape[d] || b_shape[d] != out_shape[d]) flat = false;
        sa *= a_shape[d];
        sb *= b_shape[d];
        n *= out_shape[d];
    }
    if (n == 0) return BH_OK;
    BH_CHECK_ARG(a && b && out, "null pointer");
#define BH_TYPED_LAUNCH(T) \
    hipLaunchKernelGGL(typed_binary_kernel<T>, dim3(grid_for(n)), dim3(256), 0, stream(), op, (const T*)a, (const T*)b, (T*)out, n, map, flat)
    switch (dtype) {
        case BH_DT_F32: BH_TYPED_LAUNCH(float); break;
        case BH_DT_F64: BH_TYPED_LAUNCH(double); break;
        case BH_DT_I32: BH_TYPED_LAUNCH(int32_t); break;
        default: BH_TYPED_LAUNCH(int64_t); break;
    }
#undef BH_TYPED_LAUNCH
    return BH_LAUNCH_CHECK("bh_binary_typed");
}

int bh_scalar_op_typed(int dtype, int op, const void* a, double scalar, void* out, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(dtype >= BH_DT_F32 && dtype <= BH_DT_I64, "unknown element type");
    BH_CHECK_ARG((op >= 0 && op <= 3) || (op == 5 && dtype <= BH_DT_F64), "unknown op for this element type");
    BH_CHECK_ARG(n >= 0, "bad size");
    if (n == 0) return BH_OK;
    BH_CHECK_ARG(a && out, "null pointer");
    // the scalar is narrowed to the tensor's element type first (arithmetic.c:437,455,464)
#define BH_TYPED_LAUNCH(T) \
    hipLaunchKernelGGL(typed_scalar_kernel<T>, dim3(grid_for(n)), dim3(256), 0, stream(), op, (const T*)a, (T)scalar, (T*)out, n)
    switch (dtype) {
        case BH_DT_F32: BH_TYPED_LAUNCH(float); break;
        case BH_DT_F64: BH_TYPED_LAUNCH(double); break;
        case BH_DT_I32: BH_TYPED_LAUNCH(int32_t); break;
        default: BH_TYPED_LAUNCH(int64_t); break;
    }
#undef BH_TYPED_LAUNCH
    return BH_LAUNCH_CHECK("bh_scalar_op_typed");
}

}  // extern "C"
