// bh_reduce.hip - reductions and row softmax family.
//
//   full sum                      src/ops/arithmetic.c:611-691 (boat_sum)
//   column sum (bias gradient)    src/layers/dense.c:286-291, src/layers/attention.c:1257-1268
//   softmax / log-softmax, last axis, forward and backward
//                                 src/autodiff.c:1701-1883, 1885-2068
//   fused softmax + cross-entropy gradient replacing the tape chain
//   log_softmax -> mul(onehot) -> sum -> mul(-1/B) of examples/mnist/mnist_autodiff.c:397-522
//
// The reference adds left to right in fp32; these kernels add in wavefront trees, so
// results agree to rounding (a few ulp), not bit for bit.
#include "bh_common.h"

#include <float.h>

namespace bh {

constexpr int kRBlock = 256;

// ---- full sum: per-block partials, then one block folds them (double accumulator) ----
__global__ __launch_bounds__(kRBlock) void sum_partial_kernel(const float* x, float* partial, int64_t n) {
    __shared__ float red[kRBlock / 64];
    float acc = 0.f;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) acc += x[i];
    float t = block_sum<kRBlock / 64>(acc, red);
    if (threadIdx.x == 0) partial[blockIdx.x] = t;
}
// small inputs: one workgroup does both stages
__global__ __launch_bounds__(kRBlock) void sum_small_kernel(const float* x, float* out, int64_t n) {
    __shared__ double red[kRBlock / 64];
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int64_t i = threadIdx.x;
    for (; i + 3 * kRBlock < n; i += 4 * kRBlock) {
        a0 += x[i];
        a1 += x[i + kRBlock];
        a2 += x[i + 2 * kRBlock];
        a3 += x[i + 3 * kRBlock];
    }
    for (; i < n; i += kRBlock) a0 += x[i];
    double acc = wave_sum_f64((double)((a0 + a1) + (a2 + a3)));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int w = 0; w < kRBlock / 64; w++) t += red[w];
        out[0] = (float)t;
    }
}
__global__ __launch_bounds__(kRBlock) void sum_final_kernel(const float* partial, float* out, int n, float scale) {
    __shared__ double red[kRBlock / 64];
    double acc = 0.0;
    for (int i = threadIdx.x; i < n; i += blockDim.x) acc += (double)partial[i];
    acc = wave_sum_f64(acc);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int i = 0; i < kRBlock / 64; i++) t += red[i];
        out[0] = (float)t * scale;
    }
}

// ---- column sum: partial[rb][c] over row chunks, then fold_rows_kernel folds the chunks ----
// Row chunk y of Y takes rows y, y+Y, y+2Y, ...: the resident workgroups read neighbouring rows.
__global__ __launch_bounds__(kRBlock) void colsum_partial_kernel(const float* __restrict__ x, float* __restrict__ partial,
                                                                 int64_t rows, int64_t cols) {
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= cols) return;
    const int64_t step = gridDim.y;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int64_t r = blockIdx.y;
    for (; r + 3 * step < rows; r += 4 * step) {
        a0 += x[r * cols + c];
        a1 += x[(r + step) * cols + c];
        a2 += x[(r + 2 * step) * cols + c];
        a3 += x[(r + 3 * step) * cols + c];
    }
    for (; r < rows; r += step) a0 += x[r * cols + c];
    partial[(int64_t)blockIdx.y * cols + c] = (a0 + a1) + (a2 + a3);
}

// the same for up to four matrices of one shape in one launch (blockIdx.z picks the matrix): partial[rb][g*cols + c]
struct ColsumTab {
    const float* x[4];
    float* out[4];
};
__global__ __launch_bounds__(kRBlock) void colsum_partial_tab_kernel(ColsumTab t, float* __restrict__ partial, int64_t rows, int64_t cols) {
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= cols) return;
    const float* __restrict__ x = t.x[blockIdx.z];
    const int64_t step = gridDim.y;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int64_t r = blockIdx.y;
    for (; r + 3 * step < rows; r += 4 * step) {
        a0 += x[r * cols + c];
        a1 += x[(r + step) * cols + c];
        a2 += x[(r + 2 * step) * cols + c];
        a3 += x[(r + 3 * step) * cols + c];
    }
    for (; r < rows; r += step) a0 += x[r * cols + c];
    partial[((int64_t)blockIdx.y * gridDim.z + blockIdx.z) * cols + c] = (a0 + a1) + (a2 + a3);
}
// folds the row chunks of that launch: column c of matrix g from partial[rb][g][c]; the arithmetic and its order are
// fold_rows_kernel's (16 row lanes per column, four running sums each, folded through LDS in lane order)
__global__ __launch_bounds__(kFoldCols * kFoldLanes) void fold_rows_tab_kernel(const float* __restrict__ partial, int64_t nrows, int64_t cols,
                                                                               int groups, ColsumTab t, int accumulate) {
    __shared__ float red[kFoldLanes][kFoldCols + 1];
    const int tx = threadIdx.x % kFoldCols, ty = threadIdx.x / kFoldCols;
    const int64_t gc = (int64_t)blockIdx.x * kFoldCols + tx;      // column of the [rb][groups * cols] matrix
    const int64_t ncols = (int64_t)groups * cols;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    if (gc < ncols) {
        int64_t r = ty;
        for (; r + 3 * kFoldLanes < nrows; r += 4 * kFoldLanes) {
            a0 += partial[r * ncols + gc];
            a1 += partial[(r + kFoldLanes) * ncols + gc];
            a2 += partial[(r + 2 * kFoldLanes) * ncols + gc];
            a3 += partial[(r + 3 * kFoldLanes) * ncols + gc];
        }
        for (; r < nrows; r += kFoldLanes) a0 += partial[r * ncols + gc];
    }
    red[ty][tx] = (a0 + a1) + (a2 + a3);
    __syncthreads();
    if (ty == 0 && gc < ncols) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < kFoldLanes; i++) acc += red[i][tx];
        float* dst = t.out[gc / cols] + gc % cols;
        *dst = accumulate ? *dst + acc : acc;
    }
}

// ---- row kernels: one wavefront per row, 4 rows per block ----
// MODE 0 softmax fwd, 1 softmax bwd, 2 log-softmax fwd, 3 log-softmax bwd
template <int MODE>
__global__ __launch_bounds__(kRBlock) void row_softmax_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                              float* __restrict__ out, int64_t rows, int64_t cols) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (kRBlock / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* ar = a + row * cols;
    const float* br = b ? b + row * cols : nullptr;
    float* orow = out + row * cols;
    if (MODE == 0 || MODE == 2) {
        float mx = -FLT_MAX;
        for (int64_t i = lane; i < cols; i += 64) mx = fmaxf(mx, ar[i]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int64_t i = lane; i < cols; i += 64) sum += expf(ar[i] - mx);
        sum = wave_sum(sum);
        if (MODE == 0) {
            const float inv = 1.0f / sum;
            for (int64_t i = lane; i < cols; i += 64) {
                float e = expf(ar[i] - mx);
                orow[i] = sum != 0.0f ? e * inv : e;
            }
        } else {
            const float lse = logf(fmaxf(sum, FLT_MIN));
            for (int64_t i = lane; i < cols; i += 64) orow[i] = ar[i] - mx - lse;
        }
    } else if (MODE == 1) {   // a = y, b = dy : dx = y*(dy - sum(y*dy))
        float t = 0.f;
        for (int64_t i = lane; i < cols; i += 64) t += ar[i] * br[i];
        t = wave_sum(t);
        for (int64_t i = lane; i < cols; i += 64) orow[i] = ar[i] * (br[i] - t);
    } else {                  // a = y (log-probs), b = dy : dx = dy - exp(y)*sum(dy)
        float g = 0.f;
        for (int64_t i = lane; i < cols; i += 64) g += br[i];
        g = wave_sum(g);
        for (int64_t i = lane; i < cols; i += 64) orow[i] = br[i] - expf(ar[i]) * g;
    }
}

// The same four row operations for rows of up to 64 * NR elements: the row (both rows, backward) is read once into NR
// registers per lane and every later pass runs over the registers.  Lane l still owns elements l, l + 64, ... and adds
// them in that order, and an exponential kept from the sum is the one the kernel above computes a second time, so the
// results are the same bits (8192x1024 softmax forward: 13 us against 23).
template <int MODE, int NR>
__global__ __launch_bounds__(kRBlock) void row_softmax_cached_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                                     float* __restrict__ out, int64_t rows, int cols) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (kRBlock / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* ar = a + row * cols;
    float* orow = out + row * cols;
    float av[NR];
#pragma unroll
    for (int j = 0; j < NR; j++) av[j] = lane + 64 * j < cols ? ar[lane + 64 * j] : 0.f;
    if (MODE == 0 || MODE == 2) {
        float mx = -FLT_MAX;
#pragma unroll
        for (int j = 0; j < NR; j++)
            if (lane + 64 * j < cols) mx = fmaxf(mx, av[j]);
        mx = wave_max(mx);
        float ev[NR];
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < NR; j++)
            if (lane + 64 * j < cols) {
                ev[j] = expf(av[j] - mx);
                sum += ev[j];
            }
        sum = wave_sum(sum);
        if (MODE == 0) {
            const float inv = 1.0f / sum;
#pragma unroll
            for (int j = 0; j < NR; j++)
                if (lane + 64 * j < cols) orow[lane + 64 * j] = sum != 0.0f ? ev[j] * inv : ev[j];
        } else {
            const float lse = logf(fmaxf(sum, FLT_MIN));
#pragma unroll
            for (int j = 0; j < NR; j++)
                if (lane + 64 * j < cols) orow[lane + 64 * j] = av[j] - mx - lse;
        }
    } else {
        const float* br = b + row * cols;
        float bv[NR];
#pragma unroll
        for (int j = 0; j < NR; j++) bv[j] = lane + 64 * j < cols ? br[lane + 64 * j] : 0.f;
        if (MODE == 1) {      // a = y, b = dy : dx = y*(dy - sum(y*dy))
            float t = 0.f;
#pragma unroll
            for (int j = 0; j < NR; j++)
                if (lane + 64 * j < cols) t += av[j] * bv[j];
            t = wave_sum(t);
#pragma unroll
            for (int j = 0; j < NR; j++)
                if (lane + 64 * j < cols) orow[lane + 64 * j] = av[j] * (bv[j] - t);
        } else {              // a = y (log-probs), b = dy : dx = dy - exp(y)*sum(dy)
            float g = 0.f;
#pragma unroll
            for (int j = 0; j < NR; j++)
                if (lane + 64 * j < cols) g += bv[j];
            g = wave_sum(g);
#pragma unroll
            for (int j = 0; j < NR; j++)
                if (lane + 64 * j < cols) orow[lane + 64 * j] = bv[j] - expf(av[j]) * g;
        }
    }
}

// Backward of loss = f * sum(w o log_softmax(z)) in one kernel: the chain rule of mul, sum, mul and log-softmax with the
// operations of the separate kernels in their order (dls = (seed*f) * w ; g = sum_j dls_j ; dz_j = dls_j - expf(y_j) * g),
// so the result is the chain's bit for bit.  y = log_softmax(z) as the forward pass left it.
__global__ __launch_bounds__(kRBlock) void log_softmax_weighted_bwd_kernel(const float* __restrict__ y, const float* __restrict__ w,
                                                                           const float* __restrict__ seed, const float* __restrict__ f,
                                                                           float* __restrict__ dz, int64_t rows, int64_t cols) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (kRBlock / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float c = (seed ? seed[0] : 1.0f) * f[0];
    const float* yr = y + row * cols;
    const float* wr = w + row * cols;
    float* out = dz + row * cols;
    float g = 0.f;
    for (int64_t i = lane; i < cols; i += 64) g += c * wr[i];
    g = wave_sum(g);
    for (int64_t i = lane; i < cols; i += 64) out[i] = c * wr[i] - expf(yr[i]) * g;
}

// The same for a small matrix, followed in the same launch by the column sums of dz (the bias gradient of the dense layer that
// produced z): one workgroup, rows dealt to its 16 wavefronts, dz kept in LDS, then fold_rows_kernel's own summation (64
// columns x 16 row lanes, four running sums each, folded in lane order), so the sums are bh_colsum's bit for bit.
constexpr int kLswTile = 8192;                  // rows * cols the LDS copy of dz holds
__global__ __launch_bounds__(kFoldCols * kFoldLanes) void lsw_bwd_colsum_small_kernel(const float* __restrict__ y, const float* __restrict__ w,
                                                                                      const float* __restrict__ seed, const float* __restrict__ f,
                                                                                      float* __restrict__ dz, float* __restrict__ colsum,
                                                                                      int rows, int cols, int accumulate) {
    __shared__ float tile[kLswTile];
    __shared__ float red[kFoldLanes][kFoldCols + 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float c = (seed ? seed[0] : 1.0f) * f[0];
    for (int row = wave; row < rows; row += kFoldCols * kFoldLanes / 64) {
        const float* yr = y + (int64_t)row * cols;
        const float* wr = w + (int64_t)row * cols;
        float g = 0.f;
        for (int i = lane; i < cols; i += 64) g += c * wr[i];
        g = wave_sum(g);
        for (int i = lane; i < cols; i += 64) {
            const float v = c * wr[i] - expf(yr[i]) * g;
            dz[(int64_t)row * cols + i] = v;
            tile[row * cols + i] = v;
        }
    }
    __syncthreads();
    const int tx = threadIdx.x % kFoldCols, ty = threadIdx.x / kFoldCols;
    for (int cb = 0; cb < cols; cb += kFoldCols) {
        const int col = cb + tx;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        if (col < cols) {
            int r = ty;
            for (; r + 3 * kFoldLanes < rows; r += 4 * kFoldLanes) {
                a0 += tile[r * cols + col];
                a1 += tile[(r + kFoldLanes) * cols + col];
                a2 += tile[(r + 2 * kFoldLanes) * cols + col];
                a3 += tile[(r + 3 * kFoldLanes) * cols + col];
            }
            for (; r < rows; r += kFoldLanes) a0 += tile[r * cols + col];
        }
        red[ty][tx] = (a0 + a1) + (a2 + a3);
        __syncthreads();
        if (ty == 0 && col < cols) {
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < kFoldLanes; i++) acc += red[i][tx];
            colsum[col] = accumulate ? colsum[col] + acc : acc;
        }
        __syncthreads();
    }
}

// fused softmax + cross-entropy gradient; row_ll receives log_softmax(z)[label] per row
__global__ __launch_bounds__(kRBlock) void softmax_ce_kernel(const float* __restrict__ z, const int32_t* __restrict__ labels,
                                                             float* __restrict__ dz, float* __restrict__ row_ll,
                                                             int64_t rows, int64_t cols, float f) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (kRBlock / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* zr = z + row * cols;
    float mx = -FLT_MAX;
    for (int64_t i = lane; i < cols; i += 64) mx = fmaxf(mx, zr[i]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int64_t i = lane; i < cols; i += 64) sum += expf(zr[i] - mx);
    sum = wave_sum(sum);
    const float lse = logf(fmaxf(sum, FLT_MIN));
    const int32_t label = labels[row];
    const bool valid = label >= 0 && label < cols;
    // backward of the tape chain: d(ls)_j = f*onehot_j, dz_j = d(ls)_j - exp(ls_j) * sum_j d(ls)_j
    const float g = valid ? f : 0.0f;
    for (int64_t i = lane; i < cols; i += 64) {
        const float ls = zr[i] - mx - lse;
        const float dls = (valid && i == label) ? f : 0.0f;
        if (dz) dz[row * cols + i] = dls - expf(ls) * g;
        if (valid && i == label && row_ll) row_ll[row] = ls;
    }
    if (!valid && lane == 0 && row_ll) row_ll[row] = 0.0f;
}

}  // namespace bh

using namespace bh;

extern "C" {

int bh_sum_all(const float* x, float* out1, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n >= 0 && out1 && (x || n == 0), "bad argument");
    if (n <= 16 * kRBlock) {   // a few elements per lane: one launch
        hipLaunchKernelGGL(sum_small_kernel, dim3(1), dim3(kRBlock), 0, stream(), x, out1, n);
        return BH_LAUNCH_CHECK("bh_sum_all");
    }
    int blocks = (int)ceil_div(n > 0 ? n : 1, (int64_t)kRBlock * 8);
    if (blocks > 1024) blocks = 1024;
    float* partial = (float*)bh_malloc(sizeof(float) * (size_t)blocks);
    if (!partial) return BH_ENOMEM;
    hipLaunchKernelGGL(sum_partial_kernel, dim3(blocks), dim3(kRBlock), 0, stream(), x, partial, n);
    hipLaunchKernelGGL(sum_final_kernel, dim3(1), dim3(kRBlock), 0, stream(), partial, out1, blocks, 1.0f);
    bh_free(partial);
    return BH_LAUNCH_CHECK("bh_sum_all");
}

int bh_mse_loss(const float* pred, const float* target, float* loss_out, int64_t n);  // defined below
int bh_mse_grad(const float* pred, const float* target, float* grad, int64_t n);

int bh_colsum(const float* x, float* out, int64_t rows, int64_t cols, int accumulate) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(rows >= 0 && cols >= 0 && (out || cols == 0) && (x || rows * cols == 0), "bad argument");
    if (cols == 0) return BH_OK;
    ProfScope prof(BH_PROF_COLSUM, 4.0 * (double)rows * (double)cols);
    if (rows <= 256) {   // few rows: the fold kernel (64 columns x 16 row lanes per workgroup) is the whole column sum
        hipLaunchKernelGGL(fold_rows_kernel, dim3((unsigned)ceil_div(cols, kFoldCols)), dim3(kFoldCols * kFoldLanes), 0, stream(),
                           x, rows, cols, out, (float*)nullptr, cols, accumulate);
        return BH_LAUNCH_CHECK("bh_colsum");
    }
    const int col_blocks = (int)ceil_div(cols, kRBlock);
    // enough row chunks to put ~2k blocks on the chip, at least 32 rows each
    int64_t chunks = ceil_div(2048, col_blocks);
    if (chunks > ceil_div(rows, 32)) chunks = ceil_div(rows, 32);
    if (chunks < 1) chunks = 1;
    float* partial = (float*)bh_malloc(sizeof(float) * (size_t)(chunks * cols));
    if (!partial) return BH_ENOMEM;
    hipLaunchKernelGGL(colsum_partial_kernel, dim3(col_blocks, (unsigned)chunks), dim3(kRBlock), 0, stream(), x, partial,
                       rows, cols);
    hipLaunchKernelGGL(fold_rows_kernel, dim3((unsigned)ceil_div(cols, kFoldCols)), dim3(kFoldCols * kFoldLanes), 0, stream(),
                       partial, chunks, cols, out, (float*)nullptr, cols, accumulate);
    bh_free(partial);
    return BH_LAUNCH_CHECK("bh_colsum");
}

#define BH_ROW_LAUNCH(MODE, a, b, out, name)                                                                   \
    do {                                                                                                       \
        BH_REQUIRE_INIT();                                                                                     \
        BH_CHECK_ARG(rows >= 0 && cols >= 0, "negative shape");                                                \
        if (rows * cols == 0) return BH_OK;                                                                    \
        BH_CHECK_ARG((a) && (out), "null pointer");                                                            \
        const dim3 row_grid((unsigned)ceil_div(rows, kRBlock / 64));                                           \
        if (cols <= 64 * 4)                                                                                    \
            hipLaunchKernelGGL((row_softmax_cached_kernel<MODE, 4>), row_grid, dim3(kRBlock), 0, stream(), a, b, out, rows, (int)cols); \
        else if (cols <= 64 * 16)                                                                              \
            hipLaunchKernelGGL((row_softmax_cached_kernel<MODE, 16>), row_grid, dim3(kRBlock), 0, stream(), a, b, out, rows, (int)cols); \
        else if (cols <= 64 * 32)                                                                              \
            hipLaunchKernelGGL((row_softmax_cached_kernel<MODE, 32>), row_grid, dim3(kRBlock), 0, stream(), a, b, out, rows, (int)cols); \
        else                                                                                                   \
            hipLaunchKernelGGL((row_softmax_kernel<MODE>), row_grid, dim3(kRBlock), 0, stream(), a, b, out, rows, cols); \
        return BH_LAUNCH_CHECK(name);                                                                          \
    } while (0)

// out[g][c] (+)= sum_r x[g][r][c] for up to four matrices of one shape: one partial launch and one fold where bh_colsum
// takes two per matrix; the sums and their order are bh_colsum's, so the results are the same bits
int bh_colsum_grouped(const float* const* x, float* const* out, int groups, int64_t rows, int64_t cols, int accumulate) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(groups >= 1 && groups <= 4 && rows >= 0 && cols >= 0 && x && out, "bad argument");
    if (cols == 0) return BH_OK;
    for (int g = 0; g < groups; g++) BH_CHECK_ARG(out[g] && (x[g] || rows == 0), "null pointer");
    if (groups == 1 || rows <= 256) {
        for (int g = 0; g < groups; g++) {
            const int rc = bh_colsum(x[g], out[g], rows, cols, accumulate);
            if (rc != BH_OK) return rc;
        }
        return BH_OK;
    }
    ProfScope prof(BH_PROF_COLSUM, 4.0 * (double)rows * (double)cols * groups);
    const int col_blocks = (int)ceil_div(cols, kRBlock);
    int64_t chunks = ceil_div(2048, col_blocks);          // per matrix, as bh_colsum cuts it
    if (chunks > ceil_div(rows, 32)) chunks = ceil_div(rows, 32);
    if (chunks < 1) chunks = 1;
    float* partial = (float*)bh_malloc(sizeof(float) * (size_t)(chunks * groups * cols));
    if (!partial) return BH_ENOMEM;
    ColsumTab t = {};
    for (int g = 0; g < groups; g++) {
        t.x[g] = x[g];
        t.out[g] = out[g];
    }
    hipLaunchKernelGGL(colsum_partial_tab_kernel, dim3(col_blocks, (unsigned)chunks, (unsigned)groups), dim3(kRBlock), 0, stream(), t, partial,
                       rows, cols);
    hipLaunchKernelGGL(fold_rows_tab_kernel, dim3((unsigned)ceil_div((int64_t)groups * cols, kFoldCols)), dim3(kFoldCols * kFoldLanes), 0, stream(),
                       partial, chunks, cols, groups, t, accumulate);
    bh_free(partial);
    return BH_LAUNCH_CHECK("bh_colsum_grouped");
}

int bh_softmax_forward(const float* x, float* y, int64_t rows, int64_t cols) {
    BH_ROW_LAUNCH(0, x, (const float*)nullptr, y, "bh_softmax_forward");
}
int bh_softmax_backward(const float* y, const float* dy, float* dx, int64_t rows, int64_t cols) {
    BH_CHECK_ARG(dy || rows * cols == 0, "null dy");
    BH_ROW_LAUNCH(1, y, dy, dx, "bh_softmax_backward");
}
int bh_log_softmax_forward(const float* x, float* y, int64_t rows, int64_t cols) {
    BH_ROW_LAUNCH(2, x, (const float*)nullptr, y, "bh_log_softmax_forward");
}
int bh_log_softmax_backward(const float* y, const float* dy, float* dx, int64_t rows, int64_t cols) {
    BH_CHECK_ARG(dy || rows * cols == 0, "null dy");
    BH_ROW_LAUNCH(3, y, dy, dx, "bh_log_softmax_backward");
}

int bh_log_softmax_weighted_backward(const float* y, const float* w, const float* seed, const float* f, float* dz,
                                     int64_t rows, int64_t cols) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(rows >= 0 && cols >= 0, "negative shape");
    if (rows * cols == 0) return BH_OK;
    BH_CHECK_ARG(y && w && f && dz, "null pointer");
    hipLaunchKernelGGL(log_softmax_weighted_bwd_kernel, dim3((unsigned)ceil_div(rows, kRBlock / 64)), dim3(kRBlock), 0, stream(),
                       y, w, seed, f, dz, rows, cols);
    return BH_LAUNCH_CHECK("bh_log_softmax_weighted_backward");
}

int bh_log_softmax_weighted_backward_colsum(const float* y, const float* w, const float* seed, const float* f, float* dz,
                                            float* colsum, int64_t rows, int64_t cols, int accumulate) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(rows >= 0 && cols >= 0 && (colsum || cols == 0), "bad argument");
    if (cols == 0) return BH_OK;
    if (rows == 0) return accumulate ? BH_OK : bh_memset_zero(colsum, sizeof(float) * (size_t)cols);
    BH_CHECK_ARG(y && w && f && dz, "null pointer");
    if (rows <= 256 && rows * cols <= kLswTile) {
        hipLaunchKernelGGL(lsw_bwd_colsum_small_kernel, dim3(1), dim3(kFoldCols * kFoldLanes), 0, stream(), y, w, seed, f, dz, colsum,
                           (int)rows, (int)cols, accumulate);
        return BH_LAUNCH_CHECK("bh_log_softmax_weighted_backward_colsum");
    }
    const int rc = bh_log_softmax_weighted_backward(y, w, seed, f, dz, rows, cols);
    return rc != BH_OK ? rc : bh_colsum(dz, colsum, rows, cols, accumulate);
}

int bh_softmax_ce_grad(const float* logits, const int32_t* labels, float* dlogits, float* loss_out, int64_t rows,
                       int64_t cols) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(rows > 0 && cols > 0 && logits && labels, "bad argument");
    float* row_ll = nullptr;
    if (loss_out) {
        row_ll = (float*)bh_malloc(sizeof(float) * (size_t)rows);
        if (!row_ll) return BH_ENOMEM;
    }
    const float f = -1.0f / (float)(size_t)rows;
    hipLaunchKernelGGL(softmax_ce_kernel, dim3((unsigned)ceil_div(rows, kRBlock / 64)), dim3(kRBlock), 0, stream(),
                       logits, labels, dlogits, row_ll, rows, cols, f);
    if (loss_out && rows <= 16 * kRBlock) {   // a few values per lane: the final stage alone sums them (in double)
        hipLaunchKernelGGL(sum_final_kernel, dim3(1), dim3(kRBlock), 0, stream(), row_ll, loss_out, (int)rows, f);
        bh_free(row_ll);
    } else if (loss_out) {
        int blocks = (int)ceil_div(rows, (int64_t)kRBlock * 8);
        if (blocks > 1024) blocks = 1024;
        float* partial = (float*)bh_malloc(sizeof(float) * (size_t)blocks);
        if (!partial) {
            bh_free(row_ll);
            return BH_ENOMEM;
        }
        hipLaunchKernelGGL(sum_partial_kernel, dim3(blocks), dim3(kRBlock), 0, stream(), row_ll, partial, rows);
        hipLaunchKernelGGL(sum_final_kernel, dim3(1), dim3(kRBlock), 0, stream(), partial, loss_out, blocks, f);
        bh_free(partial);
        bh_free(row_ll);
    }
    return BH_LAUNCH_CHECK("bh_softmax_ce_grad");
}

}  // extern "C"

// ---- mean squared error value (src/loss/mse.c:70-78) ----
namespace bh {
__global__ __launch_bounds__(kRBlock) void sse_partial_kernel(const float* p, const float* t, float* partial, int64_t n) {
    __shared__ float red[kRBlock / 64];
    float acc = 0.f;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float d = p[i] - t[i];
        acc += d * d;
    }
    float s = block_sum<kRBlock / 64>(acc, red);
    if (threadIdx.x == 0) partial[blockIdx.x] = s;
}
// the same sum with the gradient 2*(p - t)/n written on the way (one read of p and t for both): 16-byte pieces
typedef float red_f32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(kRBlock) void sse_grad_partial_kernel(const float* __restrict__ p, const float* __restrict__ t,
                                                                   float* __restrict__ grad, float* __restrict__ partial,
                                                                   int64_t n4, float nf) {
    __shared__ float red[kRBlock / 64];
    float acc = 0.f;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const red_f32x4* p4 = reinterpret_cast<const red_f32x4*>(p);
    const red_f32x4* t4 = reinterpret_cast<const red_f32x4*>(t);
    red_f32x4* g4 = reinterpret_cast<red_f32x4*>(grad);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        const red_f32x4 d = __builtin_nontemporal_load(p4 + i) - __builtin_nontemporal_load(t4 + i);
        acc += (d.x * d.x + d.y * d.y) + (d.z * d.z + d.w * d.w);
        const red_f32x4 g = {2.0f * d.x / nf, 2.0f * d.y / nf, 2.0f * d.z / nf, 2.0f * d.w / nf};   // as FMseGrad: 2*(p-t)/n
        __builtin_nontemporal_store(g, g4 + i);
    }
    float s = block_sum<kRBlock / 64>(acc, red);
    if (threadIdx.x == 0) partial[blockIdx.x] = s;
}
// per-element loss terms of the reference's loss objects, summed: kind 0 (p-t)^2 (src/loss/mse.c:72-76),
// 1 t*logf(clip(p, 1e-7, 1-1e-7)) (src/loss/cross_entropy.c:35-44, 91-95), 2 Huber with threshold delta (src/loss/huber.c)
__global__ __launch_bounds__(kRBlock) void loss_terms_partial_kernel(int kind, const float* p, const float* t, float* partial,
                                                                     int64_t n, float delta) {
    __shared__ float red[kRBlock / 64];
    float acc = 0.f;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const float pv = p[i], tv = t[i];
        if (kind == 0) {
            const float d = pv - tv;
            acc += d * d;
        } else if (kind == 1) {
            const float eps = 1e-7f;
            const float c = pv < eps ? eps : (pv > 1.0f - eps ? 1.0f - eps : pv);
            acc += tv * logf(c);
        } else {
            const float d = fabsf(pv - tv);
            acc += d <= delta ? 0.5f * d * d : delta * (d - 0.5f * delta);
        }
    }
    float s = block_sum<kRBlock / 64>(acc, red);
    if (threadIdx.x == 0) partial[blockIdx.x] = s;
}
}  // namespace bh

extern "C" int bh_loss_terms_sum(int kind, const float* pred, const float* target, float* sum_out, int64_t n, float delta) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(kind >= 0 && kind <= 2 && n >= 0 && sum_out && ((pred && target) || n == 0), "bad argument");
    int blocks = (int)bh::ceil_div(n > 0 ? n : 1, (int64_t)bh::kRBlock * 8);
    if (blocks > 1024) blocks = 1024;
    float* partial = (float*)bh_malloc(sizeof(float) * (size_t)blocks);
    if (!partial) return BH_ENOMEM;
    hipLaunchKernelGGL(bh::loss_terms_partial_kernel, dim3(blocks), dim3(bh::kRBlock), 0, bh::stream(), kind, pred, target,
                       partial, n, delta);
    hipLaunchKernelGGL(bh::sum_final_kernel, dim3(1), dim3(bh::kRBlock), 0, bh::stream(), partial, sum_out, blocks, 1.0f);
    bh_free(partial);
    return BH_LAUNCH_CHECK("bh_loss_terms_sum");
}

// loss = mean((p-t)^2) and grad = 2*(p-t)/n in one pass over p and t (what a training loop asks for together);
// the gradient is bit for bit bh_mse_grad's, the loss sums in another order than bh_mse_loss
extern "C" int bh_mse_loss_grad(const float* pred, const float* target, float* loss_out, float* grad, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n > 0 && pred && target && loss_out && grad, "bad argument");
    const bool vec = n % 4 == 0 && ((reinterpret_cast<uintptr_t>(pred) | reinterpret_cast<uintptr_t>(target) | reinterpret_cast<uintptr_t>(grad)) & 15) == 0;
    if (!vec) {
        const int rc = bh_mse_loss(pred, target, loss_out, n);
        return rc != BH_OK ? rc : bh_mse_grad(pred, target, grad, n);
    }
    const int64_t n4 = n / 4;
    int blocks = (int)ceil_div(n4, (int64_t)kRBlock * 2);
    if (blocks > 2048) blocks = 2048;
    float* partial = (float*)bh_malloc(sizeof(float) * (size_t)blocks);
    if (!partial) return BH_ENOMEM;
    hipLaunchKernelGGL(bh::sse_grad_partial_kernel, dim3(blocks), dim3(bh::kRBlock), 0, bh::stream(), pred, target, grad, partial, n4,
                       (float)(size_t)n);
    hipLaunchKernelGGL(bh::sum_final_kernel, dim3(1), dim3(bh::kRBlock), 0, bh::stream(), partial, loss_out, blocks,
                       1.0f / (float)(size_t)n);
    bh_free(partial);
    return BH_LAUNCH_CHECK("bh_mse_loss_grad");
}

extern "C" int bh_mse_loss(const float* pred, const float* target, float* loss_out, int64_t n) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(n > 0 && pred && target && loss_out, "bad argument");
    int blocks = (int)ceil_div(n, (int64_t)kRBlock * 8);
    if (blocks > 1024) blocks = 1024;
    float* partial = (float*)bh_malloc(sizeof(float) * (size_t)blocks);
    if (!partial) return BH_ENOMEM;
    hipLaunchKernelGGL(bh::sse_partial_kernel, dim3(blocks), dim3(bh::kRBlock), 0, bh::stream(), pred, target, partial, n);
    hipLaunchKernelGGL(bh::sum_final_kernel, dim3(1), dim3(bh::kRBlock), 0, bh::stream(), partial, loss_out, blocks,
                       1.0f / (float)(size_t)n);
    bh_free(partial);
    return BH_LAUNCH_CHECK("bh_mse_loss");
}
