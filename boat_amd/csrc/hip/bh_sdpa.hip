// bh_sdpa.hip - scaled dot-product attention on [bh, s, d] blocks, forward and backward.
//
// Forward follows scaled_dot_product_attention_impl, src/layers/attention.c:997-1073:
//   score = (q.k) * scale ; causal: score[j>i] = -1e9 ; row softmax (max-subtract, expf, /sum) ; out = A.v
// but keeps the row log-sum-exp (max + logf(sum)) instead of the [bh,s,s] matrix A the
// reference caches (:1049-1059).  Backward follows attention_backward, :1417-1520:
//   dV = A^T.dO ; dA = dO.V^T ; dS = A*(dA - rowsum(dA*A)) * scale ; dQ = dS.K ; dK = dS^T.Q
// with A recomputed as exp(score - lse).  The row term rowsum(dA*A) is evaluated as
// rowsum(dO*O), which is the same number (A.V = O) without needing A.
//
// Three implementations behind one entry point:
//   * general kernels (any s, d): one workgroup per query row (forward, dQ) or per key row
//     (dK, dV); scores of one row live in LDS.
//   * the reference's own decomposition on the matrix cores for any other shape with s >= 64: batched GEMMs through
//     bh_gemm for Q.K^T, P.V, P^T.dO, dO.V^T, dS.K, dS^T.Q with row kernels for softmax and dS in between; the [s, s]
//     matrices exist for a bounded chunk of heads at a time.
//   * MFMA kernels for d == 64 and s >= 32 (the shapes of the attention benchmarks; a length that is not a
//     multiple of 128 is handled by clamped loads, masked scores and guarded stores).
#include "bh_common.h"

#include <float.h>

namespace bh {

constexpr int kSBlock = 256;
constexpr int kMaxRowFloats = 12288;   // general path: one score row (or two) must fit in LDS

template <int NW>
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float t = red[0];
#pragma unroll
    for (int i = 1; i < NW; i++) t = fmaxf(t, red[i]);
    return t;
}

// ---- general forward: block per (head-block, query row) ----
__global__ __launch_bounds__(kSBlock) void sdpa_fwd_row_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                               const float* __restrict__ v, float scale, int causal,
                                                               float* __restrict__ out, float* __restrict__ lse,
                                                               float* __restrict__ attn, int64_t s, int64_t d) {
    extern __shared__ float row[];                 // s scores, then d floats of q
    __shared__ float red[kSBlock / 64];
    float* qrow = row + s;
    const int64_t i = blockIdx.x, h = blockIdx.y;
    const float* qh = q + h * s * d;
    const float* kh = k + h * s * d;
    const float* vh = v + h * s * d;
    for (int64_t t = threadIdx.x; t < d; t += kSBlock) qrow[t] = qh[i * d + t];
    __syncthreads();
    float mx = -FLT_MAX;
    for (int64_t j = threadIdx.x; j < s; j += kSBlock) {
        float sum = 0.f;
        for (int64_t t = 0; t < d; t++) sum += qrow[t] * kh[j * d + t];
        float sc = sum * scale;
        if (causal && j > i) sc = -1e9f;
        row[j] = sc;
        mx = fmaxf(mx, sc);
    }
    mx = block_max<kSBlock / 64>(mx, red);
    float sum = 0.f;
    for (int64_t j = threadIdx.x; j < s; j += kSBlock) {
        float e = expf(row[j] - mx);
        row[j] = e;
        sum += e;
    }
    sum = block_sum<kSBlock / 64>(sum, red);
    for (int64_t j = threadIdx.x; j < s; j += kSBlock) {
        float p = sum != 0.0f ? row[j] / sum : row[j];
        row[j] = p;
        if (attn) attn[(h * s + i) * s + j] = p;
    }
    if (threadIdx.x == 0 && lse) lse[h * s + i] = mx + logf(sum);
    __syncthreads();
    for (int64_t t = threadIdx.x; t < d; t += kSBlock) {
        float acc = 0.f;
        for (int64_t j = 0; j < s; j++) acc += row[j] * vh[j * d + t];
        out[(h * s + i) * d + t] = acc;
    }
}

// delta for head sizes that are a multiple of 4 and at most 256: d/4 lanes per row (a power of two), each one 16-byte
// piece of O and dO, rows packed into the wavefront; the lanes of a row fold through the wavefront
template <int LANES>
__global__ __launch_bounds__(kSBlock) void sdpa_delta_vec_kernel(const float* __restrict__ o, const float* __restrict__ d_out,
                                                                 float* __restrict__ delta, int64_t rows) {
    constexpr int ROWS_PER_BLOCK = kSBlock / LANES;
    const int sub = threadIdx.x % LANES;
    const int64_t r = (int64_t)blockIdx.x * ROWS_PER_BLOCK + threadIdx.x / LANES;
    float acc = 0.f;
    if (r < rows) {
        const float4 a = reinterpret_cast<const float4*>(o)[r * LANES + sub];
        const float4 b = reinterpret_cast<const float4*>(d_out)[r * LANES + sub];
        acc = (a.x * b.x + a.y * b.y) + (a.z * b.z + a.w * b.w);
    }
#pragma unroll
    for (int off = LANES / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (sub == 0 && r < rows) delta[r] = acc;
}

static void launch_delta(const float* o, const float* d_out, float* delta, int64_t rows, int64_t d);

// delta[i] = sum_d dO[i,d] * O[i,d], one wavefront per row
__global__ __launch_bounds__(kSBlock) void sdpa_delta_kernel(const float* __restrict__ o, const float* __restrict__ d_out,
                                                             float* __restrict__ delta, int64_t rows, int64_t d) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * (kSBlock / 64) + (threadIdx.x >> 6);
    if (r >= rows) return;
    float acc = 0.f;
    for (int64_t t = lane; t < d; t += 64) acc += o[r * d + t] * d_out[r * d + t];
    acc = wave_sum(acc);
    if (lane == 0) delta[r] = acc;
}

static void launch_delta(const float* o, const float* d_out, float* delta, int64_t rows, int64_t d) {
    const bool al = ((reinterpret_cast<uintptr_t>(o) | reinterpret_cast<uintptr_t>(d_out)) & 15) == 0;
#define DELTA_VEC(L)                                                                                                      \
    hipLaunchKernelGGL((sdpa_delta_vec_kernel<L>), dim3((unsigned)ceil_div(rows, kSBlock / L)), dim3(kSBlock), 0, stream(), o, \
                       d_out, delta, rows)
    if (al && d == 64 && ceil_div(rows, kSBlock / 16) <= 0x7fffffff) DELTA_VEC(16);
    else if (al && d == 128 && ceil_div(rows, kSBlock / 32) <= 0x7fffffff) DELTA_VEC(32);
    else if (al && d == 32 && ceil_div(rows, kSBlock / 8) <= 0x7fffffff) DELTA_VEC(8);
    else
        hipLaunchKernelGGL(sdpa_delta_kernel, dim3((unsigned)ceil_div(rows, kSBlock / 64)), dim3(kSBlock), 0, stream(), o, d_out,
                           delta, rows, d);
#undef DELTA_VEC
}

// ---- general backward, dQ: block per (head-block, query row) ----
__global__ __launch_bounds__(kSBlock) void sdpa_bwd_dq_row_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                                  const float* __restrict__ v, const float* __restrict__ lse,
                                                                  const float* __restrict__ delta, const float* __restrict__ d_out,
                                                                  float scale, int causal, float* __restrict__ dq, int64_t s,
                                                                  int64_t d) {
    extern __shared__ float row[];                 // s floats of dS, then q row, then dO row
    float* qrow = row + s;
    float* grow = qrow + d;
    const int64_t i = blockIdx.x, h = blockIdx.y;
    const float* kh = k + h * s * d;
    const float* vh = v + h * s * d;
    for (int64_t t = threadIdx.x; t < d; t += kSBlock) {
        qrow[t] = q[(h * s + i) * d + t];
        grow[t] = d_out[(h * s + i) * d + t];
    }
    __syncthreads();
    const float l = lse[h * s + i], dl = delta[h * s + i];
    for (int64_t j = threadIdx.x; j < s; j += kSBlock) {
        float sc = 0.f, dp = 0.f;
        for (int64_t t = 0; t < d; t++) {
            sc += qrow[t] * kh[j * d + t];
            dp += grow[t] * vh[j * d + t];
        }
        sc *= scale;
        if (causal && j > i) sc = -1e9f;
        const float p = expf(sc - l);
        row[j] = p * (dp - dl) * scale;
    }
    __syncthreads();
    for (int64_t t = threadIdx.x; t < d; t += kSBlock) {
        float acc = 0.f;
        for (int64_t j = 0; j < s; j++) acc += row[j] * kh[j * d + t];
        dq[(h * s + i) * d + t] = acc;
    }
}

// ---- general backward, dK and dV: block per (head-block, key row) ----
__global__ __launch_bounds__(kSBlock) void sdpa_bwd_dkv_row_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                                   const float* __restrict__ v, const float* __restrict__ lse,
                                                                   const float* __restrict__ delta, const float* __restrict__ d_out,
                                                                   float scale, int causal, float* __restrict__ dk,
                                                                   float* __restrict__ dv, int64_t s, int64_t d) {
    extern __shared__ float col[];                 // s floats of P, s floats of dS, k row, v row
    float* ds = col + s;
    float* krow = ds + s;
    float* vrow = krow + d;
    const int64_t j = blockIdx.x, h = blockIdx.y;
    const float* qh = q + h * s * d;
    const float* gh = d_out + h * s * d;
    for (int64_t t = threadIdx.x; t < d; t += kSBlock) {
        krow[t] = k[(h * s + j) * d + t];
        vrow[t] = v[(h * s + j) * d + t];
    }
    __syncthreads();
    for (int64_t i = threadIdx.x; i < s; i += kSBlock) {
        float sc = 0.f, dp = 0.f;
        for (int64_t t = 0; t < d; t++) {
            sc += qh[i * d + t] * krow[t];
            dp += gh[i * d + t] * vrow[t];
        }
        sc *= scale;
        if (causal && j > i) sc = -1e9f;
        const float p = expf(sc - lse[h * s + i]);
        col[i] = p;
        ds[i] = p * (dp - delta[h * s + i]) * scale;
    }
    __syncthreads();
    for (int64_t t = threadIdx.x; t < d; t += kSBlock) {
        float av = 0.f, ak = 0.f;
        for (int64_t i = 0; i < s; i++) {
            av += col[i] * gh[i * d + t];
            ak += ds[i] * qh[i * d + t];
        }
        dv[(h * s + j) * d + t] = av;
        dk[(h * s + j) * d + t] = ak;
    }
}

// ---- row kernels of the GEMM-based path: one workgroup per row of a [rows][s] score matrix (row = head*s + query) ----

// in place: P = softmax(scale * S) with keys after the query masked; lse = max + log(sum)
__global__ __launch_bounds__(kSBlock) void sdpa_softmax_rows_kernel(float* __restrict__ sc, float* __restrict__ lse, int64_t s,
                                                                    float scale, int causal) {
    __shared__ float red[kSBlock / 64];
    const int64_t row = blockIdx.x, i = row % s;
    float* p = sc + row * s;
    const int64_t lim = causal ? i + 1 : s;            // keys j < lim are visible
    float mx = -FLT_MAX;
    for (int64_t j = threadIdx.x; j < lim; j += kSBlock) mx = fmaxf(mx, p[j] * scale);
    mx = block_max<kSBlock / 64>(mx, red);
    float sum = 0.f;
    for (int64_t j = threadIdx.x; j < lim; j += kSBlock) sum += expf(p[j] * scale - mx);
    sum = block_sum<kSBlock / 64>(sum, red);
    const float inv = 1.0f / sum;
    for (int64_t j = threadIdx.x; j < s; j += kSBlock) p[j] = j < lim ? expf(p[j] * scale - mx) * inv : 0.f;
    if (threadIdx.x == 0 && lse) lse[row] = mx + logf(sum);
}

// in place: P = exp(scale * S - lse), masked keys 0
__global__ __launch_bounds__(kSBlock) void sdpa_probs_rows_kernel(float* __restrict__ sc, const float* __restrict__ lse, int64_t s,
                                                                  float scale, int causal) {
    const int64_t row = blockIdx.x, i = row % s;
    float* p = sc + row * s;
    const float l = lse[row];
    const int64_t lim = causal ? i + 1 : s;
    for (int64_t j = threadIdx.x; j < s; j += kSBlock) p[j] = j < lim ? expf(p[j] * scale - l) : 0.f;
}

// in place on dP: dS = P * (dP - delta) * scale
__global__ __launch_bounds__(kSBlock) void sdpa_ds_rows_kernel(const float* __restrict__ prob, float* __restrict__ dp,
                                                               const float* __restrict__ delta, int64_t s, float scale) {
    const int64_t row = blockIdx.x;
    const float dl = delta[row];
    const float* p = prob + row * s;
    float* g = dp + row * s;
    for (int64_t j = threadIdx.x; j < s; j += kSBlock) g[j] = p[j] * (g[j] - dl) * scale;
}

// heads per pass of the GEMM-based path: the [heads, s, s] matrices of one pass stay under 1 GiB each
static int64_t heads_per_pass(int64_t bh_count, int64_t s) {
    int64_t h = ((int64_t)1 << 28) / (s * s);
    if (h < 1) h = 1;
    if (h > 32768) h = 32768;                          // bh_gemm's batch limit with room to spare
    return h < bh_count ? h : bh_count;
}

static int sdpa_forward_gemm(const float* q, const float* k, const float* v, float scale, int causal, float* out, float* lse,
                             float* attn_out, int64_t bh_count, int64_t s, int64_t d) {
    const int64_t hp = heads_per_pass(bh_count, s);
    float* scratch = attn_out ? nullptr : (float*)bh_malloc(sizeof(float) * (size_t)(hp * s * s));
    if (!attn_out && !scratch) return BH_ENOMEM;
    int rc = BH_OK;
    for (int64_t h0 = 0; h0 < bh_count && rc == BH_OK; h0 += hp) {
        const int64_t nh = bh_count - h0 < hp ? bh_count - h0 : hp;
        float* sc = attn_out ? attn_out + h0 * s * s : scratch;
        const int64_t off = h0 * s * d;
        rc = bh_gemm(0, 1, s, s, d, q + off, d, k + off, d, sc, s, nullptr, 0, nh);              // S = Q.K^T
        if (rc != BH_OK) break;
        hipLaunchKernelGGL(sdpa_softmax_rows_kernel, dim3((unsigned)(nh * s)), dim3(kSBlock), 0, stream(), sc,
                           lse ? lse + h0 * s : nullptr, s, scale, causal);
        rc = BH_LAUNCH_CHECK("sdpa_softmax_rows_kernel");
        if (rc == BH_OK) rc = bh_gemm(0, 0, s, d, s, sc, s, v + off, d, out + off, d, nullptr, 0, nh);   // O = P.V
    }
    if (scratch) bh_free(scratch);
    return rc;
}

static int sdpa_backward_gemm(const float* q, const float* k, const float* v, const float* lse, const float* delta,
                              const float* d_out, float scale, int causal, float* dq, float* dk, float* dv, int64_t bh_count,
                              int64_t s, int64_t d) {
    const int64_t hp = heads_per_pass(bh_count, s);
    float* prob = (float*)bh_malloc(sizeof(float) * (size_t)(hp * s * s));
    float* ds = prob ? (float*)bh_malloc(sizeof(float) * (size_t)(hp * s * s)) : nullptr;
    if (!prob || !ds) {
        if (prob) bh_free(prob);
        return BH_ENOMEM;
    }
    int rc = BH_OK;
    for (int64_t h0 = 0; h0 < bh_count && rc == BH_OK; h0 += hp) {
        const int64_t nh = bh_count - h0 < hp ? bh_count - h0 : hp;
        const int64_t off = h0 * s * d;
        const dim3 rows((unsigned)(nh * s));
        rc = bh_gemm(0, 1, s, s, d, q + off, d, k + off, d, prob, s, nullptr, 0, nh);            // S = Q.K^T
        if (rc != BH_OK) break;
        hipLaunchKernelGGL(sdpa_probs_rows_kernel, rows, dim3(kSBlock), 0, stream(), prob, lse + h0 * s, s, scale, causal);
        rc = BH_LAUNCH_CHECK("sdpa_probs_rows_kernel");
        if (rc == BH_OK) rc = bh_gemm(1, 0, s, d, s, prob, s, d_out + off, d, dv + off, d, nullptr, 0, nh);     // dV = P^T.dO
        if (rc == BH_OK) rc = bh_gemm(0, 1, s, s, d, d_out + off, d, v + off, d, ds, s, nullptr, 0, nh);        // dP = dO.V^T
        if (rc != BH_OK) break;
        hipLaunchKernelGGL(sdpa_ds_rows_kernel, rows, dim3(kSBlock), 0, stream(), prob, ds, delta + h0 * s, s, scale);
        rc = BH_LAUNCH_CHECK("sdpa_ds_rows_kernel");
        if (rc == BH_OK) rc = bh_gemm(0, 0, s, d, s, ds, s, k + off, d, dq + off, d, nullptr, 0, nh);           // dQ = dS.K
        if (rc == BH_OK) rc = bh_gemm(1, 0, s, d, s, ds, s, q + off, d, dk + off, d, nullptr, 0, nh);           // dK = dS^T.Q
    }
    bh_free(ds);
    bh_free(prob);
    return rc;
}

}  // namespace bh

using namespace bh;

namespace bh {
// MFMA path (defined in bh_sdpa_mfma.hip); returns BH_EINVAL-free "not applicable" as 1
int sdpa_forward_mfma(const float* q, const float* k, const float* v, float scale, int causal, float* out, float* lse,
                      float* scores_t, int64_t bh_count, int64_t s, int64_t d);
int sdpa_backward_mfma(const float* q, const float* k, const float* v, const float* lse, const float* delta,
                       const float* d_out, const float* scores_t, float scale, int causal, float* dq, float* dk, float* dv,
                       int64_t bh_count, int64_t s, int64_t d);
bool sdpa_scores_shape(int64_t s, int64_t d);
static int g_sdpa_force_general = 0;
}  // namespace bh

extern "C" {

// test hook: 1 forces the row kernels, 2 the GEMM-based path, even where the fused MFMA kernels apply; 0 = heuristic
int bh_sdpa_force_general(int on) {
    g_sdpa_force_general = on;
    return BH_OK;
}

int bh_sdpa_forward(const float* q, const float* k, const float* v, float scale, int causal, float* out, float* lse,
                    float* attn_out, int64_t bh_count, int64_t s, int64_t d) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(bh_count >= 0 && s >= 0 && d > 0, "bad shape");
    if (bh_count == 0 || s == 0) return BH_OK;
    BH_CHECK_ARG(q && k && v && out, "null pointer");
    ProfScope prof(BH_PROF_SDPA_FWD, 4.0 * (double)bh_count * (double)s * (double)s * (double)d);
    if (!g_sdpa_force_general && !attn_out && lse) {
        int rc = sdpa_forward_mfma(q, k, v, scale, causal, out, lse, nullptr, bh_count, s, d);
        if (rc <= 0) return rc;   // 0 done, <0 error, 1 shape not covered
    }
    // from 64 keys on the six products are worth a trip through the matrix cores
    if (g_sdpa_force_general == 2 || (g_sdpa_force_general == 0 && s >= 64 && s <= 16384))
        return sdpa_forward_gemm(q, k, v, scale, causal, out, lse, attn_out, bh_count, s, d);
    BH_CHECK_ARG(bh_count <= 65535, "too many head blocks for the general attention kernel");
    BH_CHECK_ARG(s + d <= kMaxRowFloats, "sequence too long for the general attention kernel");
    const size_t shmem = sizeof(float) * (size_t)(s + d);
    hipLaunchKernelGGL(sdpa_fwd_row_kernel, dim3((unsigned)s, (unsigned)bh_count), dim3(kSBlock), shmem, stream(), q, k, v,
                       scale, causal, out, lse, attn_out, s, d);
    return BH_LAUNCH_CHECK("sdpa_fwd_row_kernel");
}

int bh_sdpa_backward(const float* q, const float* k, const float* v, const float* out, const float* lse, const float* d_out,
                     float scale, int causal, float* dq, float* dk, float* dv, int64_t bh_count, int64_t s, int64_t d) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(bh_count >= 0 && s >= 0 && d > 0, "bad shape");
    if (bh_count == 0 || s == 0) return BH_OK;
    BH_CHECK_ARG(q && k && v && out && lse && d_out && dq && dk && dv, "null pointer");
    ProfScope prof(BH_PROF_SDPA_BWD, 8.0 * (double)bh_count * (double)s * (double)s * (double)d);
    const int64_t rows = bh_count * s;
    float* delta = (float*)bh_malloc(sizeof(float) * (size_t)rows);
    if (!delta) return BH_ENOMEM;
    launch_delta(out, d_out, delta, rows, d);
    int rc = BH_LAUNCH_CHECK("sdpa_delta_kernel");
    if (rc == BH_OK) {
        int done = 1;
        if (!g_sdpa_force_general)
            done = sdpa_backward_mfma(q, k, v, lse, delta, d_out, nullptr, scale, causal, dq, dk, dv, bh_count, s, d);
        // the matrix-core kernel's dQ workspace grows with s^2: when it cannot be had, the GEMM-based path, whose
        // [s, s] matrices are held for a bounded chunk of heads at a time, takes the shape
        if (done == BH_ENOMEM && s >= 64 && s <= 16384) done = 1;
        if (done < 0) rc = done;
        if (done == 1 && (g_sdpa_force_general == 2 || (g_sdpa_force_general == 0 && s >= 64 && s <= 16384))) {
            rc = sdpa_backward_gemm(q, k, v, lse, delta, d_out, scale, causal, dq, dk, dv, bh_count, s, d);
            done = 0;
        }
        if (done == 1) {
            if (2 * s + 2 * d > kMaxRowFloats || bh_count > 65535) {
                bh_free(delta);
                return set_error(BH_EINVAL, "bh_sdpa_backward: sequence too long or too many head blocks for the general attention kernel");
            }
            hipLaunchKernelGGL(sdpa_bwd_dq_row_kernel, dim3((unsigned)s, (unsigned)bh_count), dim3(kSBlock),
                               sizeof(float) * (size_t)(s + 2 * d), stream(), q, k, v, lse, delta, d_out, scale, causal, dq, s,
                               d);
            hipLaunchKernelGGL(sdpa_bwd_dkv_row_kernel, dim3((unsigned)s, (unsigned)bh_count), dim3(kSBlock),
                               sizeof(float) * (size_t)(2 * s + 2 * d), stream(), q, k, v, lse, delta, d_out, scale, causal,
                               dk, dv, s, d);
            rc = BH_LAUNCH_CHECK("sdpa_bwd_row_kernels");
        }
    }
    bh_free(delta);
    return rc;
}

// ---- score cache: the forward pass leaves the scaled scores for the backward pass, as the reference keeps its
// attention weights (src/layers/attention.c:424-431, 1046-1050 cache the [B, nh, S, S] softmax; :584-598 hand it to attention_backward) ----
size_t bh_sdpa_score_cache_bytes(int64_t bh_count, int64_t s, int64_t d) {
    if (bh_count <= 0 || s <= 0 || !sdpa_scores_shape(s, d)) return 0;
    return sizeof(float) * (size_t)bh_count * (size_t)s * (size_t)s;
}

int bh_sdpa_forward_cached(const float* q, const float* k, const float* v, float scale, int causal, float* out, float* lse,
                           float* scores, int64_t bh_count, int64_t s, int64_t d) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(bh_count >= 0 && s >= 0 && d > 0, "bad shape");
    if (bh_count == 0 || s == 0) return BH_OK;
    BH_CHECK_ARG(q && k && v && out && lse && scores, "null pointer");
    BH_CHECK_ARG(bh_sdpa_score_cache_bytes(bh_count, s, d) != 0, "bh_sdpa_forward_cached: head_dim 64 and a sequence length that is a multiple of 128 only");
    ProfScope prof(BH_PROF_SDPA_FWD, 4.0 * (double)bh_count * (double)s * (double)s * (double)d);
    int rc = sdpa_forward_mfma(q, k, v, scale, causal, out, lse, scores, bh_count, s, d);
    if (rc == 1) return set_error(BH_EINVAL, "bh_sdpa_forward_cached: pointers must be 16-byte aligned");
    return rc;
}

int bh_sdpa_backward_cached(const float* q, const float* k, const float* v, const float* out, const float* lse,
                            const float* scores, const float* d_out, float scale, int causal, float* dq, float* dk, float* dv,
                            int64_t bh_count, int64_t s, int64_t d) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(bh_count >= 0 && s >= 0 && d > 0, "bad shape");
    if (bh_count == 0 || s == 0) return BH_OK;
    BH_CHECK_ARG(q && k && v && out && lse && scores && d_out && dq && dk && dv, "null pointer");
    BH_CHECK_ARG(bh_sdpa_score_cache_bytes(bh_count, s, d) != 0, "bh_sdpa_backward_cached: head_dim 64 and a sequence length that is a multiple of 128 only");
    ProfScope prof(BH_PROF_SDPA_BWD, 8.0 * (double)bh_count * (double)s * (double)s * (double)d);
    const int64_t rows = bh_count * s;
    float* delta = (float*)bh_malloc(sizeof(float) * (size_t)rows);
    if (!delta) return BH_ENOMEM;
    launch_delta(out, d_out, delta, rows, d);
    int rc = BH_LAUNCH_CHECK("sdpa_delta_kernel");
    if (rc == BH_OK) {
        rc = sdpa_backward_mfma(q, k, v, lse, delta, d_out, scores, scale, causal, dq, dk, dv, bh_count, s, d);
        if (rc == 1) rc = set_error(BH_EINVAL, "bh_sdpa_backward_cached: pointers must be 16-byte aligned");
    }
    bh_free(delta);
    return rc;
}

}  // extern "C"
