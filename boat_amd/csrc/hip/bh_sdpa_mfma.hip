// bh_sdpa_mfma.hip - attention core on the fp32 matrix cores for head_dim 32, 64 and 128, any sequence length from 32 up.
//
// Same mathematics as the reference's scaled_dot_product_attention_impl / attention_backward
// (src/layers/attention.c:997-1073, 1417-1520) on one [s, 64] block per (batch, head):
//   forward   P = softmax(scale * Q.K^T)  (causal: keys after the query are masked), O = P.V,
//             lse = rowmax + log(rowsum)
//   backward  P = exp(scale*Q.K^T - lse) recomputed; dV = P^T.dO; dP = dO.V^T;
//             dS = P*(dP - delta)*scale with delta = rowsum(dO*O); dQ = dS.K; dK = dS^T.Q
// The [s, s] matrices never exist in memory.
//
// Every contraction is a chain of v_mfma_f32_32x32x2_f32.  Operand roles are chosen so that a product
// leaves the accumulator already in the register layout the next product needs as an input:
//   forward: S^T = K.Q^T puts "query = lane, key = register", which is exactly the B operand of
//            O^T = V^T.P^T; all per-query state (running max, sum, the O^T accumulator) lives in the
//            query's own lane, so the online-softmax rescale is a per-lane multiply.
//   backward: S = Q.K^T and dP = dO.V^T put "key = lane, query = register", the A operand of
//            dV += P^T.dO and dK += dS^T.Q; only dQ = dS.K needs dS with "query = lane", which is one
//            32x32 transpose per wavefront through LDS.  dK/dV accumulate in registers over the loop
//            on query tiles.  dQ of a query tile contracts over the workgroup's 128 keys: the four
//            wavefronts publish dS in LDS and each computes a 16-column slice, written as one partial
//            per (key tile, query tile); a second kernel sums the s/128 partials.  No atomics
//            anywhere, so dQ is deterministic.
// Any order of the contraction index is a valid sum, so the index order inside a chain is whatever the
// register layout gives; operands fetched from LDS use 16-byte reads along head_dim (row stride 68
// floats, conflict free) or 8-byte reads that hand one lane two interleaved output columns.
// The kernels are templates on the head size D: rows of D + 4 floats in LDS, D / 8 groups of four head-dim values per
// half-wavefront in every chain over head_dim, D / 32 interleaved 32-column accumulator tiles wherever head_dim is an
// output index (a lane owns columns NT*lane .. NT*lane + NT - 1).  The reference takes any head_size = hidden / heads
// (src/layers/attention.c:145-146, 393-397); other sizes than these three use the kernels of bh_sdpa.hip.
#include "bh_common.h"

namespace bh {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// N consecutive floats from LDS (the N interleaved head-dim columns a lane owns)
template <int N> struct FloatN;
template <> struct FloatN<1> { float v[1]; __device__ __forceinline__ void load(const float* p) { v[0] = p[0]; }
                               __device__ __forceinline__ void store(float* p) const { p[0] = v[0]; } };
template <> struct FloatN<2> { float v[2]; __device__ __forceinline__ void load(const float* p) { const float2 t = *reinterpret_cast<const float2*>(p); v[0] = t.x; v[1] = t.y; }
                               __device__ __forceinline__ void store(float* p) const { *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]); } };
template <> struct FloatN<4> { float v[4]; __device__ __forceinline__ void load(const float* p) { const float4 t = *reinterpret_cast<const float4*>(p); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
                               __device__ __forceinline__ void store(float* p) const { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); } };
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x2f32((a), (b), (c), 0, 0, 0)

__device__ __forceinline__ floatx16 zero16() {
    floatx16 z;
#pragma unroll
    for (int e = 0; e < 16; e++) z[e] = 0.f;
    return z;
}
// row index inside a 32x32 accumulator tile held by register e of a lane in half `half`
__device__ __forceinline__ int acc_row(int e, int half) { return (e >> 2) * 8 + half * 4 + (e & 3); }

// ------------------------------------------------------------------ forward
// grid (s/128, bh); 4 wavefronts, each owns 32 queries; key/value tiles of KT rows double-buffered in LDS (64 rows; 32
// for head_dim 128, whose 64-row tiles would leave room for one workgroup per compute unit only).
// EMIT: the scaled scores (log2 units, masked pairs -inf) are also written, transposed ([head][key][query]: a key's row
// is what a lane of the backward kernel reads), so that the backward pass can skip the Q.K^T recompute.  Under a causal
// mask the tiles past the diagonal are never visited and their part of the cache stays unwritten.
// The second launch-bounds figure is the least number of wavefronts per SIMD the register allocation must allow: two,
// i.e. two workgroups per compute unit (the LDS allows no more).  Left to itself the compiler gave the causal
// cache-writing form 244 registers and one wavefront per SIMD; the unmasked cache-writing form is the one that runs faster
// with its own allocation (300 against 313 us).
template <int D, int KT, bool CAUSAL, bool RAGGED, bool EMIT = false>   // RAGGED: s is not a multiple of 128; rows past s are clamped on load, masked, never stored
__global__ __launch_bounds__(256, (EMIT && !CAUSAL) ? 1 : 2) void sdpa_fwd_mfma_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                            const float* __restrict__ v, float* __restrict__ out,
                                                            float* __restrict__ lse, int s, int n_heads, float scale_log2e,
                                                            float* __restrict__ scores_t) {
    static_assert(!EMIT || (D == 64 && KT == 64), "the score cache exists for head_dim 64");
    extern __shared__ __align__(16) float smem[];
    constexpr int kD = D, kLd = D + 4;           // LDS row stride in floats (4 pad)
    constexpr int NT = D / 32;                   // 32-row tiles of O^T; a lane's A operand rows are d = NT*lane + tile
    constexpr int G = D / 8;                     // groups of four head-dim values per half-wavefront
    constexpr int ST = KT / 32;                  // 32-key tiles of S^T per key/value tile
    constexpr int TILE = KT * kLd;               // floats per K or V tile in LDS
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, r = lane & 31, half = lane >> 5;
    // Workgroups are handed out in the order of their linear id.  Read it tile-major: all heads' workgroups of one query
    // tile are neighbours, and with a causal mask the query tile with the most keys comes first, so that the short
    // workgroups fill the end of the launch instead of the long ones stretching it.
    const int lin = blockIdx.x;                  // one-dimensional grid of tiles * n_heads workgroups
    const int64_t head = lin % n_heads;
    const int n_qtiles = gridDim.x / n_heads;
    const int bx = CAUSAL ? n_qtiles - 1 - lin / n_heads : lin / n_heads;
    const float* qh = q + head * s * kD;
    const float* kh = k + head * s * kD;
    const float* vh = v + head * s * kD;
    const int q0 = bx * 128 + w * 32;            // first query of this wavefront
    const int my_q = q0 + r;
    const int ld_q = RAGGED ? min(my_q, s - 1) : my_q;

    // this lane's query row, pre-scaled so that scores come out in log2 units: step (g, e) <-> d = 8g + 4*half + e
    float qreg[4 * G];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const float4 t = *reinterpret_cast<const float4*>(qh + (int64_t)ld_q * kD + 8 * g + 4 * half);
        qreg[4 * g + 0] = t.x * scale_log2e;
        qreg[4 * g + 1] = t.y * scale_log2e;
        qreg[4 * g + 2] = t.z * scale_log2e;
        qreg[4 * g + 3] = t.w * scale_log2e;
    }
    float* sc_base = EMIT ? scores_t + ((int64_t)head * s + half * 4) * s + my_q : nullptr;
    floatx16 acc_o[NT];                          // O^T: [d tile][...]; d = NT*row + tile, query = lane
#pragma unroll
    for (int t = 0; t < NT; t++) acc_o[t] = zero16();
    float m_run = -INFINITY, l_run = 0.f;

    int n_tiles = RAGGED ? (s + KT - 1) / KT : s / KT;
    if (CAUSAL) {
        const int last = (bx * 128 + 127) / KT + 1;   // tiles that hold a key <= the last query of the workgroup
        if (last < n_tiles) n_tiles = last;
    }
    // global -> register staging: KT * D / 4 float4 per tile and operand, PER per lane (macros, not lambdas:
    // the staging registers must stay registers)
    constexpr int PER = KT * D / 4 / 256, C4 = D / 4;      // PER is 2 or 4
    float4 kst0, kst1, kst2, kst3, vst0, vst1, vst2, vst3;
#define FWD_LD(i, K, V)                                                                                   \
    if constexpr (PER > (i)) {                                                                            \
        const int idx = tid + (i) * 256, row = idx / C4, c4 = idx % C4;                                   \
        const int grow = RAGGED ? min(jt_ld * KT + row, s - 1) : jt_ld * KT + row;                        \
        K = *reinterpret_cast<const float4*>(kh + (int64_t)grow * kD + c4 * 4);                           \
        V = *reinterpret_cast<const float4*>(vh + (int64_t)grow * kD + c4 * 4);                           \
    }
#define FWD_ST(i, K, V)                                                                                   \
    if constexpr (PER > (i)) {                                                                            \
        const int idx = tid + (i) * 256, row = idx / C4, c4 = idx % C4;                                   \
        *reinterpret_cast<float4*>(st_base + row * kLd + c4 * 4) = K;                                     \
        *reinterpret_cast<float4*>(st_base + TILE + row * kLd + c4 * 4) = V;                              \
    }
#define FWD_STAGE_LOAD(JT) { const int jt_ld = (JT); FWD_LD(0, kst0, vst0) FWD_LD(1, kst1, vst1) FWD_LD(2, kst2, vst2) FWD_LD(3, kst3, vst3) }
#define FWD_STAGE_STORE(BUF) { float* st_base = smem + (BUF) * 2 * TILE; FWD_ST(0, kst0, vst0) FWD_ST(1, kst1, vst1) FWD_ST(2, kst2, vst2) FWD_ST(3, kst3, vst3) }
    FWD_STAGE_LOAD(0)
    FWD_STAGE_STORE(0)
    __syncthreads();

    for (int jt = 0; jt < n_tiles; jt++) {
        const int cur = jt & 1;
        const bool more = jt + 1 < n_tiles;
        if (more) FWD_STAGE_LOAD(jt + 1)
        const float* ks = smem + cur * 2 * TILE;
        const float* vs = ks + TILE;
        // a wavefront whose queries all precede this tile's keys has nothing to add
        if (!CAUSAL || jt * KT <= q0 + 31) {
            floatx16 acc_s[ST];                         // S^T: key = row (tile*32 + acc_row), query = lane
#pragma unroll
            for (int t = 0; t < ST; t++) acc_s[t] = zero16();
            // the wavefront's priority rises with its progress through the tile (scores 1, softmax 2, O^T 3, 0 around the
            // staging and the barrier): of the two wavefronts that share a SIMD the one nearer to its barrier goes first
            // (measured: 287 -> 273 us unmasked, 175 -> 162 us causal at B8 h16 S1024)
            __builtin_amdgcn_s_setprio(1);
            // (the K fragments of group g + 1 are read from LDS before the products of group g are issued, and further down
            // the V rows two steps ahead of the step in work: left to itself the compiler puts a read right in front of its
            // first use, and the wavefront waits out the LDS latency every few products)
            float4 a_next[ST];
#pragma unroll
            for (int t = 0; t < ST; t++) a_next[t] = *reinterpret_cast<const float4*>(ks + (t * 32 + r) * kLd + 4 * half);
#pragma unroll
            for (int g = 0; g < G; g++) {
                float4 a[ST];
#pragma unroll
                for (int t = 0; t < ST; t++) a[t] = a_next[t];
                if (g + 1 < G) {
#pragma unroll
                    for (int t = 0; t < ST; t++) a_next[t] = *reinterpret_cast<const float4*>(ks + (t * 32 + r) * kLd + 8 * (g + 1) + 4 * half);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int t = 0; t < ST; t++) acc_s[t] = MFMA(a[t].x, qreg[4 * g + 0], acc_s[t]);
#pragma unroll
                for (int t = 0; t < ST; t++) acc_s[t] = MFMA(a[t].y, qreg[4 * g + 1], acc_s[t]);
#pragma unroll
                for (int t = 0; t < ST; t++) acc_s[t] = MFMA(a[t].z, qreg[4 * g + 2], acc_s[t]);
#pragma unroll
                for (int t = 0; t < ST; t++) acc_s[t] = MFMA(a[t].w, qreg[4 * g + 3], acc_s[t]);
                __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_s_setprio(2);
            // the first two V rows of the O^T products are on their way while the softmax runs
            constexpr int NSTEP = ST * 16;
            FloatN<NT> v_buf[3];
#pragma unroll
            for (int i = 0; i < 2; i++) v_buf[i].load(vs + ((i / 16) * 32 + acc_row(i % 16, half)) * kLd + NT * r);
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < ST; t++)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    if (CAUSAL || RAGGED) {
                        const int key = jt * KT + t * 32 + acc_row(e, half);
                        if ((CAUSAL && key > my_q) || (RAGGED && key >= s)) acc_s[t][e] = -INFINITY;
                    }
                    mx = fmaxf(mx, acc_s[t][e]);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run, mx);      // finite: key 0 is never masked and tiles are visited in order
            const float alpha = exp2f(m_run - m_new);
            float psum = 0.f;
#pragma unroll
            for (int t = 0; t < ST; t++)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    // the score goes to the cache between the exponentials: row (tile's first key + t*32 + 8*(e/4) + e%4) of
                    // the lane's base, which already holds the lane-dependent part (half, query)
                    if (EMIT) __builtin_nontemporal_store(acc_s[t][e], sc_base + (int64_t)(jt * KT + t * 32 + (e >> 2) * 8 + (e & 3)) * s);
                    const float p = __builtin_amdgcn_exp2f(acc_s[t][e] - m_new);
                    acc_s[t][e] = p;
                    psum += p;
                }
            psum += __shfl_xor(psum, 32, 64);
            l_run = l_run * alpha + psum;
            m_run = m_new;
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc_o[t][e] *= alpha;
            __builtin_amdgcn_s_setprio(3);
            // O^T += V^T . P^T : step e of key tile t uses key row t*32 + acc_row(e, half)
#pragma unroll
            for (int i = 0; i < NSTEP; i++) {
                if (i + 2 < NSTEP) v_buf[(i + 2) % 3].load(vs + (((i + 2) / 16) * 32 + acc_row((i + 2) % 16, half)) * kLd + NT * r);
                __builtin_amdgcn_sched_barrier(0);
                const FloatN<NT> a = v_buf[i % 3];
#pragma unroll
                for (int n = 0; n < NT; n++) acc_o[n] = MFMA(a.v[n], acc_s[i / 16][i % 16], acc_o[n]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __builtin_amdgcn_s_setprio(0);
        if (more) FWD_STAGE_STORE(cur ^ 1)
        __syncthreads();
    }
#undef FWD_LD
#undef FWD_ST
#undef FWD_STAGE_LOAD
#undef FWD_STAGE_STORE

    // O = O^T / l, transposed through LDS so that rows are written whole
    const float inv_l = 1.0f / l_run;
    float* os = smem + w * 32 * kLd;             // 32 x (D + 4) floats per wavefront, tiles are no longer needed
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int e = 0; e < 16; e++) os[r * kLd + NT * acc_row(e, half) + t] = acc_o[t][e] * inv_l;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float* oh = out + head * s * kD;
    constexpr int RPI = 64 / C4;                 // rows one pass of the wavefront stores (C4 lanes per row)
#pragma unroll
    for (int it = 0; it < 32 / RPI; it++) {
        const int row = it * RPI + lane / C4, c4 = lane % C4;
        const float4 val = *reinterpret_cast<const float4*>(os + row * kLd + c4 * 4);
        if (!RAGGED || q0 + row < s) *reinterpret_cast<float4*>(oh + (int64_t)(q0 + row) * kD + c4 * 4) = val;
    }
    if (half == 0 && (!RAGGED || my_q < s)) lse[head * s + my_q] = (m_run + log2f(l_run)) * kLn2;
}

// ----------------------------------------------------------------- backward
// grid (s/128, bh); 4 wavefronts, each owns 32 keys (dK, dV rows) and loops over query tiles of 32.
// Two workgroups fit a CU at head_dim 32 and 64 (71 and 69 KB of LDS, <= 256 registers per lane), so a SIMD always has a second
// wavefront to run while one waits at a barrier or on LDS; head_dim 128 (119 KB of LDS, 128 accumulator registers for
// dK and dV alone) runs one workgroup per compute unit.
// LDS per workgroup: the 128 K rows, one Q tile and one dO tile (refilled through registers between the
// two barriers of an iteration), a [32 queries][128 keys] dS tile, and the tile's lse/delta.
// V never enters LDS: a lane keeps the 32 values of V it feeds to dP = dO.V^T in registers for the
// whole kernel.
// dQ = dS.K of a query tile contracts over all 128 keys of the workgroup, so the four wavefronts first
// publish their dS blocks in LDS and then each computes a [32 queries][D/4 head-dim columns] slice (head_dim 32: a
// [16 queries][16 columns] quarter) with
// v_mfma_f32_16x16x4_f32 (as the transposed product, so that a lane holds four consecutive head-dim columns of a query
// row) and stores it straight to the key tile's partial dQ with 16-byte stores: no cross-wavefront sum.
typedef float floatx4 __attribute__((ext_vector_type(4)));
#define MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32((a), (b), (c), 0, 0, 0)

template <int D, int KW = 4> struct BwdSmem {          // KW: wavefronts (32 keys each) per workgroup
    static constexpr int kLd = D + 4;
    // queries per turn of the loop: 32, or two sub-tiles of 32 at head_dim 32, where a 32-query turn holds half the matrix
    // work of head_dim 64 for the same two barriers, the same staging and the same dQ store
    static constexpr int QSUB = D == 32 ? 2 : 1;
    static constexpr int QROWS = 32 * QSUB;
    static constexpr int KEYS = 32 * KW;                // keys per workgroup
    static constexpr int K = KEYS * kLd;                // K rows of the workgroup
    static constexpr int QT = QROWS * kLd;              // one Q (or dO) tile
    static constexpr int kDsLd = KEYS + 4;              // dS row stride: the workgroup's keys + 4 pad
    // The tiles that are read row by row with constant steps come first: an LDS instruction's immediate offset reaches
    // 64 KB, and whatever lies beyond costs an address register per access (with K first, the 256-key form spent some forty
    // registers on the addresses of its Q and dO rows).
    static constexpr int OFF_Q = 0;
    static constexpr int OFF_DO = OFF_Q + QT;
    static constexpr int OFF_DS = OFF_DO + QT;          // [QROWS][kDsLd]
    static constexpr int OFF_STAT = OFF_DS + QROWS * kDsLd; // [2][QROWS]: lse*log2e, delta
    static constexpr int OFF_K = OFF_STAT + 2 * QROWS;
    static constexpr int TOTAL = OFF_K + K;
};

// RAGGED: rows past s are clamped on load; padding keys are masked, padding queries contribute nothing because their
// dO rows and delta are staged as zeros; stores are guarded
// CACHED: the forward pass left the scaled scores (log2 units, [head][key][query]); S = Q.K^T is read instead of recomputed
template <int D, bool CAUSAL, bool RAGGED, bool CACHED = false, int KW = 4>
__global__ __launch_bounds__(64 * KW, (D == 128 || KW == 8) ? 1 : 2) void sdpa_bwd_mfma_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                               const float* __restrict__ v, const float* __restrict__ lse,
                                                               const float* __restrict__ delta, const float* __restrict__ d_out,
                                                               float* __restrict__ dq_partial, float* __restrict__ dk,
                                                               float* __restrict__ dv, int s, int n_heads, float scale,
                                                               int mirror, const float* __restrict__ scores_t) {
    static_assert(!CACHED || D == 64, "the score cache exists for head_dim 64");
    extern __shared__ __align__(16) float smem[];
    using Smem = BwdSmem<D, KW>;
    constexpr int kD = D, kLd = D + 4, NT = D / 32, G = D / 8, C4 = D / 4, NTHR = 64 * KW, KEYS = 32 * KW;
    constexpr int QSUB = Smem::QSUB, QROWS = Smem::QROWS;
    const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, r = lane & 31, half = lane >> 5;
    const int i16 = lane & 15, kk = lane >> 4;   // operand coordinates of the 16x16x4 products
    // tile-major reading of the linear workgroup id, as in the forward kernel: key tile 0, which meets every query tile
    // under a causal mask, is handed out first for all heads
    // mirror: the second of two launches that share one set of dQ partials.  Workgroup px of the first launch takes key
    // tile px, workgroup px of the second takes key tile tiles-1-px and adds its dQ contribution to the rows its
    // counterpart stored (the stream orders the launches; a partial is read and written by one workgroup per launch).
    const int lin = blockIdx.x;
    const int64_t head = lin % n_heads;
    const int px = lin / n_heads;
    const int bx = mirror ? (s + KEYS - 1) / KEYS - 1 - px : px;
    const float* qh = q + head * s * kD;
    const float* kh = k + head * s * kD;
    const float* vh = v + head * s * kD;
    const float* gh = d_out + head * s * kD;
    const float* lh = lse + head * s;
    const float* dh = delta + head * s;
    // partial dQ of this workgroup: [px][bh][s][64]
    float* dqh = dq_partial + ((int64_t)px * n_heads + head) * s * kD;
    const int kv_wg = bx * KEYS;         // first key of the workgroup
    const int kv0 = kv_wg + w * 32;              // first key of this wavefront
    const float c1 = scale * kLog2e;

    float* kall = smem + Smem::OFF_K;         // all 128 K rows
    float* ks = kall + w * 32 * kLd;             // this wavefront's 32
    float* qs = smem + Smem::OFF_Q;
    float* gs = smem + Smem::OFF_DO;
    float* dsb = smem + Smem::OFF_DS;
    float* st = smem + Smem::OFF_STAT;
    // this wavefront's K rows -> LDS (each lane: D/8 float4)
#pragma unroll
    for (int i = 0; i < G; i++) {
        const int idx = lane + i * 64, row = idx / C4, c4 = idx % C4;
        const int grow = RAGGED ? min(kv0 + row, s - 1) : kv0 + row;
        *reinterpret_cast<float4*>(ks + row * kLd + c4 * 4) = *reinterpret_cast<const float4*>(kh + (int64_t)grow * kD + c4 * 4);
    }
    // this lane's slice of V: key kv0 + r, head-dim 8g + 4*half .. +3 for g = 0..G-1
    float4 vreg[G];
#pragma unroll
    for (int g = 0; g < G; g++)
        vreg[g] = *reinterpret_cast<const float4*>(vh + (int64_t)(RAGGED ? min(kv0 + r, s - 1) : kv0 + r) * kD + 8 * g + 4 * half);

    floatx16 acc_dk[NT], acc_dv[NT];             // [d tile]: key = acc_row, d = NT*lane + tile
#pragma unroll
    for (int t = 0; t < NT; t++) acc_dk[t] = acc_dv[t] = zero16();

    const int n_qt = RAGGED ? (s + QROWS - 1) / QROWS : s / QROWS;
    const int first_qt = CAUSAL ? kv_wg / QROWS : 0;   // earlier query tiles see none of this workgroup's keys
    // their partial dQ rows are zero (a mirror launch leaves them as its counterpart wrote them)
    if (!mirror)
        for (int i = tid; i < first_qt * QROWS * (kD / 4); i += NTHR)
            reinterpret_cast<float4*>(dqh)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    // staging: a Q tile and a dO tile are QROWS * D / 4 float4 each, 2 or 4 per lane and operand
    constexpr int PERQ = QROWS * D / (4 * NTHR);  // 2, 2 or 4 (1, 1 or 2 with eight wavefronts)
    float4 qst0, qst1, qst2, qst3, gst0, gst1, gst2, gst3;
    float stat = 0.f;
#define BWD_LD(i, Q, G_)                                                                                  \
    if constexpr (PERQ > (i)) {                                                                           \
        const int idx = tid + (i) * NTHR, row = idx / C4, c4 = idx % C4;                                  \
        const int grow = RAGGED ? min(qt_ld * QROWS + row, s - 1) : qt_ld * QROWS + row;                  \
        Q = *reinterpret_cast<const float4*>(qh + (int64_t)grow * kD + c4 * 4);                           \
        G_ = *reinterpret_cast<const float4*>(gh + (int64_t)grow * kD + c4 * 4);                          \
        if (RAGGED && qt_ld * QROWS + row >= s) G_ = make_float4(0.f, 0.f, 0.f, 0.f);                     \
    }
#define BWD_ST(i, Q, G_)                                                                                  \
    if constexpr (PERQ > (i)) {                                                                           \
        const int idx = tid + (i) * NTHR, row = idx / C4, c4 = idx % C4;                                  \
        *reinterpret_cast<float4*>(qs + row * kLd + c4 * 4) = Q;                                          \
        *reinterpret_cast<float4*>(gs + row * kLd + c4 * 4) = G_;                                         \
    }
#define BWD_STAGE_LOAD(QT)                                                 \
    {                                                                      \
        const int qt_ld = (QT);                                            \
        BWD_LD(0, qst0, gst0) BWD_LD(1, qst1, gst1) BWD_LD(2, qst2, gst2) BWD_LD(3, qst3, gst3)                    \
        if (tid < QROWS) stat = lh[RAGGED ? min(qt_ld * QROWS + tid, s - 1) : qt_ld * QROWS + tid] * kLog2e;       \
        else if (tid < 2 * QROWS) {                                                                                \
            stat = dh[RAGGED ? min(qt_ld * QROWS + tid - QROWS, s - 1) : qt_ld * QROWS + tid - QROWS];             \
            if (RAGGED && qt_ld * QROWS + tid - QROWS >= s) stat = 0.f;                                            \
        }                                                                                                          \
    }
#define BWD_STAGE_STORE()                                                  \
    {                                                                      \
        BWD_ST(0, qst0, gst0) BWD_ST(1, qst1, gst1) BWD_ST(2, qst2, gst2) BWD_ST(3, qst3, gst3)                    \
        if (tid < 2 * QROWS) st[tid] = stat;                               \
    }
    if (first_qt < n_qt) {
        BWD_STAGE_LOAD(first_qt)
        BWD_STAGE_STORE()
    }
    __syncthreads();

    const int my_key = kv0 + r;
    const bool key_pad = RAGGED && my_key >= s;
    // cached scores of this lane's key: row my_key of the head's [key][query] matrix
    const float* sc_row = CACHED ? scores_t + ((int64_t)head * s + my_key) * s : nullptr;
    // cached scores of the tile in work and of the next one (fetched a whole iteration ahead: a trip to HBM takes longer
    // than the dP chain that could hide it inside one iteration)
    float4 sc_cur[4], sc_next[4];
    if (CACHED) {
#pragma unroll
        for (int j = 0; j < 4; j++) sc_cur[j] = sc_next[j] = *reinterpret_cast<const float4*>(sc_row + first_qt * 32 + 8 * j + 4 * half);
    }
    for (int qt = first_qt; qt < n_qt; qt++) {
        const bool more = qt + 1 < n_qt;
        if (more) BWD_STAGE_LOAD(qt + 1)
        if (CACHED && more) {
#pragma unroll
            for (int j = 0; j < 4; j++) sc_next[j] = *reinterpret_cast<const float4*>(sc_row + (qt + 1) * 32 + 8 * j + 4 * half);
        }
        const int q0 = qt * QROWS;
#pragma unroll
        for (int u = 0; u < QSUB; u++) {                 // the turn's sub-tiles of 32 queries, one after the other
        const int qu = q0 + 32 * u;
        const float* qsu = qs + 32 * u * kLd;
        const float* gsu = gs + 32 * u * kLd;
        const float* stu = st + 32 * u;
        float* dsu = dsb + 32 * u * Smem::kDsLd;
        // (head_dim 128 takes no branch here: with 128 accumulator registers flowing around it the kernel would not fit
        // the register file; the masked pairs of the few tiles it would skip contribute exact zeros)
        if (D == 128 || !CAUSAL || qu + 31 >= kv0) {
            // S = Q.K^T and dP = dO.V^T : query = row (acc_row), key = lane
            floatx16 acc_s = zero16(), acc_dp = zero16();
            // The wavefront's priority rises with its progress through the iteration (1 here, 2 in the row loop, 3 in
            // the dQ product, 0 around the barriers and the staging): of the two wavefronts that share a matrix core the
            // one nearer to its barrier goes first, so its workgroup's other wavefronts wait less.  Measured: 1 % on the
            // recomputing kernel, 3 % on the one that reads the score cache.
            __builtin_amdgcn_s_setprio(1);
            // what the first two rows of the row loop need from LDS is on its way while the score and dP products run
            FloatN<NT> bg_buf[2], bq_buf[2];
            float lse_buf[2], delta_buf[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int row_i = acc_row(i, half);
                bg_buf[i].load(gsu + row_i * kLd + NT * r);
                bq_buf[i].load(qsu + row_i * kLd + NT * r);
                lse_buf[i] = stu[row_i];
                delta_buf[i] = stu[QROWS + row_i];
            }
            if (CACHED) {
                // registers 4j .. 4j+3 are query rows 8j + 4*half .. +3: the four 16-byte pieces fetched an iteration ago
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    acc_s[4 * j + 0] = sc_cur[j].x;
                    acc_s[4 * j + 1] = sc_cur[j].y;
                    acc_s[4 * j + 2] = sc_cur[j].z;
                    acc_s[4 * j + 3] = sc_cur[j].w;
                }
                floatx16 acc_dp2 = zero16();     // two chains, so that a product never waits for its predecessor
                // (the operands of group g + 1 are read from LDS before the products of group g are issued: left to
                // itself the compiler places a read right in front of its first use and the wavefront waits out the
                // LDS latency once per group)
                float4 ag_next = *reinterpret_cast<const float4*>(gsu + r * kLd + 4 * half);
#pragma unroll
                for (int g = 0; g < G; g++) {
                    const float4 ag = ag_next;
                    if (g + 1 < G) ag_next = *reinterpret_cast<const float4*>(gsu + r * kLd + 8 * (g + 1) + 4 * half);
                    const float4 bv = vreg[g];
                    __builtin_amdgcn_sched_barrier(0);
                    acc_dp = MFMA(ag.x, bv.x, acc_dp);
                    acc_dp2 = MFMA(ag.y, bv.y, acc_dp2);
                    acc_dp = MFMA(ag.z, bv.z, acc_dp);
                    acc_dp2 = MFMA(ag.w, bv.w, acc_dp2);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int e = 0; e < 16; e++) acc_dp[e] += acc_dp2[e];
            } else {
                const int off0 = r * kLd + 4 * half;
                float4 aq_next = *reinterpret_cast<const float4*>(qsu + off0);
                float4 bk_next = *reinterpret_cast<const float4*>(ks + off0);
                float4 ag_next = *reinterpret_cast<const float4*>(gsu + off0);
#pragma unroll
                for (int g = 0; g < G; g++) {
                    const float4 aq = aq_next, bk = bk_next, ag = ag_next;
                    if (g + 1 < G) {             // group g + 1's operands, read before group g's products are issued
                        const int off = off0 + 8 * (g + 1);
                        aq_next = *reinterpret_cast<const float4*>(qsu + off);
                        bk_next = *reinterpret_cast<const float4*>(ks + off);
                        ag_next = *reinterpret_cast<const float4*>(gsu + off);
                    }
                    const float4 bv = vreg[g];
                    __builtin_amdgcn_sched_barrier(0);
                    acc_s = MFMA(aq.x, bk.x, acc_s);
                    acc_dp = MFMA(ag.x, bv.x, acc_dp);
                    acc_s = MFMA(aq.y, bk.y, acc_s);
                    acc_dp = MFMA(ag.y, bv.y, acc_dp);
                    acc_s = MFMA(aq.z, bk.z, acc_s);
                    acc_dp = MFMA(ag.z, bv.z, acc_dp);
                    acc_s = MFMA(aq.w, bk.w, acc_s);
                    acc_dp = MFMA(ag.w, bv.w, acc_dp);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            __builtin_amdgcn_s_setprio(2);
            // Row by row: P and dS of query row acc_row(e, half), dS published for the dQ product, then the row's four
            // products dV += P^T.dO, dK += dS^T.Q (step e contracts that query row).  The exponential and the
            // arithmetic of row e + 1 are issued while the matrix core still works on row e.
            // Software pipelined by hand, two rows deep: while the matrix core works on row e, the vector unit computes
            // P and dS of row e + 1 (between the products, not after them) and LDS delivers the operands of row e + 2.
            // In the compiler's own order a row's exponential chain sits in front of its products, and the two
            // wavefronts of a SIMD, which run in step, leave the matrix core idle for that long once per row.
            float p_cur, ds_cur;
            {
                const int row0 = acc_row(0, half);
                p_cur = __builtin_amdgcn_exp2f(CACHED ? acc_s[0] - lse_buf[0] : acc_s[0] * c1 - lse_buf[0]);
                // masked pairs and padding keys carry no probability (padding queries need no mask: their dO rows
                // and delta were staged as zeros, so everything they contribute below is zero)
                if ((CAUSAL && my_key > qu + row0) || key_pad) p_cur = 0.f;
                ds_cur = p_cur * (acc_dp[0] - delta_buf[0]) * scale;
                dsu[row0 * Smem::kDsLd + w * 32 + r] = ds_cur;
            }
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const FloatN<NT> bg = bg_buf[e & 1], bq = bq_buf[e & 1];
                const float p = p_cur, ds = ds_cur;
                __builtin_amdgcn_sched_barrier(0);
                acc_dv[0] = MFMA(p, bg.v[0], acc_dv[0]);
                __builtin_amdgcn_sched_barrier(0);
                if (e + 1 < 16) {
                    const int nrow = acc_row(e + 1, half);
                    p_cur = __builtin_amdgcn_exp2f(CACHED ? acc_s[e + 1] - lse_buf[(e + 1) & 1] : acc_s[e + 1] * c1 - lse_buf[(e + 1) & 1]);
                    if ((CAUSAL && my_key > qu + nrow) || key_pad) p_cur = 0.f;
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int t = 1; t < NT; t++) acc_dv[t] = MFMA(p, bg.v[t], acc_dv[t]);
                acc_dk[0] = MFMA(ds, bq.v[0], acc_dk[0]);
                __builtin_amdgcn_sched_barrier(0);
                if (e + 1 < 16) {
                    const int nrow = acc_row(e + 1, half);
                    ds_cur = p_cur * (acc_dp[e + 1] - delta_buf[(e + 1) & 1]) * scale;
                    dsu[nrow * Smem::kDsLd + w * 32 + r] = ds_cur;
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int t = 1; t < NT; t++) acc_dk[t] = MFMA(ds, bq.v[t], acc_dk[t]);
                if (e + 2 < 16) {                // row e + 2 into the buffers row e has just left
                    const int row2 = acc_row(e + 2, half);
                    bg_buf[e & 1].load(gsu + row2 * kLd + NT * r);
                    bq_buf[e & 1].load(qsu + row2 * kLd + NT * r);
                    lse_buf[e & 1] = stu[row2];
                    delta_buf[e & 1] = stu[QROWS + row2];
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_s_setprio(0);
        } else {
#pragma unroll
            for (int e = 0; e < 16; e++) dsu[acc_row(e, half) * Smem::kDsLd + w * 32 + r] = 0.f;
        }
        }
        __syncthreads();   // dS complete; every wavefront is done with the Q and dO tiles
        if (more) BWD_STAGE_STORE()
        // dQ[32 queries][D] = dS[32][128 keys] . K[128][D] in 16x16 output tiles: a wavefront owns column tiles
        // ct0 .. ct0+NCT-1 of both 16-row tiles (head_dim 32: one column tile of one row tile); lane (i16, kk) reads four
        // consecutive keys of its dS row at once and feeds them to four successive products (the order
        // of the contraction index is free as long as both operands use the same one)
        // (head_dim 32 with its 64-query turns: column tile w & 1 of row tiles w >> 1 and (w >> 1) + 2)
        // (eight wavefronts, head_dim 32 or 64: the turn's eight 16x16 tiles, one each -- column tile w % (D/16) of row
        // tile w / (D/16) -- over 256 keys, as two chains of products over alternate key groups so that a product never
        // waits for its predecessor)
        constexpr bool WIDE = KW == 8;
        static_assert(!WIDE || D == 64 || D == 32, "eight wavefronts per workgroup exist for head_dim 32 and 64");
        constexpr int NCT = WIDE ? 1 : (D >= 64 ? D / 64 : 1), NRT = 2, RSTEP = WIDE ? 0 : (D >= 64 ? 1 : 2);
        const int ct0 = WIDE ? (w % (D / 16)) : (D >= 64 ? w * NCT : (w & 1)), rt0 = WIDE ? (w / (D / 16)) : (D >= 64 ? 0 : (w >> 1));
        floatx4 acc_dq[NCT][NRT];
#pragma unroll
        for (int c = 0; c < NCT; c++)
#pragma unroll
            for (int t = 0; t < NRT; t++) acc_dq[c][t] = floatx4{0.f, 0.f, 0.f, 0.f};
        __builtin_amdgcn_s_setprio(3);
        float* dq_row0 = dqh + (int64_t)(q0 + 16 * rt0 + i16) * kD + 16 * ct0 + 4 * kk;   // tile (c, t) at + 16*RSTEP*t rows, + 16*c columns
        // mirror launch (never under a causal mask): what the first launch stored here, in flight while the products below run
        constexpr int NST = WIDE ? 1 : NRT;     // row tiles this wavefront stores (the two chains of the wide form are one tile)
        float4 old[CAUSAL ? 1 : NCT][CAUSAL ? 1 : NST];
        if constexpr (!CAUSAL) {
#pragma unroll
            for (int c = 0; c < NCT; c++)
#pragma unroll
                for (int t = 0; t < NST; t++) {
                    old[c][t] = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (mirror && (!RAGGED || q0 + 16 * (rt0 + RSTEP * t) + i16 < s))
                        old[c][t] = *reinterpret_cast<const float4*>(dq_row0 + (int64_t)16 * RSTEP * t * kD + 16 * c);
                }
        }
        constexpr int GN = KEYS / 16;           // groups of 16 keys
        const int g_lim = CAUSAL ? min(GN, (q0 + QROWS - kv_wg + 15) / 16) : GN;   // keys past the tile's last query are masked
        for (int g0 = 0; g0 < g_lim; g0 += (WIDE ? 2 : 1)) {
            float4 a[NRT];
#pragma unroll
            for (int t = 0; t < NRT; t++) {
                // the wide form's second chain takes the next key group of the same rows (an odd g_lim: its last turn adds zeros)
                const int g = WIDE ? min(g0 + t, g_lim - 1) : g0;
                a[t] = *reinterpret_cast<const float4*>(dsb + (16 * (rt0 + RSTEP * t) + i16) * Smem::kDsLd + 16 * g + 4 * kk);
                if (WIDE && g0 + t >= g_lim) a[t] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
            float b[WIDE ? 2 : NCT][4];
#pragma unroll
            for (int c = 0; c < (WIDE ? 2 : NCT); c++) {
                const int g = WIDE ? min(g0 + c, g_lim - 1) : g0;
                const float* kb = kall + (16 * g + 4 * kk) * kLd + 16 * (ct0 + (WIDE ? 0 : c)) + i16;
                b[c][0] = kb[0]; b[c][1] = kb[kLd]; b[c][2] = kb[2 * kLd]; b[c][3] = kb[3 * kLd];
            }
            // operands swapped: the product is the transpose dQ^T[d][query], so a lane ends up with four consecutive
            // head-dim columns of one query row and stores them as one 16-byte piece
#pragma unroll
            for (int c = 0; c < NCT; c++)
#pragma unroll
                for (int t = 0; t < NRT; t++) acc_dq[c][t] = MFMA16(b[WIDE ? t : c][0], a[t].x, acc_dq[c][t]);
#pragma unroll
            for (int c = 0; c < NCT; c++)
#pragma unroll
                for (int t = 0; t < NRT; t++) acc_dq[c][t] = MFMA16(b[WIDE ? t : c][1], a[t].y, acc_dq[c][t]);
#pragma unroll
            for (int c = 0; c < NCT; c++)
#pragma unroll
                for (int t = 0; t < NRT; t++) acc_dq[c][t] = MFMA16(b[WIDE ? t : c][2], a[t].z, acc_dq[c][t]);
#pragma unroll
            for (int c = 0; c < NCT; c++)
#pragma unroll
                for (int t = 0; t < NRT; t++) acc_dq[c][t] = MFMA16(b[WIDE ? t : c][3], a[t].w, acc_dq[c][t]);
        }
        __builtin_amdgcn_s_setprio(0);
        if constexpr (WIDE) {
#pragma unroll
            for (int e = 0; e < 4; e++) acc_dq[0][0][e] += acc_dq[0][1][e];
        }
        // accumulator register e of lane (i16, kk) is head-dim column 16*ct + 4*kk + e of query row i16 of the 16-row tile
#pragma unroll
        for (int c = 0; c < NCT; c++)
#pragma unroll
            for (int t = 0; t < NST; t++)
                if (!RAGGED || q0 + 16 * (rt0 + RSTEP * t) + i16 < s) {
                    float4 o = make_float4(acc_dq[c][t][0], acc_dq[c][t][1], acc_dq[c][t][2], acc_dq[c][t][3]);
                    if constexpr (!CAUSAL) {
                        o.x += old[c][t].x; o.y += old[c][t].y; o.z += old[c][t].z; o.w += old[c][t].w;
                    }
                    *reinterpret_cast<float4*>(dq_row0 + (int64_t)16 * RSTEP * t * kD + 16 * c) = o;
                }
        __syncthreads();   // dS tile free again; the next Q and dO tiles are in place
        if (CACHED) {
#pragma unroll
            for (int j = 0; j < 4; j++) sc_cur[j] = sc_next[j];
        }
    }
#undef BWD_LD
#undef BWD_ST
#undef BWD_STAGE_LOAD
#undef BWD_STAGE_STORE

    float* dkh = dk + head * s * kD;
    float* dvh = dv + head * s * kD;
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const int64_t row = kv0 + acc_row(e, half);
        if (RAGGED && row >= s) continue;
        FloatN<NT> ok, ov;
#pragma unroll
        for (int t = 0; t < NT; t++) {
            ok.v[t] = acc_dk[t][e];
            ov.v[t] = acc_dv[t][e];
        }
        ok.store(dkh + row * kD + NT * r);
        ov.store(dvh + row * kD + NT * r);
    }
}

// dq = sum over key tiles of the partials: out[i] = sum_t partial[t][i], float4 per lane, streamed
typedef float f32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void dq_partial_sum_kernel(const float* __restrict__ partial, float* __restrict__ out,
                                                             int64_t n4, int tiles) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    f32x4 acc = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(partial) + i);
    for (int t = 1; t < tiles; t++) acc += __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(partial) + (int64_t)t * n4 + i);
    __builtin_nontemporal_store(acc, reinterpret_cast<f32x4*>(out) + i);
}

// head_dim 32, 64 or 128; any sequence length from 32 up (a length that is not a multiple of 128 takes the kernels' ragged form)
static bool mfma_shape(int64_t s, int64_t d) { return (d == 32 || d == 64 || d == 128) && s >= 32 && s <= (1 << 24); }
// the grids are one-dimensional (tiles * heads workgroups): no 65535 limit on the number of heads
static bool grid_fits(int64_t s, int64_t bh_count) { return ceil_div(s, 128) * bh_count <= 0x7fffffff && bh_count <= 0x7fffffff; }

// shapes whose scaled scores the forward pass can leave for the backward pass: head_dim 64, whole 128-row tiles
bool sdpa_scores_shape(int64_t s, int64_t d) { return d == 64 && mfma_shape(s, d) && s % 128 == 0; }

int g_sdpa_wide = -1;   // test hook: 1 = the backward kernel's 256-key workgroups wherever they exist, 0 = never, -1 = by shape

// one launch of one instantiation; the first call raises the kernel's dynamic LDS limit
template <int D, int KT, bool CAUSAL, bool RAGGED, bool EMIT>
static int fwd_launch(dim3 grid, const float* q, const float* k, const float* v, float* out, float* lse, int s, int heads, float sl,
                      float* scores_t) {
    constexpr size_t lds = sizeof(float) * 2 * 2 * KT * (D + 4);
    static bool attr = false;
    if (!attr) {
        int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&sdpa_fwd_mfma_kernel<D, KT, CAUSAL, RAGGED, EMIT>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), "hipFuncSetAttribute");
        if (rc) return rc;
        attr = true;
    }
    hipLaunchKernelGGL((sdpa_fwd_mfma_kernel<D, KT, CAUSAL, RAGGED, EMIT>), grid, dim3(256), lds, stream(), q, k, v, out, lse, s, heads, sl,
                       scores_t);
    return BH_LAUNCH_CHECK("sdpa_fwd_mfma_kernel");
}
template <int D, int KT>
static int fwd_dispatch(dim3 grid, bool causal, bool ragged, const float* q, const float* k, const float* v, float* out, float* lse, int s,
                        int heads, float sl) {
    if (causal && ragged) return fwd_launch<D, KT, true, true, false>(grid, q, k, v, out, lse, s, heads, sl, nullptr);
    if (causal) return fwd_launch<D, KT, true, false, false>(grid, q, k, v, out, lse, s, heads, sl, nullptr);
    if (ragged) return fwd_launch<D, KT, false, true, false>(grid, q, k, v, out, lse, s, heads, sl, nullptr);
    return fwd_launch<D, KT, false, false, false>(grid, q, k, v, out, lse, s, heads, sl, nullptr);
}

int sdpa_forward_mfma(const float* q, const float* k, const float* v, float scale, int causal, float* out, float* lse,
                      float* scores_t, int64_t bh_count, int64_t s, int64_t d) {
    if (!mfma_shape(s, d) || !grid_fits(s, bh_count)) return 1;
    if (scores_t && !sdpa_scores_shape(s, d)) return 1;
    const auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (!al(q) || !al(k) || !al(v) || !al(out)) return 1;
    dim3 grid((unsigned)(ceil_div(s, 128) * bh_count));
    const bool ragged = s % 128 != 0;
    const float sl = scale * kLog2e;
    const int si = (int)s, hi = (int)bh_count;
    if (scores_t)
        return causal ? fwd_launch<64, 64, true, false, true>(grid, q, k, v, out, lse, si, hi, sl, scores_t)
                      : fwd_launch<64, 64, false, false, true>(grid, q, k, v, out, lse, si, hi, sl, scores_t);
    if (d == 32) return fwd_dispatch<32, 64>(grid, causal != 0, ragged, q, k, v, out, lse, si, hi, sl);
    if (d == 64) return fwd_dispatch<64, 64>(grid, causal != 0, ragged, q, k, v, out, lse, si, hi, sl);
    return fwd_dispatch<128, 32>(grid, causal != 0, ragged, q, k, v, out, lse, si, hi, sl);
}

template <int D, bool CAUSAL, bool RAGGED, bool CACHED, int KW = 4>
static int bwd_launch(int64_t grid, int mirror, const float* q, const float* k, const float* v, const float* lse, const float* delta,
                      const float* d_out, float* partial, float* dk, float* dv, int s, int heads, float scale, const float* scores_t) {
    constexpr size_t lds = sizeof(float) * BwdSmem<D, KW>::TOTAL;
    static bool attr = false;
    if (!attr) {
        int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&sdpa_bwd_mfma_kernel<D, CAUSAL, RAGGED, CACHED, KW>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), "hipFuncSetAttribute");
        if (rc) return rc;
        attr = true;
    }
    hipLaunchKernelGGL((sdpa_bwd_mfma_kernel<D, CAUSAL, RAGGED, CACHED, KW>), dim3((unsigned)grid), dim3(64 * KW), lds, stream(), q, k, v, lse, delta,
                       d_out, partial, dk, dv, s, heads, scale, mirror, scores_t);
    return BH_LAUNCH_CHECK("sdpa_bwd_mfma_kernel");
}
template <int D, int KW = 4>
static int bwd_dispatch(int64_t grid, int mirror, bool causal, bool ragged, const float* q, const float* k, const float* v, const float* lse,
                        const float* delta, const float* d_out, float* partial, float* dk, float* dv, int s, int heads, float scale) {
    if (causal && ragged) return bwd_launch<D, true, true, false, KW>(grid, mirror, q, k, v, lse, delta, d_out, partial, dk, dv, s, heads, scale, nullptr);
    if (causal) return bwd_launch<D, true, false, false, KW>(grid, mirror, q, k, v, lse, delta, d_out, partial, dk, dv, s, heads, scale, nullptr);
    if (ragged) return bwd_launch<D, false, true, false, KW>(grid, mirror, q, k, v, lse, delta, d_out, partial, dk, dv, s, heads, scale, nullptr);
    return bwd_launch<D, false, false, false, KW>(grid, mirror, q, k, v, lse, delta, d_out, partial, dk, dv, s, heads, scale, nullptr);
}

int sdpa_backward_mfma(const float* q, const float* k, const float* v, const float* lse, const float* delta,
                       const float* d_out, const float* scores_t, float scale, int causal, float* dq, float* dk, float* dv,
                       int64_t bh_count, int64_t s, int64_t d) {
    if (!mfma_shape(s, d) || !grid_fits(s, bh_count)) return 1;
    if (scores_t && !sdpa_scores_shape(s, d)) return 1;
    const auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (!al(q) || !al(k) || !al(v) || !al(d_out) || !al(dq) || !al(dk) || !al(dv)) return 1;
    // Eight wavefronts and 256 keys per workgroup, one workgroup per compute unit (head_dim 32 and 64; the score-cache
    // kernel only unmasked and over whole 256-key tiles): half as many dQ partials to write, add to and fold -- none at
    // all when two mirrored launches cover the sequence, as at 512 keys -- and one dQ tile per wavefront and turn.  It
    // pays when the launch still fills the chip twice over (B8 h16 S1024 D64: 0.684 against 0.699 ms; 256 heads of
    // S512 with the score cache: 0.319 against 0.336 ms); with fewer workgroups the 128-key form's finer grain wins (32
    // heads of S1024: 0.217 against 0.333 ms).
    const bool wide_exists = (d == 64 || d == 32) && (!scores_t || (s % 256 == 0 && !causal));
    const bool wide = wide_exists && (g_sdpa_wide > 0 || (g_sdpa_wide < 0 && ceil_div(s, 256) * bh_count >= 2 * (int64_t)bh_device_cu_count()));
    const int keys = wide ? 256 : 128;
    const int key_tiles = (int)ceil_div(s, keys);
    // Two launches that share one set of dQ partials (the second takes the key tiles in mirrored order and adds to what
    // the first stored) when each launch still fills every compute unit with the workgroups it can hold (two; one at
    // head_dim 128): half as many partials to write and fold, and each launch is a single round of workgroups that start
    // and finish together instead of two rounds whose second runs out unevenly.  Not under a causal mask, where a launch
    // would hold tiles of unequal work.
    const int64_t resident = ((d == 128 || wide) ? 1 : 2) * (int64_t)bh_device_cu_count();
    const bool two_launches = !causal && key_tiles >= 2 && (int64_t)(key_tiles / 2) * bh_count >= resident;
    const int tiles = two_launches ? (key_tiles + 1) / 2 : key_tiles;      // dQ partials per head
    const bool ragged = s % keys != 0;
    const int64_t n = bh_count * s * d;
    float* partial = tiles > 1 ? (float*)bh_malloc(sizeof(float) * (size_t)(tiles * n)) : dq;   // one partial: dq itself
    if (!partial) return BH_ENOMEM;
    const int si = (int)s, hi = (int)bh_count;
    int rc = BH_OK;
    for (int pass = 0; pass < (two_launches ? 2 : 1) && rc == BH_OK; pass++) {
        const int64_t grid = (pass == 0 ? tiles : key_tiles / 2) * bh_count;
        if (scores_t && wide)
            rc = bwd_launch<64, false, false, true, 8>(grid, pass, q, k, v, lse, delta, d_out, partial, dk, dv, si, hi, scale, scores_t);
        else if (scores_t)
            rc = causal ? bwd_launch<64, true, false, true>(grid, pass, q, k, v, lse, delta, d_out, partial, dk, dv, si, hi, scale, scores_t)
                        : bwd_launch<64, false, false, true>(grid, pass, q, k, v, lse, delta, d_out, partial, dk, dv, si, hi, scale, scores_t);
        else if (wide && d == 32) rc = bwd_dispatch<32, 8>(grid, pass, causal != 0, ragged, q, k, v, lse, delta, d_out, partial, dk, dv, si, hi, scale);
        else if (wide) rc = bwd_dispatch<64, 8>(grid, pass, causal != 0, ragged, q, k, v, lse, delta, d_out, partial, dk, dv, si, hi, scale);
        else if (d == 32) rc = bwd_dispatch<32>(grid, pass, causal != 0, ragged, q, k, v, lse, delta, d_out, partial, dk, dv, si, hi, scale);
        else if (d == 64) rc = bwd_dispatch<64>(grid, pass, causal != 0, ragged, q, k, v, lse, delta, d_out, partial, dk, dv, si, hi, scale);
        else rc = bwd_dispatch<128>(grid, pass, causal != 0, ragged, q, k, v, lse, delta, d_out, partial, dk, dv, si, hi, scale);
    }
    if (tiles > 1) {
        if (rc == BH_OK) {
            const int64_t n4 = n / 4;
            hipLaunchKernelGGL(dq_partial_sum_kernel, dim3((unsigned)ceil_div(n4, 256)), dim3(256), 0, stream(), partial, dq, n4, tiles);
            rc = BH_LAUNCH_CHECK("dq_partial_sum_kernel");
        }
        bh_free(partial);
    }
    return rc;
}

}  // namespace bh

// test/benchmark hook: 1 = 256-key workgroups in the attention backward wherever that form exists, 0 = never, -1 = by shape
extern "C" int bh_sdpa_force_wide(int mode) {
    bh::g_sdpa_wide = mode;
    return BH_OK;
}
