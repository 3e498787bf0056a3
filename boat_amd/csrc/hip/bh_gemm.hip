// bh_gemm.hip - fp32 GEMM on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32).
//
// Replaces boat_matmul (src/ops/linear.c:12-170) together with the materialised
// boat_transpose calls (src/ops/linear.c:238-406) that the reference's backward passes
// wrap around it:
//   dense forward   Y  = X.W (+ b)      src/layers/dense.c:150-185
//   dense backward  dX = dY.W^T         src/layers/dense.c:219-228
//                   dW += X^T.dY        src/layers/dense.c:230-261
//   attention projections and their backward, src/layers/attention.c:247-308, 1186-1285
// Transposed operands are read in place: an operand is either "k-contiguous" (the
// contraction index is the fast index in memory) or "row-contiguous" (the output index is
// the fast one); each has its own LDS layout and fragment read, so no transpose is ever
// written to memory.
//
// Tiling (wave64, gfx950):
//   macro tile BM x BN per workgroup (256x256, 256x128, 128x256 or 128x128), k-tile BK=16, LDS double buffered, next k-tile
//   prefetched into registers while the current one feeds the MFMAs (one barrier per k-tile)
//   each wavefront owns a (32*TM) x (32*TN) block = TM*TN accumulators of 16 VGPRs
//   A-fragment for MFMA step s comes from one ds_read_b128 / ds_read_b64:
//     k-contiguous operand   [rows][BK+4] : lane (r, half) reads k = kb+4*half .. +3 of row r;
//                                            element s feeds step s (any k order is a valid sum)
//     row-contiguous operand [BK][rows+4] : lane (r, half) reads rows T*r .. T*r+T-1 of k-row
//                                            kb+4*half+s; element t feeds tile t, i.e. tile t
//                                            owns the interleaved rows {base + T*i + t}
//   workgroup -> tile map is XCD-aware: consecutive tiles of a group land on the same XCD
//   (same L2), and tiles are walked in groups of 8 tile-rows.
// Small or unaligned problems take a bounds-checked LDS-tiled fallback kernel; problems with a
// small output and a long contraction (weight gradients) are split along K into a workspace and
// folded by a second kernel (deterministic, no atomics).
#include "bh_common.h"

#include <stdint.h>
#include <type_traits>

namespace bh {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kBK = 16;
constexpr int kPad = 4;

template <int T> struct FragT;             // T consecutive floats from LDS
template <> struct FragT<1> { float v[1]; __device__ __forceinline__ void load(const float* p) { v[0] = p[0]; } };
template <> struct FragT<2> { float v[2]; __device__ __forceinline__ void load(const float* p) { float2 t = *reinterpret_cast<const float2*>(p); v[0] = t.x; v[1] = t.y; } };
template <> struct FragT<4> { float v[4]; __device__ __forceinline__ void load(const float* p) { float4 t = *reinterpret_cast<const float4*>(p); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; } };

template <int BM_, int BN_, int WGM_, int WGN_>
struct GemmCfg {
    static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
    static constexpr int NT = WGM * WGN * 64;
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int TM = WM / 32, TN = WN / 32;
};

// LDS floats for one operand tile of R rows
template <bool KC, int R> struct TileShape {
    static constexpr int ld = KC ? (kBK + kPad) : (R + kPad);
    static constexpr int floats = KC ? R * ld : kBK * ld;
};

struct GemmArgs {
    const float* a; const float* b; float* c; const float* bias;
    int64_t m, n, k;
    int64_t lda, ldb, ldc;
    int64_t stride_a, stride_b, stride_c;   // per batch
    int accumulate;
    int k_splits;        // >1: write partials to c (workspace [split][batch][m][n], ldc == n)
    int64_t k_per_split; // multiple of kBK
    int tiles_m, tiles_n;
};

// Operand tables of a grouped launch (up to kMaxGroups problems of one shape).  Two forms:
//   k_segments == 1: blockIdx.y picks the group: c[g] (+)= op(a[g]) . op(b[g]) (+ bias[g])
//   k_segments  > 1: ONE product whose contraction runs over the operand pairs in turn,
//                    c[0] (+)= sum_s op(a[s]) . op(b[s]) (+ bias[0]), seg_k of the contraction per pair
// (the three input projections of self-attention: one launch for the forward products, one for the three weight
// gradients, one contraction for the summed input gradient dQ.Wq^T + dK.Wk^T + dV.Wv^T)
constexpr int kMaxGroups = 4;
constexpr int kMaxSegments = 3;
struct GemmTab {
    const float* a[kMaxGroups];
    const float* b[kMaxGroups];
    float* c[kMaxGroups];
    const float* bias[kMaxGroups];
    int k_segments;
    int64_t seg_k;       // multiple of 2 * kBK
};

// Global -> registers for one operand tile.  KC: tile is [R rows][kBK], row r at base + r*ld.
// !KC: tile is [kBK k-rows][R], k-row kk at base + kk*ld.
template <bool KC, int R, int NT>
struct TileLoader {
    static constexpr int F4 = R * kBK / 4;
    static constexpr int PER = (F4 + NT - 1) / NT;
    float4 reg[PER];

    __device__ __forceinline__ void load(const float* __restrict__ base, int64_t ld, int64_t row0, int64_t row_lim,
                                         int64_t k0, int64_t k_lim, int tid) {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int idx = tid + i * NT;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (F4 % NT == 0 || idx < F4) {
                if (KC) {
                    const int r = idx / (kBK / 4), kq = idx % (kBK / 4);
                    const int64_t gr = row0 + r, gk = k0 + kq * 4;
                    if (gr < row_lim && gk < k_lim) v = *reinterpret_cast<const float4*>(base + gr * ld + gk);
                } else {
                    const int kk = idx / (R / 4), c4 = idx % (R / 4);
                    const int64_t gk = k0 + kk, gr = row0 + c4 * 4;
                    if (gk < k_lim && gr < row_lim) v = *reinterpret_cast<const float4*>(base + gk * ld + gr);
                }
            }
            reg[i] = v;
        }
    }
    __device__ __forceinline__ void store(float* lds, int tid) const {
        constexpr int ld = TileShape<KC, R>::ld;
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int idx = tid + i * NT;
            if (F4 % NT == 0 || idx < F4) {
                if (KC) {
                    const int r = idx / (kBK / 4), kq = idx % (kBK / 4);
                    *reinterpret_cast<float4*>(lds + r * ld + kq * 4) = reg[i];
                } else {
                    const int kk = idx / (R / 4), c4 = idx % (R / 4);
                    *reinterpret_cast<float4*>(lds + kk * ld + c4 * 4) = reg[i];
                }
            }
        }
    }
};

// Fragments of one operand for one k-group (8 k values = 4 MFMA steps), T tiles.
template <bool KC, int R, int T>
struct Frags {
    float v[4][T];   // [step][tile]
    __device__ __forceinline__ void load(const float* lds, int wave_off, int kb, int r, int half) {
        constexpr int ld = TileShape<KC, R>::ld;
        if (KC) {
#pragma unroll
            for (int t = 0; t < T; t++) {
                float4 q = *reinterpret_cast<const float4*>(lds + (wave_off + t * 32 + r) * ld + kb + 4 * half);
                v[0][t] = q.x; v[1][t] = q.y; v[2][t] = q.z; v[3][t] = q.w;
            }
        } else {
#pragma unroll
            for (int s = 0; s < 4; s++) {
                FragT<T> f;
                f.load(lds + (kb + 4 * half + s) * ld + wave_off + T * r);
#pragma unroll
                for (int t = 0; t < T; t++) v[s][t] = f.v[t];
            }
        }
    }
};


// ---- direct-to-LDS operand path (global_load_lds_dwordx4: no staging registers, no ds_write) ----
// One instruction moves 1 KB: lane l supplies the address of its 16 bytes, and the 64 pieces land contiguously at the
// LDS address in M0.  A k-tile (kBK = 16) of an R-row operand is R/16 such blocks:
//   k-contiguous operand   block = 16 rows x 16 k.  Row stride is 16 floats with no room for padding, so the four
//                          16-byte chunks of a row are swizzled instead: chunk q of row r sits in slot q ^ ((r >> 2) & 3),
//                          which makes the fragment reads of 16 consecutive rows hit 16 different bank groups.
//   row-contiguous operand block = 256 consecutive floats of k-rows (one k-row for R = 256, two for R = 128, four for R = 64), blocks
//                          padded by 4 floats so that the two half-wavefronts of a fragment read use different banks.
// Rows or columns past the matrix edge are clamped to the last valid ones (their products are never stored); the
// contraction range must be a multiple of kBK because nothing zero-fills a k tail.
typedef __attribute__((address_space(3))) void* lds_ptr_t;

template <bool KC, int R> struct DirectTile {
    static_assert(R == 64 || R == 128 || R == 256, "operand tiles of 64, 128 or 256 rows");
    static constexpr int blocks = R / 16;
    static constexpr int block_stride = KC ? 256 : 260;   // floats
    static constexpr int floats = blocks * block_stride;
};

__device__ __forceinline__ void load_block_to_lds(const float* base, unsigned lane_byte_offset, unsigned lds_byte_addr) {
    // M0 carries the LDS address of the block.  It is a reserved register that the compiler neither allocates nor keeps
    // live in these kernels (no s_movrel / s_sendmsg / GWS), so nothing of its own is disturbed.
    // The address is a scalar base (the same for the whole workgroup, advanced from k-tile to k-tile by scalar
    // instructions) plus a 32-bit byte offset per lane that never changes: the main loop spends no vector instruction
    // on addresses -- it has no issue slot to spare between two matrix instructions.
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 ::"v"(lane_byte_offset), "s"(base), "s"(lds_byte_addr) : "memory");
}
__device__ __forceinline__ void wait_direct_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <bool KC, int R, int NW>
struct DirectLoader {
    static constexpr int PER = DirectTile<KC, R>::blocks / NW;   // blocks per wavefront and k-tile
    static_assert(DirectTile<KC, R>::blocks % NW == 0, "blocks must divide among the wavefronts");
    const float* base;      // the workgroup's tile at the next k-tile to issue (the same for every lane)
    unsigned off[PER];      // this lane's byte offset from base (the host keeps leading dimensions below 2^22, so 256 rows fit)
    unsigned dst[PER];      // LDS byte address inside stage 0
    int64_t step;           // floats from one k-tile to the next

    __device__ __forceinline__ void init(const float* mat, int64_t ld, int64_t row0, int64_t row_lim, int64_t k_begin,
                                         const float* lds_tile, int wave, int lane) {
        step = KC ? kBK : kBK * ld;
        base = KC ? mat + row0 * ld + k_begin : mat + k_begin * ld;
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const int blk = wave + j * NW;
            if (KC) {
                int64_t row = row0 + 16 * blk + (lane >> 2);
                if (row > row_lim - 1) row = row_lim - 1;
                const int chunk = (lane & 3) ^ ((lane >> 4) & 3);
                off[j] = (unsigned)(((row - row0) * ld + 4 * chunk) * (int64_t)sizeof(float));
            } else {
                const int krow = R == 256 ? blk : R == 128 ? 2 * blk + (lane >> 5) : 4 * blk + (lane >> 4);
                int64_t col = row0 + 4 * (R == 256 ? lane : R == 128 ? (lane & 31) : (lane & 15));
                if (col > row_lim - 4) col = row_lim - 4;
                off[j] = (unsigned)((krow * ld + col) * (int64_t)sizeof(float));
            }
            const unsigned addr = (unsigned)(uintptr_t)(lds_ptr_t)(lds_tile + blk * DirectTile<KC, R>::block_stride);
            dst[j] = __builtin_amdgcn_readfirstlane(addr);
        }
    }
    // continue at the start (k = 0) of another matrix of the same shape: the lane offsets stay what they are
    __device__ __forceinline__ void rebase(const float* mat, int64_t ld, int64_t row0) { base = KC ? mat + row0 * ld : mat; }
    // issue this wavefront's blocks of the next k-tile into the stage at byte offset stage_bytes
    __device__ __forceinline__ void issue(unsigned stage_bytes) {
#pragma unroll
        for (int j = 0; j < PER; j++) load_block_to_lds(base, off[j], dst[j] + stage_bytes);
        base += step;
    }
};

// Fragments from a direct-to-LDS tile: same register meaning as Frags.
template <bool KC, int R, int T>
struct DirectFrags {
    float v[4][T];
    __device__ __forceinline__ void load(const float* lds, int wave_off, int kb, int r, int half) {
        if (KC) {
            const int slot = ((kb >> 2) + half) ^ ((r >> 2) & 3);
#pragma unroll
            for (int t = 0; t < T; t++) {
                float4 q = *reinterpret_cast<const float4*>(lds + (wave_off + t * 32 + r) * 16 + slot * 4);
                v[0][t] = q.x; v[1][t] = q.y; v[2][t] = q.z; v[3][t] = q.w;
            }
        } else {
#pragma unroll
            for (int s = 0; s < 4; s++) {
                const int kk = kb + 4 * half + s;
                FragT<T> f;
                f.load(lds + (R == 256 ? kk * 260 : R == 128 ? (kk >> 1) * 260 + (kk & 1) * 128 : (kk >> 2) * 260 + (kk & 3) * 64) + wave_off + T * r);
#pragma unroll
                for (int t = 0; t < T; t++) v[s][t] = f.v[t];
            }
        }
    }
};

// (the four-wavefront tile is held to the registers of three workgroups per compute unit -- 146, its accumulators among
// them -- which its 33 KB of LDS allow as well: a third resident workgroup is worth 0.3-0.9 % on the block's shapes)
template <typename Cfg, bool A_KC, bool B_KC, bool DIRECT, int KT = 1, bool TAB = false>   // KT: k-tiles per LDS stage (and per barrier); TAB: operands from tables
__global__ __launch_bounds__(Cfg::NT, Cfg::NT == 256 ? 3 : 1) void gemm_mfma_kernel(GemmArgs g, GemmTab t) {
    static_assert(!TAB || DIRECT, "grouped launches use the direct-to-LDS loaders");
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NT = Cfg::NT, TM = Cfg::TM, TN = Cfg::TN;
    constexpr int A_FLOATS = DIRECT ? DirectTile<A_KC, BM>::floats : TileShape<A_KC, BM>::floats;
    constexpr int B_FLOATS = DIRECT ? DirectTile<B_KC, BN>::floats : TileShape<B_KC, BN>::floats;
    extern __shared__ __align__(16) float smem[];
    constexpr int STAGE = A_FLOATS + B_FLOATS;   // stage `cur` holds A at smem+cur*STAGE, B right after it

    // ---- workgroup -> (tile_m, tile_n): XCD-aware, grouped ----
    const int total = g.tiles_m * g.tiles_n;
    int pid = blockIdx.x;
    if (total % kNumXcd == 0) pid = (pid % kNumXcd) * (total / kNumXcd) + pid / kNumXcd;
    constexpr int GROUP = 8;
    const int per_group = GROUP * g.tiles_n;
    const int group_id = pid / per_group;
    const int first_m = group_id * GROUP;
    const int gsz = min(g.tiles_m - first_m, GROUP);
    const int tile_m = first_m + (pid % per_group) % gsz;
    const int tile_n = (pid % per_group) / gsz;

    const int batch = blockIdx.y;
    const int split = blockIdx.z;
    const int64_t k_begin = (int64_t)split * g.k_per_split;
    int64_t k_end = g.k_splits > 1 ? k_begin + g.k_per_split : g.k;
    if (k_end > g.k) k_end = g.k;

    const float* A = TAB ? t.a[batch] : g.a + (int64_t)batch * g.stride_a;
    const float* B = TAB ? t.b[batch] : g.b + (int64_t)batch * g.stride_b;
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    // a segmented contraction: the operand pairs that follow the first, picked by scalar selects when the issue stream
    // crosses into the next segment (blockIdx.y is 0 then)
    const float* A1 = TAB ? t.a[1] : nullptr;
    const float* A2 = TAB ? t.a[2] : nullptr;
    const float* B1 = TAB ? t.b[1] : nullptr;
    const float* B2 = TAB ? t.b[2] : nullptr;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave / Cfg::WGN, wn = wave % Cfg::WGN;
    const int r = lane & 31, half = lane >> 5;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    if constexpr (DIRECT && KT == 2) {
        // Two k-tiles per stage and one barrier per pair: the same pipeline as below with the barrier (where every
        // matrix core of the workgroup drains) paid once per 32 k instead of once per 16.  The contraction range is a
        // multiple of 32 here (the host checks), so every stage is whole.
        constexpr int NW = NT / 64;
        constexpr unsigned TILE_BYTES = (unsigned)(STAGE * sizeof(float));
        DirectLoader<A_KC, BM, NW> da;
        DirectLoader<B_KC, BN, NW> db;
        da.init(A, g.lda, m0, g.m, k_begin, smem, wave, lane);
        db.init(B, g.ldb, n0, g.n, k_begin, smem + A_FLOATS, wave, lane);
        const int pairs = (int)((k_end - k_begin) / (2 * kBK));
        DirectFrags<A_KC, BM, TM> fa0, fa1;
        DirectFrags<B_KC, BN, TN> fb0, fb1;
        auto products = [&](const DirectFrags<A_KC, BM, TM>& fa, const DirectFrags<B_KC, BN, TN>& fb) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 4; s++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa.v[s][i], fb.v[s][j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        };
        int seg = 0, seg_left = TAB && t.k_segments > 1 ? (int)(t.seg_k / (2 * kBK)) : 0x7fffffff;   // pairs to issue before the next segment
        auto issue_pair = [&](unsigned stage) {     // the next two k-tiles of this wavefront's blocks into stage `stage`
            da.issue(stage * 2 * TILE_BYTES);
            db.issue(stage * 2 * TILE_BYTES);
            da.issue(stage * 2 * TILE_BYTES + TILE_BYTES);
            db.issue(stage * 2 * TILE_BYTES + TILE_BYTES);
            if constexpr (TAB) {
                if (--seg_left == 0) {
                    seg++;
                    seg_left = (int)(t.seg_k / (2 * kBK));
                    da.rebase(seg == 1 ? A1 : A2, g.lda, m0);
                    db.rebase(seg == 1 ? B1 : B2, g.ldb, n0);
                }
            }
        };
        if (pairs > 0) issue_pair(0);
        if (pairs > 1) issue_pair(1);
        wait_direct_loads();
        __syncthreads();
        if (pairs > 0) {
            fa0.load(smem, wm * Cfg::WM, 0, r, half);
            fb0.load(smem + A_FLOATS, wn * Cfg::WN, 0, r, half);
        }
        // A wavefront whose load cannot be queued issues nothing else, matrix instructions included, and eight
        // wavefronts that issue their 64 KB of loads at the same point queue behind each other for about a thousand
        // cycles per pair.  So only half of them issue right after the barrier; the other half issue the same pair one
        // group of products later, into the stage that barrier freed (8192x4096x4096: 1.94 -> 1.89 ms, the same bits).
        // More than two issue points were measured and are slower.
        const bool late = NW >= 8 && __builtin_amdgcn_readfirstlane(wave) >= NW / 2;
        // The stage a pair sits in is a compile-time constant of its iteration (two iterations per trip of the loop), so
        // every fragment address is one of a few per-lane registers plus an immediate offset: no vector instruction for
        // addresses between the matrix instructions.
        const auto iteration = [&](auto stage_const, int p) {
            constexpr int cur = decltype(stage_const)::value;
            const float* sa0 = smem + cur * 2 * STAGE;     // first k-tile of the pair: A, then B
            const float* sa1 = sa0 + STAGE;                // second k-tile
            fa1.load(sa0, wm * Cfg::WM, 8, r, half);
            fb1.load(sa0 + A_FLOATS, wn * Cfg::WN, 8, r, half);
            products(fa0, fb0);
            if (late && p >= 1 && p + 1 < pairs) issue_pair((unsigned)(cur ^ 1));     // pair p+1; pairs 0 and 1 were issued up front
            fa0.load(sa1, wm * Cfg::WM, 0, r, half);
            fb0.load(sa1 + A_FLOATS, wn * Cfg::WN, 0, r, half);
            products(fa1, fb1);
            fa1.load(sa1, wm * Cfg::WM, 8, r, half);
            fb1.load(sa1 + A_FLOATS, wn * Cfg::WN, 8, r, half);
            products(fa0, fb0);
            wait_direct_loads();       // pair p+1, issued a whole pair (or, by the late half, two groups of products) ago
            __syncthreads();           // ... is visible to everyone, and everyone has the last fragments of stage cur in registers
            if (!late && p + 2 < pairs) issue_pair((unsigned)cur);
            if (p + 1 < pairs) {
                const float* na = smem + (cur ^ 1) * 2 * STAGE;
                fa0.load(na, wm * Cfg::WM, 0, r, half);
                fb0.load(na + A_FLOATS, wn * Cfg::WN, 0, r, half);
            }
            products(fa1, fb1);
        };
        int p = 0;
        for (; p + 1 < pairs; p += 2) {
            iteration(std::integral_constant<int, 0>{}, p);
            iteration(std::integral_constant<int, 1>{}, p + 1);
        }
        if (p < pairs) iteration(std::integral_constant<int, 0>{}, p);
    } else if constexpr (DIRECT) {
        // tile kt+1 streams straight into the other LDS stage while tile kt feeds the MFMAs; the wait for this
        // wavefront's own loads and the barrier at the end of the k-tile publish it to the workgroup
        constexpr int NW = NT / 64;
        DirectLoader<A_KC, BM, NW> da;
        DirectLoader<B_KC, BN, NW> db;
        da.init(A, g.lda, m0, g.m, k_begin, smem, wave, lane);
        db.init(B, g.ldb, n0, g.n, k_begin, smem + A_FLOATS, wave, lane);
        const int kt_count = (int)((k_end - k_begin) / kBK);
        // Two tiles are in flight ahead of the arithmetic and the fragments are software pipelined across the one
        // barrier of a k-tile, which sits between its two halves: the fragments of the second half are read while the
        // first half's products run, those of the next tile's first half right after the barrier while the second
        // half's products run, so no product ever waits for an LDS read it has just issued.
        DirectFrags<A_KC, BM, TM> fa0, fa1;
        DirectFrags<B_KC, BN, TN> fb0, fb1;
        int seg = 0, seg_left = TAB && t.k_segments > 1 ? (int)(t.seg_k / kBK) : 0x7fffffff;   // k-tiles to issue before the next segment
        const auto issue_tile = [&](unsigned stage_bytes) {
            da.issue(stage_bytes);
            db.issue(stage_bytes);
            if constexpr (TAB) {
                if (--seg_left == 0) {
                    seg++;
                    seg_left = (int)(t.seg_k / kBK);
                    da.rebase(seg == 1 ? A1 : A2, g.lda, m0);
                    db.rebase(seg == 1 ? B1 : B2, g.ldb, n0);
                }
            }
        };
        if (kt_count > 0) issue_tile(0);
        if (kt_count > 1) issue_tile((unsigned)(STAGE * sizeof(float)));
        wait_direct_loads();
        __syncthreads();
        if (kt_count > 0) {
            fa0.load(smem, wm * Cfg::WM, 0, r, half);
            fb0.load(smem + A_FLOATS, wn * Cfg::WN, 0, r, half);
        }
        // the stage is a compile-time constant of the iteration (two per trip of the loop): fragment addresses are
        // per-lane registers plus immediates, no vector instruction for addresses between the matrix instructions
        const auto iteration = [&](auto stage_const, int kt) {
            constexpr int cur = decltype(stage_const)::value;
            const float* sa = smem + cur * STAGE;
            const float* sb = sa + A_FLOATS;
            fa1.load(sa, wm * Cfg::WM, 8, r, half);
            fb1.load(sb, wn * Cfg::WN, 8, r, half);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 4; s++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa0.v[s][i], fb0.v[s][j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            wait_direct_loads();       // tile kt+1, issued a whole tile ago
            __syncthreads();           // ... is visible to everyone, and everyone has its fragments of stage cur in registers
            if (kt + 2 < kt_count) {
                constexpr unsigned stage_bytes = (unsigned)(cur * STAGE * sizeof(float));
                issue_tile(stage_bytes);
            }
            if (kt + 1 < kt_count) {
                const float* na = smem + (cur ^ 1) * STAGE;
                fa0.load(na, wm * Cfg::WM, 0, r, half);
                fb0.load(na + A_FLOATS, wn * Cfg::WN, 0, r, half);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 4; s++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa1.v[s][i], fb1.v[s][j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        };
        int kt = 0;
        for (; kt + 1 < kt_count; kt += 2) {
            iteration(std::integral_constant<int, 0>{}, kt);
            iteration(std::integral_constant<int, 1>{}, kt + 1);
        }
        if (kt < kt_count) iteration(std::integral_constant<int, 0>{}, kt);
    } else {
        TileLoader<A_KC, BM, NT> la;
        TileLoader<B_KC, BN, NT> lb;

        const int64_t kt_count = (k_end - k_begin + kBK - 1) / kBK;
        if (kt_count > 0) {
            la.load(A, g.lda, m0, g.m, k_begin, k_end, tid);
            lb.load(B, g.ldb, n0, g.n, k_begin, k_end, tid);
            la.store(smem, tid);
            lb.store(smem + A_FLOATS, tid);
        }
        __syncthreads();

        int cur = 0;
        for (int64_t kt = 0; kt < kt_count; kt++) {
            const bool more = kt + 1 < kt_count;
            if (more) {
                const int64_t k0 = k_begin + (kt + 1) * kBK;
                la.load(A, g.lda, m0, g.m, k0, k_end, tid);
                lb.load(B, g.ldb, n0, g.n, k0, k_end, tid);
            }
            const float* sa = smem + cur * STAGE;
            const float* sb = sa + A_FLOATS;
    #pragma unroll
            for (int kb = 0; kb < kBK; kb += 8) {
                Frags<A_KC, BM, TM> fa;
                Frags<B_KC, BN, TN> fb;
                fa.load(sa, wm * Cfg::WM, kb, r, half);
                fb.load(sb, wn * Cfg::WN, kb, r, half);
    #pragma unroll
                for (int s = 0; s < 4; s++)
    #pragma unroll
                    for (int i = 0; i < TM; i++)
    #pragma unroll
                        for (int j = 0; j < TN; j++)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa.v[s][i], fb.v[s][j], acc[i][j], 0, 0, 0);
            }
            if (more) {
                la.store(smem + (cur ^ 1) * STAGE, tid);
                lb.store(smem + (cur ^ 1) * STAGE + A_FLOATS, tid);
            }
            __syncthreads();
            cur ^= 1;
        }

    }

    // ---- epilogue ----
    // (a split launch writes partials to the workspace in g.c, [split][group][m][n], tables or not)
    float* C = TAB && g.k_splits <= 1 ? t.c[batch] : g.c + (int64_t)batch * g.stride_c;
    if (g.k_splits > 1) C += (int64_t)split * gridDim.y * g.stride_c;
    const bool add_c = g.accumulate && g.k_splits <= 1;
    const float* bias = g.k_splits <= 1 ? (TAB ? t.bias[batch] : g.bias) : nullptr;
    // a lane's TN columns are the same for every row it stores: their bias values are fetched once, not once per element
    float bias_v[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int64_t col = B_KC ? n0 + wn * Cfg::WN + j * 32 + r : n0 + wn * Cfg::WN + TN * r + j;
        bias_v[j] = (bias && col < g.n) ? bias[col] : 0.f;
    }
    // A tile that lies wholly inside the matrix (every tile of a shape that is a multiple of the tile) needs no bounds
    // checks, and its addresses are one per-lane pointer plus row and column steps that are the same for every lane: the
    // row step goes through the scalar unit, the column step into the store's immediate offset.  The general code below
    // spends about fifteen vector instructions per stored element on indices, comparisons and 64-bit address arithmetic,
    // a thousand per wavefront, in the one phase of the kernel in which no matrix instruction is in flight.
    if (m0 + BM <= g.m && n0 + BN <= g.n) {
        const int64_t ldc = g.ldc;
        float* lp = C + (m0 + wm * Cfg::WM + (A_KC ? half * 4 : TM * half * 4)) * ldc + n0 + wn * Cfg::WN + (B_KC ? r : TN * r);
        constexpr int GR = TM * TN <= 4 ? 8 : 4;      // rows whose old values are fetched together when accumulating
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int eg = 0; eg < 16; eg += GR) {
                if (add_c) {       // the same sums in the same order as the general code: (acc + bias) + old
                    float prev[GR][TN];
#pragma unroll
                    for (int e = 0; e < GR; e++) {
                        const int ec = eg + e;
                        const int rc = A_KC ? i * 32 + (ec >> 2) * 8 + (ec & 3) : TM * ((ec >> 2) * 8 + (ec & 3)) + i;
                        const float* rp = lp + rc * ldc;
#pragma unroll
                        for (int j = 0; j < TN; j++) prev[e][j] = __builtin_nontemporal_load(rp + (B_KC ? j * 32 : j));
                    }
#pragma unroll
                    for (int e = 0; e < GR; e++) {
                        const int ec = eg + e;
                        const int rc = A_KC ? i * 32 + (ec >> 2) * 8 + (ec & 3) : TM * ((ec >> 2) * 8 + (ec & 3)) + i;
                        float* rp = lp + rc * ldc;
#pragma unroll
                        for (int j = 0; j < TN; j++)
                            rp[B_KC ? j * 32 : j] = GR == 8 ? (acc[i][j][ec] + prev[e][j]) + bias_v[j] : (acc[i][j][ec] + bias_v[j]) + prev[e][j];
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < GR; e++) {
                        const int ec = eg + e;
                        const int rc = A_KC ? i * 32 + (ec >> 2) * 8 + (ec & 3) : TM * ((ec >> 2) * 8 + (ec & 3)) + i;
                        float* rp = lp + rc * ldc;
#pragma unroll
                        for (int j = 0; j < TN; j++) rp[B_KC ? j * 32 : j] = acc[i][j][ec] + bias_v[j];
                    }
                }
            }
        }
        return;
    }
    // accumulate: the old values of one 32-row slab are fetched by loads that depend on nothing, then added; a load
    // placed between the stores below would have to wait for them (the compiler cannot tell the rows apart)
    // (with wavefront tiles of 128x64 the addresses, which the stores need again, would not fit the register file
    // next to the accumulators: those tiles take the pipelined groups further down)
    constexpr bool kPrefetchC = TM * TN <= 4;
    if (kPrefetchC && add_c) {
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int eg = 0; eg < 16; eg += 8) {
                float prev[8][TN];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int ri = ((eg + e) >> 2) * 8 + half * 4 + (e & 3);
                    const int64_t row = m0 + wm * Cfg::WM + (A_KC ? i * 32 + ri : TM * ri + i);
                    const float* crow = C + row * g.ldc;
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const int64_t col = B_KC ? n0 + wn * Cfg::WN + j * 32 + r : n0 + wn * Cfg::WN + TN * r + j;
                        prev[e][j] = (row < g.m && col < g.n) ? __builtin_nontemporal_load(crow + col) : 0.f;
                    }
                }
#pragma unroll
                for (int e = 0; e < 8; e++)
#pragma unroll
                    for (int j = 0; j < TN; j++) acc[i][j][eg + e] += prev[e][j];
            }
        }
    }
    if (!kPrefetchC && add_c) {
        // the larger wavefront tiles: groups of four rows, the old values of the next group fetched before the current
        // group is stored (a load behind a store has to stay there: the compiler cannot tell the rows apart), so that
        // one trip to memory is exposed per wavefront instead of one per group, and a group's addresses die with it
        constexpr int NG = TM * 4;
        float prev[2][4][TN];
        const auto fetch = [&](int G, float (&pv)[4][TN]) {
            const int i = G >> 2, eq = G & 3;
#pragma unroll
            for (int e4 = 0; e4 < 4; e4++) {
                const int ri = eq * 8 + half * 4 + e4;
                const int64_t row = m0 + wm * Cfg::WM + (A_KC ? i * 32 + ri : TM * ri + i);
                const float* crow = C + row * g.ldc;
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int64_t col = B_KC ? n0 + wn * Cfg::WN + j * 32 + r : n0 + wn * Cfg::WN + TN * r + j;
                    pv[e4][j] = (row < g.m && col < g.n) ? __builtin_nontemporal_load(crow + col) : 0.f;
                }
            }
        };
        fetch(0, prev[0]);
#pragma unroll
        for (int G = 0; G < NG; G++) {
            if (G + 1 < NG) fetch(G + 1, prev[(G + 1) & 1]);
            const int i = G >> 2, eq = G & 3;
#pragma unroll
            for (int e4 = 0; e4 < 4; e4++) {
                const int ri = eq * 8 + half * 4 + e4;
                const int64_t row = m0 + wm * Cfg::WM + (A_KC ? i * 32 + ri : TM * ri + i);
                if (row >= g.m) continue;
                float* crow = C + row * g.ldc;
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int64_t col = B_KC ? n0 + wn * Cfg::WN + j * 32 + r : n0 + wn * Cfg::WN + TN * r + j;
                    if (col < g.n) crow[col] = acc[i][j][eq * 4 + e4] + bias_v[j] + prev[G & 1][e4][j];
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int ri = (e >> 2) * 8 + half * 4 + (e & 3);    // row inside the 32x32 tile
            const int64_t row = m0 + wm * Cfg::WM + (A_KC ? i * 32 + ri : TM * ri + i);
            if (row >= g.m) continue;
            float* crow = C + row * g.ldc;
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int64_t col = B_KC ? n0 + wn * Cfg::WN + j * 32 + r : n0 + wn * Cfg::WN + TN * r + j;
                if (col < g.n) {
                    crow[col] = acc[i][j][e] + bias_v[j];
                }
            }
        }
    }
}

// ---- fold split-K partials: c (+)= sum_s ws[s] (+ bias) ----
__global__ __launch_bounds__(256) void splitk_fold_kernel(const float* __restrict__ ws, float* __restrict__ c,
                                                          const float* __restrict__ bias, int64_t m, int64_t n, int64_t ldc,
                                                          int splits, int64_t batch_count, int64_t stride_c, int accumulate) {
    const int64_t per = m * n;
    const int64_t total = per * batch_count;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t bt = i / per, rem = i % per, row = rem / n, col = rem % n;
        float acc = 0.f;
        for (int s = 0; s < splits; s++) acc += ws[((int64_t)s * batch_count + bt) * per + rem];
        float* dst = c + bt * stride_c + row * ldc + col;
        if (bias) acc += bias[col];
        *dst = accumulate ? *dst + acc : acc;
    }
}

// the same for a dense output (ldc == n, batches back to back) whose size is a multiple of 4: one 16-byte piece per
// lane, single-wavefront workgroups, the grid as large as the output, everything streamed once.  The partials are
// summed in the order of the splits, as in the scalar kernel.
typedef float fold_f32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(64) void splitk_fold_vec_kernel(const float* __restrict__ ws, float* __restrict__ c,
                                                             const float* __restrict__ bias, int64_t total4, int64_t n,
                                                             int splits, int accumulate) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= total4) return;
    const fold_f32x4* w4 = reinterpret_cast<const fold_f32x4*>(ws);
    fold_f32x4 acc = __builtin_nontemporal_load(w4 + i);
    // four partials in flight at a time
    int sp = 1;
    for (; sp + 3 < splits; sp += 4) {
        const fold_f32x4 a = __builtin_nontemporal_load(w4 + (int64_t)sp * total4 + i);
        const fold_f32x4 b = __builtin_nontemporal_load(w4 + (int64_t)(sp + 1) * total4 + i);
        const fold_f32x4 d = __builtin_nontemporal_load(w4 + (int64_t)(sp + 2) * total4 + i);
        const fold_f32x4 e = __builtin_nontemporal_load(w4 + (int64_t)(sp + 3) * total4 + i);
        acc += a;
        acc += b;
        acc += d;
        acc += e;
    }
    for (; sp < splits; sp++) acc += __builtin_nontemporal_load(w4 + (int64_t)sp * total4 + i);
    if (bias) {
        const int64_t col = (i * 4) % n;    // n % 4 == 0: the four elements share a row
        acc += *reinterpret_cast<const fold_f32x4*>(bias + col);
    }
    fold_f32x4* dst = reinterpret_cast<fold_f32x4*>(c) + i;
    if (accumulate) acc = __builtin_nontemporal_load(dst) + acc;
    __builtin_nontemporal_store(acc, dst);
}

// the same for a grouped launch: blockIdx.y picks the group, whose partials sit at [split][group][m*n] in the workspace
__global__ __launch_bounds__(64) void splitk_fold_vec_tab_kernel(const float* __restrict__ ws, GemmTab t, int64_t per4, int64_t n,
                                                                 int splits, int accumulate) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= per4) return;
    const int grp = blockIdx.y;
    const int64_t split_stride = per4 * gridDim.y;
    const fold_f32x4* w4 = reinterpret_cast<const fold_f32x4*>(ws) + grp * per4 + i;
    fold_f32x4 acc = __builtin_nontemporal_load(w4);
    int sp = 1;
    for (; sp + 3 < splits; sp += 4) {
        const fold_f32x4 a = __builtin_nontemporal_load(w4 + (int64_t)sp * split_stride);
        const fold_f32x4 b = __builtin_nontemporal_load(w4 + (int64_t)(sp + 1) * split_stride);
        const fold_f32x4 d = __builtin_nontemporal_load(w4 + (int64_t)(sp + 2) * split_stride);
        const fold_f32x4 e = __builtin_nontemporal_load(w4 + (int64_t)(sp + 3) * split_stride);
        acc += a;
        acc += b;
        acc += d;
        acc += e;
    }
    for (; sp < splits; sp++) acc += __builtin_nontemporal_load(w4 + (int64_t)sp * split_stride);
    const float* bias = t.bias[grp];
    if (bias) acc += *reinterpret_cast<const fold_f32x4*>(bias + (i * 4) % n);
    fold_f32x4* dst = reinterpret_cast<fold_f32x4*>(t.c[grp]) + i;
    if (accumulate) acc = __builtin_nontemporal_load(dst) + acc;
    __builtin_nontemporal_store(acc, dst);
}

// many partials of a small output (a long contraction cut into hundreds of chunks): one wavefront per output element,
// the lanes striding over the partials
__global__ __launch_bounds__(256) void splitk_fold_wide_kernel(const float* __restrict__ ws, float* __restrict__ c,
                                                               const float* __restrict__ bias, int64_t m, int64_t n, int64_t ldc,
                                                               int splits, int64_t batch_count, int64_t stride_c, int accumulate) {
    const int lane = threadIdx.x & 63;
    const int64_t per = m * n, total = per * batch_count;
    const int64_t i = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= total) return;
    const int64_t bt = i / per, rem = i % per, row = rem / n, col = rem % n;
    float acc = 0.f;
    for (int s = lane; s < splits; s += 64) acc += ws[((int64_t)s * batch_count + bt) * per + rem];
    acc = wave_sum(acc);
    if (lane == 0) {
        float* dst = c + bt * stride_c + row * ldc + col;
        if (bias) acc += bias[col];
        *dst = accumulate ? *dst + acc : acc;
    }
}

// ---- small problems: one trip to memory per workgroup ----
// A 64x64 output tile per workgroup (four wavefronts, one 32x32 accumulator each) and a k-chunk of at most kSmallK
// that is loaded WHOLE into LDS before the first MFMA: a tiny GEMM is bound by the number of dependent round trips to
// memory (about 2 us each), not by flops, so the chunk loop of the big kernels is replaced by one load phase, one
// barrier and one MFMA chain; longer contractions are split over workgroups (blockIdx.z) and folded afterwards.
// Loads are scalar and bounds-checked (any alignment, any leading dimension), walk the operand's contiguous
// direction and are all issued before the first LDS store; both panels sit k-contiguous in LDS, rows padded by 4.
constexpr int kSmallK = 128;   // two 64 x (128+4) panels = 66 KB of dynamic LDS
constexpr int kSmallLd = kSmallK + 4;

template <bool a_kfast, bool b_kfast, int KCH>   // operand's k index is the fast one in memory; panel width (>= the k-chunk)
__global__ __launch_bounds__(256) void gemm_small_kernel(GemmArgs g) {
    extern __shared__ __align__(16) float smem[];
    float* as = smem;
    float* bs = smem + 64 * kSmallLd;
    const int tid = threadIdx.x;
    const int tile_m = blockIdx.x % g.tiles_m, tile_n = blockIdx.x / g.tiles_m;
    const int batch = blockIdx.y, split = blockIdx.z;
    const int64_t k_begin = (int64_t)split * g.k_per_split;
    int64_t k_end = k_begin + g.k_per_split;
    if (k_end > g.k) k_end = g.k;
    const int kc = (int)(k_end - k_begin);               // <= kSmallK
    const int kc8 = (kc + 7) & ~7;                       // MFMA groups of 8; the tail is zero-filled
    const float* A = g.a + (int64_t)batch * g.stride_a;
    const float* B = g.b + (int64_t)batch * g.stride_b;
    const int64_t m0 = (int64_t)tile_m * 64, n0 = (int64_t)tile_n * 64;

    // Panel element (row, kk) of an operand whose k index is the fast one in memory sits at base[row*ld + kk], else at
    // base[kk*ld + row].  All loads of a thread are issued before the first LDS store, so they are in flight together.
    constexpr int PER = 64 * KCH / 256;     // loads per lane and operand: a narrow chunk pays for a narrow panel only
    float va[PER], vb[PER];
    // out-of-range elements read a clamped (valid) address and are zeroed afterwards: no divergent branches, so the
    // loads really are issued back to back
    const int64_t m_last = g.m - 1, n_last = g.n - 1;
    const int k_last = kc > 0 ? kc - 1 : 0;
#pragma unroll
    for (int i = 0; i < PER; i++) va[i] = vb[i] = 0.f;
    if (kc > 0) {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int idx = tid + i * 256;
            const int row = a_kfast ? idx / KCH : idx & 63, kk = a_kfast ? idx % KCH : idx >> 6;
            const int64_t gr = min(m0 + row, m_last), gk = k_begin + min(kk, k_last);
            va[i] = a_kfast ? A[gr * g.lda + gk] : A[gk * g.lda + gr];
            const int col = b_kfast ? idx / KCH : idx & 63, kk2 = b_kfast ? idx % KCH : idx >> 6;
            const int64_t gc = min(n0 + col, n_last), gk2 = k_begin + min(kk2, k_last);
            vb[i] = b_kfast ? B[gc * g.ldb + gk2] : B[gk2 * g.ldb + gc];
        }
    }
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const int idx = tid + i * 256;
        const int row = a_kfast ? idx / KCH : idx & 63, kk = a_kfast ? idx % KCH : idx >> 6;
        if (m0 + row > m_last || kk >= kc) va[i] = 0.f;
        const int col = b_kfast ? idx / KCH : idx & 63, kk2 = b_kfast ? idx % KCH : idx >> 6;
        if (n0 + col > n_last || kk2 >= kc) vb[i] = 0.f;
    }
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const int idx = tid + i * 256;
        const int row = a_kfast ? idx / KCH : idx & 63, kk = a_kfast ? idx % KCH : idx >> 6;
        as[row * kSmallLd + kk] = va[i];
        const int col = b_kfast ? idx / KCH : idx & 63, kk2 = b_kfast ? idx % KCH : idx >> 6;
        bs[col * kSmallLd + kk2] = vb[i];
    }
    __syncthreads();

    const int wave = tid >> 6, lane = tid & 63, r = lane & 31, half = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;
    floatx16 acc0, acc1;                                 // two chains, even and odd k-groups
#pragma unroll
    for (int e = 0; e < 16; e++) acc0[e] = acc1[e] = 0.f;
    const float* pa = as + (wm * 32 + r) * kSmallLd + 4 * half;
    const float* pb = bs + (wn * 32 + r) * kSmallLd + 4 * half;
    for (int kb = 0; kb < kc8; kb += 16) {
        const float4 a0 = *reinterpret_cast<const float4*>(pa + kb);
        const float4 b0 = *reinterpret_cast<const float4*>(pb + kb);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.x, b0.x, acc0, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.y, b0.y, acc0, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.z, b0.z, acc0, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.w, b0.w, acc0, 0, 0, 0);
        if (kb + 8 < kc8) {
            const float4 a1 = *reinterpret_cast<const float4*>(pa + kb + 8);
            const float4 b1 = *reinterpret_cast<const float4*>(pb + kb + 8);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.x, b1.x, acc1, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.y, b1.y, acc1, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.z, b1.z, acc1, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.w, b1.w, acc1, 0, 0, 0);
        }
    }

    float* C = g.c + (int64_t)batch * g.stride_c;
    if (g.k_splits > 1) C += (int64_t)split * gridDim.y * g.stride_c;
    const bool add_c = g.accumulate && g.k_splits <= 1;
    const float* bias = g.k_splits <= 1 ? g.bias : nullptr;
    const int64_t col = n0 + wn * 32 + r;
    if (col < g.n) {
        const float bv = bias ? bias[col] : 0.f;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int64_t row = m0 + wm * 32 + (e >> 2) * 8 + half * 4 + (e & 3);
            if (row < g.m) {
                float v = acc0[e] + acc1[e];
                if (bias) v += bv;
                float* dst = C + row * g.ldc + col;
                *dst = add_c ? *dst + v : v;
            }
        }
    }
}

// ---- tiny problems: latency, not throughput ----
// A problem of a few million multiply-adds (the layers of a small MLP at batch 64) is over in the time one trip to memory
// and one chain of products take, so this kernel makes both as short as they can be: a workgroup owns a 32x32 tile of
// C and splits the contraction among its NW wavefronts in groups of 8 (a wavefront count and fetch depth that keep the kernel
// free of register spills: one kernel that needs scratch memory slows every later launch of the process); every lane fetches its operand values straight
// from global memory into the registers the products read (no staging, no barrier before the arithmetic), all of a
// wavefront's fetches in flight together; the NW partial tiles are then summed through LDS in wavefront order (so the
// result does not depend on timing) and stored with bias and accumulation applied.  No workspace, no second launch.
template <bool a_kfast, bool b_kfast, int NW, int U>   // wavefronts per tile; groups of 8 k one wavefront fetches together
__global__ __launch_bounds__(64 * NW) void gemm_tiny_kernel(GemmArgs g, int a_vec, int b_vec) {
    __shared__ float red[NW * 1024];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 31, half = lane >> 5;
    const int tile_m = blockIdx.x % g.tiles_m, tile_n = blockIdx.x / g.tiles_m;
    const int64_t batch = blockIdx.y;
    const int64_t m0 = (int64_t)tile_m * 32, n0 = (int64_t)tile_n * 32;
    // rows and columns past the edge read the last valid one: they only feed outputs that are never stored
    const int64_t row = min(m0 + r, g.m - 1), col = min(n0 + r, g.n - 1);
    const float* pa = g.a + batch * g.stride_a + (a_kfast ? row * g.lda : row);
    const float* pb = g.b + batch * g.stride_b + (b_kfast ? col * g.ldb : col);
    const int64_t sa = a_kfast ? 1 : g.lda, sb = b_kfast ? 1 : g.ldb;   // distance between consecutive k
    const int K = (int)g.k;
    const int groups = (K + 7) >> 3;

    floatx16 acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.f;
    for (int g0 = wave; g0 < groups; g0 += NW * U) {
        float av[U][4], bv[U][4];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int kk = (g0 + u * NW) * 8 + 4 * half;      // this lane's four k of the group; may lie past K
            if (a_kfast && a_vec) {                          // K % 4 == 0 here: kk < K implies kk + 3 < K
                const float4 t = *reinterpret_cast<const float4*>(pa + min(kk, K - 4));
                av[u][0] = t.x; av[u][1] = t.y; av[u][2] = t.z; av[u][3] = t.w;
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) av[u][j] = pa[(int64_t)min(kk + j, K - 1) * sa];
            }
            if (b_kfast && b_vec) {
                const float4 t = *reinterpret_cast<const float4*>(pb + min(kk, K - 4));
                bv[u][0] = t.x; bv[u][1] = t.y; bv[u][2] = t.z; bv[u][3] = t.w;
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) bv[u][j] = pb[(int64_t)min(kk + j, K - 1) * sb];
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int kk = (g0 + u * NW) * 8 + 4 * half;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const bool in = kk + j < K;                    // both operands are zero past the end of the contraction
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(in ? av[u][j] : 0.f, in ? bv[u][j] : 0.f, acc, 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 16; e++) red[wave * 1024 + e * 64 + lane] = acc[e];
    __syncthreads();

    float* C = g.c + batch * g.stride_c;
    for (int o = tid; o < 1024; o += 64 * NW) {
        float v = red[o];
#pragma unroll
        for (int w = 1; w < NW; w++) v += red[w * 1024 + o];
        const int e = o >> 6, l = o & 63;
        const int64_t orow = m0 + (e >> 2) * 8 + (l >> 5) * 4 + (e & 3), ocol = n0 + (l & 31);
        if (orow < g.m && ocol < g.n) {
            if (g.bias) v += g.bias[ocol];
            float* dst = C + orow * g.ldc + ocol;
            *dst = g.accumulate ? *dst + v : v;
        }
    }
}

// ---- tiny problems with a long contraction and an operand whose k index is the fast one in memory ----
// Fetching such an operand straight into the MFMA layout makes every lane of a load touch a cache line of its own (one
// row each), and the rate at which the vector cache looks lines up then bounds the kernel (measured: 7-16 us per trip).
// Here a wavefront owns a contiguous range of k, fetches its 32 x 64 slice of a k-fast operand with whole lines
// (16 lanes per row) and turns it into the MFMA layout through a slice of LDS that only this wavefront touches, so no
// workgroup barrier stands before the arithmetic; a row-fast operand is fetched straight into registers as in
// gemm_tiny_kernel.  The partial tiles meet in LDS at the end, summed in wavefront order.
constexpr int kWidePanel = 32 * 68;   // floats of one staged 32 x 64 slice (rows padded by 4)

template <bool a_kfast, bool b_kfast, int NW>
__global__ __launch_bounds__(64 * NW) void gemm_tiny_wide_kernel(GemmArgs g, int a_vec, int b_vec) {
    static_assert(a_kfast || b_kfast, "gemm_tiny_kernel covers two row-fast operands");
    extern __shared__ __align__(16) float smem[];
    constexpr int PER_WAVE = (a_kfast ? kWidePanel : 0) + (b_kfast ? kWidePanel : 0);   // >= 1024 floats: the partial tile fits
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 31, half = lane >> 5;
    const int tile_m = blockIdx.x % g.tiles_m, tile_n = blockIdx.x / g.tiles_m;
    const int64_t batch = blockIdx.y;
    const int64_t m0 = (int64_t)tile_m * 32, n0 = (int64_t)tile_n * 32;
    const float* A = g.a + batch * g.stride_a;
    const float* B = g.b + batch * g.stride_b;
    const int K = (int)g.k;
    // a very long contraction is cut over blockIdx.z first (partial tiles go to the workspace and are folded afterwards)
    const int ks0 = g.k_splits > 1 ? (int)(blockIdx.z * g.k_per_split) : 0;
    const int ks1 = g.k_splits > 1 ? min(K, ks0 + (int)g.k_per_split) : K;
    const int groups = (ks1 - ks0 + 7) >> 3;
    const int gpw = (groups + NW - 1) / NW;                // groups of 8 k per wavefront
    const int kw0 = ks0 + wave * gpw * 8;
    const int kw1 = min(ks1, kw0 + gpw * 8);               // this wavefront contracts k in [kw0, kw1)
    float* mine = smem + wave * PER_WAVE;
    float* as = mine;
    float* bs = mine + (a_kfast ? kWidePanel : 0);
    // rows and columns past the edge read the last valid one: they only feed outputs that are never stored
    const int64_t row = min(m0 + r, g.m - 1), col = min(n0 + r, g.n - 1);

    floatx16 acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.f;
    for (int kc = kw0; kc < kw1; kc += 64) {
        // row-fast operands: this lane's values for the eight groups of the chunk, straight from memory
        float av[8][4], bv[8][4];
        if (!a_kfast) {
#pragma unroll
            for (int u = 0; u < 8; u++)
#pragma unroll
                for (int j = 0; j < 4; j++) av[u][j] = A[(int64_t)min(kc + 8 * u + 4 * half + j, K - 1) * g.lda + row];
        }
        if (!b_kfast) {
#pragma unroll
            for (int u = 0; u < 8; u++)
#pragma unroll
                for (int j = 0; j < 4; j++) bv[u][j] = B[(int64_t)min(kc + 8 * u + 4 * half + j, K - 1) * g.ldb + col];
        }
        // k-fast operands: 32 rows x 64 k as 512 16-byte pieces, 8 per lane, 16 lanes along a row
        float4 sa[8], sb[8];
        if (a_kfast) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int f = lane + 64 * i, rr = f >> 4, kk = kc + 4 * (f & 15);
                const float* p = A + min(m0 + rr, g.m - 1) * g.lda;
                if (a_vec) sa[i] = *reinterpret_cast<const float4*>(p + min(kk, K - 4));
                else sa[i] = make_float4(p[min(kk, K - 1)], p[min(kk + 1, K - 1)], p[min(kk + 2, K - 1)], p[min(kk + 3, K - 1)]);
            }
        }
        if (b_kfast) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int f = lane + 64 * i, rr = f >> 4, kk = kc + 4 * (f & 15);
                const float* p = B + min(n0 + rr, g.n - 1) * g.ldb;
                if (b_vec) sb[i] = *reinterpret_cast<const float4*>(p + min(kk, K - 4));
                else sb[i] = make_float4(p[min(kk, K - 1)], p[min(kk + 1, K - 1)], p[min(kk + 2, K - 1)], p[min(kk + 3, K - 1)]);
            }
        }
        if (a_kfast) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int f = lane + 64 * i;
                *reinterpret_cast<float4*>(as + (f >> 4) * 68 + 4 * (f & 15)) = sa[i];
            }
        }
        if (b_kfast) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int f = lane + 64 * i;
                *reinterpret_cast<float4*>(bs + (f >> 4) * 68 + 4 * (f & 15)) = sb[i];
            }
        }
        // the slice is private to this wavefront: its own LDS writes are ordered before its reads, the fences only keep
        // the compiler from moving one across the other
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int kk = kc + 8 * u + 4 * half;
            float a4[4], b4[4];
            if (a_kfast) {
                const float4 t = *reinterpret_cast<const float4*>(as + r * 68 + 8 * u + 4 * half);
                a4[0] = t.x; a4[1] = t.y; a4[2] = t.z; a4[3] = t.w;
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) a4[j] = av[u][j];
            }
            if (b_kfast) {
                const float4 t = *reinterpret_cast<const float4*>(bs + r * 68 + 8 * u + 4 * half);
                b4[0] = t.x; b4[1] = t.y; b4[2] = t.z; b4[3] = t.w;
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) b4[j] = bv[u][j];
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const bool in = kk + j < kw1;                  // past this wavefront's range (or the contraction): no contribution
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(in ? a4[j] : 0.f, in ? b4[j] : 0.f, acc, 0, 0, 0);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    // the partial tile goes where the wavefront's slices were
#pragma unroll
    for (int e = 0; e < 16; e++) mine[e * 64 + lane] = acc[e];
    __syncthreads();

    float* C = g.c + batch * g.stride_c;
    if (g.k_splits > 1) C += (int64_t)blockIdx.z * gridDim.y * g.stride_c;
    const bool last_word = g.k_splits <= 1;                // bias and accumulation belong to the fold otherwise
    for (int o = tid; o < 1024; o += 64 * NW) {
        float v = smem[o];
#pragma unroll
        for (int w = 1; w < NW; w++) v += smem[w * PER_WAVE + o];
        const int e = o >> 6, l = o & 63;
        const int64_t orow = m0 + (e >> 2) * 8 + (l >> 5) * 4 + (e & 3), ocol = n0 + (l & 31);
        if (orow < g.m && ocol < g.n) {
            if (last_word && g.bias) v += g.bias[ocol];
            float* dst = C + orow * g.ldc + ocol;
            *dst = last_word && g.accumulate ? *dst + v : v;
        }
    }
}

// ---- fallback: bounds-checked 32x32 LDS tiles, any shape / alignment ----
__global__ __launch_bounds__(256) void gemm_fallback_kernel(GemmArgs g, int trans_a, int trans_b) {
    __shared__ float ta[32][33];
    __shared__ float tb[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
    const int64_t m0 = (int64_t)blockIdx.y * 32, n0 = (int64_t)blockIdx.x * 32;
    const float* A = g.a + (int64_t)blockIdx.z * g.stride_a;
    const float* B = g.b + (int64_t)blockIdx.z * g.stride_b;
    float* C = g.c + (int64_t)blockIdx.z * g.stride_c;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int64_t k0 = 0; k0 < g.k; k0 += 32) {
        for (int p = 0; p < 4; p++) {
            const int rr = ty + p * 8;
            // ta[rr][tx] = A(m0+rr, k0+tx) ; tb[rr][tx] = B(k0+rr, n0+tx)
            const int64_t am = m0 + rr, ak = k0 + tx;
            ta[rr][tx] = (am < g.m && ak < g.k) ? (trans_a ? A[ak * g.lda + am] : A[am * g.lda + ak]) : 0.f;
            const int64_t bk = k0 + rr, bn = n0 + tx;
            tb[rr][tx] = (bk < g.k && bn < g.n) ? (trans_b ? B[bn * g.ldb + bk] : B[bk * g.ldb + bn]) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int kk = 0; kk < 32; kk++) {
            const float bv = tb[kk][tx];
#pragma unroll
            for (int p = 0; p < 4; p++) acc[p] += ta[ty + p * 8][kk] * bv;
        }
        __syncthreads();
    }
    for (int p = 0; p < 4; p++) {
        const int64_t row = m0 + ty + p * 8, col = n0 + tx;
        if (row < g.m && col < g.n) {
            float v = acc[p];
            if (g.bias) v += g.bias[col];
            if (g.accumulate) v += C[row * g.ldc + col];
            C[row * g.ldc + col] = v;
        }
    }
}

// ---- out-of-place transpose of the last two dims (for boat_transpose callers) ----
__global__ __launch_bounds__(256) void transpose_kernel(const float* __restrict__ a, float* __restrict__ out, int64_t rows,
                                                        int64_t cols) {
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const float* ab = a + (int64_t)blockIdx.z * rows * cols;
    float* ob = out + (int64_t)blockIdx.z * rows * cols;
    const int64_t r0 = (int64_t)blockIdx.y * 32, c0 = (int64_t)blockIdx.x * 32;
    for (int p = 0; p < 4; p++) {
        const int64_t rr = r0 + ty + p * 8, cc = c0 + tx;
        if (rr < rows && cc < cols) tile[ty + p * 8][tx] = ab[rr * cols + cc];
    }
    __syncthreads();
    for (int p = 0; p < 4; p++) {
        const int64_t cc = c0 + ty + p * 8, rr = r0 + tx;
        if (rr < rows && cc < cols) ob[cc * rows + rr] = tile[tx][ty + p * 8];
    }
}

using CfgBig = GemmCfg<256, 256, 2, 4>;   // 8 waves, 128x64 per wave
using CfgMid = GemmCfg<128, 128, 2, 2>;   // 4 waves, 64x64 per wave
using CfgTall = GemmCfg<256, 128, 4, 2>;  // 8 waves, 64x64 per wave
using CfgWide = GemmCfg<128, 256, 2, 4>;  // 8 waves, 64x64 per wave
using CfgSmall = GemmCfg<64, 64, 2, 2>;   // 4 waves, 32x32 per wave

// out[a][d1][b][d0][c] = in[a][d0][b][d1][c]: two dimensions of a dense tensor swapped, anything between and after
// them carried along (the general case of boat_transpose, linear.c:238-406).  One output element per lane and trip;
// consecutive lanes write consecutive addresses, and read consecutive ones whenever c has an extent.
template <typename T>
__global__ __launch_bounds__(256) void swap_dims_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t d0,
                                                        int64_t b, int64_t d1, int64_t c, int64_t total) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        int64_t t = i;
        const int64_t ic = t % c; t /= c;
        const int64_t i0 = t % d0; t /= d0;
        const int64_t ib = t % b; t /= b;
        const int64_t i1 = t % d1;
        const int64_t ia = t / d1;
        out[i] = in[(((ia * d0 + i0) * b + ib) * d1 + i1) * c + ic];
    }
}

template <typename Cfg, bool A_KC, bool B_KC, bool DIRECT, int KT = 1, bool TAB = false>
static int launch_mfma(const GemmArgs& g, int64_t batch, const GemmTab* tab = nullptr) {
    constexpr size_t lds = KT * 2 * sizeof(float) *
        (DIRECT ? DirectTile<A_KC, Cfg::BM>::floats + DirectTile<B_KC, Cfg::BN>::floats
                : TileShape<A_KC, Cfg::BM>::floats + TileShape<B_KC, Cfg::BN>::floats);
    static bool attr_set = false;
    if (!attr_set) {
        int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_mfma_kernel<Cfg, A_KC, B_KC, DIRECT, KT, TAB>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                           "hipFuncSetAttribute");
        if (rc) return rc;
        attr_set = true;
    }
    dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch, (unsigned)(g.k_splits > 1 ? g.k_splits : 1));
    GemmTab none = {};
    hipLaunchKernelGGL((gemm_mfma_kernel<Cfg, A_KC, B_KC, DIRECT, KT, TAB>), grid, dim3(Cfg::NT), lds, stream(), g, tab ? *tab : none);
    return BH_LAUNCH_CHECK("gemm_mfma_kernel");
}

template <typename Cfg, bool DIRECT>
static int launch_mfma_layout2(const GemmArgs& g, int64_t batch, bool a_kc, bool b_kc) {
    if (a_kc && b_kc) return launch_mfma<Cfg, true, true, DIRECT>(g, batch);
    if (a_kc && !b_kc) return launch_mfma<Cfg, true, false, DIRECT>(g, batch);
    if (!a_kc && b_kc) return launch_mfma<Cfg, false, true, DIRECT>(g, batch);
    return launch_mfma<Cfg, false, false, DIRECT>(g, batch);
}

// an eight-wavefront tile with two k-tiles per barrier (direct loads, every workgroup's contraction range a multiple of 32)
template <typename Cfg>
static int launch_mfma_pairs(const GemmArgs& g, int64_t batch, bool a_kc, bool b_kc) {
    if (a_kc && b_kc) return launch_mfma<Cfg, true, true, true, 2>(g, batch);
    if (a_kc && !b_kc) return launch_mfma<Cfg, true, false, true, 2>(g, batch);
    if (!a_kc && b_kc) return launch_mfma<Cfg, false, true, true, 2>(g, batch);
    return launch_mfma<Cfg, false, false, true, 2>(g, batch);
}

// the same tiles with their operands taken from tables (grouped launches); KT as the tile would have it ungrouped
template <typename Cfg, int KT>
static int launch_mfma_tab(const GemmArgs& g, int64_t batch, bool a_kc, bool b_kc, const GemmTab* tab) {
    if (a_kc && b_kc) return launch_mfma<Cfg, true, true, true, KT, true>(g, batch, tab);
    if (a_kc && !b_kc) return launch_mfma<Cfg, true, false, true, KT, true>(g, batch, tab);
    if (!a_kc && b_kc) return launch_mfma<Cfg, false, true, true, KT, true>(g, batch, tab);
    return launch_mfma<Cfg, false, false, true, KT, true>(g, batch, tab);
}

template <typename Cfg>
static int launch_mfma_layout(const GemmArgs& g, int64_t batch, bool a_kc, bool b_kc, bool direct) {
    return direct ? launch_mfma_layout2<Cfg, true>(g, batch, a_kc, b_kc) : launch_mfma_layout2<Cfg, false>(g, batch, a_kc, b_kc);
}

template <bool A_KFAST, bool B_KFAST, int KCH>
static int launch_small_one(const GemmArgs& g, dim3 grid, size_t lds) {
    static bool attr_set = false;
    if (!attr_set) {
        int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_small_kernel<A_KFAST, B_KFAST, KCH>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), "hipFuncSetAttribute");
        if (rc) return rc;
        attr_set = true;
    }
    hipLaunchKernelGGL((gemm_small_kernel<A_KFAST, B_KFAST, KCH>), grid, dim3(256), lds, stream(), g);
    return BH_OK;
}
template <bool A_KFAST, bool B_KFAST>
static int launch_small(int kch, const GemmArgs& g, dim3 grid, size_t lds) {
    if (kch == 32) return launch_small_one<A_KFAST, B_KFAST, 32>(g, grid, lds);
    if (kch == 64) return launch_small_one<A_KFAST, B_KFAST, 64>(g, grid, lds);
    return launch_small_one<A_KFAST, B_KFAST, kSmallK>(g, grid, lds);
}

// fold `splits` partial results in ws into c (one launch)
static int launch_fold(const float* ws, float* c, const float* bias, int64_t m, int64_t n, int64_t ldc, int splits, int64_t batch,
                       int64_t stride_c, int accumulate) {
    const int64_t total = m * n * batch;
    if (splits >= 32 && total <= 16384) {
        hipLaunchKernelGGL(splitk_fold_wide_kernel, dim3((unsigned)ceil_div(total, 4)), dim3(256), 0, stream(), ws, c, bias, m, n, ldc,
                           splits, batch, stride_c, accumulate);
    } else if (ldc == n && (batch == 1 || stride_c == m * n) && n % 4 == 0 &&
               ((reinterpret_cast<uintptr_t>(ws) | reinterpret_cast<uintptr_t>(c) | reinterpret_cast<uintptr_t>(bias)) & 15) == 0 &&
               ceil_div(total / 4, 64) <= 0x7fffffff) {
        hipLaunchKernelGGL(splitk_fold_vec_kernel, dim3((unsigned)ceil_div(total / 4, 64)), dim3(64), 0, stream(), ws, c, bias,
                           total / 4, n, splits, accumulate);
    } else {
        int64_t blocks = ceil_div(total, 256);
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(splitk_fold_kernel, dim3((unsigned)blocks), dim3(256), 0, stream(), ws, c, bias, m, n, ldc, splits, batch,
                           stride_c, accumulate);
    }
    return BH_LAUNCH_CHECK("splitk_fold_kernel");
}

// ---- which tile, and how many cuts of the contraction: a cost model instead of a table of shapes ----
// A workgroup's time is (its share of k) x (us per k of its tile) + a fixed part (launch of the round, first trip to
// memory, pipeline fill, the store of its tile); a launch takes as many such rounds as the busiest compute unit gets
// workgroups; a split contraction pays a fold that streams its partials once.  The constants are measured on MI355X
// (first a least-squares fit to a sweep of every tile at 1..32 cuts over 120 shapes from 256 to 8192 in each dimension,
// two operand layouts; then, after the epilogue lost its index arithmetic and the 128x128 tile took a third resident
// workgroup, straight lines through one-round launches at k = 512 .. 4096):
//   256x256 (8 wavefronts, one workgroup per CU)   0.2192 us per k, 14.6 us per round
//   256x128 / 128x256 (8 wavefronts, one per CU)   0.1126 us per k (half the products at 2.6 % less than the big tile's
//                                                  rate), 9.0 us per round
//   128x128 (4 wavefronts, up to three per CU)     resident workgroups take turns on the matrix cores: 0.0559 us per k
//                                                  each while two share a unit, 0.0558 with three, 0.0585 for one that has
//                                                  the unit to itself (one wavefront per SIMD hides less); fixed part
//                                                  6.5, 8.0 and 8.8 us.  A launch hands its workgroups round the units
//                                                  in turn, so what is left after whole rounds of three per unit runs
//                                                  one, two or three to a unit
//   64x64 (4 wavefronts, eight resident per CU)    4.0 us (11 beyond eight per unit) + k x (0.01432 us x workgroups per
//                                                  unit + 0.00336 us): 91-93 % of the matrix rate from two per unit on
//                                                  (one alone: 0.0185 us per k up to k = 1024, 0.0226 beyond), measured
//                                                  at 1 .. 16 per unit and k = 128 .. 4096; it reads its operands twice as
//                                                  often as the 128x128 tile and is offered up to sixteen per unit
//                                                  (1024^3: 20 us against 27; 3072x3072x1024, nine per unit where the
//                                                  128x128 tile has two and a quarter: 152 against 180)
//   fold of a cut contraction                      5 us + (cuts + 1) x output bytes at 6.2 TB/s (the partials mostly
//                                                  still sit in the last-level cache)
// Padding is paid automatically (a tile costs the same full or not), and so is the quantisation of rounds: 384 big
// tiles are two rounds, the second half empty, where 768 tiles of half the size are three full ones.
struct TilePlan {
    int cfg, splits;
    double us;
};
static double tile_us(int cfg, int64_t m, int64_t n, int64_t k, int64_t batch, int64_t splits, bool accumulate, int cus) {
    static const int bms[8] = {0, 128, 256, 256, 128, 0, 0, 64}, bns[8] = {0, 128, 256, 128, 256, 0, 0, 64};
    const int64_t tiles = ceil_div(m, bms[cfg]) * ceil_div(n, bns[cfg]) * batch;
    const int64_t unit = (k % (2 * kBK) == 0 && cfg != 1 && cfg != 7) ? 2 * kBK : kBK;
    const int64_t ks = splits > 1 ? ceil_div(ceil_div(k, splits), unit) * unit : k;
    const int64_t real_splits = splits > 1 ? ceil_div(k, ks) : 1;
    const int64_t wgs = tiles * real_splits;
    double us;
    if (cfg == 1) {
        // us per k and workgroup, and the fixed part of a round, when one, two or three workgroups share a compute unit
        // (the tile's registers and LDS let three be resident; a launch hands its workgroups round the units in turn)
        static const double rate[4] = {0.0, 0.0585, 0.0559, 0.0558}, fixed[4] = {0.0, 6.5, 8.0, 8.8};
        const int64_t full = wgs / (3 * cus), rest = wgs - full * 3 * cus;
        us = full * (3 * ks * rate[3] + fixed[3]);
        if (rest > 0) {
            const int64_t share = ceil_div(rest, cus);
            us += share * ks * rate[share] + fixed[share];
        }
    } else if (cfg == 7) {
        // the workgroups of a compute unit (the hardware keeps eight resident and refills as they end) take turns
        const int64_t share = ceil_div(wgs, cus);
        us = (share <= 8 ? 4.0 : 11.0) + ks * (share == 1 ? (ks <= 1024 ? 0.0185 : 0.0226) : share * 0.01432 + 0.00336);
        if (share > 8) us *= 1.05;      // past one set of resident workgroups the figure has been up to 10 % low: the larger tiles get the benefit of the doubt
    } else {
        const double per_k = cfg == 2 ? 0.2192 : 0.1126, fixed = cfg == 2 ? 14.6 : 9.0;
        us = ceil_div(wgs, cus) * (ks * per_k + fixed);
    }
    if (real_splits > 1) {
        const double bytes = (double)(real_splits + 1 + (accumulate ? 1 : 0)) * (double)(m * n * batch) * 4.0;
        us += 5.1 + bytes / 6.2e6;
    }
    return us;
}
static TilePlan plan_tiles(int64_t m, int64_t n, int64_t k, int64_t batch, bool segmented, bool accumulate, bool tables) {
    int cus = bh_device_cu_count();
    if (cus <= 0) cus = 256;
    TilePlan best{1, 1, 1e30};
    for (int cfg = 1; cfg <= 7; cfg++) {
        if (cfg == 5 || cfg == 6) continue;     // not tiles of this kernel
        if (cfg == 7 && (tables || ceil_div(m, 64) * ceil_div(n, 64) * batch > 16 * (int64_t)cus)) continue;
        if (cfg == 3 && m < 192) continue;      // a 256-row tile over fewer rows than that is mostly padding ...
        if (cfg == 4 && n < 192) continue;      // ... and the model's fixed part does not shrink with it
        if (cfg == 2 && (m < 192 || n < 192)) continue;
        const int64_t max_splits = segmented ? 1 : (k / 128 < 32 ? (k / 128 < 1 ? 1 : k / 128) : 32);
        for (int64_t sp = 1; sp <= max_splits; sp++) {
            const double us = tile_us(cfg, m, n, k, batch, sp, accumulate, cus);
            if (us < best.us * 0.995) best = TilePlan{cfg, (int)sp, us};   // ties go to the earlier (smaller) choice
        }
    }
    return best;
}
// the number of cuts the model would choose for a tile shape somebody forced (test hook)
static int64_t default_splits(int cfg, int64_t m, int64_t n, int64_t k, int64_t batch) {
    int cus = bh_device_cu_count();
    if (cus <= 0) cus = 256;
    double best = 1e30;
    int64_t best_sp = 1;
    const int64_t max_splits = k / 128 < 32 ? (k / 128 < 1 ? 1 : k / 128) : 32;
    for (int64_t sp = 1; sp <= max_splits; sp++) {
        const double us = tile_us(cfg, m, n, k, batch, sp, false, cus);
        if (us < best * 0.995) {
            best = us;
            best_sp = sp;
        }
    }
    return best_sp;
}

static int g_force_splits = 0;    // test hook: > 0 = this many k-splits for the MFMA tiles
static int g_pairs = 1;           // test hook: 0 = every tile keeps one k-tile per barrier
static int g_force_direct = -1;   // test hook: 0 = staged through registers, 1 / -1 = direct to LDS whenever eligible
static int g_no_tables = 0;       // test hook: 1 = grouped launches fall back to one launch per group
static int g_force_cfg = -1;   // test hook: 0 = fallback, 1..4 = MFMA tile shapes, 5 = small-problem kernel, 6 = tiny, -1 = heuristic

}  // namespace bh

using namespace bh;

extern "C" {

// test/benchmark hook: pin the kernel choice (-1 restores the heuristic)
int bh_gemm_force_config(int cfg) {
    g_force_cfg = cfg;
    return BH_OK;
}

// test/benchmark hook: number of k-splits where the heuristic would split (0 restores the heuristic)
int bh_gemm_force_splits(int splits) {
    g_force_splits = splits;
    return BH_OK;
}

// test/benchmark hook: 0 stages operand tiles through registers even where the direct-to-LDS loader applies
int bh_gemm_force_direct(int mode) {
    g_pairs = !(mode & 2);       // bit 1 set: one k-tile per barrier also for the eight-wavefront tiles
    g_force_direct = mode < 0 ? -1 : (mode & 1);
    return BH_OK;
}

}  // extern "C"

// `tab` != NULL: a grouped launch (operands from the tables, a/b/c/bias unused; k is the whole contraction of a segmented
// product).  Returns kTabUnsupported, having launched nothing, when the shape does not take one of the table kernels.
constexpr int kTabUnsupported = -1000;
static int gemm_core(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, const float* a, int64_t lda, const float* b,
                     int64_t ldb, float* c, int64_t ldc, const float* bias, int accumulate, int64_t batch, const GemmTab* tab) {

    GemmArgs g;
    g.a = a; g.b = b; g.c = c; g.bias = bias;
    g.m = m; g.n = n; g.k = k;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc;
    g.stride_a = (trans_a ? k : m) * lda;
    g.stride_b = (trans_b ? n : k) * ldb;
    g.stride_c = m * ldc;
    g.accumulate = accumulate;
    g.k_splits = 1;
    g.k_per_split = k;

    const bool a_kc = !trans_a, b_kc = trans_b != 0;
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (tab) {
        const int count = tab->k_segments > 1 ? tab->k_segments : (int)batch;
        a = tab->a[0];
        b = tab->b[0];
        for (int i = 1; i < count; i++)
            if (!al16(tab->a[i]) || !al16(tab->b[i])) return kTabUnsupported;
        for (int i = 0; i < (tab->k_segments > 1 ? 1 : count); i++)
            if (!al16(tab->c[i]) || !al16(tab->bias[i])) return kTabUnsupported;
    }
    // float4 global loads need: 16 B aligned bases, leading dimensions and the contiguous extent % 4
    bool vec_ok = al16(a) && al16(b) && (lda % 4 == 0) && (ldb % 4 == 0) && k > 0;
    vec_ok = vec_ok && ((a_kc ? k : m) % 4 == 0) && ((b_kc ? k : n) % 4 == 0);
    int cfg;   // 0 fallback, 1 = 128x128, 2 = 256x256, 3 = 256x128, 4 = 128x256, 7 = 64x64
    int plan_splits = 1;   // k-splits that come with the tile choice
    double plan_us = 1e30; // what the cost model expects of that choice
    const bool segmented = tab && tab->k_segments > 1;     // one product over several operand pairs: never split
    if (!vec_ok || m * n < 64 * 64) {
        cfg = 0;
    } else {
        const TilePlan plan = plan_tiles(m, n, k, batch, segmented, accumulate != 0, tab != nullptr);
        cfg = plan.cfg;
        plan_splits = plan.splits;
        plan_us = plan.us;
    }
    // Up to about 2^25 multiply-adds the problem is latency bound.  The 64x64 tile, cut as the cost model says, is the
    // fastest kernel there wherever its 16-byte loads apply (256x256x512: 8.4 us against 12.6 for the kernel that stages
    // a whole k-chunk per workgroup, which keeps the shapes the tile cannot load)
    const bool small_problem = m * n <= ((int64_t)1 << 25) / (k > 0 ? k : 1);
    if (small_problem) cfg = 5;
    // so is a contraction of at most 64 under an output of a few million elements, where the larger tiles spend their
    // time filling and draining their pipeline (288x12544x64: 15.7 against 20.0 us; 4096x4096x64 is past it: 56 against 37)
    if (k > 0 && k <= 64 && m * n <= ((int64_t)1 << 22)) cfg = 5;
    const bool small_tile_ok = vec_ok && m * n >= 64 * 64 && !tab;
    const auto take_small_tile = [&]() {
        int cus = bh_device_cu_count();
        if (cus <= 0) cus = 256;
        cfg = 7;
        plan_splits = (int)default_splits(7, m, n, k, batch);
        plan_us = tile_us(7, m, n, k, batch, plan_splits, accumulate != 0, cus);
    };
    if (cfg == 5 && small_tile_ok && small_problem) take_small_tile();
    // A few million multiply-adds in at most a few hundred 32x32 tiles: the kernels without workgroup-wide staging.
    // Measured against the staged small-problem kernel plus its fold (11-14 us beyond k = 128): two row-fast operands
    // 6-10 us up to k = 1024; one k-fast operand 7.5-8 us up to k = 512 (one trip) and 12 us up to 1024 (two trips);
    // two k-fast operands 9-11 us up to k = 512 and slower beyond.
    const int64_t tiles32 = ceil_div(m, 32) * ceil_div(n, 32) * batch;
    // (with a k-fast operand the 64x64 tile is as fast or faster wherever it applies -- 64x128x1024: 8.3 against 12.5 us --
    // so the kernel keeps the shapes with two row-fast operands, where it wins -- 512x512x512: 6.9 against 9.4 -- up to
    // the long contractions under small outputs that the tile cuts -- 64x128x1024: 8.0 against 10.5 --, and those
    // the tile cannot load)
    if (k > 0 && m * n * k <= ((int64_t)1 << (k <= 128 ? 25 : 24)) && tiles32 <= 512 &&
        (k <= 512 || (k <= 1024 && !(a_kc && b_kc)) || (!a_kc && !b_kc))) {
        if (small_tile_ok && (a_kc || b_kc || (k >= 1024 && m * n <= ((int64_t)1 << 17)))) take_small_tile();
        else cfg = 6;
    }
    // (two row-fast operands over a contraction of 257 .. 512: the tiny kernel's one trip per wavefront beats the tile
    // up to 256 tiles of 32x32 -- 512x512x512: 6.8 against 9.4 us, 784x128x512: 6.7 against 8.8)
    if (!a_kc && !b_kc && k > 256 && k <= 512 && tiles32 <= 256) cfg = 6;
    // A small output with a very long contraction over k-fast operands (the weight gradient of a convolution: 64 x 288
    // outputs, k = 12544): chunks of 512 k per workgroup of the same kernel, partials folded afterwards.
    // Its 32x32 tiles read every operand value once per tile row or column, k*m*n/4 bytes in all, at 3.2 TB/s when both
    // operands are k-fast and 4.3 TB/s with one (measured from 64x288 to 256x256 outputs, k 2048 to 32768); the 128x128
    // tiles with a cut contraction read a quarter of that and win from about 128x256x12544 on, which the cost model's figure
    // for them shows (256x256x8192: 43 us here against 31 us there).  Where the 64x64 tile was taken it stays: it cuts
    // such a contraction itself (64x128x2048: 8.7 against 14.1 us).
    bool tiny_split = false;
    if (cfg != 7 && k >= 2048 && tiles32 <= 64 && (a_kc || b_kc) && ceil_div(k, 512) <= 65535 &&
        8.0 + 0.25 * (double)k * (double)m * (double)n * (double)batch / ((a_kc && b_kc) ? 3.2e6 : 4.3e6) <= plan_us) {
        cfg = 6;
        tiny_split = true;
    }
    const int cfg_planned = cfg;
    if (g_force_cfg >= 0 && g_force_cfg <= 7 && (vec_ok || g_force_cfg == 0 || g_force_cfg == 5 || g_force_cfg == 6)) cfg = g_force_cfg;
    if (cfg == 6 && k == 0) cfg = 5;
    if (cfg != 6) tiny_split = false;
    if (tab && (cfg == 0 || cfg >= 5)) return kTabUnsupported;     // (the 64x64 tile, 7, has no table form either)

    if (cfg == 6) {
        g.tiles_m = (int)ceil_div(m, 32);
        g.tiles_n = (int)ceil_div(n, 32);
        BH_CHECK_ARG((int64_t)g.tiles_m * g.tiles_n <= 0x7fffffff && k <= 0x7ffffff0, "problem too large for the tiny-GEMM kernel");
        // 16-byte fetches along k need the operand's rows to start on 16 bytes and k % 4 == 0
        const int a_vec = a_kc && al16(a) && lda % 4 == 0 && k % 4 == 0 && (g.stride_a % 4 == 0 || batch == 1);
        const int b_vec = b_kc && al16(b) && ldb % 4 == 0 && k % 4 == 0 && (g.stride_b % 4 == 0 || batch == 1);
        const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch);
        if (k > 128 && (a_kc || b_kc)) {
            // long contraction with a k-fast operand: slices staged per wavefront (8 wavefronts, 64 k each per trip)
            const size_t lds = sizeof(float) * 8 * (size_t)((a_kc ? kWidePanel : 0) + (b_kc ? kWidePanel : 0));
            GemmArgs run = g;
            float* ws = nullptr;
            if (tiny_split) {
                // one trip (512 k) per workgroup unless that makes more workgroups than the chip holds at once
                g.k_per_split = tiles32 * ceil_div(k, 512) > 384 ? 1024 : 512;
                g.k_splits = (int)ceil_div(k, g.k_per_split);
                ws = (float*)bh_malloc(sizeof(float) * (size_t)(g.k_splits * batch * m * n));
                if (!ws) return BH_ENOMEM;
                run = g;
                run.c = ws;
                run.ldc = n;
                run.stride_c = m * n;
            }
            const dim3 wgrid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch, (unsigned)(g.k_splits > 1 ? g.k_splits : 1));
            int lrc = BH_OK;
#define WIDE_LAUNCH(AK, BK)                                                                                               \
    {                                                                                                                     \
        static bool attr = false;                                                                                         \
        if (!attr) {                                                                                                      \
            lrc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tiny_wide_kernel<AK, BK, 8>),         \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),                    \
                            "hipFuncSetAttribute");                                                                       \
            attr = lrc == BH_OK;                                                                                          \
        }                                                                                                                 \
        if (lrc == BH_OK)                                                                                                 \
            hipLaunchKernelGGL((gemm_tiny_wide_kernel<AK, BK, 8>), wgrid, dim3(512), lds, stream(), run, a_vec, b_vec);   \
    }
            if (a_kc && b_kc) WIDE_LAUNCH(true, true)
            else if (a_kc) WIDE_LAUNCH(true, false)
            else WIDE_LAUNCH(false, true)
#undef WIDE_LAUNCH
            if (lrc == BH_OK) lrc = BH_LAUNCH_CHECK("gemm_tiny_wide_kernel");
            if (lrc == BH_OK && g.k_splits > 1) lrc = launch_fold(ws, c, bias, m, n, ldc, g.k_splits, batch, g.stride_c, accumulate);
            if (ws) bh_free(ws);
            return lrc;
        }
        const bool wide = k > 128;    // two row-fast operands: 8 wavefronts share a long contraction, 4 a short one
#define TINY_LAUNCH(AK, BK)                                                                                               \
    if (wide) hipLaunchKernelGGL((gemm_tiny_kernel<AK, BK, 8, 8>), grid, dim3(512), 0, stream(), g, a_vec, b_vec);          \
    else hipLaunchKernelGGL((gemm_tiny_kernel<AK, BK, 4, 4>), grid, dim3(256), 0, stream(), g, a_vec, b_vec)
        if (a_kc && b_kc) { TINY_LAUNCH(true, true); }
        else if (a_kc) { TINY_LAUNCH(true, false); }
        else if (b_kc) { TINY_LAUNCH(false, true); }
        else { TINY_LAUNCH(false, false); }
#undef TINY_LAUNCH
        return BH_LAUNCH_CHECK("gemm_tiny_kernel");
    }

    if (cfg == 5) {
        g.tiles_m = (int)ceil_div(m, 64);
        g.tiles_n = (int)ceil_div(n, 64);
        const int64_t splits = k > kSmallK ? ceil_div(k, kSmallK) : 1;
        g.k_per_split = k > 0 ? ceil_div(ceil_div(k, splits), 8) * 8 : 8;
        g.k_splits = (int)(k > 0 ? ceil_div(k, g.k_per_split) : 1);
        BH_CHECK_ARG((int64_t)g.tiles_m * g.tiles_n <= 0x7fffffff && g.k_splits <= 65535, "problem too large for the small-GEMM kernel");
        GemmArgs run = g;
        float* ws = nullptr;
        if (g.k_splits > 1) {
            ws = (float*)bh_malloc(sizeof(float) * (size_t)(g.k_splits * batch * m * n));
            if (!ws) return BH_ENOMEM;
            run.c = ws;
            run.ldc = n;
            run.stride_c = m * n;
        }
        dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)batch, (unsigned)g.k_splits);
        constexpr size_t lds = 2 * 64 * kSmallLd * sizeof(float);
        const int kch = g.k_per_split <= 32 ? 32 : g.k_per_split <= 64 ? 64 : kSmallK;
        int lrc;
        if (a_kc && b_kc) lrc = launch_small<true, true>(kch, run, grid, lds);
        else if (a_kc) lrc = launch_small<true, false>(kch, run, grid, lds);
        else if (b_kc) lrc = launch_small<false, true>(kch, run, grid, lds);
        else lrc = launch_small<false, false>(kch, run, grid, lds);
        if (lrc) {
            if (ws) bh_free(ws);
            return lrc;
        }
        int rc = BH_LAUNCH_CHECK("gemm_small_kernel");
        if (rc == BH_OK && g.k_splits > 1) rc = launch_fold(ws, c, bias, m, n, ldc, g.k_splits, batch, g.stride_c, accumulate);
        if (ws) bh_free(ws);
        return rc;
    }

    if (cfg == 0) {
        if (k == 0 && !accumulate && !bias) {   // empty contraction: zeros (linear.c zero-fills its output)
            for (int64_t bt = 0; bt < batch; bt++)
                for (int64_t r = 0; r < m; r++) bh_memset_zero(c + bt * g.stride_c + r * ldc, sizeof(float) * (size_t)n);
            return BH_OK;
        }
        dim3 grid((unsigned)ceil_div(n, 32), (unsigned)ceil_div(m, 32), (unsigned)batch);
        BH_CHECK_ARG(grid.y <= 65535, "m too large for the fallback kernel");
        hipLaunchKernelGGL(gemm_fallback_kernel, grid, dim3(256), 0, stream(), g, trans_a, trans_b);
        return BH_LAUNCH_CHECK("gemm_fallback_kernel");
    }

    const int bm = cfg == 7 ? 64 : (cfg == 2 || cfg == 3) ? 256 : 128, bn = cfg == 7 ? 64 : (cfg == 2 || cfg == 4) ? 256 : 128;
    g.tiles_m = (int)ceil_div(m, bm);
    g.tiles_n = (int)ceil_div(n, bn);
    float* ws = nullptr;
    {
        int64_t splits = (((g_force_cfg >= 1 && g_force_cfg <= 4) || g_force_cfg == 7) && g_force_cfg != cfg_planned) ? default_splits(cfg, m, n, k, batch) : plan_splits;
        if (g_force_splits > 0 && g_force_splits <= k / kBK) splits = g_force_splits;
        if (segmented) splits = 1;
        if (splits > 1) {
            // whole pairs of k-tiles per workgroup where the contraction allows it (the paired main loop needs them)
            const int64_t unit = (k % (2 * kBK) == 0 && cfg != 1 && cfg != 7) ? 2 * kBK : kBK;
            g.k_per_split = ceil_div(ceil_div(k, splits), unit) * unit;
            g.k_splits = (int)ceil_div(k, g.k_per_split);
        }
    }
    // the direct-to-LDS loader cannot zero-fill a k tail, and its edge clamps need 4 valid floats in a row
    // (and it addresses a tile with 32-bit byte offsets from the tile's first row: leading dimensions below 2^22)
    const bool direct = g_force_direct != 0 && k % kBK == 0 && k >= kBK && (a_kc || m >= 4) && (b_kc || n >= 4) &&
                        lda < ((int64_t)1 << 22) && ldb < ((int64_t)1 << 22);
    // the eight-wavefront tiles take two k-tiles per barrier whenever every workgroup's contraction range is whole pairs
    // (measured at the block's shapes with the staggered loads: 1.5-3 % faster than one tile per barrier on all three)
    const bool pairs = direct && g_pairs && k % (2 * kBK) == 0 && (g.k_splits == 1 || g.k_per_split % (2 * kBK) == 0);
    if (tab) {
        // table kernels exist for the direct loaders only: paired k-tiles on the eight-wavefront tiles, single ones on 128x128;
        // a split launch folds with 16-byte pieces into dense outputs
        if (!direct || (cfg != 1 && !pairs)) return kTabUnsupported;
        if (g.k_splits > 1 && (ldc != n || n % 4 != 0 || ceil_div(m * n / 4, 64) > 0x7fffffff)) return kTabUnsupported;
        if (segmented && tab->seg_k % (2 * kBK) != 0) return kTabUnsupported;
    }
    GemmArgs run = g;
    if (g.k_splits > 1) {
        ws = (float*)bh_malloc(sizeof(float) * (size_t)(g.k_splits * batch * m * n));
        if (!ws) return BH_ENOMEM;
        run.c = ws;
        run.ldc = n;
        run.stride_c = m * n;
    }
    int rc;
    if (tab) {
        switch (cfg) {
            case 2: rc = launch_mfma_tab<CfgBig, 2>(run, batch, a_kc, b_kc, tab); break;
            case 3: rc = launch_mfma_tab<CfgTall, 2>(run, batch, a_kc, b_kc, tab); break;
            case 4: rc = launch_mfma_tab<CfgWide, 2>(run, batch, a_kc, b_kc, tab); break;
            default: rc = launch_mfma_tab<CfgMid, 1>(run, batch, a_kc, b_kc, tab); break;
        }
        if (rc == BH_OK && g.k_splits > 1) {
            const int64_t per4 = m * n / 4;
            hipLaunchKernelGGL(splitk_fold_vec_tab_kernel, dim3((unsigned)ceil_div(per4, 64), (unsigned)batch), dim3(64), 0, stream(),
                               ws, *tab, per4, n, g.k_splits, accumulate);
            rc = BH_LAUNCH_CHECK("splitk_fold_vec_tab_kernel");
        }
        if (ws) bh_free(ws);
        return rc;
    }
    switch (cfg) {
        case 2: rc = pairs ? launch_mfma_pairs<CfgBig>(run, batch, a_kc, b_kc) : launch_mfma_layout<CfgBig>(run, batch, a_kc, b_kc, direct); break;
        case 3: rc = pairs ? launch_mfma_pairs<CfgTall>(run, batch, a_kc, b_kc) : launch_mfma_layout<CfgTall>(run, batch, a_kc, b_kc, direct); break;
        case 4: rc = pairs ? launch_mfma_pairs<CfgWide>(run, batch, a_kc, b_kc) : launch_mfma_layout<CfgWide>(run, batch, a_kc, b_kc, direct); break;
        case 7: rc = launch_mfma_layout<CfgSmall>(run, batch, a_kc, b_kc, direct); break;
        default: rc = launch_mfma_layout<CfgMid>(run, batch, a_kc, b_kc, direct); break;
    }
    if (rc == BH_OK && g.k_splits > 1) rc = launch_fold(ws, c, bias, m, n, ldc, g.k_splits, batch, g.stride_c, accumulate);
    if (ws) bh_free(ws);
    return rc;
}

extern "C" {

int bh_gemm(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, const float* a, int64_t lda, const float* b,
            int64_t ldb, float* c, int64_t ldc, const float* bias, int accumulate, int64_t batch) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(m >= 0 && n >= 0 && k >= 0 && batch >= 0, "negative dimension");
    if (m == 0 || n == 0 || batch == 0) return BH_OK;
    BH_CHECK_ARG(a && b && c, "null pointer");
    BH_CHECK_ARG(lda >= (trans_a ? m : k) && ldb >= (trans_b ? k : n) && ldc >= n, "leading dimension too small");
    BH_CHECK_ARG(batch <= 65535, "batch too large");
    ProfScope prof(BH_PROF_GEMM, 2.0 * (double)m * (double)n * (double)k * (double)batch);
    return gemm_core(trans_a, trans_b, m, n, k, a, lda, b, ldb, c, ldc, bias, accumulate, batch, nullptr);
}

// c[g] (+)= op(a[g]) . op(b[g]) (+ bias[g]) for `groups` problems of one shape: one launch where the shape takes the
// matrix-core tiles with direct loads, the same kernels one after the other otherwise (the same products; a long
// contraction may be cut differently for the group than for a single product)
int bh_gemm_grouped(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, int groups, const float* const* a, int64_t lda,
                    const float* const* b, int64_t ldb, float* const* c, int64_t ldc, const float* const* bias, int accumulate) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(m >= 0 && n >= 0 && k >= 0, "negative dimension");
    BH_CHECK_ARG(groups >= 1 && groups <= kMaxGroups, "1 to 4 groups");
    BH_CHECK_ARG(a && b && c, "null table");
    if (m == 0 || n == 0) return BH_OK;
    for (int i = 0; i < groups; i++) BH_CHECK_ARG(a[i] && b[i] && c[i], "null pointer");
    BH_CHECK_ARG(lda >= (trans_a ? m : k) && ldb >= (trans_b ? k : n) && ldc >= n, "leading dimension too small");
    ProfScope prof(BH_PROF_GEMM, 2.0 * (double)m * (double)n * (double)k * (double)groups);   // the launches below nest inside it
    if (groups > 1 && !g_no_tables) {
        GemmTab t = {};
        for (int i = 0; i < groups; i++) {
            t.a[i] = a[i]; t.b[i] = b[i]; t.c[i] = c[i];
            t.bias[i] = bias ? bias[i] : nullptr;
        }
        t.k_segments = 1;
        const int rc = gemm_core(trans_a, trans_b, m, n, k, nullptr, lda, nullptr, ldb, nullptr, ldc, nullptr, accumulate, groups, &t);
        if (rc != kTabUnsupported) return rc;
    }
    for (int i = 0; i < groups; i++) {
        const int rc = bh_gemm(trans_a, trans_b, m, n, k, a[i], lda, b[i], ldb, c[i], ldc, bias ? bias[i] : nullptr, accumulate, 1);
        if (rc != BH_OK) return rc;
    }
    return BH_OK;
}

// c (+)= sum_s op(a[s]) . op(b[s]) (+ bias): one product whose contraction runs over `segments` operand pairs of k each.
// One launch where the shape takes the matrix-core tiles with direct loads; otherwise the pairs one after the other,
// each adding into c.  The two forms add the segments' products in different orders (one long chain against partial
// sums), so they agree to fp32 rounding, not bit for bit; which form runs depends on the shape only.
int bh_gemm_ksegments(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, int segments, const float* const* a, int64_t lda,
                      const float* const* b, int64_t ldb, float* c, int64_t ldc, const float* bias, int accumulate) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(m >= 0 && n >= 0 && k >= 0, "negative dimension");
    BH_CHECK_ARG(segments >= 1 && segments <= kMaxSegments, "1 to 3 segments");
    BH_CHECK_ARG(a && b && c, "null pointer");
    if (m == 0 || n == 0) return BH_OK;
    for (int i = 0; i < segments; i++) BH_CHECK_ARG(a[i] && b[i], "null pointer");
    BH_CHECK_ARG(lda >= (trans_a ? m : k) && ldb >= (trans_b ? k : n) && ldc >= n, "leading dimension too small");
    ProfScope prof(BH_PROF_GEMM, 2.0 * (double)m * (double)n * (double)k * (double)segments);
    if (segments > 1 && k > 0 && !g_no_tables) {
        GemmTab t = {};
        for (int i = 0; i < segments; i++) {
            t.a[i] = a[i]; t.b[i] = b[i];
        }
        t.c[0] = c;
        t.bias[0] = bias;
        t.k_segments = segments;
        t.seg_k = k;
        const int rc = gemm_core(trans_a, trans_b, m, n, k * segments, nullptr, lda, nullptr, ldb, nullptr, ldc, nullptr, accumulate, 1, &t);
        if (rc != kTabUnsupported) return rc;
    }
    for (int i = 0; i < segments; i++) {
        const int rc = bh_gemm(trans_a, trans_b, m, n, k, a[i], lda, b[i], ldb, c, ldc, i == 0 ? bias : nullptr, i == 0 ? accumulate : 1, 1);
        if (rc != BH_OK) return rc;
    }
    return BH_OK;
}

// test/benchmark hook: 1 = grouped entry points always run their problems one after the other
int bh_gemm_no_tables(int off) {
    g_no_tables = off != 0;
    return BH_OK;
}

int bh_transpose_last2(const float* a, float* out, int64_t batch, int64_t rows, int64_t cols) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(batch >= 0 && rows >= 0 && cols >= 0, "negative dimension");
    if (batch * rows * cols == 0) return BH_OK;
    BH_CHECK_ARG(a && out && batch <= 65535, "bad argument");
    dim3 grid((unsigned)ceil_div(cols, 32), (unsigned)ceil_div(rows, 32), (unsigned)batch);
    BH_CHECK_ARG(grid.y <= 65535, "too many rows");
    hipLaunchKernelGGL(transpose_kernel, grid, dim3(256), 0, stream(), a, out, rows, cols);
    return BH_LAUNCH_CHECK("transpose_kernel");
}

}  // extern "C"

template <typename T>
static int swap_dims(const T* in, T* out, int64_t a, int64_t d0, int64_t b, int64_t d1, int64_t c) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(a >= 0 && d0 >= 0 && b >= 0 && d1 >= 0 && c >= 0, "negative dimension");
    const double elems = (double)a * (double)d0 * (double)b * (double)d1 * (double)c;
    BH_CHECK_ARG(elems < 9.0e18 / sizeof(T), "tensor too large");
    const int64_t total = a * d0 * b * d1 * c;
    if (total == 0) return BH_OK;
    BH_CHECK_ARG(in && out, "null pointer");
    int64_t blocks = ceil_div(total, 256);
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL((swap_dims_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream(), in, out, d0, b, d1, c, total);
    return BH_LAUNCH_CHECK("swap_dims_kernel");
}

extern "C" {

int bh_swap_dims(const float* in, float* out, int64_t a, int64_t d0, int64_t b, int64_t d1, int64_t c) {
    if (in && out && a > 0 && d0 > 0 && d1 > 0 && b == 1 && c == 1 && a <= 65535 && ceil_div(d0, 32) <= 65535)
        return bh_transpose_last2(in, out, a, d0, d1);
    return swap_dims<float>(in, out, a, d0, b, d1, c);
}

int bh_swap_dims_f64(const double* in, double* out, int64_t a, int64_t d0, int64_t b, int64_t d1, int64_t c) {
    return swap_dims<double>(in, out, a, d0, b, d1, c);
}

int bh_dense_backward(const float* x, const float* w, const float* dy, float* dx, float* gw, float* gb, int64_t m,
                      int64_t k, int64_t n, int accumulate) {
    return bh_dense_backward_into(x, w, dy, dx, gw, gb, m, k, n, accumulate, 0);
}

int bh_dense_backward_into(const float* x, const float* w, const float* dy, float* dx, float* gw, float* gb, int64_t m,
                           int64_t k, int64_t n, int accumulate, int accumulate_dx) {
    BH_REQUIRE_INIT();
    BH_CHECK_ARG(m >= 0 && k >= 0 && n >= 0, "negative dimension");
    BH_CHECK_ARG(x && w && dy, "null pointer");
    int rc = BH_OK;
    // dX[m,k] (+)= dY[m,n] . W[k,n]^T
    if (dx) rc = bh_gemm(0, 1, m, k, n, dy, n, w, n, dx, k, nullptr, accumulate_dx, 1);
    // dW[k,n] (+)= X[m,k]^T . dY[m,n]
    // (running the two products side by side on two streams was measured: 6.30 ms per block step against 5.88)
    if (rc == BH_OK && gw) rc = bh_gemm(1, 0, k, n, m, x, k, dy, n, gw, n, nullptr, accumulate, 1);
    if (rc == BH_OK && gb) rc = bh_colsum(dy, gb, m, n, accumulate);
    return rc;
}

}  // extern "C"
