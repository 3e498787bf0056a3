// bh_conv.hip - 2-D convolution (NCHW, square kernel) and max pooling, forward and backward.
//
// Replaces the loops of the reference's convolution and pooling layers:
//   boat_conv_layer_forward            src/layers/conv.c:326-437
//   compute_weight_gradient            src/layers/conv.c:105-163
//   compute_bias_gradient              src/layers/conv.c:165-201
//   compute_input_gradient             src/layers/conv.c:46-103
//   boat_pool_layer_forward/backward   src/layers/pool.c:63-218
//
// Forward is a direct gather, one lane per output element, in the reference's fp32 operation order (per input
// channel a running sum over the taps, added to the output, bias last): bit-identical, so the pooling layer behind it
// picks the same maxima as the reference.
//
// Backward is three contractions on the matrix cores through bh_gemm, with K = in_channels*k*k and P = batch*ho*wo:
//   dyp [oc][P]   = dy regrouped from [batch][oc][ho*wo]      (one permute kernel)
//   col [P][K]    = patches of x (im2col, zero outside the image)
//   gw  [oc][K]  (+)= dyp . col                                (the contraction runs over all P output positions)
//   dcol[P][K]    = dyp^T . w                                  then dx gathers its <= k*k entries of dcol (col2im)
//   gb  [oc]     (+)= row sums of dyp
// No atomics; every result element is written once (deterministic).  The gradient sums run in MFMA and tree order,
// so they agree with the reference to rounding, not bit for bit.
//
// Input gradient.  The reference pairs tap (kh, kw) of the scatter ih = oh*stride - pad + kh with the weight
// of the mirrored tap (k-1-kh, k-1-kw) (conv.c:86-88); that is the gradient of a different layer, and its own
// gradient check only looks at weight and bias gradients (tests/unit/test_conv_gradient_check.c:317-332).
// flip_taps == 0 computes the true gradient dx[ih,iw] = sum w[oc,ic,kh,kw]*dy[oh,ow]; flip_taps != 0 reproduces
// the reference's pairing (the weights are mirrored into a scratch copy first), so that its numbers can be checked.
#include "bh_common.h"
#include <type_traits>

#include <math.h>

namespace bh {

constexpr int kCBlock = 256;
typedef float floatx16 __attribute__((ext_vector_type(16)));

struct ConvShape {
    int batch, ic, h, w, oc, k, stride, pad, ho, wo;
};

// One lane per output position, kOcTile output channels per lane: the k x k patch of an input channel is loaded once
// and feeds kOcTile running sums; the weights of a workgroup's channel group are wave-uniform (the group comes from
// blockIdx), so they arrive through the scalar path as whole k*k rows.  Per output element the operation order is the
// reference's: for each input channel a sum over the taps in (kh, kw) order, taps outside the image skipped, added to
// the output; bias last (conv.c:398-436).  "Skipped" is a select, not a branch: a tap outside the image reads a clamped
// (valid) address and leaves the running sum untouched.
template <int K, int kOcTile>   // kernel size (compile time: the taps live in registers) and output channels per lane
__global__ __launch_bounds__(kCBlock) void conv2d_fwd_kernel(const float* __restrict__ x, const float* __restrict__ wt,
                                                             const float* __restrict__ bias, float* __restrict__ y,
                                                             ConvShape c) {
    const int per = c.ho * c.wo;
    const int p = blockIdx.x * kCBlock + threadIdx.x;
    const int oc0 = blockIdx.y * kOcTile;
    const int b = blockIdx.z;
    if (p >= per) return;
    const int oh = p / c.wo, ow = p % c.wo;
    const int ih0 = oh * c.stride - c.pad, iw0 = ow * c.stride - c.pad;
    bool valid[K * K];
    int off[K * K];
#pragma unroll
    for (int kh = 0; kh < K; kh++)
#pragma unroll
        for (int kw = 0; kw < K; kw++) {
            const int ih = ih0 + kh, iw = iw0 + kw;
            valid[kh * K + kw] = ih >= 0 && ih < c.h && iw >= 0 && iw < c.w;
            off[kh * K + kw] = min(max(ih, 0), c.h - 1) * c.w + min(max(iw, 0), c.w - 1);
        }
    const float* wrow[kOcTile];      // channel group rows, clamped to the last real channel (extra lanes are not stored)
#pragma unroll
    for (int o = 0; o < kOcTile; o++) wrow[o] = wt + (int64_t)min(oc0 + o, c.oc - 1) * c.ic * K * K;
    float out[kOcTile];
#pragma unroll
    for (int o = 0; o < kOcTile; o++) out[o] = 0.f;
    // The loop on input channels is software pipelined: the taps of channel ci+1 are in flight while channel ci is summed
    // (the weights are the same for the whole workgroup and come through the scalar cache).
    const float* xp = x + (int64_t)b * c.ic * c.h * c.w;
    const int plane = c.h * c.w;
    float xv[K * K];
#pragma unroll
    for (int t = 0; t < K * K; t++) xv[t] = xp[off[t]];
    const auto add_channel = [&](int ci) {
#pragma unroll
        for (int o = 0; o < kOcTile; o++) {
            const float* wp = wrow[o] + ci * K * K;
            float sum = 0.f;
#pragma unroll
            for (int t = 0; t < K * K; t++) {
                const float term = sum + xv[t] * wp[t];
                sum = valid[t] ? term : sum;
            }
            out[o] += sum;
        }
    };
    for (int ci = 0; ci + 1 < c.ic; ci++) {
        float xn[K * K];
#pragma unroll
        for (int t = 0; t < K * K; t++) xn[t] = xp[(int64_t)(ci + 1) * plane + off[t]];
        add_channel(ci);
#pragma unroll
        for (int t = 0; t < K * K; t++) xv[t] = xn[t];
    }
    add_channel(c.ic - 1);
#pragma unroll
    for (int o = 0; o < kOcTile; o++) {
        if (oc0 + o >= c.oc) break;
        float v = out[o];
        if (bias) v += bias[oc0 + o];
        y[((int64_t)b * c.oc + oc0 + o) * per + p] = v;
    }
}

// any kernel size: one lane per output element, taps looped at run time, same operation order
__global__ __launch_bounds__(kCBlock) void conv2d_fwd_generic_kernel(const float* __restrict__ x, const float* __restrict__ wt,
                                                                     const float* __restrict__ bias, float* __restrict__ y,
                                                                     ConvShape c, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * kCBlock + threadIdx.x;
    if (i >= total) return;
    const int ow = (int)(i % c.wo);
    const int oh = (int)((i / c.wo) % c.ho);
    const int oc = (int)((i / ((int64_t)c.wo * c.ho)) % c.oc);
    const int b = (int)(i / ((int64_t)c.wo * c.ho * c.oc));
    const int ih0 = oh * c.stride - c.pad, iw0 = ow * c.stride - c.pad;
    float out = 0.f;
    for (int ci = 0; ci < c.ic; ci++) {
        const float* xp = x + ((int64_t)b * c.ic + ci) * c.h * c.w;
        const float* wp = wt + ((int64_t)oc * c.ic + ci) * c.k * c.k;
        float sum = 0.f;
        for (int kh = 0; kh < c.k; kh++) {
            const int ih = ih0 + kh;
            if (ih < 0 || ih >= c.h) continue;
            for (int kw = 0; kw < c.k; kw++) {
                const int iw = iw0 + kw;
                if (iw < 0 || iw >= c.w) continue;
                sum += xp[ih * c.w + iw] * wp[kh * c.k + kw];
            }
        }
        out += sum;
    }
    if (bias) out += bias[oc];
    y[i] = out;
}

// ---- forward on the matrix cores, 3x3 kernels (opt-in: the sums run in MFMA order, so the result agrees with the
// reference to rounding, not bit for bit, and a pooling layer behind it may pick another of two near-equal maxima) ----
// The convolution as one contraction y[oc][n] = sum_kk w[oc][kk] * patch[kk][n], kk = (ci, kh, kw), n = (b, oh, ow),
// on v_mfma_f32_32x32x2_f32 without a patch matrix in memory: output channel = accumulator row, output position =
// lane, so a lane fetches the patch values of its own position straight from x (neighbouring lanes read neighbouring
// pixels; taps outside the image and channels past the last read a clamped address and count as zero) and the stores
// of one accumulator register are 32 consecutive positions of one channel plane.  One matrix instruction contracts two
// consecutive kk; the lane half decides which of the two a lane supplies, so per pair of input channels (18 kk) a lane
// needs nine patch values and, per 32 output channels, nine weights.  The weights of the workgroup's 64 output channels
// and of up to 32 input channels sit in LDS, split by kk parity ([oc][kk & 1][kk >> 1], row stride odd: conflict free
// 4-byte reads).
// Workgroup: 2 * SPLIT wavefronts = 64 channels x 64 positions; a wavefront owns 32 positions, both 32-channel halves
// (a patch value feeds two products) and every SPLIT-th pair of input channels; the SPLIT partial sums are added in a
// fixed order through LDS.  SPLIT = 4 (512 lanes, one workgroup per CU) for small layers: they are bound by the latency
// of the patch loads, and four wavefronts per position tile have four times the loads in flight.  SPLIT = 2 (256 lanes,
// two workgroups per CU) for layers with many workgroups: one workgroup's staging, reduction and stores run under the
// other's products.  grid (ceil(P/64), ceil(oc/64)).
// Kernel sizes 3 and 5 (template parameter K, T = K*K taps): a lane holds four buffers of T patch values, and a 7x7
// kernel's 196 would not leave room for anything else.  The weights of 32 input channels x 64 output channels x 25 taps
// do not fit LDS, so a 32-channel stage is staged in NSUB parts of CI channels (3x3: one of 32, 5x5: two of 16).
constexpr int kFmStage = 32;                    // input channels per stage (the unit in which the patch buffers rotate)
template <int K> struct FmGeom {
    static constexpr int T = K * K;                          // taps per channel
    static constexpr int CI = K == 3 ? 32 : 16;              // input channels per LDS part
    static constexpr int NSUB = kFmStage / CI;               // parts per stage
    static constexpr int KK = CI * T;                        // contraction indices per part (a multiple of 16)
    static constexpr int ROW = KK + 1;                       // LDS row stride in floats (odd: conflict-free 4-byte reads)
    static constexpr size_t kLds = sizeof(float) * (64 * ROW + 64);      // weights + bias
};
constexpr int64_t kFmBlocksSplit2 = 257;        // from this many workgroups on (more than the part has CUs) a 3x3 layer runs with SPLIT = 2

template <int SPLIT, int K>                     // wavefronts that share a position tile: 2 or 4; kernel size 3 or 5
__global__ __launch_bounds__(128 * SPLIT, 2) void conv2d_fwd_mfma_kernel(const float* __restrict__ x, const float* __restrict__ wt,
                                                                 const float* __restrict__ bias, float* __restrict__ y,
                                                                 ConvShape c, int positions) {
    using Geo = FmGeom<K>;
    constexpr int T = Geo::T, CI = Geo::CI, NSUB = Geo::NSUB, KK = Geo::KK, ROW = Geo::ROW;
    constexpr int TPS = CI / 2 / SPLIT;                    // turns (pairs of channels) of a wavefront per part: 2, 4 or 8
    // how many turns ahead the patch values are fetched.  3x3: three (four buffers of 9 that rotate in fours); 5x5: one (two
    // buffers of 25 -- four would not fit the register file, and one turn is 50 matrix instructions, longer than a trip to memory)
    constexpr int AHEAD = K == 3 ? 3 : 1;
    static_assert(KK % 16 == 0 && TPS % (AHEAD + 1) == 0, "the patch buffers rotate in step with the parts");
    extern __shared__ __align__(16) float wl[];          // [64][ROW] + bias[64]; the weights' part holds the partial sums afterwards
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, half = lane >> 5;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);     // in a scalar register: what follows from it is the same for the whole wavefront
    const int wn = wv & 1, kg = wv >> 1;
    const int oc0 = blockIdx.y * 64;
    const int per = c.ho * c.wo, plane = c.h * c.w;
    const int n_raw = blockIdx.x * 64 + wn * 32 + r;
    const int n = min(n_raw, positions - 1);
    const int b = n / per, p = n - b * per;
    const int oh = p / c.wo, ow = p - oh * c.wo;
    const int ih0 = oh * c.stride - c.pad, iw0 = ow * c.stride - c.pad;
    // the T contraction indices 2j + half of a channel pair: byte offset of the lane's patch value from the first
    // channel's plane in image 0 (the second channel lies one plane further; byte offsets fit 32 bits, a tensor has fewer
    // than 2^30 elements), and whether the tap lies inside the image.  The T conditions live as wavefront masks in
    // scalar registers, so that a turn costs one vector instruction per load and one per select: anything more per
    // patch value competes with the matrix instructions for issue slots.
    unsigned offb[T];
    bool in[T];
#pragma unroll
    for (int j = 0; j < T; j++) {
        const int kk = 2 * j + half, cp = kk >= T ? 1 : 0, tap = kk - T * cp;
        const int kh = tap / K, kw = tap - K * kh;
        const int ih = ih0 + kh, iw = iw0 + kw;
        in[j] = ih >= 0 && ih < c.h && iw >= 0 && iw < c.w;
        offb[j] = 4u * (unsigned)((b * c.ic + cp) * plane + min(max(ih, 0), c.h - 1) * c.w + min(max(iw, 0), c.w - 1));
    }
    const float* wrow = wl + r * ROW + half * (KK / 2);
    // the second 32 channels' rows lie beyond the reach of a paired LDS read's offsets from wrow: their own base, kept
    // in a register of its own (the empty statement hides that it is wrow plus a constant, which the compiler would
    // otherwise add again in every turn)
    int far_row = (r + 32) * ROW + half * (KK / 2);
    asm volatile("" : "+v"(far_row));
    floatx16 acc[2];
#pragma unroll
    for (int e = 0; e < 16; e++) acc[0][e] = acc[1][e] = 0.f;

    // patch values of channels ci, ci + 1: the loads go to clamped (valid) addresses and nothing looks at their results
    // until mask() runs three turns later -- a select right behind a load would make the wavefront wait for it there
    const auto fetch = [&](int ci, float (&v)[T]) {
        const char* xc = reinterpret_cast<const char*>(x + (int64_t)ci * plane);     // the same for every lane
#pragma unroll
        for (int j = 0; j < T; j++) {
            // the empty statement (it leaves the offset as it is) keeps the offset's widening next to the load, where it
            // folds into the load's scalar-base-plus-32-bit-offset form; hoisted out of the loop it would hold T
            // register pairs
            asm volatile("" : "+v"(offb[j]));
            v[j] = *reinterpret_cast<const float*>(xc + offb[j]);
        }
    };
    const auto mask = [&](float (&v)[T]) {                 // taps outside the image count as zero
#pragma unroll
        for (int j = 0; j < T; j++) v[j] = in[j] ? v[j] : 0.f;
    };
    const int l16 = tid & 15, rg = tid >> 4;               // weight staging: 16 lanes per row, 8 * SPLIT rows per pass
    // the bias of the 64 channels travels with the first part's weights and waits in LDS behind them: fetched at the end
    // it would cost a trip to memory of its own
    float* bl = wl + 64 * ROW;
    float bias_in = 0.f;
    if (tid < 64 && bias && oc0 + tid < c.oc) bias_in = bias[oc0 + tid];
    // this wavefront's pairs of input channels are kg, kg + SPLIT, ... over the whole layer: a multiple of the number of
    // patch buffers to a part, so the buffers take turns in step with the parts (a register copy would have to wait for the
    // loads it copies) and the patch values run AHEAD turns ahead, across part boundaries too (a 3x3 turn's 18 products
    // take a quarter of a trip to memory)
    const int all_pairs = c.ic / 2;                        // an odd channel count's last channel follows behind its part
    float x0[T], x1[T], x2[T], x3[T];
    // a fetch past the last pair re-reads the last pair (valid memory, never used): with the same number of loads on
    // every path the waits the compiler places in front of a turn's selects count exactly the three turns in flight
    // (a fetch under a condition makes it wait for everything but the current turn's loads)
    const auto fetch_pair = [&](int pair, float (&v)[T]) { fetch(2 * min(pair, all_pairs - 1), v); };
    if (all_pairs > 0) {
        fetch_pair(kg, x0);
        if constexpr (AHEAD == 3) {
            fetch_pair(kg + SPLIT, x1);
            fetch_pair(kg + 2 * SPLIT, x2);
        }
    }
    bool first_part = true;
    // one part of a stage: CI channels from cs on; FULL: all its pairs of channels exist, so every turn runs unconditionally
    const auto part = [&](int cs, auto full_const) {
        constexpr bool FULL = decltype(full_const)::value;
        if (!first_part) __syncthreads();                  // every wavefront is done with the previous part's weights
        const int real = min(CI, c.ic - cs) * T;
        // weights of the part: row oc of w holds its ic*T values contiguously, so a part's run of chunk*T is contiguous;
        // what lies past it (an odd channel count's partner, a short last part) is zero.  A lane's loads of RQ rows are
        // in flight together before their LDS stores.
        constexpr int RQ = K == 3 ? 2 : 1;                  // rows a lane has in flight (5x5: a row is 25 loads, and registers are short)
#pragma unroll
        for (int q0 = 0; q0 < 8 / SPLIT; q0 += RQ) {
            float v[RQ][KK / 16];
#pragma unroll
            for (int q = 0; q < RQ; q++) {
                const int o = rg + 8 * SPLIT * (q0 + q);
                const float* src = wt + ((int64_t)min(oc0 + o, c.oc - 1) * c.ic + cs) * T;
                if constexpr (K == 3) {
#pragma unroll
                    for (int i = 0; i < KK / 16; i++) {
                        const int kk = l16 + 16 * i;
                        v[q][i] = src[FULL ? kk : min(kk, real - 1)];     // a valid address in any case; what does not exist becomes zero below
                    }
                } else {
                    // 25 clamped addresses would take 50 registers: a short part reads on into the next rows of w, whose values
                    // become zeros below like everything past the part; only where that would leave the tensor (its last
                    // rows) are the indices clamped, a few at a time
                    if (FULL || src + KK <= wt + (int64_t)c.oc * c.ic * T) {
#pragma unroll
                        for (int i = 0; i < KK / 16; i++) v[q][i] = src[l16 + 16 * i];
                    } else {
#pragma unroll
                        for (int i0 = 0; i0 < KK / 16; i0 += 5) {
#pragma unroll
                            for (int i = i0; i < i0 + 5; i++) v[q][i] = src[min(l16 + 16 * i, real - 1)];
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            }
#pragma unroll
            for (int q = 0; q < RQ; q++) {
                const int o = rg + 8 * SPLIT * (q0 + q);
                float* dst = wl + o * ROW;
                // kk = l16 + 16 i lands at [kk & 1][kk >> 1]: the parity is the lane's, the rest a constant step of 8
                const int lbase = (l16 & 1) * (KK / 2) + (l16 >> 1);
#pragma unroll
                for (int i = 0; i < KK / 16; i++) {
                    const int kk = l16 + 16 * i;
                    dst[lbase + 8 * i] = (oc0 + o < c.oc && (FULL || kk < real)) ? v[q][i] : 0.f;
                }
            }
        }
        if (first_part && tid < 64) bl[tid] = bias_in;
        first_part = false;
        __syncthreads();
        const int first = cs / 2 + kg;                     // this wavefront's first pair of the part
        const auto products = [&](int turn, float (&cur)[T], float (&ahead)[T]) {
            const int gp = first + turn * SPLIT;
            if (FULL) fetch_pair(gp + AHEAD * SPLIT, ahead);
            else if (gp + AHEAD * SPLIT < all_pairs) fetch(2 * (gp + AHEAD * SPLIT), ahead);
            // nothing moves across this line: left to itself the scheduler lifts the selects of a later turn up to their
            // loads, three turns early, and the wavefront waits for those loads there
            __builtin_amdgcn_sched_barrier(0);
            mask(cur);
            const float* wp = wrow + (kg + turn * SPLIT) * T;
            const float* wq = wl + far_row + (kg + turn * SPLIT) * T;
            if constexpr (K == 3) {
#pragma unroll
                for (int j = 0; j < T; j++) {
                    acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(wp[j], cur[j], acc[0], 0, 0, 0);
                    acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(wq[j], cur[j], acc[1], 0, 0, 0);
                }
            } else {
                // K taps at a time, the next K taps' weights read from LDS while these run: left alone the compiler reads all
                // 2T weights of the turn first, and they do not fit beside the patch buffers
                float wa[K], wb[K];
#pragma unroll
                for (int i = 0; i < K; i++) {
                    wa[i] = wp[i];
                    wb[i] = wq[i];
                }
#pragma unroll
                for (int ch = 0; ch < K; ch++) {
                    float na[K], nb[K];
                    if (ch + 1 < K) {
#pragma unroll
                        for (int i = 0; i < K; i++) {
                            na[i] = wp[(ch + 1) * K + i];
                            nb[i] = wq[(ch + 1) * K + i];
                        }
                    }
#pragma unroll
                    for (int i = 0; i < K; i++) {
                        acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(wa[i], cur[ch * K + i], acc[0], 0, 0, 0);
                        acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(wb[i], cur[ch * K + i], acc[1], 0, 0, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if (ch + 1 < K) {
#pragma unroll
                        for (int i = 0; i < K; i++) {
                            wa[i] = na[i];
                            wb[i] = nb[i];
                        }
                    }
                }
            }
        };
        const auto have = [&](int turn) { return FULL || first + turn * SPLIT < all_pairs; };
        if constexpr (AHEAD == 1) {
#pragma unroll
            for (int turn = 0; turn < TPS; turn += 2) {
                if (have(turn)) products(turn, x0, x1);
                if (have(turn + 1)) products(turn + 1, x1, x0);
            }
        } else if (FULL) {
#pragma unroll
            for (int turn = 0; turn < TPS; turn += 4) {
                products(turn, x0, x3);
                products(turn + 1, x1, x0);
                products(turn + 2, x2, x1);
                products(turn + 3, x3, x2);
            }
        } else {
            for (int turn = 0; turn < TPS && have(turn); turn += 4) {
                products(turn, x0, x3);
                if (have(turn + 1)) products(turn + 1, x1, x0);
                if (have(turn + 2)) products(turn + 2, x2, x1);
                if (have(turn + 3)) products(turn + 3, x3, x2);
            }
        }
        // the single last channel of an odd count: one wavefront per position half takes it with its lanes of the
        // pair's second channel reading the first and counting as zero (the weights past the last channel are zero too)
        const int single = c.ic / 2 - cs / 2;             // its pair's index within this part
        if ((c.ic & 1) && cs + CI >= c.ic && kg == single % SPLIT) {
            const char* xc = reinterpret_cast<const char*>(x + (int64_t)(c.ic - 1) * plane);
            const float* wp = wrow + single * T;
#pragma unroll
            for (int j = 0; j < T; j++) {
                const bool other = 2 * j + half >= T;
                float v = *reinterpret_cast<const float*>(xc + (offb[j] - (other ? 4u * (unsigned)plane : 0u)));
                v = (in[j] && !other) ? v : 0.f;
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(wp[j], v, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(wp[32 * ROW + j], v, acc[1], 0, 0, 0);
            }
        }
    };
    int cs_run = 0;
    for (; cs_run + kFmStage <= 2 * all_pairs; cs_run += kFmStage) {       // full stages
        part(cs_run, std::true_type{});
        if constexpr (NSUB == 2) part(cs_run + CI, std::true_type{});
    }
    // a short last stage (at most one: it holds fewer than 32 channels); its parts as far as they hold channels
    if (cs_run < c.ic) {
        part(cs_run, std::false_type{});
        if constexpr (NSUB == 2)
            if (cs_run + CI < c.ic) part(cs_run + CI, std::false_type{});
    }
    __syncthreads();                                       // the weights are no longer needed: their LDS holds the partial sums
    if (kg > 0) {
        float* red = wl + (((kg - 1) * 2 + wn) * 32) * 64 + lane;  // [kg - 1][wn][t * 16 + e][lane]
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int e = 0; e < 16; e++) red[(t * 16 + e) * 64] = acc[t][e];
    }
    __syncthreads();
    if (kg > 0 || n_raw >= positions) return;
#pragma unroll
    for (int g = 0; g < SPLIT - 1; g++) {
        const float* src = wl + ((g * 2 + wn) * 32) * 64 + lane;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[t][e] += src[(t * 16 + e) * 64];
    }
    float* yp = y + (int64_t)b * c.oc * per + p;
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int oc = oc0 + t * 32 + (e >> 2) * 8 + half * 4 + (e & 3);
            if (oc < c.oc) yp[(int64_t)oc * per] = acc[t][e] + bl[oc - oc0];
        }
}

// dyp[oc][b][p] = dy[b][oc][p], p over the ho*wo output positions
// The three rearrangement kernels of the backward pass do no arithmetic, so their index computation is their cost:
// the grid carries the outer indices (y, z) and a lane only splits its position inside one image plane (one 32-bit
// division).  Written with a flat index and 64-bit div/mod they ran at a seventh of the memory rate.

// dyp[oc][b][p] = dy[b][oc][p], p over the ho*wo output positions; grid (ceil(per/256), oc, batch)
__global__ __launch_bounds__(kCBlock) void nchw_to_cnhw_kernel(const float* __restrict__ dy, float* __restrict__ dyp, ConvShape c) {
    const unsigned per = (unsigned)(c.ho * c.wo);
    const unsigned p = blockIdx.x * kCBlock + threadIdx.x;
    if (p >= per) return;
    const unsigned oc = blockIdx.y, b = blockIdx.z;
    dyp[((int64_t)oc * c.batch + b) * per + p] = dy[((int64_t)b * c.oc + oc) * per + p];
}

// col[(ic, kh, kw)][(b, oh, ow)] = x[b, ic, oh*stride - pad + kh, ow*stride - pad + kw], zero outside the image.
// The output position is the fast index of the patch matrix: neighbouring lanes read neighbouring pixels and write
// neighbouring elements.  grid (ceil(per/256), ic, batch); a lane writes all k*k taps of its position and channel
// (one workgroup per tap made the launch itself the cost: 18432 workgroups of one element per lane).
__global__ __launch_bounds__(kCBlock) void im2col_kernel(const float* __restrict__ x, float* __restrict__ col, ConvShape c,
                                                         int64_t positions) {
    const unsigned per = (unsigned)(c.ho * c.wo);
    const unsigned p = blockIdx.x * kCBlock + threadIdx.x;
    if (p >= per) return;
    const int ci = blockIdx.y, b = blockIdx.z;                    // uniform over the workgroup
    const int oh = (int)(p / (unsigned)c.wo), ow = (int)(p - (unsigned)oh * (unsigned)c.wo);
    const int ih0 = oh * c.stride - c.pad, iw0 = ow * c.stride - c.pad;
    const float* xp = x + ((int64_t)b * c.ic + ci) * c.h * c.w;
    float* out = col + (int64_t)ci * c.k * c.k * positions + (int64_t)b * per + p;
    for (int kh = 0; kh < c.k; kh++) {
        const int ih = ih0 + kh;
        for (int kw = 0; kw < c.k; kw++) {
            const int iw = iw0 + kw;
            const bool inside = ih >= 0 && ih < c.h && iw >= 0 && iw < c.w;
            out[(int64_t)(kh * c.k + kw) * positions] = inside ? xp[ih * c.w + iw] : 0.f;
        }
    }
}

// dx[b, ic, ih, iw] = sum over the taps (kh, kw) whose output position (oh, ow) exists of dcol[(ic, kh, kw)][(b, oh, ow)];
// grid (ceil(h*w/256), ic, batch)
__global__ __launch_bounds__(kCBlock) void col2im_kernel(const float* __restrict__ dcol, float* __restrict__ dx, ConvShape c,
                                                         int64_t positions) {
    const unsigned plane = (unsigned)(c.h * c.w);
    const unsigned q = blockIdx.x * kCBlock + threadIdx.x;
    if (q >= plane) return;
    const int ci = blockIdx.y, b = blockIdx.z;
    const int ih = (int)(q / (unsigned)c.w), iw = (int)(q - (unsigned)ih * (unsigned)c.w);
    const float* base = dcol + (int64_t)b * c.ho * c.wo;
    float acc = 0.f;
    for (int kh = 0; kh < c.k; kh++) {
        const int t = ih + c.pad - kh;
        if (t < 0) continue;
        const int oh = c.stride == 1 ? t : t / c.stride;
        if (oh * c.stride != t || oh >= c.ho) continue;
        for (int kw = 0; kw < c.k; kw++) {
            const int u = iw + c.pad - kw;
            if (u < 0) continue;
            const int ow = c.stride == 1 ? u : u / c.stride;
            if (ow * c.stride != u || ow >= c.wo) continue;
            acc += base[(int64_t)((ci * c.k + kh) * c.k + kw) * positions + oh * c.wo + ow];
        }
    }
    dx[((int64_t)b * c.ic + ci) * plane + q] = acc;
}

// wf[oc, ic, kh, kw] = w[oc, ic, k-1-kh, k-1-kw]
__global__ __launch_bounds__(kCBlock) void mirror_taps_kernel(const float* __restrict__ w, float* __restrict__ wf, int taps,
                                                              int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * kCBlock + threadIdx.x;
    if (i >= total) return;
    const int64_t plane = i / taps;
    const int t = (int)(i % taps);
    wf[i] = w[plane * taps + (taps - 1 - t)];
}

// Row sums of a [rows][n] matrix in two stages: workgroup (r, ch) sums chunk ch of row r into partial[ch][r]; the
// partials are then folded by fold_rows_kernel.  (One workgroup per row left 32-64 workgroups streaming 200 KB each.)
__global__ __launch_bounds__(kCBlock) void rowsum_partial_kernel(const float* __restrict__ a, float* __restrict__ partial, int64_t n,
                                                                 int64_t chunk) {
    __shared__ float red[kCBlock / 64];
    const int64_t begin = (int64_t)blockIdx.y * chunk;
    const int64_t end = begin + chunk < n ? begin + chunk : n;
    const float* row = a + (int64_t)blockIdx.x * n;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int64_t i = begin + threadIdx.x;
    for (; i + 3 * kCBlock < end; i += 4 * kCBlock) {
        a0 += row[i];
        a1 += row[i + kCBlock];
        a2 += row[i + 2 * kCBlock];
        a3 += row[i + 3 * kCBlock];
    }
    for (; i < end; i += kCBlock) a0 += row[i];
    const float total = block_sum<kCBlock / 64>((a0 + a1) + (a2 + a3), red);
    if (threadIdx.x == 0) partial[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = total;
}

struct PoolShape {
    int64_t planes;   // batch * channels
    int h, w, ho, wo, pool, stride, pad;
};

// first maximum in row-major scan order wins (strict >, pool.c:118-123); index is the offset inside the plane, -1 if none
// grid (planes, ceil(ho*wo/256)): the plane comes from the grid, a lane splits only its position inside the plane
__global__ __launch_bounds__(kCBlock) void maxpool_fwd_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                              int32_t* __restrict__ idx, PoolShape p) {
    const unsigned q = blockIdx.y * kCBlock + threadIdx.x;
    if (q >= (unsigned)(p.ho * p.wo)) return;
    const int oh = (int)(q / (unsigned)p.wo), ow = (int)(q - (unsigned)oh * (unsigned)p.wo);
    const int64_t plane = blockIdx.x;
    const int64_t i = plane * p.ho * p.wo + q;
    const float* xp = x + plane * p.h * p.w;
    int h0 = oh * p.stride - p.pad, w0 = ow * p.stride - p.pad;
    int h1 = h0 + p.pool, w1 = w0 + p.pool;
    h0 = h0 < 0 ? 0 : h0;
    w0 = w0 < 0 ? 0 : w0;
    h1 = h1 > p.h ? p.h : h1;
    w1 = w1 > p.w ? p.w : w1;
    float best = -INFINITY;
    int where = -1;
    for (int ph = h0; ph < h1; ph++)
        for (int pw = w0; pw < w1; pw++) {
            const float v = xp[ph * p.w + pw];
            if (v > best) {
                best = v;
                where = ph * p.w + pw;
            }
        }
    y[i] = best;
    idx[i] = where;
}

// dx[plane, ih, iw] = sum of dy over the windows whose maximum sits at (ih, iw), visited in increasing output
// index, which is the order in which the reference's scatter loop adds them (pool.c:207-212)
__global__ __launch_bounds__(kCBlock) void maxpool_bwd_kernel(const float* __restrict__ dy, const int32_t* __restrict__ idx,
                                                              float* __restrict__ dx, PoolShape p) {
    const unsigned q = blockIdx.y * kCBlock + threadIdx.x;     // grid (planes, ceil(h*w/256))
    if (q >= (unsigned)(p.h * p.w)) return;
    const int ih = (int)(q / (unsigned)p.w), iw = (int)(q - (unsigned)ih * (unsigned)p.w);
    const int64_t plane = blockIdx.x;
    const int64_t i = plane * p.h * p.w + q;
    const int me = ih * p.w + iw;
    // windows covering row ih: oh*stride - pad <= ih < oh*stride - pad + pool
    int oh_lo = ih + p.pad - p.pool + 1;
    oh_lo = oh_lo <= 0 ? 0 : (oh_lo + p.stride - 1) / p.stride;
    int oh_hi = (ih + p.pad) / p.stride;
    if (oh_hi >= p.ho) oh_hi = p.ho - 1;
    int ow_lo = iw + p.pad - p.pool + 1;
    ow_lo = ow_lo <= 0 ? 0 : (ow_lo + p.stride - 1) / p.stride;
    int ow_hi = (iw + p.pad) / p.stride;
    if (ow_hi >= p.wo) ow_hi = p.wo - 1;
    const float* gp = dy + plane * p.ho * p.wo;
    const int32_t* ip = idx + plane * p.ho * p.wo;
    float acc = 0.f;
    for (int oh = oh_lo; oh <= oh_hi; oh++)
        for (int ow = ow_lo; ow <= ow_hi; ow++)
            if (ip[oh * p.wo + ow] == me) acc += gp[oh * p.wo + ow];
    dx[i] = acc;
}

static int make_conv_shape(ConvShape& c, int64_t batch, int64_t ic, int64_t h, int64_t w, int64_t oc, int64_t k, int64_t stride,
                           int64_t pad) {
    if (batch < 0 || ic <= 0 || h <= 0 || w <= 0 || oc <= 0 || k <= 0 || stride <= 0 || pad < 0)
        return set_error(BH_EINVAL, "conv2d: bad shape");
    const int64_t ho = (h + 2 * pad - k) / stride + 1, wo = (w + 2 * pad - k) / stride + 1;
    if (h + 2 * pad < k || w + 2 * pad < k || ho <= 0 || wo <= 0) return set_error(BH_EINVAL, "conv2d: kernel larger than the padded image");
    const int64_t lim = (int64_t)1 << 30;
    if (batch * ic * h * w >= lim || batch * oc * ho * wo >= lim || oc * ic * k * k >= lim)
        return set_error(BH_EINVAL, "conv2d: tensor too large for 32-bit indexing");
    c.batch = (int)batch; c.ic = (int)ic; c.h = (int)h; c.w = (int)w; c.oc = (int)oc; c.k = (int)k;
    c.stride = (int)stride; c.pad = (int)pad; c.ho = (int)ho; c.wo = (int)wo;
    return BH_OK;
}

}  // namespace bh

using namespace bh;

extern "C" {

int bh_conv2d_forward(const float* x, const float* w, const float* bias, float* y, int64_t batch, int64_t in_channels,
                      int64_t height, int64_t width, int64_t out_channels, int64_t kernel, int64_t stride, int64_t pad) {
    BH_REQUIRE_INIT();
    ConvShape c;
    int rc = make_conv_shape(c, batch, in_channels, height, width, out_channels, kernel, stride, pad);
    if (rc) return rc;
    if (batch == 0) return BH_OK;
    BH_CHECK_ARG(x && w && y, "null pointer");
    // Output channels per lane: eight amortise the patch loads best, but a small layer then has too few workgroups to
    // hide the latency of its serial channel loop (MNIST's 32->64 layer at batch 64: 0.396 ms per training step with
    // eight, 0.365 with four), so the tile shrinks until the launch has about four workgroups per compute unit.
    // 5x5 kernels stop at four: 25 taps of more channels would not fit the register file.
    const int64_t wg_per_oc_group = ceil_div((int64_t)c.ho * c.wo, kCBlock) * c.batch;
    int oc_tile = c.k == 3 ? 8 : 4;
    while (oc_tile > 2 && wg_per_oc_group * ceil_div(c.oc, oc_tile) < 1024) oc_tile >>= 1;
    const dim3 grid((unsigned)ceil_div((int64_t)c.ho * c.wo, kCBlock), (unsigned)ceil_div(c.oc, oc_tile), (unsigned)c.batch);
    if (c.k == 3 && grid.y <= 65535 && grid.z <= 65535) {
        if (oc_tile == 8) hipLaunchKernelGGL((conv2d_fwd_kernel<3, 8>), grid, dim3(kCBlock), 0, stream(), x, w, bias, y, c);
        else if (oc_tile == 4) hipLaunchKernelGGL((conv2d_fwd_kernel<3, 4>), grid, dim3(kCBlock), 0, stream(), x, w, bias, y, c);
        else hipLaunchKernelGGL((conv2d_fwd_kernel<3, 2>), grid, dim3(kCBlock), 0, stream(), x, w, bias, y, c);
    } else if (c.k == 5 && grid.y <= 65535 && grid.z <= 65535) {
        if (oc_tile == 4) hipLaunchKernelGGL((conv2d_fwd_kernel<5, 4>), grid, dim3(kCBlock), 0, stream(), x, w, bias, y, c);
        else hipLaunchKernelGGL((conv2d_fwd_kernel<5, 2>), grid, dim3(kCBlock), 0, stream(), x, w, bias, y, c);
    } else {
        const int64_t total = (int64_t)c.batch * c.oc * c.ho * c.wo;
        hipLaunchKernelGGL(conv2d_fwd_generic_kernel, dim3((unsigned)ceil_div(total, kCBlock)), dim3(kCBlock), 0, stream(), x, w,
                           bias, y, c, total);
    }
    return BH_LAUNCH_CHECK("conv2d_fwd_kernel");
}

int bh_conv2d_forward_mfma(const float* x, const float* w, const float* bias, float* y, int64_t batch, int64_t in_channels,
                           int64_t height, int64_t width, int64_t out_channels, int64_t kernel, int64_t stride, int64_t pad) {
    BH_REQUIRE_INIT();
    ConvShape c;
    int rc = make_conv_shape(c, batch, in_channels, height, width, out_channels, kernel, stride, pad);
    if (rc) return rc;
    BH_CHECK_ARG(kernel == 3 || kernel == 5, "conv2d on the matrix cores: 3x3 and 5x5 kernels only");
    if (batch == 0) return BH_OK;
    BH_CHECK_ARG(x && w && y, "null pointer");
    const int64_t positions = (int64_t)c.batch * c.ho * c.wo;
    BH_CHECK_ARG(ceil_div(c.oc, 64) <= 65535, "conv2d on the matrix cores: too many output channels");
    static bool attr = false;
    if (!attr) {
        rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv2d_fwd_mfma_kernel<4, 3>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)FmGeom<3>::kLds), "hipFuncSetAttribute");
        if (rc) return rc;
        rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv2d_fwd_mfma_kernel<2, 3>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)FmGeom<3>::kLds), "hipFuncSetAttribute");
        if (rc) return rc;
        rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv2d_fwd_mfma_kernel<4, 5>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)FmGeom<5>::kLds), "hipFuncSetAttribute");
        if (rc) return rc;
        attr = true;
    }
    const dim3 grid((unsigned)ceil_div(positions, 64), (unsigned)ceil_div(c.oc, 64));
    // the split follows the shape alone, not the device: a layer's sums always run in the same order.  (5x5: the weights of a
    // part fill more than half of a compute unit's LDS, so a second workgroup would not fit beside the first whatever the split.)
    if (kernel == 5)
        hipLaunchKernelGGL((conv2d_fwd_mfma_kernel<4, 5>), grid, dim3(512), FmGeom<5>::kLds, stream(), x, w, bias, y, c, (int)positions);
    else if ((int64_t)grid.x * grid.y >= kFmBlocksSplit2)
        hipLaunchKernelGGL((conv2d_fwd_mfma_kernel<2, 3>), grid, dim3(256), FmGeom<3>::kLds, stream(), x, w, bias, y, c, (int)positions);
    else
        hipLaunchKernelGGL((conv2d_fwd_mfma_kernel<4, 3>), grid, dim3(512), FmGeom<3>::kLds, stream(), x, w, bias, y, c, (int)positions);
    return BH_LAUNCH_CHECK("conv2d_fwd_mfma_kernel");
}

int bh_conv2d_backward(const float* x, const float* w, const float* dy, float* dx, float* gw, float* gb, int64_t batch,
                       int64_t in_channels, int64_t height, int64_t width, int64_t out_channels, int64_t kernel,
                       int64_t stride, int64_t pad, int accumulate, int flip_taps) {
    BH_REQUIRE_INIT();
    ConvShape c;
    int rc = make_conv_shape(c, batch, in_channels, height, width, out_channels, kernel, stride, pad);
    if (rc) return rc;
    const int64_t taps = (int64_t)c.k * c.k, kk = (int64_t)c.ic * taps;      // contraction length of the forward
    const int64_t positions = (int64_t)c.batch * c.ho * c.wo;
    if (batch == 0) {   // empty sums: the parameter gradients are zero (or left alone when accumulating)
        if (gw && !accumulate) rc = bh_memset_zero(gw, sizeof(float) * (size_t)(c.oc * kk));
        if (rc == BH_OK && gb && !accumulate) rc = bh_memset_zero(gb, sizeof(float) * (size_t)c.oc);
        return rc;
    }
    BH_CHECK_ARG(dy, "null pointer");
    BH_CHECK_ARG(!gw || x, "null pointer");
    BH_CHECK_ARG(!dx || w, "null pointer");
    BH_CHECK_ARG(positions * kk < ((int64_t)1 << 40), "conv2d: patch matrix too large");
    if (!dx && !gw && !gb) return BH_OK;
    auto blocks = [](int64_t n) { return dim3((unsigned)ceil_div(n, kCBlock)); };
    // the rearrangement kernels carry channel and batch indices in grid.y / grid.z
    BH_CHECK_ARG(c.oc <= 65535 && c.batch <= 65535 && c.ic <= 65535, "conv2d backward: more than 65535 channels or images");
    float *dyp = nullptr, *col = nullptr, *wf = nullptr;
    dyp = (float*)bh_malloc(sizeof(float) * (size_t)(c.oc * positions));
    if (!dyp) return BH_ENOMEM;
    const unsigned per_blocks = (unsigned)ceil_div((int64_t)c.ho * c.wo, kCBlock);
    hipLaunchKernelGGL(nchw_to_cnhw_kernel, dim3(per_blocks, (unsigned)c.oc, (unsigned)c.batch), dim3(kCBlock), 0, stream(), dy, dyp, c);
    rc = BH_LAUNCH_CHECK("nchw_to_cnhw_kernel");
    if (rc == BH_OK && gb) {
        int64_t chunks = ceil_div(512, c.oc);                       // about two workgroups per compute unit ...
        if (chunks > ceil_div(positions, 2048)) chunks = ceil_div(positions, 2048);   // ... of at least 2048 elements each
        if (chunks > 65535) chunks = 65535;
        const int64_t chunk = ceil_div(positions, chunks);
        chunks = ceil_div(positions, chunk);
        float* partial = (float*)bh_malloc(sizeof(float) * (size_t)(chunks * c.oc));
        if (!partial) rc = BH_ENOMEM;
        if (rc == BH_OK) {
            hipLaunchKernelGGL(rowsum_partial_kernel, dim3((unsigned)c.oc, (unsigned)chunks), dim3(kCBlock), 0, stream(), dyp, partial,
                               positions, chunk);
            rc = BH_LAUNCH_CHECK("rowsum_partial_kernel");
        }
        if (rc == BH_OK) {
            hipLaunchKernelGGL(fold_rows_kernel, dim3((unsigned)ceil_div(c.oc, kFoldCols)), dim3(kFoldCols * kFoldLanes), 0, stream(),
                               partial, chunks, (int64_t)c.oc, gb, (float*)nullptr, (int64_t)c.oc, accumulate);
            rc = BH_LAUNCH_CHECK("fold_rows_kernel");
        }
        if (partial) bh_free(partial);
    }
    if (rc == BH_OK && (gw || dx)) {
        col = (float*)bh_malloc(sizeof(float) * (size_t)(positions * kk));   // patches for gw, then reused as dcol
        if (!col) rc = BH_ENOMEM;
    }
    if (rc == BH_OK && gw) {
        hipLaunchKernelGGL(im2col_kernel, dim3(per_blocks, (unsigned)c.ic, (unsigned)c.batch), dim3(kCBlock), 0, stream(), x, col, c, positions);
        rc = BH_LAUNCH_CHECK("im2col_kernel");
        // gw[oc][kk] (+)= dyp[oc][positions] . col[kk][positions]^T : both operands contiguous along the contraction
        if (rc == BH_OK) rc = bh_gemm(0, 1, c.oc, kk, positions, dyp, positions, col, positions, gw, kk, nullptr, accumulate, 1);
    }
    if (rc == BH_OK && dx) {
        const float* wsrc = w;
        if (flip_taps) {
            wf = (float*)bh_malloc(sizeof(float) * (size_t)(c.oc * kk));
            if (!wf) rc = BH_ENOMEM;
            if (rc == BH_OK) {
                hipLaunchKernelGGL(mirror_taps_kernel, blocks(c.oc * kk), dim3(kCBlock), 0, stream(), w, wf, (int)taps, c.oc * kk);
                rc = BH_LAUNCH_CHECK("mirror_taps_kernel");
                wsrc = wf;
            }
        }
        // dcol[kk][positions] = w^T[kk][oc] . dyp[oc][positions]  (the stream orders it after the gw product that read col)
        if (rc == BH_OK) rc = bh_gemm(1, 0, kk, positions, c.oc, wsrc, kk, dyp, positions, col, positions, nullptr, 0, 1);
        if (rc == BH_OK) {
            hipLaunchKernelGGL(col2im_kernel, dim3((unsigned)ceil_div((int64_t)c.h * c.w, kCBlock), (unsigned)c.ic, (unsigned)c.batch),
                               dim3(kCBlock), 0, stream(), col, dx, c, positions);
            rc = BH_LAUNCH_CHECK("col2im_kernel");
        }
    }
    if (wf) bh_free(wf);
    if (col) bh_free(col);
    bh_free(dyp);
    return rc;
}

static int make_pool_shape(PoolShape& p, int64_t planes, int64_t h, int64_t w, int64_t pool, int64_t stride, int64_t pad) {
    if (planes < 0 || h <= 0 || w <= 0 || pool <= 0 || stride <= 0 || pad < 0) return set_error(BH_EINVAL, "maxpool2d: bad shape");
    const int64_t ho = (h + 2 * pad - pool) / stride + 1, wo = (w + 2 * pad - pool) / stride + 1;
    if (h + 2 * pad < pool || w + 2 * pad < pool || ho <= 0 || wo <= 0) return set_error(BH_EINVAL, "maxpool2d: window larger than the padded image");
    if (h * w >= ((int64_t)1 << 30)) return set_error(BH_EINVAL, "maxpool2d: plane too large for 32-bit indexing");
    p.planes = planes; p.h = (int)h; p.w = (int)w; p.ho = (int)ho; p.wo = (int)wo;
    p.pool = (int)pool; p.stride = (int)stride; p.pad = (int)pad;
    return BH_OK;
}

int bh_maxpool2d_forward(const float* x, float* y, int32_t* argmax, int64_t planes, int64_t height, int64_t width, int64_t pool,
                         int64_t stride, int64_t pad) {
    BH_REQUIRE_INIT();
    PoolShape p;
    int rc = make_pool_shape(p, planes, height, width, pool, stride, pad);
    if (rc) return rc;
    if (planes == 0) return BH_OK;
    BH_CHECK_ARG(x && y && argmax, "null pointer");
    const int64_t per_blocks = ceil_div((int64_t)p.ho * p.wo, kCBlock);
    BH_CHECK_ARG(planes <= 0x7fffffff && per_blocks <= 65535, "tensor too large");
    hipLaunchKernelGGL(maxpool_fwd_kernel, dim3((unsigned)planes, (unsigned)per_blocks), dim3(kCBlock), 0, stream(), x, y, argmax, p);
    return BH_LAUNCH_CHECK("maxpool_fwd_kernel");
}

int bh_maxpool2d_backward(const float* dy, const int32_t* argmax, float* dx, int64_t planes, int64_t height, int64_t width,
                          int64_t pool, int64_t stride, int64_t pad) {
    BH_REQUIRE_INIT();
    PoolShape p;
    int rc = make_pool_shape(p, planes, height, width, pool, stride, pad);
    if (rc) return rc;
    if (planes == 0) return BH_OK;
    BH_CHECK_ARG(dy && argmax && dx, "null pointer");
    const int64_t per_blocks = ceil_div((int64_t)p.h * p.w, kCBlock);
    BH_CHECK_ARG(planes <= 0x7fffffff && per_blocks <= 65535, "tensor too large");
    hipLaunchKernelGGL(maxpool_bwd_kernel, dim3((unsigned)planes, (unsigned)per_blocks), dim3(kCBlock), 0, stream(), dy, argmax, dx, p);
    return BH_LAUNCH_CHECK("maxpool_bwd_kernel");
}

}  // extern "C"
