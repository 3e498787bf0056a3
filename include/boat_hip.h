/* boat_hip.h - C-ABI of the MI355X (gfx950) device layer under Boat's training hot path.
 *
 * One process, one GPU, one HIP stream.  Every entry point takes plain pointers and
 * sizes; device pointers come from bh_malloc()/bh_buffer_ptr().  Kernels are enqueued
 * on the library's single stream and return without waiting; bh_synchronize() or any
 * device-to-host copy waits.  All tensors are dense, row-major, contiguous fp32.
 *
 * Return value: 0 on success, a negative BH_E* code otherwise; bh_last_error() gives the
 * message of the most recent failure.  No entry point falls back to host arithmetic.
 *
 * Each kernel entry point names the reference routine (file:line under the Boat tree)
 * whose arithmetic it replaces.
 */
#ifndef BOAT_HIP_H
#define BOAT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BH_OK          0
#define BH_EINVAL     -1   /* bad argument / shape the kernel cannot take */
#define BH_EDEVICE    -2   /* HIP runtime failure */
#define BH_ENOMEM     -3

/* ---- runtime: replaces the device seam src/core/memory.c:46-74,174-186,230-247 ---- */
int         bh_init(void);                       /* idempotent; picks device 0, creates the stream */
int         bh_shutdown(void);
int         bh_synchronize(void);
const char* bh_last_error(void);
const char* bh_device_name(void);
int         bh_device_cu_count(void);
void*       bh_stream(void);                     /* the hipStream_t, for callers that time or profile */

/* raw device memory from a size-bucketed cache (stream-ordered reuse, no hipFree per call) */
void*  bh_malloc(size_t nbytes);
void   bh_free(void* dptr);
int    bh_cache_release(void);                   /* hand cached blocks back to the driver */
size_t bh_bytes_in_use(void);
size_t bh_bytes_cached(void);

/* reference-counted device buffer: the device twin of boat_tensor_t's ref/unref (src/core/tensor.c:164-191) */
typedef struct bh_buffer bh_buffer_t;
bh_buffer_t* bh_buffer_create(size_t nbytes, int zero_fill);
void         bh_buffer_ref(bh_buffer_t* b);
void         bh_buffer_unref(bh_buffer_t* b);
void*        bh_buffer_ptr(const bh_buffer_t* b);
size_t       bh_buffer_nbytes(const bh_buffer_t* b);
int          bh_buffer_refcount(const bh_buffer_t* b);

int bh_memcpy_h2d(void* dst_dev, const void* src_host, size_t nbytes);
int bh_memcpy_d2h(void* dst_host, const void* src_dev, size_t nbytes);   /* waits for the stream */
int bh_memcpy_d2d(void* dst_dev, const void* src_dev, size_t nbytes);
int bh_memset_zero(void* dst_dev, size_t nbytes);
/* page-locked host memory (hipHostMalloc) and copies to and from it that are queued on the stream and do NOT wait: the
 * host side of a transfer the library stages itself (src/core/memory.c:46-247 is the reference's allocator seam; it has
 * no device).  The memory must stay untouched until the stream has passed the copy (bh_synchronize). */
void* bh_host_alloc(size_t nbytes);
void  bh_host_free(void* p);
int bh_memcpy_h2d_async(void* dst_dev, const void* src_pinned, size_t nbytes);
int bh_memcpy_d2h_async(void* dst_pinned, const void* src_dev, size_t nbytes);

/* events on the library stream: for timing, and for waiting until the stream has passed one queued copy among several */
typedef struct bh_event bh_event_t;
bh_event_t* bh_event_create(void);
void        bh_event_destroy(bh_event_t* e);
int         bh_event_record(bh_event_t* e);
int         bh_event_wait(bh_event_t* e);                                /* returns when the stream has passed the record */
float       bh_event_elapsed_ms(bh_event_t* start, bh_event_t* stop);    /* synchronises on stop */

/* ---- per-class timing of the library's own launches, for benchmarks that drive whole training steps through Boat's API
 * and still need the duration of one kernel family inside the step.  bh_profile_enable(max_calls > 0) creates
 * 2*max_calls events and starts recording one start/stop pair on the library stream around each instrumented entry point
 * (an entry point called from another instrumented one is not recorded twice); bh_profile_enable(0) stops and frees.
 * Each call to enable starts a fresh recording.  bh_profile_read waits for the stream and sums, for one class, the
 * event-to-event time in ms, the algorithmic work the calls declared (flops for the matrix classes, bytes for the
 * memory-bound ones) and the number of calls.  Calls beyond max_calls are not recorded.  A hook for single-threaded
 * benchmarks: while profiling is on, only one host thread may call into the library. */
#define BH_PROF_GEMM       0   /* bh_gemm: 2*m*n*k*batch flops */
#define BH_PROF_SDPA_FWD   1   /* bh_sdpa_forward: 2 * 2*bh*s*s*d flops */
#define BH_PROF_SDPA_BWD   2   /* bh_sdpa_backward: 4 * 2*bh*s*s*d flops (the reference's four contractions) */
#define BH_PROF_NORM       3   /* LayerNorm / RMSNorm forward (2 passes) and backward (3 passes): bytes of x, y or x, dy, dx */
#define BH_PROF_OPTIMIZER  4   /* Adam (28 B/param), RMSprop / Adagrad (20 B/param) */
#define BH_PROF_COLSUM     5   /* bh_colsum: bytes read */
int bh_profile_enable(int max_calls);
int bh_profile_read(int cls, double* total_ms, double* total_work, int64_t* calls);

/* ---- elementwise (src/ops/arithmetic.c:157-285,362-484; src/autodiff.c:1002-1452) ---- */
int bh_fill(float* x, float value, int64_t n);
int bh_add_inplace(float* a, const float* b, int64_t n);                              /* boat_add_ */
int bh_binary(int op, const float* a, const float* b, float* out, int64_t n);         /* 0 add 1 sub 2 mul 3 div */
/* broadcasting binary op, numpy rules, shapes right-aligned to ndim<=8 (arithmetic.c:78-104,199-203) */
int bh_binary_broadcast(int op, const float* a, const int64_t* a_shape,
                        const float* b, const int64_t* b_shape,
                        float* out, const int64_t* out_shape, int ndim);
/* out[i] = in[i] * scalar[0] (in == NULL: out[i] = scalar[0]) with the scalar read on the device: the gradient rules of
 * sum and dot scale by grad_output[0] (src/autodiff.c:1228, 1536), which here never leaves HBM */
int bh_scale_by_device_scalar(const float* in, const float* scalar, float* out, int64_t n);
int bh_copy_f32(float* dst, const float* src, int64_t n);   /* dst = src on the stream (bh_memcpy_d2d uses it for whole floats) */
int bh_scalar_op(int op, const float* a, float s, float* out, int64_t n);             /* boat_*_scalar */
/* d(a/b)/db = (dy*-1) * (a/(b*b))  (src/autodiff.c:1172-1201) */
int bh_div_backward_b(const float* a, const float* b, const float* dy, float* db, int64_t n);

#define BH_ACT_RELU    0
#define BH_ACT_SIGMOID 1
#define BH_ACT_TANH    2
#define BH_ACT_GELU    3   /* exact erf form; the reference's boat_gelu is a stub (src/ops/activation.c:298-302) */
int bh_activation_forward(int act, const float* x, float* y, int64_t n);             /* autodiff.c:808-909 */
/* saved = op input for RELU/GELU, op output for SIGMOID/TANH (autodiff.c:1244-1452).
 * accumulate!=0 adds into dx instead of assigning. */
int bh_activation_backward(int act, const float* saved, const float* dy, float* dx, int64_t n, int accumulate);
/* The same on a [rows, cols] matrix, and in the same pass colsum[c] (+)= sum_r dx[r][c]: the activation sat behind a dense
 * layer, so dx is that layer's grad_output and its column sums are the bias gradient (src/layers/dense.c:286-291), which
 * would otherwise read dx once more.  dx and the sums are bit for bit those of bh_activation_backward followed by bh_colsum. */
int bh_activation_backward_colsum(int act, const float* saved, const float* dy, float* dx, float* colsum, int64_t rows,
                                  int64_t cols, int accumulate);

/* the reference's elementwise arithmetic on its other element types (src/ops/arithmetic.c:157-360 with boat_mod,
 * :425-560 scalar ops and boat_pow_scalar): op 0 add, 1 sub, 2 mul, 3 div, 4 mod (fmodf / fmod / %), 5 pow (scalar form,
 * float types only).  Shapes are right-aligned to ndim <= 8, numpy broadcasting.  An integer division by zero yields 0. */
#define BH_DT_F32 0
#define BH_DT_F64 1
#define BH_DT_I32 2
#define BH_DT_I64 3
int bh_binary_typed(int dtype, int op, const void* a, const int64_t* a_shape, const void* b, const int64_t* b_shape,
                    void* out, const int64_t* out_shape, int ndim);
int bh_scalar_op_typed(int dtype, int op, const void* a, double scalar, void* out, int64_t n);

int bh_bias_add_rows(float* y, const float* bias, int64_t rows, int64_t cols);        /* dense.c:180-184 */
int bh_mse_grad(const float* pred, const float* target, float* grad, int64_t n);      /* tests/test_attention_training.c:28-41 */
/* sum over the elements of the loss terms of the reference's loss objects (src/loss/mse.c, cross_entropy.c, huber.c):
 * kind 0 (p-t)^2, 1 t*logf(clip(p, 1e-7, 1-1e-7)), 2 Huber(|p-t|, delta); sum_out is one float in device memory */
int bh_loss_terms_sum(int kind, const float* pred, const float* target, float* sum_out, int64_t n, float delta);
int bh_mse_loss(const float* pred, const float* target, float* loss_out, int64_t n);  /* src/loss/mse.c:70-78 */
/* both in one pass over pred and target (the loop of tests/test_attention_training.c:28-41 computes them together) */
int bh_mse_loss_grad(const float* pred, const float* target, float* loss_out, float* grad, int64_t n);
int bh_sgd_update(float* p, float* g, float lr, int64_t n, int zero_grad);            /* dense.c:297-329 */

/* ---- reductions / softmax (src/ops/arithmetic.c:611-691; src/autodiff.c:1701-2068; dense.c:286-291) ---- */
int bh_sum_all(const float* x, float* out1, int64_t n);
int bh_colsum(const float* x, float* out, int64_t rows, int64_t cols, int accumulate);
/* the same for up to 4 matrices of one shape in one pair of launches (the bias gradients of an attention layer's four
 * projections, src/layers/attention.c:1262-1279 four times); the same sums in the same order as bh_colsum */
int bh_colsum_grouped(const float* const* x, float* const* out, int groups, int64_t rows, int64_t cols, int accumulate); /* db (+)= sum_rows dY */
int bh_softmax_forward(const float* x, float* y, int64_t rows, int64_t cols);
int bh_softmax_backward(const float* y, const float* dy, float* dx, int64_t rows, int64_t cols);
int bh_log_softmax_forward(const float* x, float* y, int64_t rows, int64_t cols);
int bh_log_softmax_backward(const float* y, const float* dy, float* dx, int64_t rows, int64_t cols);
/* Backward of the loss chain loss = f * sum(w o log_softmax(z)) as the MNIST example writes it (w = one-hot labels, f = -1/B;
 * examples/mnist/mnist_autodiff.c:397-522) in one launch: dz_j = c*w_j - expf(y_j) * sum_j c*w_j with c = seed[0]*f[0]
 * (seed NULL = 1), y = log_softmax(z) from the forward pass.  The operations and their order are those of the four
 * separate gradient rules (src/autodiff.c:1115-1147, 1498-1548, 1975-2068), so the result is theirs bit for bit. */
int bh_log_softmax_weighted_backward(const float* y, const float* w, const float* seed, const float* f, float* dz,
                                     int64_t rows, int64_t cols);
/* The same, and colsum[c] (+)= sum_r dz[r][c] with it: z came out of a dense layer, so dz is that layer's grad_output and its
 * column sums are the bias gradient (src/layers/dense.c:286-291).  A small batch (at most 256 rows, 8192 elements) takes one
 * launch for both; dz and the sums are those of bh_log_softmax_weighted_backward followed by bh_colsum, bit for bit. */
int bh_log_softmax_weighted_backward_colsum(const float* y, const float* w, const float* seed, const float* f, float* dz,
                                            float* colsum, int64_t rows, int64_t cols, int accumulate);
/* fused replacement of the chain log_softmax -> mul(onehot) -> sum -> mul(-1/B) and its backward
 * (examples/mnist/mnist_autodiff.c:397-522): loss_out[0] = -(1/B) sum onehot*log_softmax(z),
 * dlogits = (softmax(z) - onehot)/B.  labels are class indices. */
int bh_softmax_ce_grad(const float* logits, const int32_t* labels, float* dlogits, float* loss_out,
                       int64_t rows, int64_t cols);

/* ---- LayerNorm (forward: src/layers/norm.c:184-317; backward: stub there, :397-402) ---- */
int bh_layernorm_forward(const float* x, const float* gamma, const float* beta, float* y,
                         float* mean, float* rstd, int64_t rows, int64_t hidden, float eps);
/* dx (assigned), dgamma/dbeta (assigned unless accumulate).  gamma may be NULL (no affine). */
int bh_layernorm_backward(const float* x, const float* gamma, const float* dy,
                          const float* mean, const float* rstd,
                          float* dx, float* dgamma, float* dbeta,
                          int64_t rows, int64_t hidden, int accumulate);

/* ---- RMSNorm (forward: src/layers/norm.c:212-229,319-395; backward: stub there, :404-409) ----
 * r = sqrtf(mean_h(x^2)), s = 1/(r + eps) (eps outside the root, as the reference), y = x*s*weight.  inv_rms (may be
 * NULL) receives s per row.  backward: dx (assigned) and dweight (assigned unless accumulate) from the saved s;
 * weight may be NULL (no scale). */
int bh_rmsnorm_forward(const float* x, const float* weight, float* y, float* inv_rms, int64_t rows, int64_t hidden, float eps);
int bh_rmsnorm_backward(const float* x, const float* weight, const float* dy, const float* inv_rms,
                        float* dx, float* dweight, int64_t rows, int64_t hidden, float eps, int accumulate);

/* The same with dx = (the LayerNorm input gradient) + add[rows, hidden]: a variable that feeds a LayerNorm and a residual
 * connection (x1 in y = x1 + f(LN(x1))) gets both gradients in the LayerNorm kernel's one store instead of in an adding
 * pass of its own (the sum the reference's tape makes with boat_add_, src/autodiff.c:1002-1061).  add must not overlap dx. */
int bh_layernorm_backward_add(const float* x, const float* gamma, const float* dy,
                              const float* mean, const float* rstd, const float* add,
                              float* dx, float* dgamma, float* dbeta,
                              int64_t rows, int64_t hidden, int accumulate);

/* bh_layernorm_backward for callers that cannot allocate device memory (tight serving loops, harnesses that
 * forbid hipMalloc; it launches on the library's own stream, so it is not for a caller's graph capture).  It has no counterpart in the reference.  Same arguments, same kernels and
 * the same results as bh_layernorm_backward; the per-workgroup dgamma/dbeta partials live in a 16 MiB device array
 * that is part of the library image (one copy per GPU, held until the process ends) instead of coming from bh_malloc.
 * It calls no hipMalloc/hipFree and sets nothing up: bh_init() must have returned BH_OK before.  hidden must be a
 * multiple of 4 and at most BH_LN_NOALLOC_MAX_HIDDEN, and x, dy, dx, gamma 16-byte aligned; anything else returns
 * BH_EINVAL with a message.  Every call on a GPU uses that GPU's one array: calls that overlap in time race. */
#define BH_LN_NOALLOC_MAX_HIDDEN 8192
int bh_layernorm_backward_noalloc(const float* x, const float* gamma, const float* dy,
                                  const float* mean, const float* rstd,
                                  float* dx, float* dgamma, float* dbeta,
                                  int64_t rows, int64_t hidden, int accumulate);

/* ---- GEMM on fp32 MFMA (src/ops/linear.c:12-170 with the transposes of :238-406 folded in) ----
 * C[M,N] (+)= op(A) . op(B) (+ bias[N]), row-major.
 *   trans_a == 0: A is [M,K] with leading dimension lda;  trans_a != 0: A is stored [K,M]
 *   trans_b == 0: B is [K,N] with leading dimension ldb;  trans_b != 0: B is stored [N,K]
 * dense forward  Y  = X.W + b   : trans_a=0 trans_b=0          (dense.c:150-185)
 * dense backward dX = dY.W^T    : trans_a=0 trans_b=1          (dense.c:219-228)
 *                dW += X^T.dY   : trans_a=1 trans_b=0, accumulate=1 (dense.c:230-261)
 * batch > 1 strides all three operands by their full matrix size (linear.c:116-130). */
int bh_gemm(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
            const float* a, int64_t lda, const float* b, int64_t ldb,
            float* c, int64_t ldc, const float* bias, int accumulate, int64_t batch);
/* Up to 4 products of ONE shape whose operands are separate tensors: c[g] (+)= op(a[g]) . op(b[g]) (+ bias[g]), arguments
 * as bh_gemm with tables of `groups` pointers (bias may be NULL, or hold NULLs).  The three input projections of a
 * self-attention layer (src/layers/attention.c:363-365: the same input times Wq, Wk, Wv) and the weight gradients of its
 * four projections (:1186-1285 run four times) are one launch each this way, with the kernels of bh_gemm; the number of cuts of a long
 * contraction is chosen for the group as a whole, so a product agrees with a separate bh_gemm call to fp32 rounding. */
int bh_gemm_grouped(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, int groups,
                    const float* const* a, int64_t lda, const float* const* b, int64_t ldb,
                    float* const* c, int64_t ldc, const float* const* bias, int accumulate);
/* One product whose contraction runs over up to 3 operand pairs of k each: c (+)= sum_s op(a[s]) . op(b[s]) (+ bias).
 * The summed input gradient of self-attention, dQ.Wq^T + dK.Wk^T + dV.Wv^T (what the reference's caller adds up after
 * three linear_projection_backward calls, src/autodiff.c:2458-2532), is one launch without read-modify-write this way.
 * Shapes that do not take the matrix-core tiles run pair by pair, adding into c: the same sum in another order. */
int bh_gemm_ksegments(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, int segments,
                      const float* const* a, int64_t lda, const float* const* b, int64_t ldb,
                      float* c, int64_t ldc, const float* bias, int accumulate);
int bh_transpose_last2(const float* a, float* out, int64_t batch, int64_t rows, int64_t cols); /* linear.c:238-406 */
/* out[a][d1][b][d0][c] = in[a][d0][b][d1][c]: boat_transpose of any two dimensions of a dense tensor (linear.c:238-406;
 * a, b, c are the products of the extents before, between and after the two) */
int bh_swap_dims(const float* in, float* out, int64_t a, int64_t d0, int64_t b, int64_t d1, int64_t c);
/* the same for 8-byte elements (the float64 case of boat_transpose, linear.c:339-398): data movement only */
int bh_swap_dims_f64(const double* in, double* out, int64_t a, int64_t d0, int64_t b, int64_t d1, int64_t c);
/* dense layer backward in one call: dx = dy.W^T, gw += x^T.dy, gb += colsum(dy)  (dense.c:190-295) */
int bh_dense_backward(const float* x, const float* w, const float* dy,
                      float* dx, float* gw, float* gb, int64_t m, int64_t k, int64_t n,
                      int accumulate);
/* the same with the input gradient added into dx when accumulate_dx != 0 (the key and value projections of a
 * self-attention layer add into the query projection's input gradient, src/layers/attention.c:1186-1285 run three times
 * on one input) */
int bh_dense_backward_into(const float* x, const float* w, const float* dy,
                           float* dx, float* gw, float* gb, int64_t m, int64_t k, int64_t n,
                           int accumulate, int accumulate_dx);

/* ---- scaled dot-product attention on [bh, s, d] blocks (src/layers/attention.c:882-1079,1388-1534) ----
 * forward keeps O and the row log-sum-exp instead of the reference's [bh,s,s] softmax matrix;
 * backward recomputes P = exp(scale*QK^T - lse).  attn_out (may be NULL) receives the softmax
 * matrix when a caller wants the reference's cache. */
int bh_sdpa_forward(const float* q, const float* k, const float* v, float scale, int causal,
                    float* out, float* lse, float* attn_out, int64_t bh, int64_t s, int64_t d);
int bh_sdpa_backward(const float* q, const float* k, const float* v, const float* out, const float* lse,
                     const float* d_out, float scale, int causal,
                     float* dq, float* dk, float* dv, int64_t bh, int64_t s, int64_t d);
/* The same pair with a score cache: the forward pass also leaves the scaled scores ([bh, s(key), s(query)] floats, an
 * opaque layout) and the backward pass reads them instead of recomputing Q.K^T -- the trade the reference makes when it
 * keeps its [B, nh, S, S] attention weights for attention_backward (attention.c:424-431 and 1046-1050 store them, :584-598 hand them to attention_backward).  One contraction
 * of five less in the backward pass for bh*s*s*4 bytes of HBM.  head_dim 64 and s a multiple of 128 only:
 * bh_sdpa_score_cache_bytes returns the size of the cache, 0 for shapes without this path. */
size_t bh_sdpa_score_cache_bytes(int64_t bh, int64_t s, int64_t d);
int bh_sdpa_forward_cached(const float* q, const float* k, const float* v, float scale, int causal,
                           float* out, float* lse, float* scores, int64_t bh, int64_t s, int64_t d);
int bh_sdpa_backward_cached(const float* q, const float* k, const float* v, const float* out, const float* lse,
                            const float* scores, const float* d_out, float scale, int causal,
                            float* dq, float* dk, float* dv, int64_t bh, int64_t s, int64_t d);

/* ---- 2-D convolution and max pooling, NCHW, square kernel/window (src/layers/conv.c:46-201,326-437; src/layers/pool.c:63-218) ----
 * x [batch, in_channels, height, width]; w [out_channels, in_channels, kernel, kernel]; bias [out_channels] or NULL;
 * y / dy [batch, out_channels, ho, wo] with ho = (height + 2*pad - kernel)/stride + 1.
 * backward: dx (assigned; may be NULL), gw and gb (assigned unless accumulate; may be NULL).  flip_taps == 0 gives the
 * true input gradient; flip_taps != 0 pairs each tap with the mirrored weight as conv.c:86-88 does. */
int bh_conv2d_forward(const float* x, const float* w, const float* bias, float* y, int64_t batch, int64_t in_channels,
                      int64_t height, int64_t width, int64_t out_channels, int64_t kernel, int64_t stride, int64_t pad);
/* the same forward (conv.c:326-437) as one contraction on the matrix cores, 3x3 and 5x5 kernels (any stride and padding): sums in MFMA order, so it
 * agrees with the reference to fp32 rounding instead of bit for bit (a max-pooling layer behind it may then pick the other
 * of two nearly equal maxima); several times faster on layers with many channels */
int bh_conv2d_forward_mfma(const float* x, const float* w, const float* bias, float* y, int64_t batch, int64_t in_channels,
                           int64_t height, int64_t width, int64_t out_channels, int64_t kernel, int64_t stride, int64_t pad);
int bh_conv2d_backward(const float* x, const float* w, const float* dy, float* dx, float* gw, float* gb, int64_t batch,
                       int64_t in_channels, int64_t height, int64_t width, int64_t out_channels, int64_t kernel,
                       int64_t stride, int64_t pad, int accumulate, int flip_taps);
/* planes = batch*channels images of [height, width]; argmax holds, per output, the offset of the window's first maximum
 * inside its plane (-1 when the window holds no comparable value) */
int bh_maxpool2d_forward(const float* x, float* y, int32_t* argmax, int64_t planes, int64_t height, int64_t width, int64_t pool,
                         int64_t stride, int64_t pad);
int bh_maxpool2d_backward(const float* dy, const int32_t* argmax, float* dx, int64_t planes, int64_t height, int64_t width,
                          int64_t pool, int64_t stride, int64_t pad);

/* ---- Adam (src/optimizers/adam.c:180-240) ----
 * timestep is the pre-increment value the reference passes to powf(beta, (float)(t+1)). */
int bh_adam_update(float* p, const float* g, float* m, float* v, int64_t n,
                   float lr, float beta1, float beta2, float eps, int64_t timestep);
/* benchmark hook: Adam's four read and three written streams with one add each instead of Adam's arithmetic (p += g,
 * m += g, v += g; n % 4 == 0, 16-byte aligned pointers): the rate the same grid reaches on this memory pattern */
int bh_stream_probe_4r3w(float* p, const float* g, float* m, float* v, int64_t n);
/* one launch over a table of tensors (host arrays of device pointers and element counts) */
int bh_adam_update_multi(float* const* p, const float* const* g, float* const* m, float* const* v,
                         const int64_t* n, int count,
                         float lr, float beta1, float beta2, float eps, int64_t timestep);

/* ---- RMSprop (src/optimizers/rmsprop.c:181-211) and Adagrad (src/optimizers/adagrad.c:167-197) ----
 * one state tensor each: sq = alpha*sq + (1-alpha)*g*g, resp. sum += g*g; then p -= lr*g/(sqrtf(state)+eps) */
int bh_rmsprop_update(float* p, const float* g, float* sq, int64_t n, float lr, float alpha, float eps);
int bh_adagrad_update(float* p, const float* g, float* sum, int64_t n, float lr, float eps);
int bh_rmsprop_update_multi(float* const* p, const float* const* g, float* const* sq, const int64_t* n, int count,
                            float lr, float alpha, float eps);
int bh_adagrad_update_multi(float* const* p, const float* const* g, float* const* sum, const int64_t* n, int count,
                            float lr, float eps);

/* zero `count` tensors in one launch: adam_optimizer_zero_grad's per-tensor memset loop (src/optimizers/adam.c:243-263) */
int bh_zero_multi(float* const* p, const int64_t* n, int count);

/* ---- test hooks (no arithmetic of their own) ----
 * bh_gemm_force_config: 0 = bounds-checked fallback, 1 = 128x128, 2 = 256x256, 3 = 256x128, 4 = 128x256 MFMA tile,
 * 5 = small-problem kernel (whole k-chunk in LDS, one trip to memory), 6 = tiny-problem kernel (operands straight
 * into the MFMA registers, contraction split among a workgroup's wavefronts), 7 = 64x64 MFMA tile (mid-sized and
 * small problems), -1 = heuristic (default).
 * bh_gemm_force_direct: 0 = MFMA tiles stage their operands through registers; 1 or -1 (default) = operands go
 * straight to LDS (global_load_lds) whenever the contraction length is a multiple of 16, and the eight-wavefront
 * tiles keep two k-tiles per LDS stage (one barrier per 32 k) when every workgroup's share of it is a multiple of 32;
 * 3 = straight to LDS with one k-tile per stage everywhere.
 * bh_sdpa_force_general: 0 = heuristic (default); 1 = always the row kernels; 2 = always the GEMM-based path (batched
 * bh_gemm products with row kernels for softmax and dS in between, what shapes other than head_dim 64 use from 64 keys on). */
int bh_gemm_force_config(int cfg);
int bh_gemm_force_direct(int mode);
/* bh_gemm_force_splits: where the MFMA tiles would split the contraction, split it this many ways (0 = heuristic) */
int bh_gemm_force_splits(int splits);
/* bh_gemm_no_tables: 1 = bh_gemm_grouped / bh_gemm_ksegments run their products one launch after the other (0 = one launch
 * where the shape allows) */
int bh_gemm_no_tables(int off);
int bh_sdpa_force_general(int on);
/* bh_sdpa_force_wide: 1 = the attention backward's 256-key workgroups (eight wavefronts) wherever that form exists
 * (head_dim 32 and 64), 0 = never, -1 = chosen by shape (the default) */
int bh_sdpa_force_wide(int mode);
/* bh_layernorm_tune: cap on the workgroups of the LayerNorm backward (each writes one dgamma/dbeta partial) and of
 * the forward; 0 keeps the current value. */
int bh_layernorm_tune(int bwd_blocks, int fwd_blocks);

#ifdef __cplusplus
}
#endif
#endif
