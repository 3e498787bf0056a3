/* boat_oracle.h - CPU restatement of Boat's training hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product library links, loads or
 * calls this file; it exists so that tests, the smoke check and the CPU
 * baseline leg of the benchmark have something to compare the HIP path with
 * (and to time beside it).  Every routine follows the loop order and the
 * floating-point types of the reference C sources cited above it, so that on
 * the same inputs it reproduces the reference's results bit for bit (checked
 * against the compiled reference in oracle/_ref and the committed golden
 * vectors).
 *
 * Routines whose names end in _f64 have NO counterpart in the reference (the
 * reference ships stubs for them): LayerNorm and RMSNorm backward, GELU
 * forward/backward and the MSE gradient.  They are double-precision closed forms, pinned by
 * finite differences and by an independent autograd library's vectors, and
 * their parity with the reference is by construction "unpinned".
 *
 * All tensors are dense, row-major, contiguous fp32 unless stated.
 */
#ifndef BOAT_ORACLE_H
#define BOAT_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* src/ops/linear.c:116-130 (batched i-j-l loop, fp32 running sum). */
void bo_matmul(const float* a, const float* b, float* c,
               int64_t batch, int64_t m, int64_t k, int64_t n);
/* src/ops/linear.c:238-406 restricted to swapping the last two dims. */
void bo_transpose_last2(const float* a, float* out, int64_t batch, int64_t rows, int64_t cols);

/* src/ops/arithmetic.c:362-419 / 157-285 / 425-484 / 611-691 (same-shape case). */
void bo_add_inplace(float* a, const float* b, int64_t n);
void bo_mul(const float* a, const float* b, float* out, int64_t n);
void bo_div(const float* a, const float* b, float* out, int64_t n);
void bo_mul_scalar(const float* a, double s, float* out, int64_t n);
float bo_sum(const float* a, int64_t n);

/* src/autodiff.c:1115-1203: gradients of c=a*b and c=a/b (assign form). */
void bo_mul_backward(const float* a, const float* b, const float* dy, float* da, float* db, int64_t n);
void bo_div_backward(const float* a, const float* b, const float* dy, float* da, float* db, int64_t n);

/* src/autodiff.c:808-842, 1244-1296. */
void bo_relu_forward(const float* x, float* y, int64_t n);
void bo_relu_backward(const float* x, const float* dy, float* dx, int64_t n);
/* src/autodiff.c:844-909, 1298-1452 (c is the saved forward output). */
void bo_sigmoid_forward(const float* x, float* y, int64_t n);
void bo_sigmoid_backward(const float* c, const float* dy, float* dx, int64_t n);
void bo_tanh_forward(const float* x, float* y, int64_t n);
void bo_tanh_backward(const float* c, const float* dy, float* dx, int64_t n);

/* src/autodiff.c:1701-1794, 1885-1973 (last axis). */
void bo_softmax_forward(const float* x, float* y, int64_t rows, int64_t cols);
void bo_softmax_backward(const float* y, const float* dy, float* dx, int64_t rows, int64_t cols);
/* src/autodiff.c:1796-1883, 1975-2068. */
void bo_log_softmax_forward(const float* x, float* y, int64_t rows, int64_t cols);
void bo_log_softmax_backward(const float* y, const float* dy, float* dx, int64_t rows, int64_t cols);

/* The loss chain of examples/mnist/mnist_autodiff.c:397-522 and its backward
 * through src/autodiff.c (log_softmax -> mul(onehot) -> sum -> mul(-1/B)):
 * returns the loss, writes dlogits. */
float bo_ce_chain(const float* logits, const float* onehot, float* dlogits, int64_t rows, int64_t cols);

/* src/layers/dense.c:135-188 and :190-295 (gw, gb accumulate with +=). */
void bo_dense_forward(const float* x, const float* w, const float* bias, float* y,
                      int64_t m, int64_t k, int64_t n);
void bo_dense_backward(const float* x, const float* w, const float* dy,
                       float* dx, float* gw, float* gb,
                       int64_t m, int64_t k, int64_t n);

/* src/layers/attention.c:882-1079: one call covers bh = batch*heads blocks of
 * [s, d] floats.  attn receives softmax weights [bh, s, s]; lse (may be NULL)
 * receives max + logf(sum) per row, which the reference does not keep. */
void bo_sdpa_forward(const float* q, const float* k, const float* v, float scale, int causal,
                     float* attn, float* out, float* lse, int64_t bh, int64_t s, int64_t d);
/* src/layers/attention.c:1388-1534. */
void bo_sdpa_backward(const float* q, const float* k, const float* v, const float* attn,
                      const float* d_out, float scale,
                      float* dq, float* dk, float* dv, int64_t bh, int64_t s, int64_t d);

/* Whole attention layer, src/layers/attention.c:310-466 and :468-732.
 * Weights are [hidden, hidden] in [in, out] layout; biases may be NULL.
 * Caches (q_proj, k_proj, v_proj, attn, attn_out) are caller-provided. */
void bo_attention_forward(const float* query, const float* key, const float* value,
                          const float* wq, const float* wk, const float* wv, const float* wo,
                          const float* bq, const float* bk, const float* bv, const float* bo_,
                          int causal, int64_t batch, int64_t seq, int64_t hidden, int64_t heads,
                          float* q_proj, float* k_proj, float* v_proj,
                          float* attn, float* attn_out, float* out);
void bo_attention_backward(const float* query, const float* key, const float* value,
                           const float* wq, const float* wk, const float* wv, const float* wo,
                           int has_bias,
                           const float* q_proj, const float* k_proj, const float* v_proj,
                           const float* attn, const float* attn_out, const float* d_out,
                           int64_t batch, int64_t seq, int64_t hidden, int64_t heads,
                           float* d_query, float* d_key, float* d_value,
                           float* gwq, float* gwk, float* gwv, float* gwo,
                           float* gbq, float* gbk, float* gbv, float* gbo);

/* src/layers/norm.c:184-209, 231-317.  mean/rstd may be NULL. */
void bo_layernorm_forward(const float* x, const float* gamma, const float* beta, float* y,
                          float* mean, float* rstd, int64_t rows, int64_t hidden, float eps);

/* src/layers/norm.c:212-229 (rms = sqrtf(sum_sq / hidden)) and :366-389 (scale = 1/(rms + eps), then * weight).
 * weight and inv_rms may be NULL; inv_rms receives the per-row scale. */
void bo_rmsnorm_forward(const float* x, const float* weight, float* y, float* inv_rms,
                        int64_t rows, int64_t hidden, float eps);

/* src/optimizers/adam.c:180-223 for one tensor at the given (pre-increment)
 * timestep; the caller increments the timestep after all tensors (:226-240). */
void bo_adam_update(float* p, const float* g, float* m, float* v, int64_t n,
                    float lr, float beta1, float beta2, float eps, int64_t timestep);

/* src/layers/conv.c:326-437 (NCHW, weight [oc, ic, k, k], bias may be NULL). */
void bo_conv2d_forward(const float* x, const float* w, const float* bias, float* y,
                       int64_t batch, int64_t ic, int64_t h, int64_t wd, int64_t oc, int64_t k, int64_t stride, int64_t pad);
/* src/layers/conv.c:46-201; dx, gw, gb may be NULL.  flip_taps != 0 reproduces the reference's input gradient
 * (mirrored taps, :86-88); flip_taps == 0 is the true gradient. */
void bo_conv2d_backward(const float* x, const float* w, const float* dy, float* dx, float* gw, float* gb,
                        int64_t batch, int64_t ic, int64_t h, int64_t wd, int64_t oc, int64_t k, int64_t stride, int64_t pad,
                        int flip_taps);
/* src/layers/pool.c:63-218; planes = batch*channels; argmax = flat input index of each window's maximum. */
void bo_maxpool2d_forward(const float* x, float* y, int64_t* argmax, int64_t planes, int64_t h, int64_t wd,
                          int64_t pool, int64_t stride, int64_t pad);
void bo_maxpool2d_backward(const float* dy, const int64_t* argmax, float* dx, int64_t n_in, int64_t n_out);

/* src/loss/mse.c:37-88, cross_entropy.c:48-104, huber.c: kind 0 MSE, 1 cross entropy over probabilities, 2 Huber(delta). */
float bo_loss_value(int kind, const float* p, const float* t, int64_t n, float delta);

/* src/optimizers/rmsprop.c:181-211 and src/optimizers/adagrad.c:167-197: one tensor, one step. */
void bo_rmsprop_update(float* p, const float* g, float* sq, int64_t n, float lr, float alpha, float eps);
void bo_adagrad_update(float* p, const float* g, float* sum, int64_t n, float lr, float eps);

/* src/loss/mse.c:37-88 (value) -- mean over all elements, fp32 running sum. */
float bo_mse_loss(const float* pred, const float* target, int64_t n);

/* ---- no reference counterpart (stubs there): double-precision closed forms ---- */
void bo_layernorm_backward_f64(const float* x, const float* gamma, const float* dy,
                               const float* mean, const float* rstd,
                               double* dx, double* dgamma, double* dbeta,
                               int64_t rows, int64_t hidden);
/* RMSNorm backward (stub in the reference, src/layers/norm.c:404-409): derivative of y = x*w/(sqrt(mean(x^2)) + eps)
 * in double precision, straight from x (no saved statistics) */
void bo_rmsnorm_backward_f64(const float* x, const float* weight, const float* dy, double* dx, double* dweight,
                             int64_t rows, int64_t hidden, double eps);
void bo_gelu_forward_f64(const float* x, double* y, int64_t n);
void bo_gelu_backward_f64(const float* x, const float* dy, double* dx, int64_t n);
/* gradient of the mean-squared error, 2(o-t)/n, as tests/test_attention_training.c:28-41 writes it */
void bo_mse_grad(const float* pred, const float* target, float* grad, int64_t n);

#ifdef __cplusplus
}
#endif
#endif
