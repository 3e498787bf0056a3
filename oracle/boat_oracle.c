/* boat_oracle.c - CPU restatement of Boat's training hot path (see boat_oracle.h).
 *
 * TEST INFRASTRUCTURE ONLY: the checker the HIP path is compared with, and the
 * single-threaded CPU baseline timed beside it.  Build with plain -O3 and no
 * -ffast-math / -march flags so that no operation is reassociated or fused:
 * every loop below keeps the reference's operation order and operand types.
 */
#include "boat_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ linear */

/* src/ops/linear.c:116-130 */
void bo_matmul(const float* a, const float* b, float* c,
               int64_t batch, int64_t m, int64_t k, int64_t n) {
    for (int64_t bt = 0; bt < batch; bt++) {
        const float* ab = a + bt * m * k;
        const float* bb = b + bt * k * n;
        float* cb = c + bt * m * n;
        for (int64_t i = 0; i < m; i++) {
            for (int64_t j = 0; j < n; j++) {
                float sum = 0.0f;
                for (int64_t l = 0; l < k; l++) {
                    sum += ab[i * k + l] * bb[l * n + j];
                }
                cb[i * n + j] = sum;
            }
        }
    }
}

/* src/ops/linear.c:238-406 (pure data movement, so only the index map matters) */
void bo_transpose_last2(const float* a, float* out, int64_t batch, int64_t rows, int64_t cols) {
    for (int64_t bt = 0; bt < batch; bt++) {
        const float* ab = a + bt * rows * cols;
        float* ob = out + bt * rows * cols;
        for (int64_t i = 0; i < rows; i++)
            for (int64_t j = 0; j < cols; j++)
                ob[j * rows + i] = ab[i * cols + j];
    }
}

/* -------------------------------------------------------------- arithmetic */

void bo_add_inplace(float* a, const float* b, int64_t n) {      /* arithmetic.c:362-419 */
    for (int64_t i = 0; i < n; i++) a[i] += b[i];
}
void bo_mul(const float* a, const float* b, float* out, int64_t n) {   /* :157-285 */
    for (int64_t i = 0; i < n; i++) out[i] = a[i] * b[i];
}
void bo_div(const float* a, const float* b, float* out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = a[i] / b[i];
}
void bo_mul_scalar(const float* a, double s, float* out, int64_t n) {   /* :425-484, scalar narrowed first */
    float sf = (float)s;
    for (int64_t i = 0; i < n; i++) out[i] = a[i] * sf;
}
float bo_sum(const float* a, int64_t n) {                       /* :639-647 */
    float sum = 0.0f;
    for (int64_t i = 0; i < n; i++) sum += a[i];
    return sum;
}

/* src/autodiff.c:1115-1147 */
void bo_mul_backward(const float* a, const float* b, const float* dy, float* da, float* db, int64_t n) {
    if (da) for (int64_t i = 0; i < n; i++) da[i] = dy[i] * b[i];
    if (db) for (int64_t i = 0; i < n; i++) db[i] = dy[i] * a[i];
}

/* src/autodiff.c:1149-1203: da = dy/b ; db = (dy*-1) * (a / (b*b)) */
void bo_div_backward(const float* a, const float* b, const float* dy, float* da, float* db, int64_t n) {
    if (da) for (int64_t i = 0; i < n; i++) da[i] = dy[i] / b[i];
    if (db) {
        for (int64_t i = 0; i < n; i++) {
            float bsq = b[i] * b[i];
            float adb = a[i] / bsq;
            float neg = dy[i] * -1.0f;
            db[i] = neg * adb;
        }
    }
}

/* ------------------------------------------------------------- activations */

void bo_relu_forward(const float* x, float* y, int64_t n) {     /* autodiff.c:823-825 */
    for (int64_t i = 0; i < n; i++) y[i] = x[i] > 0 ? x[i] : 0.0f;
}
void bo_relu_backward(const float* x, const float* dy, float* dx, int64_t n) {   /* :1262-1287 */
    for (int64_t i = 0; i < n; i++) {
        float mask = x[i] > 0 ? 1.0f : 0.0f;
        dx[i] = dy[i] * mask;
    }
}
void bo_sigmoid_forward(const float* x, float* y, int64_t n) {  /* :855-861 */
    for (int64_t i = 0; i < n; i++) y[i] = 1.0f / (1.0f + expf(-x[i]));
}
void bo_sigmoid_backward(const float* c, const float* dy, float* dx, int64_t n) { /* :1298-1353 */
    for (int64_t i = 0; i < n; i++) {
        float omc = 1.0f - c[i];
        float t = c[i] * omc;
        dx[i] = dy[i] * t;
    }
}
void bo_tanh_forward(const float* x, float* y, int64_t n) {     /* :888-896 */
    for (int64_t i = 0; i < n; i++) {
        float ex = expf(x[i]);
        float emx = expf(-x[i]);
        y[i] = (ex - emx) / (ex + emx);
    }
}
void bo_tanh_backward(const float* c, const float* dy, float* dx, int64_t n) {    /* :1355-1452 */
    for (int64_t i = 0; i < n; i++) {
        float csq = c[i] * c[i];
        float om = 1.0f - csq;
        dx[i] = dy[i] * om;
    }
}

/* src/autodiff.c:1725-1751 */
void bo_softmax_forward(const float* x, float* y, int64_t rows, int64_t cols) {
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * cols;
        float* yr = y + r * cols;
        float mx = xr[0];
        for (int64_t i = 1; i < cols; i++) if (xr[i] > mx) mx = xr[i];
        float sum = 0.0f;
        for (int64_t i = 0; i < cols; i++) {
            float e = expf(xr[i] - mx);
            yr[i] = e;
            sum += e;
        }
        if (sum != 0.0f) {
            float inv = 1.0f / sum;
            for (int64_t i = 0; i < cols; i++) yr[i] *= inv;
        }
    }
}
/* src/autodiff.c:1921-1935 */
void bo_softmax_backward(const float* y, const float* dy, float* dx, int64_t rows, int64_t cols) {
    for (int64_t r = 0; r < rows; r++) {
        const float* yr = y + r * cols;
        const float* gr = dy + r * cols;
        float* dr = dx + r * cols;
        float t = 0.0f;
        for (int64_t i = 0; i < cols; i++) t += yr[i] * gr[i];
        for (int64_t i = 0; i < cols; i++) dr[i] = yr[i] * (gr[i] - t);
    }
}
/* src/autodiff.c:1820-1843 */
void bo_log_softmax_forward(const float* x, float* y, int64_t rows, int64_t cols) {
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * cols;
        float* yr = y + r * cols;
        float mx = xr[0];
        for (int64_t i = 1; i < cols; i++) if (xr[i] > mx) mx = xr[i];
        float sum = 0.0f;
        for (int64_t i = 0; i < cols; i++) sum += expf(xr[i] - mx);
        float lse = logf(fmaxf(sum, FLT_MIN));
        for (int64_t i = 0; i < cols; i++) yr[i] = xr[i] - mx - lse;
    }
}
/* src/autodiff.c:2014-2029 */
void bo_log_softmax_backward(const float* y, const float* dy, float* dx, int64_t rows, int64_t cols) {
    for (int64_t r = 0; r < rows; r++) {
        const float* yr = y + r * cols;
        const float* gr = dy + r * cols;
        float* dr = dx + r * cols;
        float g = 0.0f;
        for (int64_t i = 0; i < cols; i++) g += gr[i];
        for (int64_t i = 0; i < cols; i++) dr[i] = gr[i] - expf(yr[i]) * g;
    }
}

/* examples/mnist/mnist_autodiff.c:397-522 forward, then the tape walked backward:
 * loss = f * sum(onehot * log_softmax(z)), f = -1.0f/B.
 * seed 1 -> d(sum) = 1*f (autodiff.c:1134-1145) -> ones*scalar (:1510-1537)
 * -> d(ls) = d(m) * onehot (:1134-1145) -> log-softmax backward. */
float bo_ce_chain(const float* logits, const float* onehot, float* dlogits, int64_t rows, int64_t cols) {
    int64_t n = rows * cols;
    float* ls = (float*)malloc(sizeof(float) * (size_t)n);
    float* m = (float*)malloc(sizeof(float) * (size_t)n);
    bo_log_softmax_forward(logits, ls, rows, cols);
    for (int64_t i = 0; i < n; i++) m[i] = onehot[i] * ls[i];
    float s = bo_sum(m, n);
    float f = -1.0f / (float)(size_t)rows;
    float loss = f * s;
    if (dlogits) {
        float seed = 1.0f;
        float ds = seed * f;            /* grad of `sum` through mul(factor, sum) */
        for (int64_t i = 0; i < n; i++) m[i] = 1.0f * ds;            /* ones * scalar */
        for (int64_t i = 0; i < n; i++) m[i] = m[i] * onehot[i];     /* d(ls) = d(m) * onehot */
        bo_log_softmax_backward(ls, m, dlogits, rows, cols);
    }
    free(ls);
    free(m);
    return loss;
}

/* ------------------------------------------------------------------- dense */

/* src/layers/dense.c:150-185 */
void bo_dense_forward(const float* x, const float* w, const float* bias, float* y,
                      int64_t m, int64_t k, int64_t n) {
    bo_matmul(x, w, y, 1, m, k, n);
    if (bias) {
        for (int64_t i = 0; i < m; i++)
            for (int64_t j = 0; j < n; j++)
                y[i * n + j] += bias[j];
    }
}

/* src/layers/dense.c:219-291 */
void bo_dense_backward(const float* x, const float* w, const float* dy,
                       float* dx, float* gw, float* gb,
                       int64_t m, int64_t k, int64_t n) {
    float* wt = (float*)malloc(sizeof(float) * (size_t)(k * n));
    bo_transpose_last2(w, wt, 1, k, n);                 /* [n, k] */
    bo_matmul(dy, wt, dx, 1, m, n, k);                  /* dX = dY . W^T */
    free(wt);
    float* xt = (float*)malloc(sizeof(float) * (size_t)(m * k));
    float* g = (float*)malloc(sizeof(float) * (size_t)(k * n));
    bo_transpose_last2(x, xt, 1, m, k);                 /* [k, m] */
    bo_matmul(xt, dy, g, 1, k, m, n);                   /* X^T . dY */
    bo_add_inplace(gw, g, k * n);
    free(xt);
    free(g);
    if (gb) {
        for (int64_t b = 0; b < m; b++)
            for (int64_t j = 0; j < n; j++)
                gb[j] += dy[b * n + j];
    }
}

/* --------------------------------------------------------------- attention */

/* src/layers/attention.c:997-1073 */
void bo_sdpa_forward(const float* q, const float* k, const float* v, float scale, int causal,
                     float* attn, float* out, float* lse, int64_t bh, int64_t s, int64_t d) {
    float* scores = (float*)malloc(sizeof(float) * (size_t)(s * s));
    for (int64_t h = 0; h < bh; h++) {
        const float* qh = q + h * s * d;
        const float* kh = k + h * s * d;
        const float* vh = v + h * s * d;
        float* oh = out + h * s * d;
        for (int64_t i = 0; i < s; i++) {
            for (int64_t j = 0; j < s; j++) {
                float sum = 0.0f;
                for (int64_t t = 0; t < d; t++) sum += qh[i * d + t] * kh[j * d + t];
                scores[i * s + j] = sum * scale;
            }
        }
        if (causal) {
            for (int64_t i = 0; i < s; i++)
                for (int64_t j = i + 1; j < s; j++) scores[i * s + j] = -1e9f;
        }
        for (int64_t i = 0; i < s; i++) {
            float mx = scores[i * s];
            for (int64_t j = 1; j < s; j++) if (scores[i * s + j] > mx) mx = scores[i * s + j];
            float sum = 0.0f;
            for (int64_t j = 0; j < s; j++) {
                scores[i * s + j] = expf(scores[i * s + j] - mx);
                sum += scores[i * s + j];
            }
            if (sum != 0.0f) {
                for (int64_t j = 0; j < s; j++) scores[i * s + j] /= sum;
            }
            if (lse) lse[h * s + i] = mx + logf(sum);
        }
        if (attn) memcpy(attn + h * s * s, scores, sizeof(float) * (size_t)(s * s));
        for (int64_t i = 0; i < s; i++) {
            for (int64_t t = 0; t < d; t++) {
                float sum = 0.0f;
                for (int64_t j = 0; j < s; j++) sum += scores[i * s + j] * vh[j * d + t];
                oh[i * d + t] = sum;
            }
        }
    }
    free(scores);
}

/* src/layers/attention.c:1417-1520 */
void bo_sdpa_backward(const float* q, const float* k, const float* v, const float* attn,
                      const float* d_out, float scale,
                      float* dq, float* dk, float* dv, int64_t bh, int64_t s, int64_t d) {
    float* at = (float*)malloc(sizeof(float) * (size_t)(bh * s * s));
    bo_transpose_last2(attn, at, bh, s, s);
    bo_matmul(at, d_out, dv, bh, s, s, d);                       /* dV = A^T . dO */
    float* vt = (float*)malloc(sizeof(float) * (size_t)(bh * s * d));
    bo_transpose_last2(v, vt, bh, s, d);                         /* [d, s] */
    float* da = (float*)malloc(sizeof(float) * (size_t)(bh * s * s));
    bo_matmul(d_out, vt, da, bh, s, d, s);                       /* dA = dO . V^T */
    free(vt);
    float* ds = at;                                              /* reuse */
    for (int64_t r = 0; r < bh * s; r++) {
        const float* ar = attn + r * s;
        const float* gr = da + r * s;
        double sum = 0.0;
        for (int64_t j = 0; j < s; j++) sum += (double)gr[j] * (double)ar[j];
        for (int64_t j = 0; j < s; j++) ds[r * s + j] = ar[j] * (gr[j] - sum);   /* float*(float-double) -> float */
    }
    bo_mul_scalar(ds, (double)scale, ds, bh * s * s);
    bo_matmul(ds, k, dq, bh, s, s, d);                           /* dQ = dS . K */
    bo_transpose_last2(ds, da, bh, s, s);
    bo_matmul(da, q, dk, bh, s, s, d);                           /* dK = dS^T . Q */
    free(da);
    free(at);
}

/* src/layers/attention.c:247-308 applied to [batch*seq, hidden]: matmul then
 * bias broadcast through boat_add (arithmetic.c:157-285). */
static void projection(const float* x, const float* w, const float* bias, float* y,
                       int64_t rows, int64_t hidden) {
    bo_matmul(x, w, y, 1, rows, hidden, hidden);
    if (bias) {
        for (int64_t i = 0; i < rows; i++)
            for (int64_t j = 0; j < hidden; j++)
                y[i * hidden + j] = y[i * hidden + j] + bias[j];
    }
}

/* src/layers/attention.c:1186-1285 (3-D branch) */
static void projection_backward(const float* x, const float* w, const float* dy, int has_bias,
                                float* dx, float* gw, float* gb, int64_t rows, int64_t hidden) {
    float* wt = (float*)malloc(sizeof(float) * (size_t)(hidden * hidden));
    bo_transpose_last2(w, wt, 1, hidden, hidden);
    bo_matmul(dy, wt, dx, 1, rows, hidden, hidden);
    free(wt);
    float* xt = (float*)malloc(sizeof(float) * (size_t)(rows * hidden));
    bo_transpose_last2(x, xt, 1, rows, hidden);
    bo_matmul(xt, dy, gw, 1, hidden, rows, hidden);              /* overwritten, not accumulated */
    free(xt);
    if (has_bias && gb) {
        memset(gb, 0, sizeof(float) * (size_t)hidden);
        for (int64_t r = 0; r < rows; r++)
            for (int64_t j = 0; j < hidden; j++)
                gb[j] += dy[r * hidden + j];
    }
}

void bo_attention_forward(const float* query, const float* key, const float* value,
                          const float* wq, const float* wk, const float* wv, const float* wo,
                          const float* bq, const float* bk, const float* bv, const float* bo_,
                          int causal, int64_t batch, int64_t seq, int64_t hidden, int64_t heads,
                          float* q_proj, float* k_proj, float* v_proj,
                          float* attn, float* attn_out, float* out) {
    int64_t rows = batch * seq;
    int64_t hd = hidden / heads;
    projection(query, wq, bq, q_proj, rows, hidden);
    projection(key, wk, bk, k_proj, rows, hidden);
    projection(value, wv, bv, v_proj, rows, hidden);
    /* head split is a plain reshape [B,S,H] -> [B,nh,S,hd] (attention.c:393-397):
     * block (b,h) is the h-th run of S*hd contiguous floats of batch b. */
    float scale = 1.0f / sqrtf((float)hd);
    bo_sdpa_forward(q_proj, k_proj, v_proj, scale, causal, attn, attn_out, NULL, batch * heads, seq, hd);
    projection(attn_out, wo, bo_, out, rows, hidden);
}

void bo_attention_backward(const float* query, const float* key, const float* value,
                           const float* wq, const float* wk, const float* wv, const float* wo,
                           int has_bias,
                           const float* q_proj, const float* k_proj, const float* v_proj,
                           const float* attn, const float* attn_out, const float* d_out,
                           int64_t batch, int64_t seq, int64_t hidden, int64_t heads,
                           float* d_query, float* d_key, float* d_value,
                           float* gwq, float* gwk, float* gwv, float* gwo,
                           float* gbq, float* gbk, float* gbv, float* gbo) {
    int64_t rows = batch * seq;
    int64_t hd = hidden / heads;
    size_t act = sizeof(float) * (size_t)(rows * hidden);
    float* d_ao = (float*)malloc(act);
    float* dqp = (float*)malloc(act);
    float* dkp = (float*)malloc(act);
    float* dvp = (float*)malloc(act);
    projection_backward(attn_out, wo, d_out, has_bias, d_ao, gwo, gbo, rows, hidden);
    float scale = 1.0f / sqrtf((float)hd);
    bo_sdpa_backward(q_proj, k_proj, v_proj, attn, d_ao, scale, dqp, dkp, dvp, batch * heads, seq, hd);
    projection_backward(query, wq, dqp, has_bias, d_query, gwq, gbq, rows, hidden);
    projection_backward(key, wk, dkp, has_bias, d_key, gwk, gbk, rows, hidden);
    projection_backward(value, wv, dvp, has_bias, d_value, gwv, gbv, rows, hidden);
    free(d_ao);
    free(dqp);
    free(dkp);
    free(dvp);
}

/* --------------------------------------------------------------- layernorm */

/* src/layers/norm.c:184-209 (stats) and :283-305 (normalise + affine) */
void bo_layernorm_forward(const float* x, const float* gamma, const float* beta, float* y,
                          float* mean, float* rstd, int64_t rows, int64_t hidden, float eps) {
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * hidden;
        float* yr = y + r * hidden;
        float sum = 0.0f;
        for (int64_t h = 0; h < hidden; h++) sum += xr[h];
        float m = sum / (float)(size_t)hidden;
        float var_sum = 0.0f;
        for (int64_t h = 0; h < hidden; h++) {
            float diff = xr[h] - m;
            var_sum += diff * diff;
        }
        float var = var_sum / (float)(size_t)hidden;
        float scale = 1.0f / sqrtf(var + eps);
        for (int64_t h = 0; h < hidden; h++) {
            float nrm = (xr[h] - m) * scale;
            if (gamma) nrm = nrm * gamma[h];
            if (beta) nrm = nrm + beta[h];
            yr[h] = nrm;
        }
        if (mean) mean[r] = m;
        if (rstd) rstd[r] = scale;
    }
}

/* src/layers/norm.c:212-229 (compute_rms) and :366-389 (apply) */
void bo_rmsnorm_forward(const float* x, const float* weight, float* y, float* inv_rms,
                        int64_t rows, int64_t hidden, float eps) {
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * hidden;
        float* yr = y + r * hidden;
        float sum_sq = 0.0f;
        for (int64_t h = 0; h < hidden; h++) {
            float val = xr[h];
            sum_sq += val * val;
        }
        float rms = sqrtf(sum_sq / (float)(size_t)hidden);
        float scale = 1.0f / (rms + eps);
        for (int64_t h = 0; h < hidden; h++) {
            float nrm = xr[h] * scale;
            if (weight) nrm = nrm * weight[h];
            yr[h] = nrm;
        }
        if (inv_rms) inv_rms[r] = scale;
    }
}

/* -------------------------------------------------------------------- adam */

/* src/optimizers/adam.c:203-222 */
void bo_adam_update(float* p, const float* g, float* m, float* v, int64_t n,
                    float lr, float beta1, float beta2, float eps, int64_t timestep) {
    float b1t = powf(beta1, (float)(timestep + 1));
    float b2t = powf(beta2, (float)(timestep + 1));
    for (int64_t i = 0; i < n; i++) {
        float gi = g[i];
        m[i] = beta1 * m[i] + (1.0f - beta1) * gi;
        v[i] = beta2 * v[i] + (1.0f - beta2) * gi * gi;
        float m_hat = m[i] / (1.0f - b1t);
        float v_hat = v[i] / (1.0f - b2t);
        p[i] -= lr * m_hat / (sqrtf(v_hat) + eps);
    }
}

/* ------------------------------------------------------------- conv / pool */

/* src/layers/conv.c:398-436: per (b, oc): for each input channel a running sum over the taps is added to the
 * output element; the bias is added last. */
void bo_conv2d_forward(const float* x, const float* w, const float* bias, float* y,
                       int64_t batch, int64_t ic, int64_t h, int64_t wd, int64_t oc, int64_t k, int64_t stride, int64_t pad) {
    const int64_t ho = (h + 2 * pad - k) / stride + 1, wo = (wd + 2 * pad - k) / stride + 1;
    memset(y, 0, sizeof(float) * (size_t)(batch * oc * ho * wo));
    for (int64_t b = 0; b < batch; b++)
        for (int64_t o = 0; o < oc; o++) {
            for (int64_t c = 0; c < ic; c++)
                for (int64_t oh = 0; oh < ho; oh++)
                    for (int64_t ow = 0; ow < wo; ow++) {
                        float sum = 0.0f;
                        for (int64_t kh = 0; kh < k; kh++) {
                            int64_t ih = oh * stride - pad + kh;
                            if (ih < 0 || ih >= h) continue;
                            for (int64_t kw = 0; kw < k; kw++) {
                                int64_t iw = ow * stride - pad + kw;
                                if (iw < 0 || iw >= wd) continue;
                                sum += x[((b * ic + c) * h + ih) * wd + iw] * w[((o * ic + c) * k + kh) * k + kw];
                            }
                        }
                        y[((b * oc + o) * ho + oh) * wo + ow] += sum;
                    }
            if (bias)
                for (int64_t i = 0; i < ho * wo; i++) y[(b * oc + o) * ho * wo + i] += bias[o];
        }
}

/* src/layers/conv.c:46-201.  All three gradients are overwritten.  flip_taps != 0 is the reference as written:
 * the input gradient pairs tap (kh, kw) with the weight of tap (k-1-kh, k-1-kw) (:86-88); flip_taps == 0 uses the
 * weight of the same tap, which is the true gradient of bo_conv2d_forward. */
void bo_conv2d_backward(const float* x, const float* w, const float* dy, float* dx, float* gw, float* gb,
                        int64_t batch, int64_t ic, int64_t h, int64_t wd, int64_t oc, int64_t k, int64_t stride, int64_t pad,
                        int flip_taps) {
    const int64_t ho = (h + 2 * pad - k) / stride + 1, wo = (wd + 2 * pad - k) / stride + 1;
    if (dx) memset(dx, 0, sizeof(float) * (size_t)(batch * ic * h * wd));
    if (gw) memset(gw, 0, sizeof(float) * (size_t)(oc * ic * k * k));
    for (int64_t b = 0; b < batch; b++)
        for (int64_t o = 0; o < oc; o++)
            for (int64_t c = 0; c < ic; c++)
                for (int64_t kh = 0; kh < k; kh++)
                    for (int64_t kw = 0; kw < k; kw++)
                        for (int64_t oh = 0; oh < ho; oh++) {
                            int64_t ih = oh * stride - pad + kh;
                            if (ih < 0 || ih >= h) continue;
                            for (int64_t ow = 0; ow < wo; ow++) {
                                int64_t iw = ow * stride - pad + kw;
                                if (iw < 0 || iw >= wd) continue;
                                const int64_t xi = ((b * ic + c) * h + ih) * wd + iw;
                                const int64_t gi = ((b * oc + o) * ho + oh) * wo + ow;
                                if (dx) {
                                    const int64_t wi = flip_taps ? ((o * ic + c) * k + (k - 1 - kh)) * k + (k - 1 - kw)
                                                                 : ((o * ic + c) * k + kh) * k + kw;
                                    dx[xi] += w[wi] * dy[gi];
                                }
                                if (gw) gw[((o * ic + c) * k + kh) * k + kw] += x[xi] * dy[gi];
                            }
                        }
    if (gb) {
        memset(gb, 0, sizeof(float) * (size_t)oc);
        for (int64_t b = 0; b < batch; b++)
            for (int64_t o = 0; o < oc; o++) {
                float sum = 0.0f;
                for (int64_t i = 0; i < ho * wo; i++) sum += dy[(b * oc + o) * ho * wo + i];
                gb[o] += sum;
            }
    }
}

/* src/layers/pool.c:100-133: window clamped to the image, first maximum wins (strict >); argmax is the flat input index or -1 */
void bo_maxpool2d_forward(const float* x, float* y, int64_t* argmax, int64_t planes, int64_t h, int64_t wd,
                          int64_t pool, int64_t stride, int64_t pad) {
    const int64_t ho = (h + 2 * pad - pool) / stride + 1, wo = (wd + 2 * pad - pool) / stride + 1;
    for (int64_t p = 0; p < planes; p++)
        for (int64_t oh = 0; oh < ho; oh++)
            for (int64_t ow = 0; ow < wo; ow++) {
                int64_t h0 = oh * stride - pad, w0 = ow * stride - pad;
                int64_t h1 = h0 + pool, w1 = w0 + pool;
                h0 = h0 < 0 ? 0 : h0;
                w0 = w0 < 0 ? 0 : w0;
                h1 = h1 > h ? h : h1;
                w1 = w1 > wd ? wd : w1;
                float best = -INFINITY;
                int64_t where = -1;
                for (int64_t ph = h0; ph < h1; ph++)
                    for (int64_t pw = w0; pw < w1; pw++) {
                        const int64_t idx = (p * h + ph) * wd + pw;
                        if (x[idx] > best) {
                            best = x[idx];
                            where = idx;
                        }
                    }
                y[(p * ho + oh) * wo + ow] = best;
                argmax[(p * ho + oh) * wo + ow] = where;
            }
}

/* src/layers/pool.c:199-213 */
void bo_maxpool2d_backward(const float* dy, const int64_t* argmax, float* dx, int64_t n_in, int64_t n_out) {
    memset(dx, 0, sizeof(float) * (size_t)n_in);
    for (int64_t i = 0; i < n_out; i++)
        if (argmax[i] >= 0 && argmax[i] < n_in) dx[argmax[i]] += dy[i];
}

/* ------------------------------------------------------------------ losses */

/* mean loss of the reference's loss objects, fp32 left-to-right sums: kind 0 src/loss/mse.c:70-80, kind 1
 * src/loss/cross_entropy.c:35-44,86-98 (returns the negated mean), kind 2 src/loss/huber.c (threshold delta) */
float bo_loss_value(int kind, const float* p, const float* t, int64_t n, float delta) {
    float sum = 0.0f;
    for (int64_t i = 0; i < n; i++) {
        if (kind == 0) {
            float diff = p[i] - t[i];
            sum += diff * diff;
        } else if (kind == 1) {
            const float eps = 1e-7f;
            float c = p[i];
            if (c < eps) c = eps;
            else if (c > 1.0f - eps) c = 1.0f - eps;
            sum += t[i] * logf(c);
        } else {
            float diff = fabsf(p[i] - t[i]);
            if (diff <= delta) sum += 0.5f * diff * diff;
            else sum += delta * (diff - 0.5f * delta);
        }
    }
    const float mean = sum / (size_t)n;
    return kind == 1 ? -mean : mean;
}

/* src/optimizers/rmsprop.c:197-210 */
void bo_rmsprop_update(float* p, const float* g, float* sq, int64_t n, float lr, float alpha, float eps) {
    for (int64_t i = 0; i < n; i++) {
        float gi = g[i];
        sq[i] = alpha * sq[i] + (1.0f - alpha) * gi * gi;
        p[i] -= lr * gi / (sqrtf(sq[i]) + eps);
    }
}

/* src/optimizers/adagrad.c:183-196 */
void bo_adagrad_update(float* p, const float* g, float* sum, int64_t n, float lr, float eps) {
    for (int64_t i = 0; i < n; i++) {
        float gi = g[i];
        sum[i] += gi * gi;
        p[i] -= lr * gi / (sqrtf(sum[i]) + eps);
    }
}

/* -------------------------------------------------------------------- loss */

/* src/loss/mse.c:70-78 */
float bo_mse_loss(const float* pred, const float* target, int64_t n) {
    float sse = 0.0f;
    for (int64_t i = 0; i < n; i++) {
        float diff = pred[i] - target[i];
        sse += diff * diff;
    }
    return sse / (float)(size_t)n;
}

/* tests/test_attention_training.c:28-41 */
void bo_mse_grad(const float* pred, const float* target, float* grad, int64_t n) {
    for (int64_t i = 0; i < n; i++) grad[i] = 2.0f * (pred[i] - target[i]) / (float)(size_t)n;
}

/* ---------------- no reference counterpart: double-precision closed forms */

/* xhat = (x-mean)*rstd ; g = dy*gamma ;
 * dx = rstd * (g - mean_h(g) - xhat * mean_h(g*xhat)) ; dgamma = sum_rows dy*xhat ; dbeta = sum_rows dy */
void bo_layernorm_backward_f64(const float* x, const float* gamma, const float* dy,
                               const float* mean, const float* rstd,
                               double* dx, double* dgamma, double* dbeta,
                               int64_t rows, int64_t hidden) {
    if (dgamma) memset(dgamma, 0, sizeof(double) * (size_t)hidden);
    if (dbeta) memset(dbeta, 0, sizeof(double) * (size_t)hidden);
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * hidden;
        const float* gr = dy + r * hidden;
        double mu = mean[r], rs = rstd[r];
        double s1 = 0.0, s2 = 0.0;
        for (int64_t h = 0; h < hidden; h++) {
            double xh = ((double)xr[h] - mu) * rs;
            double g = (double)gr[h] * (gamma ? (double)gamma[h] : 1.0);
            s1 += g;
            s2 += g * xh;
            if (dgamma) dgamma[h] += (double)gr[h] * xh;
            if (dbeta) dbeta[h] += (double)gr[h];
        }
        s1 /= (double)hidden;
        s2 /= (double)hidden;
        if (dx) {
            for (int64_t h = 0; h < hidden; h++) {
                double xh = ((double)xr[h] - mu) * rs;
                double g = (double)gr[h] * (gamma ? (double)gamma[h] : 1.0);
                dx[r * hidden + h] = rs * (g - s1 - xh * s2);
            }
        }
    }
}

/* y_j = x_j*w_j*s with s = 1/(r+eps), r = sqrt(mean_h x^2):
 * dx_j = s*g_j - s^2 * (sum_i g_i x_i) * x_j/(H r)   (g = dy*w; the second term is absent for a row of zeros);
 * dw_j = sum_rows dy_j x_j s */
void bo_rmsnorm_backward_f64(const float* x, const float* weight, const float* dy, double* dx, double* dweight,
                             int64_t rows, int64_t hidden, double eps) {
    if (dweight) memset(dweight, 0, sizeof(double) * (size_t)hidden);
    for (int64_t r = 0; r < rows; r++) {
        const float* xr = x + r * hidden;
        const float* gr = dy + r * hidden;
        double sq = 0.0, gx = 0.0;
        for (int64_t h = 0; h < hidden; h++) {
            sq += (double)xr[h] * (double)xr[h];
            gx += (double)gr[h] * (weight ? (double)weight[h] : 1.0) * (double)xr[h];
        }
        const double rms = sqrt(sq / (double)hidden);
        const double s = 1.0 / (rms + eps);
        for (int64_t h = 0; h < hidden; h++) {
            const double g = (double)gr[h] * (weight ? (double)weight[h] : 1.0);
            if (dx) dx[r * hidden + h] = s * g - (rms > 0.0 ? s * s * gx * (double)xr[h] / ((double)hidden * rms) : 0.0);
            if (dweight) dweight[h] += (double)gr[h] * (double)xr[h] * s;
        }
    }
}

/* exact (erf) GELU: y = x*Phi(x), dy/dx = Phi(x) + x*phi(x) */
void bo_gelu_forward_f64(const float* x, double* y, int64_t n) {
    for (int64_t i = 0; i < n; i++) {
        double xd = x[i];
        y[i] = 0.5 * xd * (1.0 + erf(xd * 0.70710678118654752440));
    }
}
void bo_gelu_backward_f64(const float* x, const float* dy, double* dx, int64_t n) {
    for (int64_t i = 0; i < n; i++) {
        double xd = x[i];
        double cdf = 0.5 * (1.0 + erf(xd * 0.70710678118654752440));
        double pdf = 0.39894228040143267794 * exp(-0.5 * xd * xd);
        dx[i] = (double)dy[i] * (cdf + xd * pdf);
    }
}
