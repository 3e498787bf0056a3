/* api_tour.c - one pass over the training-path API of Boat, from a plain C caller.
 *
 * Where mlp_train_step.c times one network, this program touches every family of entry points once, frees everything it
 * creates and checks a few invariants on the way (gradient shapes, losses that fall, optimizers that move parameters).
 * It is the program to run under a host-side sanitizer after changing the C side of the library:
 *
 *   gcc -fsanitize=address,undefined api_tour.c -I<repo>/include -L<dir> -lboat_amd -lm
 *
 * Every call is Boat's own API (same names and signatures as the reference's headers) except those named boat_hip_*.
 * Exit status 0 = every check held; otherwise the number of the first failed check is printed.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "boat_api.h"

static int g_failed = 0;
#define CHECK(cond)                                                                  \
    do {                                                                             \
        if (!(cond)) {                                                               \
            fprintf(stderr, "api_tour: check failed at line %d: %s\n", __LINE__, #cond); \
            if (!g_failed) g_failed = __LINE__;                                      \
        }                                                                            \
    } while (0)

static uint64_t rng_state = 0x243F6A8885A308D3ull;
static float uniform01(void) {
    uint64_t z = (rng_state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (float)(z >> 40) / 16777216.0f;
}

static boat_tensor_t* random_tensor(const int64_t* shape, size_t ndim, float scale) {
    boat_tensor_t* t = boat_tensor_create(shape, ndim, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    if (!t) return NULL;
    float* p = (float*)boat_tensor_data(t);
    const size_t n = boat_tensor_nelements(t);
    for (size_t i = 0; i < n; i++) p[i] = (2.0f * uniform01() - 1.0f) * scale;
    return t;
}

static float first_value(const boat_tensor_t* t) { return ((const float*)boat_tensor_const_data(t))[0]; }

static float sum_abs(const boat_tensor_t* t) {
    const float* p = (const float*)boat_tensor_const_data(t);
    const size_t n = boat_tensor_nelements(t);
    double s = 0.0;
    for (size_t i = 0; i < n; i++) s += fabs((double)p[i]);
    return (float)s;
}

/* ---- tensors, views, the memory seam ---- */
static void tour_tensors(void) {
    const int64_t s23[2] = {2, 3}, s6[1] = {6}, s32[2] = {3, 2};
    boat_tensor_t* a = boat_tensor_create(s23, 2, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    CHECK(a && boat_tensor_ndim(a) == 2 && boat_tensor_nelements(a) == 6 && boat_tensor_nbytes(a) == 24);
    CHECK(first_value(a) == 0.0f);                                   /* creation zero-fills */
    float* pa = (float*)boat_tensor_data(a);
    for (int i = 0; i < 6; i++) pa[i] = (float)(i + 1);
    boat_tensor_t* v = boat_tensor_reshape(a, s6, 1);                /* a view: shares the payload */
    CHECK(v && boat_tensor_nelements(v) == 6 && ((const float*)boat_tensor_const_data(v))[5] == 6.0f);
    boat_tensor_t* c = boat_tensor_clone(a);
    boat_tensor_t* like = boat_tensor_create_like(a);
    CHECK(c && like && boat_tensor_shape(like)[1] == 3);
    const float raw[6] = {1, 2, 3, 4, 5, 6};
    boat_tensor_t* f = boat_tensor_from_data(s32, 2, BOAT_DTYPE_FLOAT32, raw);
    boat_tensor_t* d = boat_tensor_to_device(a, BOAT_DEVICE_HIP);
    CHECK(f && d && boat_tensor_device(d) == BOAT_DEVICE_HIP);
    CHECK(((const float*)boat_tensor_const_data(d))[4] == 5.0f);

    boat_tensor_t* sum = boat_add(a, c);
    boat_tensor_t* prod = boat_matmul(a, f);                         /* [2,3].[3,2] */
    boat_tensor_t* tr = boat_transpose(a, 0, 1);
    boat_tensor_t* sc = boat_mul_scalar(a, 0.5);
    boat_tensor_t* total = boat_sum(a, NULL, 0, false);
    boat_tensor_t* mean = boat_mean(a, NULL, 0, false);
    boat_tensor_t* sm = boat_softmax(a, 1);
    boat_tensor_t* ge = boat_gelu(a);
    CHECK(sum && ((const float*)boat_tensor_const_data(sum))[5] == 12.0f);
    CHECK(prod && boat_tensor_shape(prod)[0] == 2 && boat_tensor_shape(prod)[1] == 2 && first_value(prod) == 22.0f);
    CHECK(tr && boat_tensor_shape(tr)[0] == 3 && ((const float*)boat_tensor_const_data(tr))[1] == 4.0f);
    CHECK(sc && first_value(sc) == 0.5f && total && first_value(total) == 21.0f && mean && first_value(mean) == 3.5f);
    CHECK(sm && fabsf(((const float*)boat_tensor_const_data(sm))[0] + ((const float*)boat_tensor_const_data(sm))[1] +
                      ((const float*)boat_tensor_const_data(sm))[2] - 1.0f) < 1e-6f);
    CHECK(ge && fabsf(first_value(ge) - 0.8413447f) < 1e-5f);
    boat_add_(a, c);
    CHECK(((const float*)boat_tensor_const_data(a))[0] == 2.0f);

    void* hostmem = boat_memory_allocate(64, BOAT_DEVICE_CPU, __FILE__, __LINE__);
    void* devmem = boat_memory_allocate_zero(64, BOAT_DEVICE_HIP, __FILE__, __LINE__);
    CHECK(hostmem && devmem);
    memset(hostmem, 7, 64);
    boat_memory_copy(devmem, hostmem, 64, BOAT_DEVICE_HIP, BOAT_DEVICE_CPU);
    memset(hostmem, 0, 64);
    boat_memory_copy(hostmem, devmem, 64, BOAT_DEVICE_CPU, BOAT_DEVICE_HIP);
    CHECK(((unsigned char*)hostmem)[63] == 7);
    boat_memory_free(devmem);
    boat_memory_free(hostmem);

    boat_tensor_t* all[] = {a, v, c, like, f, d, sum, prod, tr, sc, total, mean, sm, ge};
    for (size_t i = 0; i < sizeof(all) / sizeof(all[0]); i++) boat_tensor_unref(all[i]);
}

/* ---- the tape: every boat_var_* op once, one backward ---- */
static void tour_tape(void) {
    const int64_t s[2] = {4, 5};
    boat_tensor_t* ta = random_tensor(s, 2, 1.0f);
    boat_tensor_t* tb = random_tensor(s, 2, 1.0f);
    float* pb = (float*)boat_tensor_data(tb);
    for (int i = 0; i < 20; i++) pb[i] = 1.5f + fabsf(pb[i]);        /* a safe divisor */
    boat_variable_t* a = boat_variable_create(ta, true);
    boat_variable_t* b = boat_variable_create(tb, true);
    boat_variable_t* add = boat_var_add(a, b);
    boat_variable_t* sub = boat_var_sub(add, b);
    boat_variable_t* mul = boat_var_mul(sub, b);
    boat_variable_t* div = boat_var_div(mul, b);
    boat_variable_t* re = boat_var_relu(div);
    boat_variable_t* sg = boat_var_sigmoid(re);
    boat_variable_t* act = boat_var_tanh(sg);
    boat_variable_t* sm = boat_var_softmax(act, 1);
    boat_variable_t* lsm = boat_var_log_softmax(sm, 1);
    boat_variable_t* ge = boat_hip_var_gelu(lsm);
    boat_variable_t* fl = boat_var_flatten(ge);
    const int64_t back[2] = {5, 4};
    boat_variable_t* rs = boat_hip_var_reshape(fl, back, 2);
    boat_variable_t* mm = boat_var_matmul(rs, a);                    /* [5,4].[4,5] */
    boat_variable_t* mean = boat_var_mean(mm, NULL, 0, false);
    /* the reference's mean keeps its input's shape: the mean in element 0, zeros elsewhere (src/autodiff.c:947-985) */
    CHECK(mean && boat_tensor_nelements(boat_variable_data(mean)) == 25);
    boat_autodiff_print_graph(NULL);
    char* dot = boat_autodiff_graph_to_dot(mean);
    CHECK(dot && strstr(dot, "digraph"));
    free(dot);
    boat_variable_backward_full(mean);
    const boat_tensor_t* ga = boat_variable_grad(a);
    const boat_tensor_t* gb = boat_variable_grad(b);
    CHECK(ga && gb && boat_tensor_nelements(ga) == 20 && isfinite(sum_abs(ga)) && sum_abs(ga) > 0.0f && isfinite(sum_abs(gb)));
    CHECK(boat_var_dot(a, b) == NULL);                               /* vectors only (src/ops/linear.c:176-183) */
    const int64_t len[1] = {3};
    boat_variable_t* u = boat_variable_create_with_shape(len, 1, BOAT_DTYPE_FLOAT32, true);
    boat_variable_t* w = boat_variable_create_with_shape(len, 1, BOAT_DTYPE_FLOAT32, true);
    float* pu = (float*)boat_tensor_data(boat_variable_data(u));
    float* pw = (float*)boat_tensor_data(boat_variable_data(w));
    for (int i = 0; i < 3; i++) {
        pu[i] = (float)(i + 1);
        pw[i] = (float)(i + 4);
    }
    boat_variable_t* dotp = boat_var_dot(u, w);
    CHECK(dotp && first_value(boat_variable_data(dotp)) == 32.0f);
    boat_variable_backward(dotp, NULL);
    CHECK(boat_variable_grad(u) && first_value(boat_variable_grad(u)) == 4.0f);   /* d(u.w)/du = w */
    boat_variable_t* owned[] = {dotp, w, u, mean, mm, rs, fl, ge, lsm, sm, act, sg, re, div, mul, sub, add, b, a};
    for (size_t i = 0; i < sizeof(owned) / sizeof(owned[0]); i++) boat_variable_free(owned[i]);
    boat_autodiff_clear_computation_graph();
    boat_tensor_unref(ta);
    boat_tensor_unref(tb);
}

/* ---- layers by their hooks, a model container, losses, the three optimizers, a scheduler ---- */
static void tour_layers(void) {
    const int64_t xs[2] = {8, 16}, ys[2] = {8, 4};
    boat_tensor_t* x = random_tensor(xs, 2, 1.0f);
    boat_tensor_t* target = random_tensor(ys, 2, 1.0f);

    boat_dense_layer_t* d1 = boat_dense_layer_create(16, 32, true);
    boat_norm_layer_t* ln = boat_norm_layer_create(32, 1e-5f, true);
    boat_dense_layer_t* d2 = boat_dense_layer_create(32, 4, true);
    boat_model_t* model = boat_sequential_create();
    boat_sequential_add(model, boat_hip_layer_from_dense(d1));
    boat_sequential_add(model, boat_hip_layer_from_norm(ln));
    boat_model_add_layer(model, boat_hip_layer_gelu());
    boat_model_add_layer(model, boat_hip_layer_from_dense(d2));
    CHECK(boat_model_layer_count(model) == 4);

    boat_optimizer_t* opts[3] = {boat_adam_optimizer_create(1e-2f, 0.9f, 0.999f, 1e-8f), boat_rmsprop_optimizer_create(1e-3f, 0.99f, 1e-8f),
                                 boat_adagrad_optimizer_create(1e-2f, 1e-10f)};
    CHECK(boat_sgd_optimizer_create(0.1f, 0.0f) == NULL);            /* as the reference's stub */
    boat_scheduler_t* sched = boat_step_lr_scheduler_create(1e-2f, 2, 0.5f);
    boat_loss_t* mse = boat_mse_loss_create();
    boat_loss_t* huber = boat_huber_loss_create(1.0f);
    float first = 0.f, last = 0.f;
    for (int o = 0; o < 3; o++) {
        boat_hip_optimizer_add_dense(opts[o], d1);
        boat_hip_optimizer_add_layernorm(opts[o], ln);
        boat_hip_optimizer_add_dense(opts[o], d2);
        for (int it = 0; it < 4; it++) {
            boat_tensor_t* y = boat_model_forward(model, x);
            CHECK(y && boat_tensor_shape(y)[1] == 4);
            boat_tensor_t* grad = NULL;
            boat_tensor_t* loss = boat_hip_mse_loss(y, target, &grad);
            CHECK(loss && grad);
            const float lv = boat_loss_compute(mse, y, target);
            CHECK(fabsf(lv - first_value(loss)) <= 1e-5f * fabsf(lv) + 1e-7f && boat_loss_compute(huber, y, target) >= 0.0f);
            if (o == 0 && it == 0) first = lv;
            last = lv;
            boat_tensor_t* dx = boat_model_backward(model, grad);
            CHECK(dx && boat_tensor_shape(dx)[1] == 16);
            boat_optimizer_step(opts[o]);
            boat_optimizer_zero_grad(opts[o]);
            if (o == 0) {
                boat_scheduler_step(sched);
                boat_scheduler_update_optimizer(sched, opts[o]);
            }
            boat_tensor_unref(dx);
            boat_tensor_unref(loss);
            boat_tensor_unref(grad);
            boat_tensor_unref(y);
        }
    }
    CHECK(last < first);
    CHECK(boat_optimizer_get_learning_rate(opts[0]) < 1e-2f);                     /* the step scheduler halved it */
    boat_model_update(model, 1e-3f);                                  /* plain gradient step through the vtables */
    for (int o = 0; o < 3; o++) boat_optimizer_free(opts[o]);
    boat_scheduler_free(sched);
    boat_loss_free(mse);
    boat_loss_free(huber);
    boat_model_free(model);                                           /* frees the wrapped layers as well */
    boat_tensor_unref(x);
    boat_tensor_unref(target);
}

/* ---- attention by its hooks and on the tape, convolution / pooling / flatten on the tape ---- */
static void tour_attention_and_conv(void) {
    const int64_t qs[3] = {2, 6, 32};
    boat_tensor_t* q = random_tensor(qs, 3, 1.0f);
    boat_attention_config_t cfg;
    memset(&cfg, 0, sizeof(cfg));
    cfg.hidden_size = 32;
    cfg.num_heads = 4;
    cfg.head_size = 8;
    cfg.use_bias = true;
    boat_attention_t* att = boat_attention_create(&cfg);
    CHECK(att != NULL);
    boat_attention_set_causal(att, true);
    boat_attention_set_dropout(att, 0.0f);
    boat_tensor_t* out = boat_attention_forward(att, q, q, q, NULL);
    CHECK(out && boat_tensor_shape(out)[2] == 32);
    boat_tensor_t *gq = NULL, *gk = NULL, *gv = NULL;
    CHECK(boat_attention_backward(att, out, &gq, &gk, &gv) && gq && gk && gv);
    CHECK(boat_attention_get_grad_weight_q(att) && sum_abs(boat_attention_get_grad_weight_o(att)) > 0.0f);
    boat_attention_update(att, 1e-3f);
    boat_tensor_unref(gq);
    boat_tensor_unref(gk);
    boat_tensor_unref(gv);
    boat_tensor_unref(out);

    boat_optimizer_t* opt = boat_adam_optimizer_create(1e-3f, 0.9f, 0.999f, 1e-8f);
    boat_hip_optimizer_add_attention(opt, att);
    boat_variable_t* vq = boat_variable_create(q, true);
    boat_variable_t* va = boat_var_attention(vq, vq, vq, att, NULL);
    boat_variable_t* vs = boat_var_sum(va, NULL, 0, false);
    boat_variable_backward_full(vs);
    CHECK(boat_variable_grad(vq) && boat_tensor_nelements(boat_variable_grad(vq)) == 2 * 6 * 32);
    boat_optimizer_step(opt);
    boat_optimizer_zero_grad(opt);
    boat_variable_free(vs);
    boat_variable_free(va);
    boat_variable_free(vq);
    boat_optimizer_free(opt);
    boat_attention_free(att);
    boat_tensor_unref(q);

    boat_attention_layer_t* al = boat_attention_layer_create(32, 4, 0.0f, false);
    const int64_t xs3[3] = {2, 5, 32};
    boat_tensor_t* x3 = random_tensor(xs3, 3, 1.0f);
    boat_tensor_t* y3 = boat_attention_layer_forward(al, x3, x3, x3, NULL);
    boat_tensor_t* g3 = y3 ? boat_attention_layer_backward(al, y3) : NULL;
    CHECK(al && y3 && g3);
    boat_attention_layer_update(al, 1e-3f);
    boat_tensor_unref(g3);
    boat_tensor_unref(y3);
    boat_tensor_unref(x3);
    boat_attention_layer_free(al);

    const int64_t is[4] = {3, 2, 8, 8};
    boat_tensor_t* img = random_tensor(is, 4, 1.0f);
    boat_conv_layer_t* conv = boat_conv_layer_create(2, 4, 3, 1, 1);
    boat_pool_layer_t* pool = boat_pool_layer_create(2, 2, 0);
    boat_dense_layer_t* head = boat_dense_layer_create(4 * 4 * 4, 3, true);
    boat_optimizer_t* copt = boat_rmsprop_optimizer_create(1e-3f, 0.99f, 1e-8f);
    boat_hip_optimizer_add_conv(copt, conv);
    boat_hip_optimizer_add_dense(copt, head);
    boat_variable_t* vi = boat_variable_create(img, true);
    boat_variable_t* vc = boat_var_conv(vi, conv);
    boat_variable_t* vr = boat_var_relu(vc);
    boat_variable_t* vp = boat_var_pool(vr, pool);
    boat_variable_t* vf = boat_var_flatten(vp);
    boat_variable_t* vd = boat_var_dense(vf, head);
    boat_variable_t* vl = boat_var_sum(vd, NULL, 0, false);
    CHECK(vl != NULL);
    boat_variable_backward_full(vl);
    CHECK(boat_variable_grad(vi) && boat_tensor_nelements(boat_variable_grad(vi)) == 3 * 2 * 8 * 8);
    CHECK(sum_abs(boat_conv_layer_get_grad_weight(conv)) > 0.0f);
    boat_optimizer_step(copt);
    boat_optimizer_zero_grad(copt);
    boat_variable_t* owned[] = {vl, vd, vf, vp, vr, vc, vi};
    for (size_t i = 0; i < sizeof(owned) / sizeof(owned[0]); i++) boat_variable_free(owned[i]);
    boat_optimizer_free(copt);
    boat_dense_layer_free(head);
    boat_pool_layer_free(pool);
    boat_conv_layer_free(conv);
    boat_tensor_unref(img);

    /* the fused loss of the MNIST example */
    const int64_t ls[2] = {4, 10}, lab_s[1] = {4};
    boat_tensor_t* logits = random_tensor(ls, 2, 2.0f);
    boat_tensor_t* labels = boat_tensor_create(lab_s, 1, BOAT_DTYPE_INT32, BOAT_DEVICE_CPU);
    for (int i = 0; i < 4; i++) ((int32_t*)boat_tensor_data(labels))[i] = (i * 3) % 10;
    boat_tensor_t* dlogits = NULL;
    boat_tensor_t* ce = boat_hip_softmax_cross_entropy(logits, labels, &dlogits);
    CHECK(ce && dlogits && first_value(ce) > 0.0f && boat_tensor_nelements(dlogits) == 40);
    boat_loss_t* cel = boat_cross_entropy_loss_create();
    boat_tensor_t* probs = boat_softmax(logits, 1);
    boat_tensor_t* onehot = boat_tensor_create(ls, 2, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    for (int i = 0; i < 4; i++) ((float*)boat_tensor_data(onehot))[i * 10 + (i * 3) % 10] = 1.0f;
    CHECK(boat_loss_compute(cel, probs, onehot) > 0.0f);
    boat_loss_free(cel);
    boat_tensor_unref(onehot);
    boat_tensor_unref(probs);
    boat_tensor_unref(dlogits);
    boat_tensor_unref(ce);
    boat_tensor_unref(labels);
    boat_tensor_unref(logits);
}

/* ---- RMSNorm, the stateless norms, the public attention core, arithmetic on other element types, the opt-in paths ---- */
static void tour_norms_attention_core_and_types(void) {
    const int64_t xs[2] = {6, 32}, ns[1] = {32};
    boat_tensor_t* x = random_tensor(xs, 2, 1.0f);
    boat_rmsnorm_config_t rc;
    memset(&rc, 0, sizeof(rc));
    rc.normalized_shape = 32;
    rc.eps = 1e-6f;
    rc.elementwise_affine = true;
    boat_rmsnorm_t* rms = boat_rmsnorm_create(&rc);
    boat_tensor_t* y = boat_rmsnorm_forward(rms, x);
    boat_tensor_t* gx = y ? boat_rmsnorm_backward(rms, y) : NULL;
    CHECK(rms && y && gx && boat_tensor_nelements(gx) == 6 * 32);
    CHECK(boat_hip_rmsnorm_get_grad_weight(rms) && sum_abs(boat_hip_rmsnorm_get_grad_weight(rms)) > 0.0f);
    boat_rmsnorm_update(rms, 1e-3f);
    boat_tensor_t* ln = boat_layer_norm(x, ns, 1, 1e-5f);
    boat_tensor_t* rn = boat_rms_norm(x, ns, 1, 1e-6f);
    boat_tensor_t* rg = rn ? boat_rms_norm_grad(rn, x, rn, ns, 1, 1e-6f) : NULL;
    CHECK(ln && rn && rg);
    boat_tensor_t* owned[] = {rg, rn, ln, gx, y, x};
    for (size_t i = 0; i < sizeof(owned) / sizeof(owned[0]); i++) boat_tensor_unref(owned[i]);
    boat_rmsnorm_free(rms);

    /* attention core on [batch, heads, seq, head_size]; self-attention through a throw-away layer */
    const int64_t qs[4] = {2, 3, 10, 16};
    boat_tensor_t* q = random_tensor(qs, 4, 1.0f);
    boat_tensor_t* core = boat_scaled_dot_product_attention(q, q, q, 0.25f, NULL, true, 0.0f);
    CHECK(core && boat_tensor_nelements(core) == 2 * 3 * 10 * 16);
    const int64_t hs[3] = {2, 10, 48};
    boat_tensor_t* h = random_tensor(hs, 3, 1.0f);
    boat_tensor_t* mh = boat_multihead_attention(h, 3, 0.0f, false, NULL);
    CHECK(mh && boat_tensor_shape(mh)[2] == 48);
    boat_tensor_unref(mh);
    boat_tensor_unref(h);
    boat_tensor_unref(core);
    boat_tensor_unref(q);

    /* an attention layer whose forward pass keeps the scores for its backward pass (head size 64, 128 keys), then the
     * same with the cache switched off */
    for (int pass = 0; pass < 2; pass++) {
        boat_hip_set_attention_score_cache_limit(pass == 0 ? (size_t)1 << 30 : 0);
        boat_attention_config_t cfg;
        memset(&cfg, 0, sizeof(cfg));
        cfg.hidden_size = 128;
        cfg.num_heads = 2;
        cfg.head_size = 64;
        cfg.use_bias = true;
        boat_attention_t* att = boat_attention_create(&cfg);
        const int64_t as[3] = {1, 128, 128};
        boat_tensor_t* ax = random_tensor(as, 3, 1.0f);
        boat_tensor_t* ay = boat_attention_forward(att, ax, ax, ax, NULL);
        boat_tensor_t *gq = NULL, *gk = NULL, *gv = NULL;
        CHECK(att && ay && boat_attention_backward(att, ay, &gq, &gk, &gv) && gq && gk && gv && sum_abs(gq) > 0.0f);
        boat_tensor_t* at[] = {gq, gk, gv, ay, ax};
        for (size_t i = 0; i < sizeof(at) / sizeof(at[0]); i++) boat_tensor_unref(at[i]);
        boat_attention_free(att);
    }
    boat_hip_set_attention_score_cache_limit((size_t)1 << 30);

    /* elementwise arithmetic on float64 and integers, with broadcasting */
    const int64_t ds[2] = {3, 4}, bs[2] = {1, 4};
    boat_tensor_t* a64 = boat_tensor_create(ds, 2, BOAT_DTYPE_FLOAT64, BOAT_DEVICE_CPU);
    boat_tensor_t* b64 = boat_tensor_create(bs, 2, BOAT_DTYPE_FLOAT64, BOAT_DEVICE_CPU);
    for (int i = 0; i < 12; i++) ((double*)boat_tensor_data(a64))[i] = 1.0 + i;
    for (int i = 0; i < 4; i++) ((double*)boat_tensor_data(b64))[i] = 2.0 + i;
    boat_tensor_t* s64 = boat_add(a64, b64);
    boat_tensor_t* m64 = boat_mod(a64, b64);
    boat_tensor_t* p64 = boat_pow_scalar(a64, 2.0);
    CHECK(s64 && ((const double*)boat_tensor_const_data(s64))[5] == 6.0 + 3.0);
    CHECK(m64 && ((const double*)boat_tensor_const_data(m64))[5] == fmod(6.0, 3.0));
    CHECK(p64 && ((const double*)boat_tensor_const_data(p64))[3] == 16.0);
    boat_tensor_t* i32 = boat_tensor_create(ds, 2, BOAT_DTYPE_INT32, BOAT_DEVICE_CPU);
    for (int i = 0; i < 12; i++) ((int32_t*)boat_tensor_data(i32))[i] = 10 * i;
    boat_tensor_t* d32 = boat_div_scalar(i32, 3.0);
    boat_mul_scalar_(i32, 2.0);
    CHECK(d32 && ((const int32_t*)boat_tensor_const_data(d32))[4] == 13 && ((const int32_t*)boat_tensor_const_data(i32))[4] == 80);
    boat_tensor_t* tt[] = {d32, i32, p64, m64, s64, b64, a64};
    for (size_t i = 0; i < sizeof(tt) / sizeof(tt[0]); i++) boat_tensor_unref(tt[i]);

    /* a 3x3 convolution with enough input channels for the matrix-core forward, switched on and off again */
    const int64_t is[4] = {2, 8, 6, 6};
    boat_tensor_t* img = random_tensor(is, 4, 1.0f);
    boat_conv_layer_t* conv = boat_conv_layer_create(8, 5, 3, 1, 1);
    boat_tensor_t* direct = boat_conv_layer_forward(conv, img);
    boat_hip_conv_forward_matrix_cores(1);
    boat_tensor_t* mfma = boat_conv_layer_forward(conv, img);
    boat_hip_conv_forward_matrix_cores(0);
    CHECK(direct && mfma && fabsf(sum_abs(direct) - sum_abs(mfma)) <= 1e-3f * sum_abs(direct));
    boat_tensor_unref(mfma);
    boat_tensor_unref(direct);
    boat_conv_layer_free(conv);
    boat_tensor_unref(img);

    /* reference-exact mode: the fan-out of a non-leaf counts once per consumer, as in the reference */
    const int64_t one[1] = {1};
    for (int mode = 0; mode < 2; mode++) {
        boat_hip_set_reference_exact(mode);
        boat_tensor_t* ta = random_tensor(one, 1, 1.0f);
        boat_tensor_t* tb = random_tensor(one, 1, 1.0f);
        boat_variable_t* va = boat_variable_create(ta, true);
        boat_variable_t* vb = boat_variable_create(tb, true);
        boat_variable_t* vy = boat_var_mul(va, vb);
        boat_variable_t* vz = boat_var_add(vy, vy);
        boat_variable_backward_full(vz);
        const float want = (mode ? 4.0f : 2.0f) * first_value(tb);
        CHECK(boat_variable_grad(va) && fabsf(first_value(boat_variable_grad(va)) - want) <= 1e-6f * fabsf(want));
        boat_variable_free(vz);
        boat_variable_free(vy);
        boat_variable_free(vb);
        boat_variable_free(va);
        boat_tensor_unref(tb);
        boat_tensor_unref(ta);
    }
    boat_hip_set_reference_exact(0);
}

int main(void) {
    boat_init();
    if (boat_has_error()) {
        fprintf(stderr, "api_tour: %s\n", boat_get_last_error_message());
        return 1;
    }
    tour_tensors();
    tour_tape();
    tour_layers();
    tour_attention_and_conv();
    tour_norms_attention_core_and_types();
    boat_hip_synchronize();
    CHECK(!boat_has_error());
    const boat_memory_stats_t st = boat_memory_get_stats();
    printf("{\"failed_check_line\": %d, \"host_blocks_allocated\": %zu, \"host_blocks_freed\": %zu}\n", g_failed,
           st.allocated_blocks, st.freed_blocks);
    boat_memory_print_stats(stdout);                                  /* "device in use 0 B": nothing leaked in HBM either */
    boat_cleanup();
    return g_failed ? 2 : 0;
}
