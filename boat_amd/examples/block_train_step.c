/* block_train_step.c - one training step of a pre-LN transformer encoder block, written against Boat's C API.
 *
 *   x1 = x + attention(LN1(x));  y = x1 + dense2(gelu(dense1(LN2(x1))));  loss = mean((y - target)^2)
 *   d_model 1024, 16 heads, FFN 4096, sequence 512, batch 16 (the sizes are arguments): forward on the tape,
 *   boat_variable_backward from d(loss)/dy, boat_optimizer_step (Adam over the block's 16 parameter tensors),
 *   boat_optimizer_zero_grad.
 *
 * The layers, the tape operations, the optimizer and the tensors are Boat's (src/layers/attention.c:247-466, norm.c:231-317,
 * dense.c:135-188, src/autodiff.c, src/optimizers/adam.c); the symbols marked boat_hip_ have no counterpart in the
 * reference: tape operations for LayerNorm, GELU and reshape (the reference's LayerNorm backward and GELU are stubs,
 * norm.c:397-402, activation.c:298-302), the MSE loss with its gradient in one pass, registering layer-owned gradients
 * with the optimizer, and the device synchronisation around the timed region.
 *
 *   gcc block_train_step.c -I<repo>/include -L<repo>/boat_amd/lib -lboat_amd -Wl,-rpath,<repo>/boat_amd/lib -lm
 *
 * usage: block_train_step [steps] [warmup] [batch] [seq] [d_model] [heads] [ffn]  -> one JSON line: wall ms per step,
 * first and last loss.  The program keeps no data pointer across a call; run it with BOAT_HIP_COHERENT_POINTERS=0 to let
 * the tensors it wrote during set-up stay resident on the device.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <time.h>

#include "boat_api.h"

static uint64_t rng_state = 0x243F6A8885A308D3ull;
static float uniform01(void) {           /* splitmix64 -> [0, 1) */
    uint64_t z = (rng_state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (float)(z >> 40) / 16777216.0f;
}
static float normal01(void) {            /* Box-Muller */
    const float u = uniform01() + 5.9604645e-8f, v = uniform01();
    return sqrtf(-2.0f * logf(u)) * cosf(6.28318530718f * v);
}
static void fill_normal(boat_tensor_t* t, float std) {
    float* p = (float*)boat_tensor_data(t);
    const size_t n = boat_tensor_nelements(t);
    for (size_t i = 0; i < n; i++) p[i] = std * normal01();
}
static double now_ms(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return ts.tv_sec * 1e3 + ts.tv_nsec * 1e-6;
}

int main(int argc, char** argv) {
    const int steps = argc > 1 ? atoi(argv[1]) : 20;
    const int warmup = argc > 2 ? atoi(argv[2]) : 5;
    const int64_t B = argc > 3 ? atoll(argv[3]) : 16, S = argc > 4 ? atoll(argv[4]) : 512, H = argc > 5 ? atoll(argv[5]) : 1024;
    const int64_t heads = argc > 6 ? atoll(argv[6]) : 16, ffn = argc > 7 ? atoll(argv[7]) : 4096;
    if (steps < 1 || warmup < 0 || B < 1 || S < 1 || H < 1 || heads < 1 || H % heads || ffn < 1) return 1;

    boat_layernorm_config_t ln_cfg = {(size_t)H, 1e-5f, true, true};
    boat_layernorm_t* ln1 = boat_layernorm_create(&ln_cfg);      /* gamma = 1, beta = 0 */
    boat_layernorm_t* ln2 = boat_layernorm_create(&ln_cfg);
    boat_attention_config_t att_cfg = {(size_t)H, (size_t)heads, (size_t)(H / heads), 0.0f, false, true, false, 10000.0f};
    boat_attention_t* att = boat_attention_create(&att_cfg);
    boat_dense_layer_t* d1 = boat_dense_layer_create((size_t)H, (size_t)ffn, true);
    boat_dense_layer_t* d2 = boat_dense_layer_create((size_t)ffn, (size_t)H, true);
    if (!ln1 || !ln2 || !att || !d1 || !d2) return 2;
    fill_normal(boat_attention_get_weight_q(att), 0.02f);
    fill_normal(boat_attention_get_weight_k(att), 0.02f);
    fill_normal(boat_attention_get_weight_v(att), 0.02f);
    fill_normal(boat_attention_get_weight_o(att), 0.02f);
    fill_normal(boat_dense_layer_get_weight(d1), 0.02f);
    fill_normal(boat_dense_layer_get_weight(d2), 0.02f);

    boat_optimizer_t* opt = boat_adam_optimizer_create(1e-3f, 0.9f, 0.999f, 1e-8f);
    boat_hip_optimizer_add_layernorm(opt, ln1);
    boat_hip_optimizer_add_attention(opt, att);
    boat_hip_optimizer_add_layernorm(opt, ln2);
    boat_hip_optimizer_add_dense(opt, d1);
    boat_hip_optimizer_add_dense(opt, d2);

    const int64_t shape3[3] = {B, S, H}, shape2[2] = {B * S, H};
    boat_tensor_t* x = boat_tensor_create(shape3, 3, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    boat_tensor_t* target = boat_tensor_create(shape3, 3, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    if (!opt || !x || !target) return 2;
    fill_normal(x, 1.0f);
    fill_normal(target, 1.0f);

    float first = 0.f, last = 0.f;
    double t0 = 0.0;
    for (int it = 0; it < warmup + steps; it++) {
        if (it == warmup) {
            boat_hip_synchronize();
            t0 = now_ms();
        }
        boat_variable_t* vx = boat_variable_create(x, true);
        boat_variable_t* h1 = boat_hip_var_layernorm(vx, ln1);
        boat_variable_t* a = boat_var_attention(h1, h1, h1, att, NULL);
        boat_variable_t* x1 = boat_var_add(vx, a);
        boat_variable_t* h2 = boat_hip_var_layernorm(x1, ln2);
        boat_variable_t* h2f = boat_hip_var_reshape(h2, shape2, 2);
        boat_variable_t* f1 = boat_var_dense(h2f, d1);
        boat_variable_t* g1 = boat_hip_var_gelu(f1);
        boat_variable_t* f2 = boat_var_dense(g1, d2);
        boat_variable_t* f2r = boat_hip_var_reshape(f2, shape3, 3);
        boat_variable_t* y = boat_var_add(x1, f2r);
        if (!y) return 3;
        boat_tensor_t* grad = NULL;
        boat_tensor_t* loss = boat_hip_mse_loss(boat_variable_data(y), target, &grad);
        if (!loss || !grad) return 3;
        boat_variable_backward(y, grad);
        boat_optimizer_step(opt);
        boat_optimizer_zero_grad(opt);
        if (it == 0 || it == warmup + steps - 1) {
            const float v = ((const float*)boat_tensor_const_data(loss))[0];
            if (it == 0) first = v;
            else last = v;
        }
        boat_tensor_unref(loss);
        boat_tensor_unref(grad);
        boat_variable_t* vars[] = {y, f2r, f2, g1, f1, h2f, h2, x1, a, h1, vx};
        for (size_t i = 0; i < sizeof(vars) / sizeof(vars[0]); i++) boat_variable_free(vars[i]);
    }
    boat_hip_synchronize();
    const double ms = (now_ms() - t0) / steps;
    printf("{\"ms_per_step\": %.4f, \"steps\": %d, \"warmup\": %d, \"batch\": %lld, \"seq\": %lld, \"d_model\": %lld, \"heads\": %lld, "
           "\"ffn\": %lld, \"loss_first\": %.6f, \"loss_last\": %.6f}\n",
           ms, steps, warmup, (long long)B, (long long)S, (long long)H, (long long)heads, (long long)ffn, first, last);
    boat_optimizer_free(opt);
    boat_tensor_unref(x);
    boat_tensor_unref(target);
    boat_dense_layer_free(d1);
    boat_dense_layer_free(d2);
    boat_attention_free(att);
    boat_layernorm_free(ln1);
    boat_layernorm_free(ln2);
    return 0;
}
