/* mlp_train_step.c - the training step of Boat's MNIST example, written against Boat's C API only.
 *
 *   MLP 784 -> 128 (ReLU) -> 10, batch 64: dense, relu, dense, log_softmax, mul(onehot), sum, mul(-1/B) on the tape,
 *   boat_variable_backward_full, boat_optimizer_step (Adam), boat_optimizer_zero_grad
 *   (the step of examples/mnist/mnist_autodiff.c:2437-2488 with the loss chain of :397-522).
 *
 * Every symbol used here exists with the same signature in the reference's headers, except the two marked
 * "boat_hip_": registering layer-owned gradients with the optimizer and the final device synchronisation.  Linking
 * this file against libboat_amd.so instead of libboat is the whole switch to the GPU path:
 *
 *   gcc mlp_train_step.c -I<repo>/include -L<repo>/boat_amd/lib -lboat_amd -Wl,-rpath,<repo>/boat_amd/lib -lm
 *
 * usage: mlp_train_step [steps] [warmup] [fused]   -> one JSON line: wall ms per step, first and last loss
 *
 * With a third argument "fused" the four-op loss chain and its backward are replaced by one call of
 * boat_hip_softmax_cross_entropy (loss and d(loss)/d(logits) from one kernel), and backward starts at the logits.
 *
 * The program writes through boat_tensor_data() pointers during set-up only and never keeps one across a call; run it
 * with BOAT_HIP_COHERENT_POINTERS=0 to let the tensors it touched stay resident on the device.
 */
#include <stdio.h>
#include <stdlib.h>
#include <time.h>

#include "boat_api.h"

enum { B = 64, D_IN = 784, D_H = 128, D_OUT = 10 };

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static float uniform01(void) {           /* splitmix64 -> [0, 1) */
    uint64_t z = (rng_state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (float)(z >> 40) / 16777216.0f;
}

static double now_ms(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return ts.tv_sec * 1e3 + ts.tv_nsec * 1e-6;
}

int main(int argc, char** argv) {
    const int steps = argc > 1 ? atoi(argv[1]) : 200;
    const int warmup = argc > 2 ? atoi(argv[2]) : 20;
    const int fused = argc > 3 && argv[3][0] == 'f';

    boat_dense_layer_t* l1 = boat_dense_layer_create(D_IN, D_H, true);
    boat_dense_layer_t* l2 = boat_dense_layer_create(D_H, D_OUT, true);
    if (!l1 || !l2) return 1;
    /* Xavier-uniform weights written in place through the data pointer, zero biases */
    boat_dense_layer_t* layers[2] = {l1, l2};
    const int fan[2][2] = {{D_IN, D_H}, {D_H, D_OUT}};
    for (int l = 0; l < 2; l++) {
        float* w = (float*)boat_tensor_data(boat_dense_layer_get_weight(layers[l]));
        const float lim = 2.449489743f / __builtin_sqrtf((float)(fan[l][0] + fan[l][1]));
        for (int i = 0; i < fan[l][0] * fan[l][1]; i++) w[i] = (2.0f * uniform01() - 1.0f) * lim;
    }

    const int64_t xs[2] = {B, D_IN}, ys[2] = {B, D_OUT}, one[1] = {1};
    boat_tensor_t* x = boat_tensor_create(xs, 2, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    boat_tensor_t* onehot = boat_tensor_create(ys, 2, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    boat_tensor_t* factor = boat_tensor_create(one, 1, BOAT_DTYPE_FLOAT32, BOAT_DEVICE_CPU);
    float* px = (float*)boat_tensor_data(x);
    for (int i = 0; i < B * D_IN; i++) px[i] = uniform01();
    const int64_t ls_shape[1] = {B};
    boat_tensor_t* labels = boat_tensor_create(ls_shape, 1, BOAT_DTYPE_INT32, BOAT_DEVICE_CPU);
    float* poh = (float*)boat_tensor_data(onehot);
    int32_t* plab = (int32_t*)boat_tensor_data(labels);
    for (int b = 0; b < B; b++) {
        plab[b] = (int)(uniform01() * D_OUT) % D_OUT;
        poh[b * D_OUT + plab[b]] = 1.0f;
    }
    ((float*)boat_tensor_data(factor))[0] = -1.0f / B;

    boat_optimizer_t* opt = boat_adam_optimizer_create(1e-3f, 0.9f, 0.999f, 1e-8f);
    boat_hip_optimizer_add_dense(opt, l1);     /* = boat_optimizer_add_parameter for weight and bias of the layer */
    boat_hip_optimizer_add_dense(opt, l2);

    float first = 0.f, last = 0.f;
    double t0 = 0.0;
    for (int it = 0; it < warmup + steps; it++) {
        if (it == warmup) {
            boat_hip_synchronize();
            t0 = now_ms();
        }
        if (fused) {
            boat_variable_t* vx = boat_variable_create(x, true);
            boat_variable_t* h = boat_var_dense(vx, l1);
            boat_variable_t* r = boat_var_relu(h);
            boat_variable_t* z = boat_var_dense(r, l2);
            boat_tensor_t* dz = NULL;
            boat_tensor_t* tl = z ? boat_hip_softmax_cross_entropy(boat_variable_data(z), labels, &dz) : NULL;
            if (!tl || !dz) return 2;
            boat_variable_backward(z, dz);
            boat_optimizer_step(opt);
            boat_optimizer_zero_grad(opt);
            if (it == 0 || it == warmup + steps - 1) {
                const float v = ((const float*)boat_tensor_const_data(tl))[0];
                if (it == 0) first = v;
                else last = v;
            }
            boat_tensor_unref(tl);
            boat_tensor_unref(dz);
            boat_variable_t* vars[] = {z, r, h, vx};
            for (size_t i = 0; i < sizeof(vars) / sizeof(vars[0]); i++) boat_variable_free(vars[i]);
            continue;
        }
        boat_variable_t* vx = boat_variable_create(x, true);
        boat_variable_t* voh = boat_variable_create(onehot, false);
        boat_variable_t* vf = boat_variable_create(factor, false);
        boat_variable_t* h = boat_var_dense(vx, l1);
        boat_variable_t* r = boat_var_relu(h);
        boat_variable_t* z = boat_var_dense(r, l2);
        boat_variable_t* ls = boat_var_log_softmax(z, 1);
        boat_variable_t* m = boat_var_mul(voh, ls);
        boat_variable_t* s = boat_var_sum(m, NULL, 0, false);
        boat_variable_t* loss = boat_var_mul(vf, s);
        if (!loss) return 2;
        boat_variable_backward_full(loss);
        boat_optimizer_step(opt);
        boat_optimizer_zero_grad(opt);
        if (it == 0 || it == warmup + steps - 1) {
            const float v = ((const float*)boat_tensor_const_data(boat_variable_data(loss)))[0];
            if (it == 0) first = v;
            else last = v;
        }
        boat_variable_t* vars[] = {loss, s, m, ls, z, r, h, vf, voh, vx};
        for (size_t i = 0; i < sizeof(vars) / sizeof(vars[0]); i++) boat_variable_free(vars[i]);
    }
    boat_hip_synchronize();
    const double ms = (now_ms() - t0) / steps;
    printf("{\"ms_per_step\": %.5f, \"steps\": %d, \"warmup\": %d, \"fused_loss\": %d, \"loss_first\": %.6f, \"loss_last\": %.6f}\n",
           ms, steps, warmup, fused, first, last);
    boat_optimizer_free(opt);
    boat_tensor_unref(x);
    boat_tensor_unref(onehot);
    boat_tensor_unref(labels);
    boat_tensor_unref(factor);
    boat_dense_layer_free(l1);
    boat_dense_layer_free(l2);
    return last < first ? 0 : 3;
}
