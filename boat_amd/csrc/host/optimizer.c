/* optimizer.c - Adam, RMSprop and Adagrad behind boat_optimizer_* with one fused multi-tensor launch per step.
 *
 * Same state machines as src/optimizers/adam.c:15-308, rmsprop.c:15-300, adagrad.c:15-290 and the type
 * dispatch of src/optimizers/optimizer_common.c:108-235: the state's first field is the optimizer type;
 * parameters are registered as borrowed (param, grad) tensor pairs that must outlive the
 * optimizer; m and v are created zero at registration; `step` updates every registered tensor
 * with the bias correction of the CURRENT timestep and increments it once afterwards; `step`
 * never zeroes gradients; creation rejects lr <= 0 and betas outside (0,1).
 */
#include "boat_internal.h"

#include <stdlib.h>
#include <string.h>

typedef struct {
    boat_optimizer_type_t type;   /* must stay first: the dispatcher reads it (optimizer_common.c:108-114) */
    float learning_rate, beta1, beta2, epsilon;   /* beta1 doubles as RMSprop's alpha */
    int64_t timestep;
    boat_tensor_t** params;
    boat_tensor_t** grads;
    boat_tensor_t** m;
    boat_tensor_t** v;
    size_t num_params, capacity;
    /* launch tables, rebuilt every step (device pointers can move when a host write invalidates a copy) */
    float** tp;
    const float** tg;
    float** tm;
    float** tv;
    int64_t* tn;
} adam_state_t;

boat_optimizer_t* boat_adam_optimizer_create(float learning_rate, float beta1, float beta2, float epsilon) {
    if (learning_rate <= 0.0f) return NULL;
    if (beta1 <= 0.0f || beta1 >= 1.0f) return NULL;
    if (beta2 <= 0.0f || beta2 >= 1.0f) return NULL;
    adam_state_t* s = (adam_state_t*)calloc(1, sizeof(*s));
    if (!s) return NULL;
    s->type = BOAT_OPTIMIZER_ADAM;
    s->learning_rate = learning_rate;
    s->beta1 = beta1;
    s->beta2 = beta2;
    s->epsilon = epsilon;
    return (boat_optimizer_t*)s;
}

/* rmsprop.c:33-57: lr > 0, alpha in (0,1), eps > 0 */
boat_optimizer_t* boat_rmsprop_optimizer_create(float learning_rate, float alpha, float epsilon) {
    if (learning_rate <= 0.0f || alpha <= 0.0f || alpha >= 1.0f || epsilon <= 0.0f) return NULL;
    adam_state_t* s = (adam_state_t*)calloc(1, sizeof(*s));
    if (!s) return NULL;
    s->type = BOAT_OPTIMIZER_RMSPROP;
    s->learning_rate = learning_rate;
    s->beta1 = alpha;
    s->epsilon = epsilon;
    return (boat_optimizer_t*)s;
}

/* adagrad.c:41-50: lr > 0, eps > 0 */
boat_optimizer_t* boat_adagrad_optimizer_create(float learning_rate, float epsilon) {
    if (learning_rate <= 0.0f || epsilon <= 0.0f) return NULL;
    adam_state_t* s = (adam_state_t*)calloc(1, sizeof(*s));
    if (!s) return NULL;
    s->type = BOAT_OPTIMIZER_ADAGRAD;
    s->learning_rate = learning_rate;
    s->epsilon = epsilon;
    return (boat_optimizer_t*)s;
}

/* declared by the reference and defined as a stub that returns NULL (optimizer_common.c:62-67) */
boat_optimizer_t* boat_sgd_optimizer_create(float learning_rate, float momentum) {
    (void)learning_rate;
    (void)momentum;
    return NULL;
}

static bool known_type(const adam_state_t* s) {
    return s->type == BOAT_OPTIMIZER_ADAM || s->type == BOAT_OPTIMIZER_RMSPROP || s->type == BOAT_OPTIMIZER_ADAGRAD;
}

static bool adam_grow(adam_state_t* s) {
    const size_t cap = s->capacity ? s->capacity * 2 : 16;
#define GROW(field, type)                                              \
    do {                                                               \
        type* p = (type*)realloc(s->field, cap * sizeof(type));        \
        if (!p) return false;                                          \
        s->field = p;                                                  \
    } while (0)
    GROW(params, boat_tensor_t*);
    GROW(grads, boat_tensor_t*);
    GROW(m, boat_tensor_t*);
    GROW(v, boat_tensor_t*);
    GROW(tp, float*);
    GROW(tg, const float*);
    GROW(tm, float*);
    GROW(tv, float*);
    GROW(tn, int64_t);
#undef GROW
    s->capacity = cap;
    return true;
}

void boat_optimizer_add_parameter(boat_optimizer_t* optimizer, boat_tensor_t* param, boat_tensor_t* grad) {
    if (!optimizer) return;
    adam_state_t* s = (adam_state_t*)optimizer;
    if (!known_type(s)) return;
    if (!param || !grad) return;   /* silently ignored, as adam.c:99-101 */
    if (!bt_is_f32(param) || !bt_is_f32(grad) || param->nelements != grad->nelements) {
        boat_fail(BOAT_ERROR_INVALID_ARGUMENT, "boat_optimizer_add_parameter: param and grad must be float32 tensors of equal size");
        return;
    }
    if (s->num_params >= s->capacity && !adam_grow(s)) return;
    const size_t i = s->num_params;
    s->params[i] = param;
    s->grads[i] = grad;
    s->m[i] = boat_tensor_create(param->shape, param->ndim, param->dtype, param->device);   /* zero moments */
    /* Adam's second moment; RMSprop and Adagrad keep one state tensor (square_avg / sum_square_grad) in m */
    s->v[i] = s->type == BOAT_OPTIMIZER_ADAM ? boat_tensor_create(param->shape, param->ndim, param->dtype, param->device) : NULL;
    s->num_params++;
}

static void adam_step(adam_state_t* s) {
    const bool two = s->type == BOAT_OPTIMIZER_ADAM;
    int count = 0;
    for (size_t i = 0; i < s->num_params; i++) {
        if (!s->params[i] || !s->grads[i] || !s->m[i] || (two && !s->v[i])) continue;
        if (s->params[i]->nelements == 0) continue;
        const float* g = bt_dev_read(s->grads[i]);
        float* p = bt_dev_rw(s->params[i]);
        float* m = bt_dev_rw(s->m[i]);
        float* v = two ? bt_dev_rw(s->v[i]) : NULL;
        if (!g || !p || !m || (two && !v)) return;
        s->tp[count] = p;
        s->tg[count] = g;
        s->tm[count] = m;
        s->tv[count] = v;
        s->tn[count] = (int64_t)s->params[i]->nelements;
        count++;
    }
    if (s->type == BOAT_OPTIMIZER_RMSPROP) {
        boat_hip_ok(bh_rmsprop_update_multi(s->tp, s->tg, s->tm, s->tn, count, s->learning_rate, s->beta1, s->epsilon),
                    "boat_optimizer_step");
        return;
    }
    if (s->type == BOAT_OPTIMIZER_ADAGRAD) {
        boat_hip_ok(bh_adagrad_update_multi(s->tp, s->tg, s->tm, s->tn, count, s->learning_rate, s->epsilon), "boat_optimizer_step");
        return;
    }
    boat_hip_ok(bh_adam_update_multi(s->tp, s->tg, s->tm, s->tv, s->tn, count, s->learning_rate, s->beta1, s->beta2,
                                     s->epsilon, s->timestep),
                "boat_optimizer_step");
    s->timestep++;   /* once per step, after all tensors (adam.c:239) */
}

void boat_optimizer_step(boat_optimizer_t* optimizer) {
    if (!optimizer) return;
    adam_state_t* s = (adam_state_t*)optimizer;
    if (known_type(s)) adam_step(s);
    bt_flush_exposed();
}

void boat_optimizer_zero_grad(boat_optimizer_t* optimizer) {
    if (!optimizer) return;
    adam_state_t* s = (adam_state_t*)optimizer;
    if (!known_type(s)) return;
    /* A gradient nobody holds a pointer to becomes zero by losing its contents (the next backward writes it instead of
     * adding to it, a reader in between gets zeros filled in); the others are cleared by one launch over all of them
     * (the table arrays are sized for num_params) */
    int count = 0;
    for (size_t i = 0; i < s->num_params; i++) {
        boat_tensor_t* g = s->grads[i];
        if (!g || g->nelements == 0 || !bt_is_f32(g)) continue;
        if (bt_set_zero(g)) continue;
        float* p = bt_dev_write(g);
        if (!p) continue;
        s->tp[count] = p;
        s->tn[count] = (int64_t)g->nelements;
        count++;
    }
    if (count) boat_hip_ok(bh_zero_multi(s->tp, s->tn, count), "boat_optimizer_zero_grad");
    bt_flush_exposed();
}

void boat_optimizer_free(boat_optimizer_t* optimizer) {
    if (!optimizer) return;
    adam_state_t* s = (adam_state_t*)optimizer;
    for (size_t i = 0; i < s->num_params; i++) {
        boat_tensor_unref(s->m[i]);
        boat_tensor_unref(s->v[i]);
    }
    free(s->params);
    free(s->grads);
    free(s->m);
    free(s->v);
    free(s->tp);
    free(s->tg);
    free(s->tm);
    free(s->tv);
    free(s->tn);
    free(s);
}

float boat_optimizer_get_learning_rate(const boat_optimizer_t* optimizer) {
    return optimizer ? ((const adam_state_t*)optimizer)->learning_rate : 0.0f;
}
void boat_optimizer_set_learning_rate(boat_optimizer_t* optimizer, float learning_rate) {
    if (optimizer) ((adam_state_t*)optimizer)->learning_rate = learning_rate;
}

/* ---- registration helpers (no counterpart in the reference) ---- */

void boat_hip_optimizer_add_dense(boat_optimizer_t* opt, boat_dense_layer_t* layer) {
    if (!opt || !layer) return;
    boat_optimizer_add_parameter(opt, layer->weight, layer->grad_weight);
    if (layer->use_bias) boat_optimizer_add_parameter(opt, layer->bias, layer->grad_bias);
}

void boat_hip_optimizer_add_conv(boat_optimizer_t* opt, boat_conv_layer_t* layer) {
    if (!opt || !layer) return;
    boat_optimizer_add_parameter(opt, boat_conv_layer_get_weight(layer), boat_conv_layer_get_grad_weight(layer));
    boat_optimizer_add_parameter(opt, boat_conv_layer_get_bias(layer), boat_conv_layer_get_grad_bias(layer));
}

void boat_hip_optimizer_add_layernorm(boat_optimizer_t* opt, boat_layernorm_t* norm) {
    if (!opt || !norm) return;
    if (norm->weight) boat_optimizer_add_parameter(opt, norm->weight, norm->grad_weight);
    if (norm->bias) boat_optimizer_add_parameter(opt, norm->bias, norm->grad_bias);
}

/* The reference creates attention gradients inside the first backward (attention.c:181-188), too
 * late to register them; here they are created zero-filled on registration and every backward
 * overwrites their contents in place, so the registered pointers stay valid. */
void boat_hip_optimizer_add_attention(boat_optimizer_t* opt, boat_attention_t* a) {
    if (!opt || !a) return;
    boat_tensor_t** w[] = {&a->weight_q, &a->weight_k, &a->weight_v, &a->weight_o, &a->bias_q, &a->bias_k, &a->bias_v, &a->bias_o};
    boat_tensor_t** g[] = {&a->grad_weight_q, &a->grad_weight_k, &a->grad_weight_v, &a->grad_weight_o,
                           &a->grad_bias_q, &a->grad_bias_k, &a->grad_bias_v, &a->grad_bias_o};
    for (int i = 0; i < 8; i++) {
        if (!*w[i]) continue;
        if (!*g[i]) *g[i] = boat_tensor_create_like(*w[i]);
        boat_optimizer_add_parameter(opt, *w[i], *g[i]);
    }
}
