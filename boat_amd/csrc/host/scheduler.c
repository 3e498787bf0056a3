/* scheduler.c - learning-rate schedulers and the hook that hands their rate to an optimizer.
 *
 * Host arithmetic only (one float per training step); behaviour follows the reference:
 *   step decay        lr = base * powf(gamma, (step-1) / step_size)             src/schedulers/step_lr.c:17-84
 *   cosine annealing  lr = eta_min + 0.5*(base-eta_min)*(1 + cosf(pi*min(step,T)/T))   src/schedulers/cosine_annealing.c:17-99
 *   caller's function lr = max(fn(step, base), 0)                                 src/schedulers/lambda_lr.c:17-88
 *   dispatch, boat_scheduler_update_optimizer (ignores a rate <= 0)              src/schedulers/scheduler_common.c:41-148
 * `step` counts calls of boat_scheduler_step; before the first call the last rate is the base rate, and
 * get_next_lr previews the rate the next call will set without advancing.
 */
#include "boat_internal.h"

#include <math.h>
#include <stdlib.h>

struct boat_scheduler_t {
    boat_scheduler_type_t type;
    float base_lr, last_lr;
    int steps_taken;
    int period;                 /* step_size or T_max */
    float factor;               /* gamma or eta_min */
    float (*fn)(int step, float base_lr);
};

static boat_scheduler_t* scheduler_new(boat_scheduler_type_t type, float base_lr) {
    if (!(base_lr > 0.0f)) return NULL;
    boat_scheduler_t* s = (boat_scheduler_t*)calloc(1, sizeof(*s));
    if (!s) return NULL;
    s->type = type;
    s->base_lr = s->last_lr = base_lr;
    return s;
}

boat_scheduler_t* boat_step_lr_scheduler_create(float base_learning_rate, int step_size, float gamma) {
    if (step_size <= 0 || !(gamma > 0.0f)) return NULL;
    boat_scheduler_t* s = scheduler_new(BOAT_SCHEDULER_STEP_LR, base_learning_rate);
    if (s) {
        s->period = step_size;
        s->factor = gamma;
    }
    return s;
}

boat_scheduler_t* boat_cosine_annealing_scheduler_create(float base_learning_rate, int T_max, float eta_min) {
    if (T_max <= 0 || eta_min < 0.0f || !(eta_min < base_learning_rate)) return NULL;
    boat_scheduler_t* s = scheduler_new(BOAT_SCHEDULER_COSINE_ANNEALING, base_learning_rate);
    if (s) {
        s->period = T_max;
        s->factor = eta_min;
    }
    return s;
}

boat_scheduler_t* boat_lambda_lr_scheduler_create(float base_learning_rate, float (*lambda_fn)(int step, float base_lr)) {
    if (!lambda_fn) return NULL;
    boat_scheduler_t* s = scheduler_new(BOAT_SCHEDULER_LAMBDA_LR, base_learning_rate);
    if (s) s->fn = lambda_fn;
    return s;
}

/* the rate in force after `step` calls of boat_scheduler_step (step >= 1) */
static float rate_at(const boat_scheduler_t* s, int step) {
    switch (s->type) {
        case BOAT_SCHEDULER_STEP_LR:
            return s->base_lr * powf(s->factor, (float)((step - 1) / s->period));
        case BOAT_SCHEDULER_COSINE_ANNEALING: {
            float t = (float)step;
            const float t_max = (float)s->period;
            if (t > t_max) t = t_max;
            const float c = cosf(3.14159265358979323846f * t / t_max);
            return s->factor + 0.5f * (s->base_lr - s->factor) * (1.0f + c);
        }
        case BOAT_SCHEDULER_LAMBDA_LR: {
            const float lr = s->fn(step, s->base_lr);
            return lr < 0.0f ? 0.0f : lr;
        }
        default:
            return 0.0f;
    }
}

void boat_scheduler_step(boat_scheduler_t* s) {
    if (!s) return;
    s->steps_taken++;
    s->last_lr = rate_at(s, s->steps_taken);
}

void boat_scheduler_reset(boat_scheduler_t* s) {
    if (!s) return;
    s->steps_taken = 0;
    s->last_lr = s->base_lr;
}

float boat_scheduler_get_last_lr(const boat_scheduler_t* s) { return s ? s->last_lr : 0.0f; }
float boat_scheduler_get_next_lr(const boat_scheduler_t* s) { return s ? rate_at(s, s->steps_taken + 1) : 0.0f; }
void boat_scheduler_free(boat_scheduler_t* s) { free(s); }

void boat_scheduler_update_optimizer(const boat_scheduler_t* s, boat_optimizer_t* optimizer) {
    if (!s || !optimizer) return;
    if (s->last_lr > 0.0f) boat_optimizer_set_learning_rate(optimizer, s->last_lr);
}
