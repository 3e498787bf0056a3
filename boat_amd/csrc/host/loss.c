/* loss.c - the reference's loss objects (include/boat/loss.h:12-27): value of a loss over two equally shaped fp32 tensors.
 *
 *   MSE            sum((p - t)^2) / n                                   src/loss/mse.c:37-88
 *   cross entropy  -sum(t * logf(clip(p, 1e-7, 1 - 1e-7))) / n          src/loss/cross_entropy.c:48-104 (p are probabilities)
 *   Huber          sum(|d| <= delta ? d^2/2 : delta*(|d| - delta/2)) / n   src/loss/huber.c
 * The sum runs on the GPU (per-workgroup partials folded in double precision); the call returns a host float, so it
 * waits for the device, as the reference's callers expect.  Mismatched shapes or dtypes return 0 without a message, as
 * the reference does.  The objects also keep the reference's running sum / element count.
 */
#include "boat_internal.h"

#include <stdlib.h>

struct boat_loss_t {
    boat_loss_type_t type;
    float delta;
    float sum;
    int count;
};

static boat_loss_t* loss_new(boat_loss_type_t type, float delta) {
    boat_loss_t* l = (boat_loss_t*)calloc(1, sizeof(*l));
    if (!l) return NULL;
    l->type = type;
    l->delta = delta;
    return l;
}

boat_loss_t* boat_mse_loss_create(void) { return loss_new(BOAT_LOSS_MSE, 0.0f); }
boat_loss_t* boat_cross_entropy_loss_create(void) { return loss_new(BOAT_LOSS_CROSS_ENTROPY, 0.0f); }
boat_loss_t* boat_huber_loss_create(float delta) { return delta > 0.0f ? loss_new(BOAT_LOSS_HUBER, delta) : NULL; }
void boat_loss_free(boat_loss_t* loss) { free(loss); }

float boat_loss_compute(boat_loss_t* loss, const void* predictions, const void* targets) {
    if (!loss || !predictions || !targets) return 0.0f;
    const boat_tensor_t* p = (const boat_tensor_t*)predictions;
    const boat_tensor_t* t = (const boat_tensor_t*)targets;
    if (!bt_same_shape(p, t) || !bt_is_f32(p) || !bt_is_f32(t)) return 0.0f;
    const int kind = loss->type == BOAT_LOSS_MSE ? 0 : loss->type == BOAT_LOSS_CROSS_ENTROPY ? 1 : 2;
    const size_t n = p->nelements;
    float sum = 0.0f;
    if (n > 0) {
        const float* pp = bt_dev_read(p);
        const float* pt = bt_dev_read(t);
        float* dsum = (float*)bh_malloc(sizeof(float));
        bool ok = pp && pt && dsum &&
                  boat_hip_ok(bh_loss_terms_sum(kind, pp, pt, dsum, (int64_t)n, loss->delta), "boat_loss_compute") &&
                  boat_hip_ok(bh_memcpy_d2h(&sum, dsum, sizeof(float)), "boat_loss_compute");
        if (dsum) bh_free(dsum);
        if (!ok) return 0.0f;
    }
    loss->sum += sum;
    loss->count += (int)n;
    const float mean = sum / n;                       /* float / size_t, as in the reference; 0/0 for empty tensors */
    return kind == 1 ? -mean : mean;
}
