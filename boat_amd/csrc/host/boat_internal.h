/* boat_internal.h - private structures of the host side of libboat_amd (C11). */
#ifndef BOAT_INTERNAL_H
#define BOAT_INTERNAL_H

#include "boat_api.h"
#include "boat_hip.h"

/* Payload shared by a tensor and its views (the reference shares the raw `data`
 * pointer between a view and its parent, src/core/tensor.c:253-300). */
typedef struct boat_storage {
    void* host;            /* host mirror (malloc), NULL until first host access */
    bh_buffer_t* dev;      /* device buffer, NULL until first device access */
    size_t nbytes;
    bool host_valid;       /* host mirror holds the current values */
    bool dev_valid;        /* device buffer holds the current values */
    size_t refs;
    bool exposed;          /* coherent-pointer mode: the caller holds the host pointer and may use it at any time */
    bool pending;          /* coherent-pointer mode: written on the device since the last write-back to the host */
    void* shadow;          /* coherent-pointer mode: page-locked copy of what host mirror and device buffer both held
                              at their last transfer; a host mirror that still equals it was not written by the caller,
                              so the device copy is current without an upload; transfers are staged through it */
    bool shadow_valid;
    uint64_t upload_ticket;   /* the queued upload from `shadow` that must have run before shadow is written again */
} boat_storage_t;

struct boat_tensor_t {
    int64_t* shape;
    size_t ndim;
    boat_dtype_t dtype;
    boat_device_t device;
    boat_storage_t* st;
    size_t offset;         /* bytes into the storage; non-zero only for a slice (tensor.c:368-431) */
    size_t nbytes;
    size_t nelements;
    bool is_contiguous;
    size_t ref_count;
    bool is_view;
};

/* What exists of the reference's graph objects (include/boat/graph.h): a handle a context can carry, and the chain of
 * a model's layers seen as nodes (one per layer, in order, joined by count - 1 edges), which is all the model container
 * ever puts into its graph (src/model/model.c:434-455). */
struct boat_node_t {
    void* data;
    boat_node_type_t type;
};
struct boat_graph_t {
    boat_device_t device;
    struct boat_node_t* nodes;
    size_t node_count, node_capacity;
};

/* Coherent-pointer mode (boat_hip_set_coherent_pointers): copies every tensor whose host pointer the caller holds and
 * that this call wrote on the device back to the host.  Public functions that write tensors which existed before
 * the call end with it; a no-op in the default mode. */
void bt_flush_exposed(void);
/* device pointer for reading: uploads the host mirror first if it is the newer copy */
const float* bt_dev_read(const boat_tensor_t* t);
/* device pointer for a full overwrite: nothing is uploaded, the device copy becomes the current one */
float* bt_dev_write(boat_tensor_t* t);
/* device pointer for read-modify-write */
float* bt_dev_rw(boat_tensor_t* t);
/* A storage with no valid copy on either side is all zeros by definition (a new tensor, tensor.c:132 zero-fills) and
 * is filled in only when somebody reads it.  bt_set_zero puts a whole tensor back into that state without touching
 * memory when it can (not a slice, pointer not held by the caller) and returns whether it did; bt_dev_accumulate is the
 * pointer for `t += contribution`: while t is in the zero state the kernel may overwrite instead (*accumulate = 0), so
 * the zeros are never written and never read back. */
bool bt_set_zero(boat_tensor_t* t);
/* memcmp(a, b, n) == 0 and memcpy for the buffers of exposed tensors: on a few threads from 2 MiB on (parbytes.c) */
bool bt_bytes_equal(const void* a, const void* b, size_t n);
void bt_bytes_copy(void* dst, const void* src, size_t n);
bool bt_is_zero(const boat_tensor_t* t);
float* bt_dev_accumulate(boat_tensor_t* t, int* accumulate);
/* what boat_tensor_data() returns, for the library's own host-side writes (initial weights): the pointer does not
 * leave the library, so the tensor does not become "exposed" in coherent-pointer mode */
void* bt_host_rw(boat_tensor_t* t);
/* new fp32 tensor with the shape/device of `like`, contents unspecified (to be fully written by a kernel) */
boat_tensor_t* bt_new_like_uninit(const boat_tensor_t* like);
boat_tensor_t* bt_new_uninit(const int64_t* shape, size_t ndim, boat_device_t device);
bool bt_same_shape(const boat_tensor_t* a, const boat_tensor_t* b);
bool bt_is_f32(const boat_tensor_t* t);

/* true in reference-exact mode (boat_hip_set_reference_exact / BOAT_HIP_REFERENCE_EXACT=1) */
bool bt_reference_exact(void);

void boat_fail(boat_error_t code, const char* fmt, ...);
/* turns a bh_* return code into a Boat error; returns true when rc == 0 */
bool boat_hip_ok(int rc, const char* what);

/* layer internals shared between layers.c, autodiff.c and optimizer.c */
struct boat_dense_layer_t {
    size_t input_features, output_features;
    boat_tensor_t* weight;
    boat_tensor_t* bias;
    bool use_bias;
    boat_tensor_t* grad_weight;
    boat_tensor_t* grad_bias;
    boat_tensor_t* cache_input;
};

struct boat_layernorm_t {
    boat_layernorm_config_t config;
    boat_tensor_t* weight;
    boat_tensor_t* bias;
    boat_tensor_t* grad_weight;
    boat_tensor_t* grad_bias;
    boat_tensor_t* cache_input;
    boat_tensor_t* cache_mean;   /* [rows] */
    boat_tensor_t* cache_rstd;   /* [rows]; the reference's field is named cache_variance and never written */
};

struct boat_rmsnorm_t {
    boat_rmsnorm_config_t config;
    boat_tensor_t* weight;       /* ones at creation when elementwise_affine (norm.c:149-158) */
    boat_tensor_t* grad_weight;
    boat_tensor_t* cache_input;
    boat_tensor_t* cache_inv_rms;   /* [rows]: 1/(rms + eps); the reference's cache_rms is never written */
};

struct boat_attention_t {
    boat_attention_config_t config;
    boat_tensor_t *weight_q, *weight_k, *weight_v, *weight_o;
    boat_tensor_t *bias_q, *bias_k, *bias_v, *bias_o;
    boat_tensor_t *grad_weight_q, *grad_weight_k, *grad_weight_v, *grad_weight_o;
    boat_tensor_t *grad_bias_q, *grad_bias_k, *grad_bias_v, *grad_bias_o;
    boat_tensor_t *cache_query, *cache_key, *cache_value;
    boat_tensor_t *cache_q_proj, *cache_k_proj, *cache_v_proj;
    boat_tensor_t* cache_lse;                /* [B*nh, S] row log-sum-exp, replaces the [B,nh,S,S] weights cache */
    boat_tensor_t* cache_attention_output;   /* [B,S,H] before the output projection */
    boat_tensor_t* cache_scores;             /* [B*nh, S, S] scaled scores for the backward pass, or NULL (shape without the
                                                cached path, or larger than the score-cache limit); released by the
                                                backward pass that reads it */
    bool cache_causal;                       /* the mask the forward pass ran with: what its backward pass must use
                                                (the reference's backward works from the cached weights) */
};

/* boat_attention_backward for a layer whose query, key and value were one tensor: *grad_input = dq + dk + dv, the sums
 * made by the input projections' GEMM epilogues (used by the tape) */
bool boat_attention_backward_self(boat_attention_t* attention, const boat_tensor_t* grad_output, boat_tensor_t** grad_input);

/* layernorm backward used by both the layer hook and the tape */
boat_tensor_t* boat_layernorm_backward_impl(boat_layernorm_t* norm, const boat_tensor_t* x, const boat_tensor_t* mean,
                                            const boat_tensor_t* rstd, const boat_tensor_t* grad_output);
/* the same with `add` (may be NULL; same shape as x) added to the returned input gradient by the kernel's own store */
/* The tape's rule for an activation that sat directly behind a dense layer: dx = dy * f'(saved) together with that layer's
 * bias gradient (the column sums of dx, dense.c:286-291) in one pass; NULL when the shapes do not allow it (nothing done).
 * The dense layer's own backward is then run with bias_done, which leaves grad_bias alone. */
boat_tensor_t* bt_activation_backward_with_dense_bias(int act, const boat_tensor_t* saved, const boat_tensor_t* dy,
                                                      boat_dense_layer_t* layer);
boat_tensor_t* bt_dense_layer_backward_bias_done(boat_dense_layer_t* layer, const boat_tensor_t* grad_output);
/* where a rule that computes this layer's grad_output [rows, cols] may add that call's bias gradient itself: the device
 * pointer of grad_bias and whether to add or to write (NULL: the layer has no bias of that width; nothing is touched) */
float* bt_dense_bias_grad_target(boat_dense_layer_t* layer, int64_t cols, int* accumulate);
boat_tensor_t* boat_layernorm_backward_add_impl(boat_layernorm_t* norm, const boat_tensor_t* x, const boat_tensor_t* mean,
                                                const boat_tensor_t* rstd, const boat_tensor_t* grad_output, const boat_tensor_t* add);

#endif
