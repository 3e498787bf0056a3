/* boat_api.h - the part of Boat's public C API that lies on the training hot path, as exported
 * by libboat_amd.so.  Names, argument meaning, ownership and error conventions are those of the
 * reference headers cited beside each group, so a program written against them links unchanged;
 * all arithmetic behind them runs on the GPU through boat_hip.h (there is no host fallback).
 *
 * Host/device coherence.  A tensor created with BOAT_DEVICE_CPU keeps a host mirror and a device
 * copy with ownership flags: kernels upload a dirty host mirror before use, and
 * boat_tensor_data()/boat_tensor_const_data() wait for the stream and download a dirty device copy
 * before returning the host pointer (boat_tensor_data() also hands ownership to the host, since the
 * caller may write).  A host pointer is therefore valid until the next Boat call that takes the
 * tensor; fetch it again afterwards.  A tensor created with BOAT_DEVICE_CUDA (the reference's only
 * GPU slot, value 1; alias BOAT_DEVICE_HIP) lives in HBM only and boat_tensor_data() returns the
 * device pointer.
 *
 * Layers, the tape and the optimizers take fp32 tensors, as on the reference's hot path; the eager elementwise
 * ops also take float64, int32 and int64 tensors, like the reference's (src/ops/arithmetic.c:197-282).
 */
#ifndef BOAT_API_H
#define BOAT_API_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BOAT_API __attribute__((visibility("default")))

/* ---- include/boat/tensor.h:18-110 ---- */
typedef struct boat_tensor_t boat_tensor_t;

typedef enum {
    BOAT_DTYPE_FLOAT64, BOAT_DTYPE_FLOAT32, BOAT_DTYPE_FLOAT16, BOAT_DTYPE_FLOAT8, BOAT_DTYPE_FLOAT4,
    BOAT_DTYPE_INT64, BOAT_DTYPE_INT32, BOAT_DTYPE_UINT8, BOAT_DTYPE_BITS2, BOAT_DTYPE_BITS1,
    BOAT_DTYPE_BOOL, BOAT_DTYPE_COUNT
} boat_dtype_t;

enum boat_device_enum { BOAT_DEVICE_CPU, BOAT_DEVICE_CUDA, BOAT_DEVICE_COUNT };
typedef enum boat_device_enum boat_device_t;
#define BOAT_DEVICE_HIP BOAT_DEVICE_CUDA   /* same ABI value: the one GPU slot of tensor.h:50-55 */
#define BOAT_MAX_DIMS 8

BOAT_API boat_tensor_t* boat_tensor_create(const int64_t* shape, size_t ndim, boat_dtype_t dtype, boat_device_t device);
BOAT_API boat_tensor_t* boat_tensor_create_like(const boat_tensor_t* other);
BOAT_API boat_tensor_t* boat_tensor_from_data(const int64_t* shape, size_t ndim, boat_dtype_t dtype, const void* data);
BOAT_API void boat_tensor_free(boat_tensor_t* tensor);
BOAT_API void boat_tensor_ref(boat_tensor_t* tensor);
BOAT_API void boat_tensor_unref(boat_tensor_t* tensor);
BOAT_API const int64_t* boat_tensor_shape(const boat_tensor_t* tensor);
BOAT_API size_t boat_tensor_ndim(const boat_tensor_t* tensor);
BOAT_API boat_dtype_t boat_tensor_dtype(const boat_tensor_t* tensor);
BOAT_API boat_device_t boat_tensor_device(const boat_tensor_t* tensor);
BOAT_API size_t boat_tensor_nbytes(const boat_tensor_t* tensor);
BOAT_API size_t boat_tensor_nelements(const boat_tensor_t* tensor);
BOAT_API bool boat_tensor_is_contiguous(const boat_tensor_t* tensor);
BOAT_API void* boat_tensor_data(const boat_tensor_t* tensor);
BOAT_API const void* boat_tensor_const_data(const boat_tensor_t* tensor);
BOAT_API boat_tensor_t* boat_tensor_slice(const boat_tensor_t* tensor, const size_t* start, const size_t* end, const size_t* step);   /* tensor.h:87; a view */
BOAT_API boat_tensor_t* boat_tensor_reshape(const boat_tensor_t* tensor, const int64_t* new_shape, size_t new_ndim);
BOAT_API boat_tensor_t* boat_tensor_to_device(const boat_tensor_t* tensor, boat_device_t dev);   /* declared only in the reference (tensor.h:92) */
BOAT_API boat_tensor_t* boat_tensor_clone(const boat_tensor_t* tensor);
BOAT_API size_t boat_dtype_size(boat_dtype_t dtype);
BOAT_API const char* boat_dtype_name(boat_dtype_t dtype);

/* ---- include/boat/memory.h:17-55 ---- */
typedef struct {
    size_t allocated_bytes;
    size_t allocated_blocks;
    size_t peak_allocated_bytes;
    size_t freed_bytes;
    size_t freed_blocks;
} boat_memory_stats_t;

BOAT_API void* boat_memory_allocate(size_t size, boat_device_t device, const char* file, int line);
BOAT_API void* boat_memory_allocate_zero(size_t size, boat_device_t device, const char* file, int line);
BOAT_API void boat_memory_free(void* ptr);
BOAT_API void boat_memory_free_safe(void** ptr_ptr);
BOAT_API void* boat_memory_allocate_aligned(size_t size, size_t alignment, boat_device_t device, const char* file, int line);
BOAT_API void boat_memory_free_aligned(const void* aligned_ptr);
BOAT_API void* boat_memory_reallocate(void* ptr, size_t new_size, boat_device_t device, const char* file, int line);
BOAT_API void* boat_memory_allocate_device(size_t size, boat_device_t device, const char* file, int line);
BOAT_API void boat_memory_free_device(void* ptr, boat_device_t device);
BOAT_API void boat_memory_copy(void* dest, const void* src, size_t size, boat_device_t dest_device, boat_device_t src_device);
BOAT_API void boat_memory_set(void* dest, int value, size_t size, boat_device_t device);
BOAT_API boat_memory_stats_t boat_memory_get_stats(void);
BOAT_API void boat_memory_reset_stats(void);
BOAT_API void boat_memory_print_stats(FILE* stream);
/* include/boat/memory.h:58-77: host-side pool of equal blocks and bump arena (no GPU involvement) */
typedef struct boat_memory_pool_t boat_memory_pool_t;
BOAT_API boat_memory_pool_t* boat_memory_pool_create(size_t block_size, size_t initial_blocks);
BOAT_API void boat_memory_pool_free(boat_memory_pool_t* pool);
BOAT_API void* boat_memory_pool_alloc(boat_memory_pool_t* pool, size_t size);
BOAT_API void boat_memory_pool_free_block(boat_memory_pool_t* pool, void* block);
BOAT_API void boat_memory_pool_clear(boat_memory_pool_t* pool);
BOAT_API size_t boat_memory_pool_allocated_blocks(const boat_memory_pool_t* pool);
BOAT_API size_t boat_memory_pool_free_blocks(const boat_memory_pool_t* pool);
BOAT_API size_t boat_memory_pool_total_memory(const boat_memory_pool_t* pool);
typedef struct boat_memory_arena_t boat_memory_arena_t;
BOAT_API boat_memory_arena_t* boat_memory_arena_create(size_t initial_size);
BOAT_API void boat_memory_arena_free(boat_memory_arena_t* arena);
BOAT_API void* boat_memory_arena_alloc(boat_memory_arena_t* arena, size_t size);
BOAT_API void boat_memory_arena_reset(boat_memory_arena_t* arena);
BOAT_API size_t boat_memory_arena_used(const boat_memory_arena_t* arena);
BOAT_API size_t boat_memory_arena_capacity(const boat_memory_arena_t* arena);

/* ---- include/boat.h:64-94 (error reporting; src/core/error.c:21-62: a thread-local code and a 256-byte message) ---- */
typedef enum {
    BOAT_SUCCESS = 0, BOAT_ERROR_INVALID_ARGUMENT, BOAT_ERROR_OUT_OF_MEMORY, BOAT_ERROR_INVALID_OPERATION,
    BOAT_ERROR_DEVICE, BOAT_ERROR_FILE_IO, BOAT_ERROR_FORMAT, BOAT_ERROR_NOT_IMPLEMENTED, BOAT_ERROR_UNKNOWN
} boat_error_t;
BOAT_API void boat_init(void);      /* declared in include/boat.h, defined nowhere in the reference; here it brings the device up */
BOAT_API void boat_cleanup(void);   /* likewise; releases the stream and the cached device blocks */
BOAT_API const char* boat_error_string(boat_error_t error);
BOAT_API boat_error_t boat_get_last_error(void);
BOAT_API const char* boat_get_last_error_message(void);
BOAT_API void boat_set_error(boat_error_t error, const char* message);
BOAT_API void boat_clear_error(void);
BOAT_API void boat_set_errorf(boat_error_t error, const char* format, ...);
BOAT_API void boat_reset_error(void);
BOAT_API bool boat_has_error(void);

/* ---- include/boat/ops.h:15-60 (the ops the backward pass is built from) ---- */
BOAT_API boat_tensor_t* boat_add(const boat_tensor_t* a, const boat_tensor_t* b);
BOAT_API boat_tensor_t* boat_sub(const boat_tensor_t* a, const boat_tensor_t* b);
BOAT_API boat_tensor_t* boat_mul(const boat_tensor_t* a, const boat_tensor_t* b);
BOAT_API boat_tensor_t* boat_div(const boat_tensor_t* a, const boat_tensor_t* b);
BOAT_API boat_tensor_t* boat_mod(const boat_tensor_t* a, const boat_tensor_t* b);   /* fmodf / fmod / % by element type (arithmetic.c:288-360) */
BOAT_API void boat_add_(boat_tensor_t* a, const boat_tensor_t* b);
BOAT_API void boat_sub_(boat_tensor_t* a, const boat_tensor_t* b);
BOAT_API void boat_mul_(boat_tensor_t* a, const boat_tensor_t* b);
BOAT_API void boat_div_(boat_tensor_t* a, const boat_tensor_t* b);
BOAT_API boat_tensor_t* boat_add_scalar(const boat_tensor_t* a, double scalar);
BOAT_API boat_tensor_t* boat_sub_scalar(const boat_tensor_t* a, double scalar);
BOAT_API boat_tensor_t* boat_mul_scalar(const boat_tensor_t* a, double scalar);
BOAT_API boat_tensor_t* boat_div_scalar(const boat_tensor_t* a, double scalar);
BOAT_API boat_tensor_t* boat_pow_scalar(const boat_tensor_t* a, double scalar);     /* float32 / float64 (arithmetic.c:486-518) */
BOAT_API void boat_add_scalar_(boat_tensor_t* a, double scalar);
BOAT_API void boat_sub_scalar_(boat_tensor_t* a, double scalar);
BOAT_API void boat_mul_scalar_(boat_tensor_t* a, double scalar);
BOAT_API void boat_div_scalar_(boat_tensor_t* a, double scalar);
BOAT_API boat_tensor_t* boat_inverse(const boat_tensor_t* a);                       /* returns NULL, as the reference's stub (linear.c:409-413) */
BOAT_API boat_tensor_t* boat_matmul(const boat_tensor_t* a, const boat_tensor_t* b);
BOAT_API boat_tensor_t* boat_dot(const boat_tensor_t* a, const boat_tensor_t* b);
BOAT_API boat_tensor_t* boat_transpose(const boat_tensor_t* a, int dim0, int dim1);
BOAT_API boat_tensor_t* boat_relu(const boat_tensor_t* a);
BOAT_API boat_tensor_t* boat_sigmoid(const boat_tensor_t* a);   /* stub in the reference (activation.c:286-290); here the forward of boat_var_sigmoid */
BOAT_API boat_tensor_t* boat_tanh(const boat_tensor_t* a);      /* stub in the reference (activation.c:292-296); here the forward of boat_var_tanh */
BOAT_API boat_tensor_t* boat_softmax(const boat_tensor_t* a, int axis);
BOAT_API boat_tensor_t* boat_log_softmax(const boat_tensor_t* a, int axis);
BOAT_API boat_tensor_t* boat_gelu(const boat_tensor_t* a);                          /* stub in the reference (src/ops/activation.c:298-302) */
BOAT_API boat_tensor_t* boat_selu(const boat_tensor_t* a);                          /* returns NULL, as the reference's stub (activation.c:304-308) */
BOAT_API boat_tensor_t* boat_sum(const boat_tensor_t* a, const int64_t* dims, size_t n_dims, bool keepdim);
BOAT_API boat_tensor_t* boat_mean(const boat_tensor_t* a, const int64_t* dims, size_t n_dims, bool keepdim);
/* ---- include/boat/ops.h:107-108 (the shape rule of the elementwise ops, arithmetic.c:575-608) ---- */
BOAT_API bool boat_can_broadcast(const boat_tensor_t* a, const boat_tensor_t* b);
BOAT_API boat_tensor_t* boat_broadcast_to(const boat_tensor_t* a, const int64_t* shape, size_t ndim);   /* as the reference: a dense copy under the new shape, equal element counts only */

/* ---- include/boat/autodiff.h:15-98 ---- */
typedef struct boat_variable_t boat_variable_t;
typedef struct boat_autodiff_context_t boat_autodiff_context_t;
struct boat_dense_layer_t;
struct boat_attention_t;
struct boat_conv_layer_t;
struct boat_pool_layer_t;

BOAT_API boat_variable_t* boat_variable_create(boat_tensor_t* tensor, bool requires_grad);
BOAT_API boat_variable_t* boat_variable_create_with_shape(const int64_t* shape, size_t ndim, boat_dtype_t dtype, bool requires_grad);
BOAT_API void boat_variable_free(const boat_variable_t* variable);
BOAT_API boat_tensor_t* boat_variable_data(const boat_variable_t* variable);
BOAT_API boat_tensor_t* boat_variable_grad(const boat_variable_t* variable);
BOAT_API bool boat_variable_requires_grad(const boat_variable_t* variable);
BOAT_API void boat_variable_set_requires_grad(boat_variable_t* variable, bool requires_grad);
BOAT_API bool boat_variable_reset_data(boat_variable_t* variable, boat_tensor_t* new_tensor);
BOAT_API void boat_variable_zero_grad(boat_variable_t* variable);
BOAT_API void boat_variable_retain_grad(const boat_variable_t* variable, bool retain);
BOAT_API void boat_variable_backward(boat_variable_t* variable, boat_tensor_t* grad_output);
BOAT_API void boat_variable_backward_full(const boat_variable_t* variable);
BOAT_API boat_variable_t* boat_var_add(const boat_variable_t* a, const boat_variable_t* b);
BOAT_API boat_variable_t* boat_var_sub(const boat_variable_t* a, const boat_variable_t* b);
BOAT_API boat_variable_t* boat_var_mul(const boat_variable_t* a, const boat_variable_t* b);
BOAT_API boat_variable_t* boat_var_div(const boat_variable_t* a, const boat_variable_t* b);
BOAT_API boat_variable_t* boat_var_matmul(const boat_variable_t* a, const boat_variable_t* b);
BOAT_API boat_variable_t* boat_var_dot(const boat_variable_t* a, const boat_variable_t* b);
BOAT_API boat_variable_t* boat_var_flatten(const boat_variable_t* input);
BOAT_API void boat_autodiff_set_grad_checkpointing(bool enabled);               /* no effect, as in the reference (autodiff.c:652-655) */
BOAT_API void boat_autodiff_print_graph(const boat_variable_t* variable);        /* lists the ops behind `variable` (empty in the reference, autodiff.c:727-730) */
BOAT_API char* boat_autodiff_graph_to_dot(const boat_variable_t* variable);      /* malloc'ed Graphviz text, NULL for a leaf (returns NULL in the reference, :732-736) */
BOAT_API boat_variable_t* boat_var_dense(const boat_variable_t* input, const struct boat_dense_layer_t* layer);
BOAT_API boat_variable_t* boat_var_conv(const boat_variable_t* input, const struct boat_conv_layer_t* layer);
BOAT_API boat_variable_t* boat_var_pool(const boat_variable_t* input, const struct boat_pool_layer_t* layer);
BOAT_API boat_variable_t* boat_var_attention(const boat_variable_t* query, const boat_variable_t* key, const boat_variable_t* value,
                                             const struct boat_attention_t* attention, const boat_tensor_t* attention_mask);
BOAT_API boat_variable_t* boat_var_relu(const boat_variable_t* a);
BOAT_API boat_variable_t* boat_var_sigmoid(const boat_variable_t* a);
BOAT_API boat_variable_t* boat_var_tanh(const boat_variable_t* a);
BOAT_API boat_variable_t* boat_var_softmax(const boat_variable_t* a, int axis);
BOAT_API boat_variable_t* boat_var_log_softmax(const boat_variable_t* a, int axis);
BOAT_API boat_variable_t* boat_var_sum(const boat_variable_t* a, const int64_t* dims, size_t n_dims, bool keepdim);
BOAT_API boat_variable_t* boat_var_mean(const boat_variable_t* a, int64_t* dims, size_t n_dims, bool keepdim);
BOAT_API boat_variable_t* boat_var_max(const boat_variable_t* a, int64_t* dims, size_t n_dims, bool keepdim);   /* NULL, as in the reference (autodiff.c:595-603) */
BOAT_API boat_variable_t* boat_var_min(const boat_variable_t* a, int64_t* dims, size_t n_dims, bool keepdim);
/* include/boat/graph.h:18,41-43 and autodiff.h:87-88: an opaque handle that a context can carry for its caller.  The
 * graph IR itself (nodes, edges, traversal) is outside the training path and is not provided. */
typedef struct boat_graph_t boat_graph_t;
typedef struct boat_node_t boat_node_t;
typedef enum {   /* graph.h:23-29 */
    BOAT_NODE_TYPE_VARIABLE, BOAT_NODE_TYPE_OPERATION, BOAT_NODE_TYPE_CONSTANT, BOAT_NODE_TYPE_PLACEHOLDER, BOAT_NODE_TYPE_OUTPUT
} boat_node_type_t;
BOAT_API const char* boat_node_type_name(boat_node_type_t type);
/* read-only view of a model's layers as the chain the reference's model container records (graph.h:52-53,72-75,
 * model.h:42; src/model/model.c:434-455): node i carries layer i, consecutive nodes are joined by an edge */
BOAT_API size_t boat_graph_node_count(const boat_graph_t* graph);
BOAT_API size_t boat_graph_edge_count(const boat_graph_t* graph);
BOAT_API boat_node_t* boat_graph_get_node_at_index(const boat_graph_t* graph, size_t index);
BOAT_API void* boat_node_data(const boat_node_t* node);
BOAT_API boat_node_type_t boat_node_type(const boat_node_t* node);
BOAT_API boat_graph_t* boat_graph_create(void);
BOAT_API boat_graph_t* boat_graph_create_with_device(boat_device_t device);
BOAT_API void boat_graph_free(boat_graph_t* graph);
BOAT_API void boat_autodiff_context_set_graph(boat_autodiff_context_t* context, const boat_graph_t* graph);
BOAT_API boat_graph_t* boat_autodiff_context_get_graph(const boat_autodiff_context_t* context);
BOAT_API boat_autodiff_context_t* boat_autodiff_context_create(void);
BOAT_API void boat_autodiff_context_free(const boat_autodiff_context_t* context);
BOAT_API void boat_autodiff_context_enable_grad(boat_autodiff_context_t* context);
BOAT_API void boat_autodiff_context_disable_grad(boat_autodiff_context_t* context);   /* the reference stores the flag and never reads it (autodiff.c:625-632); here ops recorded while the current context has it off get no tape entry */
BOAT_API bool boat_autodiff_context_grad_enabled(const boat_autodiff_context_t* context);
BOAT_API void boat_autodiff_set_current_context(const boat_autodiff_context_t* context);
BOAT_API boat_autodiff_context_t* boat_autodiff_get_current_context(void);
BOAT_API void boat_autodiff_clear_computation_graph(void);

/* ---- include/boat/layers.h:23-35 (dense) ---- */
typedef struct boat_dense_layer_t boat_dense_layer_t;
BOAT_API boat_dense_layer_t* boat_dense_layer_create(size_t input_features, size_t output_features, bool use_bias);
BOAT_API void boat_dense_layer_free(boat_dense_layer_t* layer);
BOAT_API boat_tensor_t* boat_dense_layer_forward(boat_dense_layer_t* layer, const boat_tensor_t* input);
BOAT_API boat_tensor_t* boat_dense_layer_backward(boat_dense_layer_t* layer, const boat_tensor_t* grad_output);
BOAT_API void boat_dense_layer_update(boat_dense_layer_t* layer, float learning_rate);
BOAT_API void boat_dense_layer_set_weight(boat_dense_layer_t* layer, boat_tensor_t* weight);
BOAT_API void boat_dense_layer_set_bias(boat_dense_layer_t* layer, boat_tensor_t* bias);
BOAT_API boat_tensor_t* boat_dense_layer_get_weight(const boat_dense_layer_t* layer);
BOAT_API boat_tensor_t* boat_dense_layer_get_bias(const boat_dense_layer_t* layer);
BOAT_API boat_tensor_t* boat_dense_layer_get_grad_weight(const boat_dense_layer_t* layer);
BOAT_API boat_tensor_t* boat_dense_layer_get_grad_bias(const boat_dense_layer_t* layer);

/* ---- include/boat/layers.h:38-51 (2-D convolution), :68-72 (max pooling), :128-132 (flatten) ---- */
typedef struct boat_conv_layer_t boat_conv_layer_t;
BOAT_API boat_conv_layer_t* boat_conv_layer_create(size_t in_channels, size_t out_channels, size_t kernel_size, size_t stride, size_t padding);
BOAT_API void boat_conv_layer_free(boat_conv_layer_t* layer);
BOAT_API boat_tensor_t* boat_conv_layer_forward(boat_conv_layer_t* layer, const boat_tensor_t* input);
/* grad_weight/grad_bias are overwritten in place (the reference replaces the tensors, src/layers/conv.c:523-532);
 * the returned input gradient is the true one (the reference mirrors the kernel taps, conv.c:86-88) */
BOAT_API boat_tensor_t* boat_conv_layer_backward(boat_conv_layer_t* layer, const boat_tensor_t* grad_output);
BOAT_API void boat_conv_layer_update(boat_conv_layer_t* layer, float learning_rate);
BOAT_API void boat_conv_layer_set_weight(boat_conv_layer_t* layer, boat_tensor_t* weight);
BOAT_API void boat_conv_layer_set_bias(boat_conv_layer_t* layer, boat_tensor_t* bias);
BOAT_API boat_tensor_t* boat_conv_layer_get_weight(const boat_conv_layer_t* layer);
BOAT_API boat_tensor_t* boat_conv_layer_get_bias(const boat_conv_layer_t* layer);
BOAT_API boat_tensor_t* boat_conv_layer_get_grad_weight(const boat_conv_layer_t* layer);
BOAT_API boat_tensor_t* boat_conv_layer_get_grad_bias(const boat_conv_layer_t* layer);
typedef struct boat_pool_layer_t boat_pool_layer_t;
BOAT_API boat_pool_layer_t* boat_pool_layer_create(size_t pool_size, size_t stride, size_t padding);
BOAT_API void boat_pool_layer_free(boat_pool_layer_t* layer);
BOAT_API boat_tensor_t* boat_pool_layer_forward(boat_pool_layer_t* layer, const boat_tensor_t* input);
BOAT_API boat_tensor_t* boat_pool_layer_backward(boat_pool_layer_t* layer, const boat_tensor_t* grad_output);
BOAT_API void boat_pool_layer_update(boat_pool_layer_t* layer, float learning_rate);
typedef struct boat_flatten_layer_t boat_flatten_layer_t;
BOAT_API boat_flatten_layer_t* boat_flatten_layer_create(void);
BOAT_API void boat_flatten_layer_free(boat_flatten_layer_t* layer);
BOAT_API boat_tensor_t* boat_flatten_layer_forward(boat_flatten_layer_t* layer, const boat_tensor_t* input);
BOAT_API boat_tensor_t* boat_flatten_layer_backward(const boat_flatten_layer_t* layer, const boat_tensor_t* grad_output);
BOAT_API void boat_flatten_layer_update(boat_flatten_layer_t* layer, float learning_rate);

/* ---- include/boat/layers.h:95-107 (activation layers) ---- */
typedef struct boat_relu_layer_t boat_relu_layer_t;
BOAT_API boat_relu_layer_t* boat_relu_layer_create(void);
BOAT_API void boat_relu_layer_free(boat_relu_layer_t* layer);
BOAT_API boat_tensor_t* boat_relu_layer_forward(const boat_relu_layer_t* layer, const boat_tensor_t* input);
BOAT_API boat_tensor_t* boat_relu_layer_backward(boat_relu_layer_t* layer, const boat_tensor_t* grad_output);
BOAT_API void boat_relu_layer_update(boat_relu_layer_t* layer, float learning_rate);
typedef struct boat_softmax_layer_t boat_softmax_layer_t;
BOAT_API boat_softmax_layer_t* boat_softmax_layer_create(int axis);
BOAT_API void boat_softmax_layer_free(boat_softmax_layer_t* layer);
BOAT_API boat_tensor_t* boat_softmax_layer_forward(const boat_softmax_layer_t* layer, const boat_tensor_t* input);
BOAT_API boat_tensor_t* boat_softmax_layer_backward(boat_softmax_layer_t* layer, const boat_tensor_t* grad_output);
BOAT_API void boat_softmax_layer_update(boat_softmax_layer_t* layer, float learning_rate);

/* ---- include/boat/layers/norm.h:15-76, include/boat/layers.h:75-79 ---- */
typedef struct boat_layernorm_t boat_layernorm_t;
typedef boat_layernorm_t boat_norm_layer_t;
typedef struct {
    size_t normalized_shape;
    float eps;
    bool elementwise_affine;
    bool use_bias;
} boat_layernorm_config_t;
BOAT_API boat_layernorm_t* boat_layernorm_create(const boat_layernorm_config_t* config);
BOAT_API void boat_layernorm_free(boat_layernorm_t* norm);
BOAT_API boat_tensor_t* boat_layernorm_forward(boat_layernorm_t* norm, const boat_tensor_t* input);
BOAT_API boat_tensor_t* boat_layernorm_backward(boat_layernorm_t* norm, const boat_tensor_t* grad_output);   /* stub in the reference (norm.c:397-402) */
BOAT_API void boat_layernorm_update(boat_layernorm_t* norm, float learning_rate);                          /* stub in the reference (norm.c:411-415) */
BOAT_API void boat_layernorm_set_weight(boat_layernorm_t* norm, boat_tensor_t* weight);
BOAT_API void boat_layernorm_set_bias(boat_layernorm_t* norm, boat_tensor_t* bias);
/* RMSNorm (norm.h:28-32,42-46): y = x / (sqrtf(mean(x^2)) + eps) * weight, eps outside the root (norm.c:226,376);
 * backward and update are stubs in the reference (norm.c:404-421) and work here like LayerNorm's */
typedef struct boat_rmsnorm_t boat_rmsnorm_t;
typedef struct {
    size_t normalized_shape;
    float eps;
    bool elementwise_affine;
} boat_rmsnorm_config_t;
BOAT_API boat_rmsnorm_t* boat_rmsnorm_create(const boat_rmsnorm_config_t* config);
BOAT_API void boat_rmsnorm_free(boat_rmsnorm_t* norm);
BOAT_API boat_tensor_t* boat_rmsnorm_forward(boat_rmsnorm_t* norm, const boat_tensor_t* input);
BOAT_API boat_tensor_t* boat_rmsnorm_backward(boat_rmsnorm_t* norm, const boat_tensor_t* grad_output);
BOAT_API void boat_rmsnorm_update(boat_rmsnorm_t* norm, float learning_rate);
/* stateless forms over the last dimension, no affine (NULL stubs in the reference, norm.c:424-463) */
BOAT_API boat_tensor_t* boat_layer_norm(const boat_tensor_t* input, const int64_t* normalized_shape, size_t normalized_shape_len, float eps);
BOAT_API boat_tensor_t* boat_rms_norm(const boat_tensor_t* input, const int64_t* normalized_shape, size_t normalized_shape_len, float eps);
BOAT_API boat_tensor_t* boat_rms_norm_grad(const boat_tensor_t* grad_output, const boat_tensor_t* input, const boat_tensor_t* output,
                                           const int64_t* normalized_shape, size_t normalized_shape_len, float eps);
BOAT_API boat_tensor_t* boat_layer_norm_grad(const boat_tensor_t* grad_output, const boat_tensor_t* input, const boat_tensor_t* output,
                                             const int64_t* normalized_shape, size_t normalized_shape_len, float eps);  /* stub in the reference (norm.c:450-463) */
BOAT_API boat_norm_layer_t* boat_norm_layer_create(size_t normalized_shape, float eps, bool elementwise_affine);
BOAT_API void boat_norm_layer_free(boat_norm_layer_t* layer);
BOAT_API boat_tensor_t* boat_norm_layer_forward(boat_norm_layer_t* layer, const boat_tensor_t* input);
BOAT_API boat_tensor_t* boat_norm_layer_backward(boat_norm_layer_t* layer, const boat_tensor_t* grad_output);
BOAT_API void boat_norm_layer_update(boat_norm_layer_t* layer, float learning_rate);

/* ---- include/boat/layers/attention.h:17-107, include/boat/layers.h:82-92 ---- */
typedef struct boat_attention_t boat_attention_t;
typedef struct {
    size_t hidden_size;
    size_t num_heads;
    size_t head_size;
    float dropout_prob;
    bool causal_mask;
    bool use_bias;
    bool use_rotary;
    float rotary_theta;
} boat_attention_config_t;
BOAT_API boat_attention_t* boat_attention_create(const boat_attention_config_t* config);
BOAT_API void boat_attention_free(boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_forward(boat_attention_t* attention, const boat_tensor_t* query, const boat_tensor_t* key,
                                               const boat_tensor_t* value, const boat_tensor_t* attention_mask);
BOAT_API bool boat_attention_backward(boat_attention_t* attention, const boat_tensor_t* grad_output,
                                      boat_tensor_t** grad_query, boat_tensor_t** grad_key, boat_tensor_t** grad_value);
BOAT_API void boat_attention_update(boat_attention_t* attention, float learning_rate);
BOAT_API void boat_attention_set_causal(boat_attention_t* attention, bool causal);
/* attention.h:63-76: the attention core on [batch, heads, seq, head_size] operands (attention.c:1082-1092), and
 * self-attention through a throw-away layer (attention.c:830-880) */
BOAT_API boat_tensor_t* boat_multihead_attention(const boat_tensor_t* input, size_t num_heads, float dropout_prob, bool causal_mask,
                                                 const boat_tensor_t* attention_mask);
BOAT_API boat_tensor_t* boat_scaled_dot_product_attention(const boat_tensor_t* query, const boat_tensor_t* key, const boat_tensor_t* value,
                                                          float scale_factor, const boat_tensor_t* attention_mask, bool causal_mask,
                                                          float dropout_prob);
/* attention.h:79-90: not implemented in the reference (attention.c:1094-1120): NULL / no effect here too */
BOAT_API boat_tensor_t* boat_rotary_position_encoding(const boat_tensor_t* tensor, size_t seq_len, size_t head_size, float theta);
BOAT_API void boat_apply_rotary_embedding(boat_tensor_t* query, boat_tensor_t* key, size_t seq_len, size_t head_size, float theta);
BOAT_API void boat_attention_set_dropout(boat_attention_t* attention, float dropout_prob);   /* stored, not applied (attention.c:1061-1062) */
BOAT_API boat_tensor_t* boat_attention_get_weight_q(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_weight_k(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_weight_v(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_weight_o(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_bias_q(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_bias_k(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_bias_v(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_bias_o(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_grad_weight_q(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_grad_weight_k(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_grad_weight_v(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_grad_weight_o(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_grad_bias_q(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_grad_bias_k(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_grad_bias_v(const boat_attention_t* attention);
BOAT_API boat_tensor_t* boat_attention_get_grad_bias_o(const boat_attention_t* attention);
typedef struct boat_attention_layer_t boat_attention_layer_t;
BOAT_API boat_attention_layer_t* boat_attention_layer_create(size_t hidden_size, size_t num_heads, float dropout_prob, bool causal_mask);
BOAT_API void boat_attention_layer_free(boat_attention_layer_t* layer);
BOAT_API boat_tensor_t* boat_attention_layer_forward(boat_attention_layer_t* layer, const boat_tensor_t* query, const boat_tensor_t* key,
                                                     const boat_tensor_t* value, const boat_tensor_t* attention_mask);
BOAT_API boat_tensor_t* boat_attention_layer_backward(boat_attention_layer_t* layer, const boat_tensor_t* grad_output);
BOAT_API void boat_attention_layer_update(boat_attention_layer_t* layer, float learning_rate);

/* ---- include/boat/optimizers.h:15-44 ---- */
typedef enum { BOAT_OPTIMIZER_SGD, BOAT_OPTIMIZER_ADAM, BOAT_OPTIMIZER_RMSPROP, BOAT_OPTIMIZER_ADAGRAD } boat_optimizer_type_t;
typedef struct boat_optimizer_t boat_optimizer_t;
BOAT_API boat_optimizer_t* boat_sgd_optimizer_create(float learning_rate, float momentum);    /* returns NULL, as the reference's stub (optimizer_common.c:62-67) */
BOAT_API boat_optimizer_t* boat_adam_optimizer_create(float learning_rate, float beta1, float beta2, float epsilon);
BOAT_API boat_optimizer_t* boat_rmsprop_optimizer_create(float learning_rate, float alpha, float epsilon);
BOAT_API boat_optimizer_t* boat_adagrad_optimizer_create(float learning_rate, float epsilon);
BOAT_API void boat_optimizer_step(boat_optimizer_t* optimizer);
BOAT_API void boat_optimizer_zero_grad(boat_optimizer_t* optimizer);
BOAT_API void boat_optimizer_free(boat_optimizer_t* optimizer);
BOAT_API void boat_optimizer_add_parameter(boat_optimizer_t* optimizer, boat_tensor_t* param, boat_tensor_t* grad);
BOAT_API float boat_optimizer_get_learning_rate(const boat_optimizer_t* optimizer);
BOAT_API void boat_optimizer_set_learning_rate(boat_optimizer_t* optimizer, float learning_rate);

/* ---- include/boat/loss.h:12-27 (loss values; the reference has no loss-gradient function) ---- */
typedef enum { BOAT_LOSS_MSE, BOAT_LOSS_CROSS_ENTROPY, BOAT_LOSS_HUBER } boat_loss_type_t;
typedef struct boat_loss_t boat_loss_t;
BOAT_API boat_loss_t* boat_mse_loss_create(void);
BOAT_API boat_loss_t* boat_cross_entropy_loss_create(void);
BOAT_API boat_loss_t* boat_huber_loss_create(float delta);
/* predictions and targets are boat_tensor_t*; returns the mean loss on the host (waits for the device) */
BOAT_API float boat_loss_compute(boat_loss_t* loss, const void* predictions, const void* targets);
BOAT_API void boat_loss_free(boat_loss_t* loss);

/* ---- include/boat/schedulers.h:15-52 (learning-rate schedulers; host arithmetic, one float per step) ---- */
typedef enum { BOAT_SCHEDULER_STEP_LR, BOAT_SCHEDULER_COSINE_ANNEALING, BOAT_SCHEDULER_LAMBDA_LR } boat_scheduler_type_t;
typedef struct boat_scheduler_t boat_scheduler_t;
BOAT_API boat_scheduler_t* boat_step_lr_scheduler_create(float base_learning_rate, int step_size, float gamma);
BOAT_API boat_scheduler_t* boat_cosine_annealing_scheduler_create(float base_learning_rate, int T_max, float eta_min);
BOAT_API boat_scheduler_t* boat_lambda_lr_scheduler_create(float base_learning_rate, float (*lambda_fn)(int step, float base_lr));
BOAT_API void boat_scheduler_step(boat_scheduler_t* scheduler);
BOAT_API void boat_scheduler_reset(boat_scheduler_t* scheduler);
BOAT_API float boat_scheduler_get_last_lr(const boat_scheduler_t* scheduler);
BOAT_API float boat_scheduler_get_next_lr(const boat_scheduler_t* scheduler);
BOAT_API void boat_scheduler_free(boat_scheduler_t* scheduler);
BOAT_API void boat_scheduler_update_optimizer(const boat_scheduler_t* scheduler, boat_optimizer_t* optimizer);

/* ---- include/boat/model.h:17-65 ---- */
typedef struct boat_model_t boat_model_t;
typedef struct boat_layer_ops_t boat_layer_ops_t;
typedef struct boat_layer_t {
    void* data;
    const boat_layer_ops_t* ops;
} boat_layer_t;
struct boat_layer_ops_t {
    boat_tensor_t* (*forward)(const boat_layer_t* layer, const boat_tensor_t* input);
    boat_tensor_t* (*backward)(const boat_layer_t* layer, const boat_tensor_t* grad_output);
    void (*update)(const boat_layer_t* layer, float learning_rate);
    void (*free)(const boat_layer_t* layer);
};
BOAT_API boat_model_t* boat_model_create(void);
BOAT_API void boat_model_free(boat_model_t* model);
BOAT_API void boat_model_add_layer(boat_model_t* model, boat_layer_t* layer);
BOAT_API size_t boat_model_layer_count(const boat_model_t* model);
BOAT_API boat_model_t* boat_model_create_with_graph(const boat_graph_t* graph);   /* the model takes the graph over (model.c:59-83) */
BOAT_API void boat_model_set_graph(boat_model_t* model, boat_graph_t* graph);
BOAT_API void* boat_model_get_user_data(const boat_model_t* model);
BOAT_API void boat_model_set_user_data(boat_model_t* model, void* user_data, void (*free_fn)(void*));
BOAT_API boat_model_t* boat_model_load(const char* filename);                       /* NULL / false, as the reference's stubs (model.c:368-379) */
BOAT_API bool boat_model_save(const boat_model_t* model, const char* filename);
BOAT_API boat_graph_t* boat_model_graph(const boat_model_t* model);   /* model.h:42; the chain view declared with the tape's contexts above */
BOAT_API boat_tensor_t* boat_model_forward(const boat_model_t* model, const boat_tensor_t* input);
BOAT_API boat_tensor_t* boat_model_backward(const boat_model_t* model, const boat_tensor_t* grad_output);  /* stub in the reference (model.c:354-359) */
BOAT_API void boat_model_update(const boat_model_t* model, float learning_rate);                          /* stub in the reference (model.c:361-365) */
typedef boat_model_t boat_sequential_model_t;
BOAT_API boat_sequential_model_t* boat_sequential_create(void);
BOAT_API void boat_sequential_add(boat_sequential_model_t* model, boat_layer_t* layer);

/* ---- additions with no counterpart in the reference (named boat_hip_*) ---- */
/* wait for all queued GPU work */
BOAT_API void boat_hip_synchronize(void);
/* Coherent-pointer mode, for callers that keep the float* of boat_tensor_data() across calls, write through it before
 * a later call and read results through it afterwards (the reference's own tests do: test_attention_gradient_check.c:22-41,
 * test_optimizer_adam.c:96-108; there the pointer is the tensor's storage).  ON by default: a tensor whose pointer was
 * handed out is uploaded before every use and copied back after every call that writes it, so such callers run
 * unchanged, paying PCIe transfers for those tensors.  Off (this call with 0, or BOAT_HIP_COHERENT_POINTERS=0 in the
 * environment), for callers that fetch the pointer again after each call (as examples/mnist/mnist_autodiff.c does per
 * batch): a data pointer is then good until the next call that takes the tensor, and parameters stay on the device. */
BOAT_API void boat_hip_set_coherent_pointers(int enable);
/* Reference-exact mode (this call, or BOAT_HIP_REFERENCE_EXACT=1 in the environment; off by default).  In three places
 * this library computes something else than the reference on purpose; the mode switches all three to the reference's
 * behaviour at once, for callers that need its numbers:
 *   - boat_variable_backward walks the tape as the reference does (depth first, descending into a non-leaf variable once
 *     per consumer with the gradient accumulated so far, src/autodiff.c:431-450): a non-leaf used twice propagates
 *     twice (z = y + y, y = a*b gives da = 4b).  Default: every op once, the true gradient (2b).
 *   - boat_conv_layer_backward returns the reference's input gradient, which pairs each kernel tap with the mirrored
 *     weight (src/layers/conv.c:86-88).  Default: the gradient of the layer's own forward.
 *     (boat_hip_conv_reference_input_grad, when called, overrides the mode for this one.)
 *   - boat_autodiff_context_disable_grad is stored and ignored, as in the reference (src/autodiff.c:625-632).  Default:
 *     ops run while the current context has gradients off are not recorded. */
BOAT_API void boat_hip_set_reference_exact(int enable);
/* gradient tensor of a variable, created zero-filled if absent and kept across boat_variable_zero_grad
 * (which then zero-fills in place), so it can be registered with an optimizer before the first backward */
BOAT_API boat_tensor_t* boat_hip_variable_ensure_grad(boat_variable_t* variable);
/* GELU with gradient tracking (exact erf form) */
BOAT_API boat_variable_t* boat_hip_var_gelu(const boat_variable_t* a);
/* reshape with gradient tracking (boat_var_flatten generalised to any target shape of equal size), e.g.
 * [batch, seq, hidden] <-> [batch*seq, hidden] between attention (3-D) and dense (2-D) */
BOAT_API boat_variable_t* boat_hip_var_reshape(const boat_variable_t* a, const int64_t* shape, size_t ndim);
/* LayerNorm with gradient tracking; dgamma/dbeta accumulate in the layer */
BOAT_API boat_variable_t* boat_hip_var_layernorm(const boat_variable_t* a, boat_layernorm_t* norm);
BOAT_API boat_tensor_t* boat_hip_layernorm_get_weight(const boat_layernorm_t* norm);
BOAT_API boat_tensor_t* boat_hip_layernorm_get_bias(const boat_layernorm_t* norm);
BOAT_API boat_tensor_t* boat_hip_layernorm_get_grad_weight(const boat_layernorm_t* norm);
BOAT_API boat_tensor_t* boat_hip_layernorm_get_grad_bias(const boat_layernorm_t* norm);
BOAT_API boat_tensor_t* boat_hip_rmsnorm_get_weight(const boat_rmsnorm_t* norm);        /* the reference has no accessor or setter for it */
BOAT_API boat_tensor_t* boat_hip_rmsnorm_get_grad_weight(const boat_rmsnorm_t* norm);
/* fused loss + gradient of the tape chain log_softmax -> mul(onehot) -> sum -> mul(-1/B)
 * (examples/mnist/mnist_autodiff.c:397-522): labels is an INT32 or UINT8 tensor of class indices;
 * returns the [1] loss tensor and, through *dlogits, (softmax(z)-onehot)/B */
BOAT_API boat_tensor_t* boat_hip_softmax_cross_entropy(const boat_tensor_t* logits, const boat_tensor_t* labels, boat_tensor_t** dlogits);
/* mean squared error (src/loss/mse.c:70-78) and its gradient 2(o-t)/n (tests/test_attention_training.c:28-41) */
BOAT_API boat_tensor_t* boat_hip_mse_loss(const boat_tensor_t* pred, const boat_tensor_t* target, boat_tensor_t** grad);
/* ready-made vtables for boat_model_add_layer (the reference ships none; callers write these wrappers,
 * tests/test_model_graph_integration.c:8-77).  The returned boat_layer_t is freed by ops->free. */
BOAT_API boat_layer_t* boat_hip_layer_from_dense(boat_dense_layer_t* layer);
BOAT_API boat_layer_t* boat_hip_layer_from_norm(boat_norm_layer_t* layer);
BOAT_API boat_layer_t* boat_hip_layer_relu(void);
BOAT_API boat_layer_t* boat_hip_layer_gelu(void);
/* register every trainable tensor of a layer with an optimizer */
BOAT_API void boat_hip_optimizer_add_dense(boat_optimizer_t* opt, boat_dense_layer_t* layer);
BOAT_API void boat_hip_optimizer_add_conv(boat_optimizer_t* opt, boat_conv_layer_t* layer);
/* enable > 0: boat_conv_layer_backward returns the reference's input gradient (each tap paired with the mirrored
 * weight, src/layers/conv.c:86-88) instead of the true one; 0: the true one; < 0 (the initial state): whatever
 * reference-exact mode says.  Process-wide. */
BOAT_API void boat_hip_conv_reference_input_grad(int enable);
/* 1: boat_conv_layer_forward runs 3x3 and 5x5 layers that are wide enough to gain from it (at least 8 input and 32 output
 * channels, or at least 32 and 16) on the matrix cores: 1.3x to 6x faster; sums in MFMA order: equal to the reference to
 * fp32 rounding, not bit for bit.  Default 0, or BOAT_HIP_CONV_FORWARD_MFMA. */
BOAT_API void boat_hip_conv_forward_matrix_cores(int enable);
BOAT_API void boat_hip_optimizer_add_attention(boat_optimizer_t* opt, boat_attention_t* attention);
/* An attention layer keeps the scaled scores [batch*heads, seq, seq] of its forward pass for its backward pass (as the
 * reference keeps its attention weights, src/layers/attention.c:424-431) when head_size is 64, seq a multiple of 128 and
 * the matrix is no larger than this many bytes: the backward pass then skips recomputing Q.K^T.  Default 1 GiB, or
 * BOAT_HIP_ATTENTION_SCORE_CACHE; 0 = always recompute (no [seq, seq] matrix is ever stored). */
BOAT_API void boat_hip_set_attention_score_cache_limit(size_t bytes);
BOAT_API void boat_hip_optimizer_add_layernorm(boat_optimizer_t* opt, boat_layernorm_t* norm);

#ifdef __cplusplus
}
#endif
#endif
