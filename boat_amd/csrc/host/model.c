/* model.c - sequential layer container with a working backward and update.
 *
 * Container API of include/boat/model.h:17-65.  boat_model_forward walks the layers in order as the
 * sequential branch of src/model/model.c:148-179 does; boat_model_backward and boat_model_update are
 * stubs in the reference (model.c:354-365) and are implemented here as the loop the layer vtable
 * implies: g = layers[i]->ops->backward(layers[i], g) for i = n-1..0, intermediates released.
 * The graph bookkeeping the reference adds per layer (model.c:406-460) has no effect on results
 * and is not reproduced.
 */
#include "boat_internal.h"

#include <stdlib.h>

struct boat_model_t {
    boat_layer_t** layers;
    size_t layer_count, layer_capacity;
    boat_graph_t* graph;   /* the layers as a chain of nodes, for callers that look at boat_model_graph() */
    void* user_data;                  /* model.c:382-397: carried for the caller, released with the model */
    void (*free_user_data)(void*);
};

boat_model_t* boat_model_create(void) {
    boat_model_t* model = (boat_model_t*)calloc(1, sizeof(boat_model_t));
    if (model) model->graph = boat_graph_create();
    return model;
}
/* model.c:59-83: the model takes the graph over (it is freed with the model) */
boat_model_t* boat_model_create_with_graph(const boat_graph_t* graph) {
    if (!graph) return NULL;
    boat_model_t* model = (boat_model_t*)calloc(1, sizeof(boat_model_t));
    if (model) model->graph = (boat_graph_t*)graph;
    return model;
}
void boat_model_set_graph(boat_model_t* model, boat_graph_t* graph) {   /* model.c:133-145 */
    if (!model || !graph) return;
    if (model->graph && model->graph != graph) boat_graph_free(model->graph);
    model->graph = graph;
}
void* boat_model_get_user_data(const boat_model_t* model) { return model ? model->user_data : NULL; }
void boat_model_set_user_data(boat_model_t* model, void* user_data, void (*free_fn)(void*)) {
    if (!model) return;
    if (model->user_data && model->free_user_data) model->free_user_data(model->user_data);
    model->user_data = user_data;
    model->free_user_data = free_fn;
}
/* no file format exists for a model in the reference: both are stubs there too (model.c:368-379) */
boat_model_t* boat_model_load(const char* filename) {
    (void)filename;
    return NULL;
}
bool boat_model_save(const boat_model_t* model, const char* filename) {
    (void)model;
    (void)filename;
    return false;
}
boat_graph_t* boat_model_graph(const boat_model_t* model) { return model ? model->graph : NULL; }
size_t boat_graph_node_count(const boat_graph_t* graph) { return graph ? graph->node_count : 0; }
size_t boat_graph_edge_count(const boat_graph_t* graph) { return graph && graph->node_count > 1 ? graph->node_count - 1 : 0; }
boat_node_t* boat_graph_get_node_at_index(const boat_graph_t* graph, size_t index) {
    return graph && index < graph->node_count ? &graph->nodes[index] : NULL;
}
void* boat_node_data(const boat_node_t* node) { return node ? node->data : NULL; }
boat_node_type_t boat_node_type(const boat_node_t* node) { return node ? node->type : BOAT_NODE_TYPE_VARIABLE; }
const char* boat_node_type_name(boat_node_type_t type) {   /* src/graph/node.c:289-298 */
    switch (type) {
        case BOAT_NODE_TYPE_VARIABLE: return "VARIABLE";
        case BOAT_NODE_TYPE_OPERATION: return "OPERATION";
        case BOAT_NODE_TYPE_CONSTANT: return "CONSTANT";
        case BOAT_NODE_TYPE_PLACEHOLDER: return "PLACEHOLDER";
        case BOAT_NODE_TYPE_OUTPUT: return "OUTPUT";
        default: return "UNKNOWN";
    }
}
boat_sequential_model_t* boat_sequential_create(void) { return boat_model_create(); }

void boat_model_free(boat_model_t* model) {
    if (!model) return;
    for (size_t i = 0; i < model->layer_count; i++) {
        boat_layer_t* l = model->layers[i];
        if (l && l->ops && l->ops->free) l->ops->free(l);
    }
    free(model->layers);
    boat_graph_free(model->graph);
    if (model->user_data && model->free_user_data) model->free_user_data(model->user_data);
    free(model);
}

void boat_model_add_layer(boat_model_t* model, boat_layer_t* layer) {
    if (!model || !layer) return;
    if (model->layer_count >= model->layer_capacity) {
        size_t cap = model->layer_capacity ? model->layer_capacity * 2 : 4;
        boat_layer_t** grown = (boat_layer_t**)realloc(model->layers, cap * sizeof(*grown));
        if (!grown) {
            fprintf(stderr, "Failed to expand layers array\n");
            return;
        }
        model->layers = grown;
        model->layer_capacity = cap;
    }
    model->layers[model->layer_count++] = layer;
    boat_graph_t* g = model->graph;
    if (g) {   /* model.c:434-455: one operation node per layer, linked to the one before */
        if (g->node_count == g->node_capacity) {
            const size_t cap = g->node_capacity ? 2 * g->node_capacity : 8;
            struct boat_node_t* grown = (struct boat_node_t*)realloc(g->nodes, cap * sizeof(*grown));
            if (!grown) return;
            g->nodes = grown;
            g->node_capacity = cap;
        }
        g->nodes[g->node_count].data = layer;
        g->nodes[g->node_count].type = BOAT_NODE_TYPE_OPERATION;
        g->node_count++;
    }
}
void boat_sequential_add(boat_sequential_model_t* model, boat_layer_t* layer) { boat_model_add_layer(model, layer); }
size_t boat_model_layer_count(const boat_model_t* model) { return model ? model->layer_count : 0; }

boat_tensor_t* boat_model_forward(const boat_model_t* model, const boat_tensor_t* input) {
    if (!model || !input || model->layer_count == 0) return NULL;
    boat_tensor_t* current = NULL;
    for (size_t i = 0; i < model->layer_count; i++) {
        const boat_layer_t* l = model->layers[i];
        if (!l || !l->ops || !l->ops->forward) {
            boat_tensor_free(current);
            return NULL;
        }
        boat_tensor_t* next = l->ops->forward(l, current ? current : input);
        boat_tensor_free(current);
        if (!next) return NULL;
        current = next;
    }
    return current;
}

boat_tensor_t* boat_model_backward(const boat_model_t* model, const boat_tensor_t* grad_output) {
    if (!model || !grad_output || model->layer_count == 0) return NULL;
    boat_tensor_t* current = NULL;
    for (size_t i = model->layer_count; i-- > 0;) {
        const boat_layer_t* l = model->layers[i];
        if (!l || !l->ops || !l->ops->backward) {
            boat_tensor_free(current);
            return NULL;
        }
        boat_tensor_t* next = l->ops->backward(l, current ? current : grad_output);
        boat_tensor_free(current);
        if (!next) return NULL;
        current = next;
    }
    return current;
}

void boat_model_update(const boat_model_t* model, float learning_rate) {
    if (!model) return;
    for (size_t i = 0; i < model->layer_count; i++) {
        const boat_layer_t* l = model->layers[i];
        if (l && l->ops && l->ops->update) l->ops->update(l, learning_rate);
    }
}

/* ---- ready-made vtables (callers of the reference write these by hand,
 *      tests/test_model_graph_integration.c:8-77) ---- */

static boat_layer_t* wrap(void* data, const boat_layer_ops_t* ops) {
    boat_layer_t* l = (boat_layer_t*)calloc(1, sizeof(*l));
    if (!l) return NULL;
    l->data = data;
    l->ops = ops;
    return l;
}

static boat_tensor_t* dense_fwd(const boat_layer_t* l, const boat_tensor_t* x) { return boat_dense_layer_forward((boat_dense_layer_t*)l->data, x); }
static boat_tensor_t* dense_bwd(const boat_layer_t* l, const boat_tensor_t* g) { return boat_dense_layer_backward((boat_dense_layer_t*)l->data, g); }
static void dense_upd(const boat_layer_t* l, float lr) { boat_dense_layer_update((boat_dense_layer_t*)l->data, lr); }
static void dense_free(const boat_layer_t* l) {
    boat_dense_layer_free((boat_dense_layer_t*)l->data);
    free((void*)l);
}
static const boat_layer_ops_t dense_ops = {dense_fwd, dense_bwd, dense_upd, dense_free};
boat_layer_t* boat_hip_layer_from_dense(boat_dense_layer_t* layer) { return layer ? wrap(layer, &dense_ops) : NULL; }

static boat_tensor_t* norm_fwd(const boat_layer_t* l, const boat_tensor_t* x) { return boat_norm_layer_forward((boat_norm_layer_t*)l->data, x); }
static boat_tensor_t* norm_bwd(const boat_layer_t* l, const boat_tensor_t* g) { return boat_norm_layer_backward((boat_norm_layer_t*)l->data, g); }
static void norm_upd(const boat_layer_t* l, float lr) { boat_norm_layer_update((boat_norm_layer_t*)l->data, lr); }
static void norm_free(const boat_layer_t* l) {
    boat_norm_layer_free((boat_norm_layer_t*)l->data);
    free((void*)l);
}
static const boat_layer_ops_t norm_ops = {norm_fwd, norm_bwd, norm_upd, norm_free};
boat_layer_t* boat_hip_layer_from_norm(boat_norm_layer_t* layer) { return layer ? wrap(layer, &norm_ops) : NULL; }

/* activation layers that cache their input so backward applies the true mask / derivative
 * (the reference's boat_relu_layer_backward has no cache and passes the gradient through) */
typedef struct { int act; boat_tensor_t* cache_input; } act_layer_t;
static boat_tensor_t* act_fwd(const boat_layer_t* l, const boat_tensor_t* x) {
    act_layer_t* a = (act_layer_t*)l->data;
    boat_tensor_ref((boat_tensor_t*)x);
    boat_tensor_free(a->cache_input);
    a->cache_input = (boat_tensor_t*)x;
    return a->act == BH_ACT_RELU ? boat_relu(x) : boat_gelu(x);
}
static boat_tensor_t* act_bwd(const boat_layer_t* l, const boat_tensor_t* g) {
    act_layer_t* a = (act_layer_t*)l->data;
    if (!a->cache_input || !g || a->cache_input->nelements != g->nelements) return NULL;
    boat_tensor_t* dx = bt_new_like_uninit(a->cache_input);
    const float* px = bt_dev_read(a->cache_input);
    const float* pg = bt_dev_read(g);
    float* pd = dx ? bt_dev_write(dx) : NULL;
    if (!px || !pg || !pd || !boat_hip_ok(bh_activation_backward(a->act, px, pg, pd, (int64_t)g->nelements, 0), "activation layer backward")) {
        boat_tensor_free(dx);
        return NULL;
    }
    return dx;
}
static void act_upd(const boat_layer_t* l, float lr) {
    (void)l;
    (void)lr;
}
static void act_free(const boat_layer_t* l) {
    act_layer_t* a = (act_layer_t*)l->data;
    boat_tensor_free(a->cache_input);
    free(a);
    free((void*)l);
}
static const boat_layer_ops_t act_ops = {act_fwd, act_bwd, act_upd, act_free};
static boat_layer_t* act_layer(int act) {
    act_layer_t* a = (act_layer_t*)calloc(1, sizeof(*a));
    if (!a) return NULL;
    a->act = act;
    boat_layer_t* l = wrap(a, &act_ops);
    if (!l) free(a);
    return l;
}
boat_layer_t* boat_hip_layer_relu(void) { return act_layer(BH_ACT_RELU); }
boat_layer_t* boat_hip_layer_gelu(void) { return act_layer(BH_ACT_GELU); }
