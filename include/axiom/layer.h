/* axiom/layer.h — Dense, ReLU, GELU, LayerNorm and Sequential, forward only
 * (include/axiom/layer.h:30-187, src/core/layer.c; include/axiom/norm.h:33-44, src/core/norm.c).  Struct layouts and enum values follow the reference.  Sequential fuses
 * Dense+ReLU as the reference does (layer.c:188-230) and additionally Dense+GELU; in both
 * cases intermediates are released as soon as the next layer has consumed them. */
#ifndef AX_LAYER_H
#define AX_LAYER_H
#include "tensor.h"
#ifdef __cplusplus
extern "C" {
#endif

#define AX_LAYER_MAX_PARAMS 8
#define AX_LAYER_MAX_BUFFERS 4
#define AX_SEQ_MAX_LAYERS 64

typedef enum {
    AX_LAYER_DENSE = 0, AX_LAYER_RELU, AX_LAYER_SIGMOID, AX_LAYER_TANH, AX_LAYER_LEAKY_RELU,
    AX_LAYER_ELU, AX_LAYER_GELU, AX_LAYER_SWISH, AX_LAYER_SOFTMAX, AX_LAYER_CONV2D,
    AX_LAYER_MAXPOOL2D, AX_LAYER_AVGPOOL2D, AX_LAYER_GLOBAL_AVGPOOL2D, AX_LAYER_FLATTEN,
    AX_LAYER_BATCHNORM, AX_LAYER_LAYERNORM, AX_LAYER_DROPOUT, AX_LAYER_SEQUENTIAL,
    AX_LAYER_CONV_BN_RELU, AX_LAYER_MHA, AX_LAYER_TYPE_COUNT
} ax_layer_type_t;

typedef struct ax_layer ax_layer_t;

typedef struct {
    ax_tensor_t *(*forward)(ax_layer_t *self, ax_tensor_t *input);
    void (*destroy)(ax_layer_t *self);
} ax_layer_ops_t;

struct ax_layer {
    ax_layer_ops_t ops;
    ax_layer_type_t type;
    bool training;
    ax_tensor_t *params[AX_LAYER_MAX_PARAMS];
    int n_params;
    ax_tensor_t *buffers[AX_LAYER_MAX_BUFFERS];
    int n_buffers;
    int64_t input_features, output_features;
};

typedef struct {
    ax_layer_t base;
    ax_tensor_t *weight;     /* [in, out] row-major: forward is x[M,in] * weight */
    ax_tensor_t *bias;       /* [out], zeros at creation; NULL without bias */
    bool use_bias;
} ax_dense_t;

typedef struct {
    ax_layer_t base;
    ax_layer_t *layers[AX_SEQ_MAX_LAYERS];
    int n_layers;
} ax_sequential_t;

/* include/axiom/norm.h:36-42: gamma ones, beta zeros at creation; eps <= 0 means 1e-5 */
typedef struct {
    ax_layer_t base;
    int64_t num_features;
    float eps;
    ax_tensor_t *gamma;
    ax_tensor_t *beta;
} ax_layernorm_t;

ax_layer_t  *ax_layernorm_create(int64_t num_features, float eps);   /* input [N, D] or [B, S, D] */
ax_layer_t  *ax_dense_create(int64_t in_features, int64_t out_features, bool use_bias);
/* include/axiom/layer.h:120-141: stateless activation layers; the struct is public so that the
 * model file code can reach alpha / axis */
typedef struct {
    ax_layer_t base;
    float alpha;             /* leaky relu, elu */
    int axis;                /* softmax */
} ax_activation_layer_t;

ax_layer_t  *ax_relu_layer_create(void);
ax_layer_t  *ax_sigmoid_layer_create(void);
ax_layer_t  *ax_tanh_layer_create(void);
ax_layer_t  *ax_leaky_relu_layer_create(float alpha);
ax_layer_t  *ax_elu_layer_create(float alpha);
ax_layer_t  *ax_gelu_layer_create(void);
ax_layer_t  *ax_swish_layer_create(void);
ax_layer_t  *ax_softmax_layer_create(int axis);
ax_layer_t  *ax_sequential_create(void);
ax_layer_t  *ax_sequential_add(ax_layer_t *seq, ax_layer_t *layer);   /* NULL when full */
ax_tensor_t *ax_layer_forward(ax_layer_t *layer, ax_tensor_t *input);
int          ax_layer_get_params(ax_layer_t *layer, ax_tensor_t **params, int max_params);
void         ax_layer_destroy(ax_layer_t *layer);

#ifdef __cplusplus
}
#endif
#endif
