/* Dense / ReLU / GELU / LayerNorm / Sequential, forward only (Axiom's src/core/layer.c:48-103,
 * 181-300; src/core/norm.c:1278-1455). */
#include <stdio.h>
#include <stdlib.h>

#include "axiom/compute.h"
#include "axiom/error.h"
#include "axiom/init.h"
#include "axiom/layer.h"
#include "axiom/ops.h"

static ax_tensor_t *dense_bias(ax_dense_t *d) { return (d->use_bias && d->bias) ? d->bias : NULL; }

static ax_tensor_t *dense_forward(ax_layer_t *self, ax_tensor_t *x) {
    ax_dense_t *d = (ax_dense_t *)self;
    return ax_matmul_bias(x, d->weight, dense_bias(d));
}

static void dense_destroy(ax_layer_t *self) {
    ax_dense_t *d = (ax_dense_t *)self;
    ax_tensor_destroy(d->weight);
    ax_tensor_destroy(d->bias);
    free(d);
}

/* weight [in,out] Kaiming-uniform with fan_in = in, drawn at creation; bias zeros (layer.c:66-99) */
ax_layer_t *ax_dense_create(int64_t in_features, int64_t out_features, bool use_bias) {
    if (in_features <= 0 || out_features <= 0) {
        ax_err_set(AX_ERR_INVALID_SHAPE, "ax_dense_create: features must be positive");
        return NULL;
    }
    ax_dense_t *d = calloc(1, sizeof *d);
    if (!d) {
        ax_err_set(AX_ERR_ALLOC, "ax_dense_create: out of memory");
        return NULL;
    }
    d->base.ops.forward = dense_forward;
    d->base.ops.destroy = dense_destroy;
    d->base.type = AX_LAYER_DENSE;
    d->base.training = true;
    d->base.input_features = in_features;
    d->base.output_features = out_features;
    d->use_bias = use_bias;
    int64_t wshape[2] = {in_features, out_features};
    d->weight = ax_tensor_create(wshape, 2, AX_FLOAT32);
    if (!d->weight) {
        free(d);
        return NULL;
    }
    ax_init_kaiming_uniform(d->weight, in_features);
    d->weight->requires_grad = true;
    d->base.params[0] = d->weight;
    d->base.n_params = 1;
    if (use_bias) {
        d->bias = ax_tensor_zeros(&out_features, 1, AX_FLOAT32);
        if (!d->bias) {
            ax_tensor_destroy(d->weight);
            free(d);
            return NULL;
        }
        d->bias->requires_grad = true;
        d->base.params[1] = d->bias;
        d->base.n_params = 2;
    }
    return &d->base;
}

static ax_tensor_t *relu_forward(ax_layer_t *self, ax_tensor_t *x) { (void)self; return ax_relu(x); }
static ax_tensor_t *gelu_forward(ax_layer_t *self, ax_tensor_t *x) { (void)self; return ax_gelu(x); }
static ax_tensor_t *sigmoid_forward(ax_layer_t *self, ax_tensor_t *x) { (void)self; return ax_sigmoid(x); }
static ax_tensor_t *tanh_forward(ax_layer_t *self, ax_tensor_t *x) { (void)self; return ax_tanh_op(x); }
static ax_tensor_t *swish_forward(ax_layer_t *self, ax_tensor_t *x) { (void)self; return ax_swish(x); }
static ax_tensor_t *leaky_relu_forward(ax_layer_t *self, ax_tensor_t *x) {
    return ax_leaky_relu(x, ((ax_activation_layer_t *)self)->alpha);
}
static ax_tensor_t *elu_forward(ax_layer_t *self, ax_tensor_t *x) { return ax_elu(x, ((ax_activation_layer_t *)self)->alpha); }
static ax_tensor_t *softmax_forward(ax_layer_t *self, ax_tensor_t *x) {
    return ax_softmax(x, ((ax_activation_layer_t *)self)->axis);
}
static void plain_destroy(ax_layer_t *self) { free(self); }

/* layer.c:136-174 */
static ax_layer_t *activation_layer(ax_layer_type_t type, ax_tensor_t *(*fwd)(ax_layer_t *, ax_tensor_t *)) {
    ax_activation_layer_t *l = calloc(1, sizeof *l);
    if (!l) {
        ax_err_set(AX_ERR_ALLOC, "activation layer: out of memory");
        return NULL;
    }
    l->base.ops.forward = fwd;
    l->base.ops.destroy = plain_destroy;
    l->base.type = type;
    l->base.training = true;
    return &l->base;
}

ax_layer_t *ax_relu_layer_create(void) { return activation_layer(AX_LAYER_RELU, relu_forward); }
ax_layer_t *ax_gelu_layer_create(void) { return activation_layer(AX_LAYER_GELU, gelu_forward); }
ax_layer_t *ax_sigmoid_layer_create(void) { return activation_layer(AX_LAYER_SIGMOID, sigmoid_forward); }
ax_layer_t *ax_tanh_layer_create(void) { return activation_layer(AX_LAYER_TANH, tanh_forward); }
ax_layer_t *ax_swish_layer_create(void) { return activation_layer(AX_LAYER_SWISH, swish_forward); }
ax_layer_t *ax_leaky_relu_layer_create(float alpha) {
    ax_layer_t *l = activation_layer(AX_LAYER_LEAKY_RELU, leaky_relu_forward);
    if (l) ((ax_activation_layer_t *)l)->alpha = alpha;
    return l;
}
ax_layer_t *ax_elu_layer_create(float alpha) {
    ax_layer_t *l = activation_layer(AX_LAYER_ELU, elu_forward);
    if (l) ((ax_activation_layer_t *)l)->alpha = alpha;
    return l;
}
ax_layer_t *ax_softmax_layer_create(int axis) {
    ax_layer_t *l = activation_layer(AX_LAYER_SOFTMAX, softmax_forward);
    if (l) ((ax_activation_layer_t *)l)->axis = axis;
    return l;
}

/* normalises the last axis of a 2-D or 3-D input (norm.c:1281-1298); inference: nothing saved */
static ax_tensor_t *layernorm_forward(ax_layer_t *self, ax_tensor_t *x) {
    ax_layernorm_t *ln = (ax_layernorm_t *)self;
    if (!x || (x->ndim != 2 && x->ndim != 3)) return NULL;
    if (x->shape[x->ndim - 1] != ln->num_features) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "layernorm: last axis is %lld, layer has %lld features",
                   (long long)x->shape[x->ndim - 1], (long long)ln->num_features);
        return NULL;
    }
    ax_device_t prev = ax_get_default_device();
    ax_set_default_device(x->storage->device);
    ax_tensor_t *out = ax_tensor_create(x->shape, x->ndim, x->dtype);
    ax_set_default_device(prev);
    if (!out) return NULL;
    if (ax_compute_layernorm(x, ln->gamma, ln->beta, ln->eps, out, NULL, NULL) != AX_OK) {
        ax_tensor_destroy(out);
        return NULL;
    }
    return out;
}

static void layernorm_destroy(ax_layer_t *self) {
    ax_layernorm_t *ln = (ax_layernorm_t *)self;
    ax_tensor_destroy(ln->gamma);
    ax_tensor_destroy(ln->beta);
    free(ln);
}

ax_layer_t *ax_layernorm_create(int64_t num_features, float eps) {
    if (num_features <= 0) {
        ax_err_set(AX_ERR_INVALID_SHAPE, "ax_layernorm_create: features must be positive");
        return NULL;
    }
    ax_layernorm_t *ln = calloc(1, sizeof *ln);
    if (!ln) {
        ax_err_set(AX_ERR_ALLOC, "ax_layernorm_create: out of memory");
        return NULL;
    }
    ln->base.ops.forward = layernorm_forward;
    ln->base.ops.destroy = layernorm_destroy;
    ln->base.type = AX_LAYER_LAYERNORM;
    ln->base.training = true;
    ln->num_features = num_features;
    ln->eps = eps > 0 ? eps : 1e-5f;
    ln->gamma = ax_tensor_zeros(&num_features, 1, AX_FLOAT32);
    ln->beta = ax_tensor_zeros(&num_features, 1, AX_FLOAT32);
    bool ok = ln->gamma && ln->beta;
    if (ok && ln->gamma->storage->device == AX_DEVICE_CPU) {
        for (int64_t i = 0; i < num_features; i++) ((float *)ln->gamma->storage->data)[i] = 1.0f;
    } else if (ok) {
        ok = ax_compute_fill(ln->gamma, 1.0) == AX_OK;
    }
    if (!ok) {
        layernorm_destroy(&ln->base);
        return NULL;
    }
    ln->gamma->requires_grad = true;
    ln->beta->requires_grad = true;
    ln->base.params[0] = ln->gamma;
    ln->base.params[1] = ln->beta;
    ln->base.n_params = 2;
    ln->base.input_features = ln->base.output_features = num_features;
    return &ln->base;
}

/* the activation a layer type fuses into the Dense before it, or -1 */
static int fused_act_of(ax_layer_type_t t) {
    return t == AX_LAYER_RELU ? AX_ACT_RELU : t == AX_LAYER_GELU ? AX_ACT_GELU : -1;
}

/* Dense [+ ReLU / GELU] followed by a Dense of at most 16 outputs [+ ReLU / GELU], on a few rows: one backend
 * call when the backend has it (ax_matmul_bias_act_head).  Returns the result and sets *consumed to the number
 * of layers it stands for, or NULL with *consumed = 0 when the pattern or the backend does not apply (the
 * caller then goes layer by layer), or NULL with *consumed < 0 on a real error. */
static ax_tensor_t *try_dense_head(ax_sequential_t *seq, int i, ax_tensor_t *x, int *consumed) {
    *consumed = 0;
    if (seq->layers[i]->type != AX_LAYER_DENSE || x->ndim != 2 || x->shape[0] > 16) return NULL;
    int j = i + 1, act = AX_ACT_NONE, act2 = AX_ACT_NONE;
    if (j < seq->n_layers && fused_act_of(seq->layers[j]->type) >= 0) act = fused_act_of(seq->layers[j++]->type);
    if (j >= seq->n_layers || seq->layers[j]->type != AX_LAYER_DENSE || seq->layers[j]->output_features > 16) return NULL;
    ax_dense_t *d1 = (ax_dense_t *)seq->layers[i], *d2 = (ax_dense_t *)seq->layers[j++];
    if (j < seq->n_layers && fused_act_of(seq->layers[j]->type) >= 0) act2 = fused_act_of(seq->layers[j++]->type);
    /* What the backend would decline is declined here, before an output tensor is allocated for nothing: no such
     * operation, or a head whose weight rows are not packed one after the other. */
    const ax_tensor_t *w2 = d2->weight;
    if (!ax_compute_has_gemm_act_head() || !w2 || w2->ndim != 2 || w2->strides[1] != 1 || w2->strides[0] != w2->shape[1])
        return NULL;
    /* a decline must leave the caller's error state as it was */
    const ax_status_t held = ax_err_last_status();
    char held_msg[256];
    snprintf(held_msg, sizeof held_msg, "%s", ax_err_last_message());
    ax_tensor_t *y = ax_matmul_bias_act_head(x, d1->weight, dense_bias(d1), act, d2->weight, dense_bias(d2), act2);
    if (y) {
        *consumed = j - i;
    } else if (ax_err_last_status() != AX_ERR_NOT_IMPLEMENTED) {
        *consumed = -1;
    } else if (held != AX_OK) {                /* not an error: the layers run one by one */
        ax_err_set(held, "%s", held_msg);
    } else {
        ax_err_clear();
    }
    return y;
}

static ax_tensor_t *sequential_forward(ax_layer_t *self, ax_tensor_t *input) {
    ax_sequential_t *seq = (ax_sequential_t *)self;
    ax_tensor_t *x = input, *prev = NULL;
    for (int i = 0; i < seq->n_layers; i++) {
        ax_layer_t *l = seq->layers[i];
        ax_layer_type_t next_type = (i + 1 < seq->n_layers) ? seq->layers[i + 1]->type : AX_LAYER_TYPE_COUNT;
        ax_tensor_t *y;
        int consumed = 0;
        if ((y = try_dense_head(seq, i, x, &consumed)) != NULL || consumed < 0) {
            if (consumed > 0) i += consumed - 1;
        } else if (l->type == AX_LAYER_DENSE && next_type == AX_LAYER_RELU) {
            ax_dense_t *d = (ax_dense_t *)l;
            y = ax_matmul_bias_relu(x, d->weight, dense_bias(d));
            i++;
        } else if (l->type == AX_LAYER_DENSE && next_type == AX_LAYER_GELU) {
            ax_dense_t *d = (ax_dense_t *)l;
            y = ax_matmul_bias_gelu(x, d->weight, dense_bias(d));
            i++;
        } else {
            y = ax_layer_forward(l, x);
        }
        if (prev) ax_tensor_destroy(prev);      /* inference: nobody else holds the intermediate */
        if (!y) return NULL;
        prev = x = y;
    }
    return x;
}

static void sequential_destroy(ax_layer_t *self) {
    ax_sequential_t *seq = (ax_sequential_t *)self;
    for (int i = 0; i < seq->n_layers; i++) ax_layer_destroy(seq->layers[i]);
    free(seq);
}

ax_layer_t *ax_sequential_create(void) {
    ax_sequential_t *seq = calloc(1, sizeof *seq);
    if (!seq) {
        ax_err_set(AX_ERR_ALLOC, "ax_sequential_create: out of memory");
        return NULL;
    }
    seq->base.ops.forward = sequential_forward;
    seq->base.ops.destroy = sequential_destroy;
    seq->base.type = AX_LAYER_SEQUENTIAL;
    seq->base.training = true;
    return &seq->base;
}

ax_layer_t *ax_sequential_add(ax_layer_t *seq_base, ax_layer_t *layer) {
    ax_sequential_t *seq = (ax_sequential_t *)seq_base;
    if (!seq || !layer || seq->base.type != AX_LAYER_SEQUENTIAL || seq->n_layers >= AX_SEQ_MAX_LAYERS) return NULL;
    seq->layers[seq->n_layers++] = layer;
    return seq_base;
}

ax_tensor_t *ax_layer_forward(ax_layer_t *layer, ax_tensor_t *input) {
    if (!layer || !layer->ops.forward) return NULL;
    return layer->ops.forward(layer, input);
}

int ax_layer_get_params(ax_layer_t *layer, ax_tensor_t **params, int max_params) {
    if (!layer) return 0;
    int count = 0;
    if (layer->type == AX_LAYER_SEQUENTIAL) {
        ax_sequential_t *seq = (ax_sequential_t *)layer;
        for (int i = 0; i < seq->n_layers && count < max_params; i++)
            count += ax_layer_get_params(seq->layers[i], params + count, max_params - count);
        return count;
    }
    for (int i = 0; i < layer->n_params && count < max_params; i++) params[count++] = layer->params[i];
    return count;
}

void ax_layer_destroy(ax_layer_t *layer) {
    if (layer && layer->ops.destroy) layer->ops.destroy(layer);
}
