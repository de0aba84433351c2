/* Model container, inference half (Axiom's src/core/model.c:10-24, 89-100, 127-135). */
#include <stdlib.h>

#include "axiom/error.h"
#include "axiom/model.h"

ax_model_t *ax_model_create(ax_layer_t *net) {
    if (!net) {
        ax_err_set(AX_ERR_NULL_ARG, "ax_model_create: net is NULL");
        return NULL;
    }
    ax_model_t *m = calloc(1, sizeof *m);
    if (!m) {
        ax_err_set(AX_ERR_ALLOC, "ax_model_create: out of memory");
        return NULL;
    }
    m->net = net;
    m->n_params = ax_layer_get_params(net, m->params, AX_MODEL_MAX_PARAMS);
    return m;
}

ax_tensor_t *ax_model_predict(ax_model_t *model, ax_tensor_t *input) {
    if (!model) return NULL;
    return ax_layer_forward(model->net, input);
}

void ax_model_destroy(ax_model_t *model) {
    if (!model) return;
    if (model->net) ax_layer_destroy(model->net);
    free(model);
}
