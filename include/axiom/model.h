/* axiom/model.h — the model container, inference half (include/axiom/model.h:45-60,
 * src/core/model.c:10-24,89-100,127-135).  The struct layout is the reference's; opt and loss_fn
 * stay NULL here (training objects are outside this library). */
#ifndef AX_MODEL_H
#define AX_MODEL_H
#include "layer.h"
#ifdef __cplusplus
extern "C" {
#endif

#define AX_MODEL_MAX_PARAMS 256

typedef ax_tensor_t *(*ax_loss_fn_t)(ax_tensor_t *pred, ax_tensor_t *target);

typedef struct {
    ax_layer_t *net;                              /* owned */
    void *opt;                                    /* ax_optimizer_t * in the reference; unused */
    ax_loss_fn_t loss_fn;                         /* unused */
    ax_tensor_t *params[AX_MODEL_MAX_PARAMS];     /* borrowed from the layers */
    int n_params;
} ax_model_t;

ax_model_t  *ax_model_create(ax_layer_t *net);                        /* takes ownership of net */
ax_tensor_t *ax_model_predict(ax_model_t *model, ax_tensor_t *input); /* caller owns the result */
void         ax_model_destroy(ax_model_t *model);

#ifdef __cplusplus
}
#endif
#endif
