/* axiom/ops.h — tensor-level matmul family and the activations
 * (include/axiom/ops.h, src/core/ops.c:285-440; activations.c).  Each returns a new tensor on
 * the inputs' device (NULL + ax_err on failure).  Inference only: no grad_fn is attached.
 *
 * ax_matmul_bias adds bias[n] to column n.  (The reference passes axis 0 to its bias_add for
 * an [M,N] + [N] add, src/core/ops.c:357, which its backends reject or apply down rows; the
 * intended column-wise add is implemented here, as in the reference's own opt_gemm_relu.) */
#ifndef AX_OPS_H
#define AX_OPS_H
#include "tensor.h"
#ifdef __cplusplus
extern "C" {
#endif
ax_tensor_t *ax_matmul(ax_tensor_t *a, ax_tensor_t *b);                              /* [M,K]x[K,N] */
ax_tensor_t *ax_matmul_bias(ax_tensor_t *a, ax_tensor_t *b, ax_tensor_t *bias);     /* a may be [B,S,K] */
ax_tensor_t *ax_matmul_bias_relu(ax_tensor_t *a, ax_tensor_t *b, ax_tensor_t *bias);
ax_tensor_t *ax_matmul_bias_gelu(ax_tensor_t *a, ax_tensor_t *b, ax_tensor_t *bias); /* not in the reference */
/* Not in the reference: act2(act(a x b + bias) x w2 + bias2) for a second layer of at most 16 outputs, without
 * the wide intermediate, when the active backend takes the shape in one call (a few rows of a); returns NULL
 * with the thread's error status at AX_ERR_NOT_IMPLEMENTED when it does not — the caller then runs the two
 * layers separately — and NULL with another status on a real error.  act, act2: ax_activation_t. */
ax_tensor_t *ax_matmul_bias_act_head(ax_tensor_t *a, ax_tensor_t *b, ax_tensor_t *bias, int act, ax_tensor_t *w2,
                                     ax_tensor_t *bias2, int act2);
ax_tensor_t *ax_relu(ax_tensor_t *a);
ax_tensor_t *ax_gelu(ax_tensor_t *a);                                                /* tanh form */
/* src/core/ops.c:509-537, src/core/activations.c:79,141,363,598 — on the tensor's device */
ax_tensor_t *ax_sigmoid(ax_tensor_t *a);
ax_tensor_t *ax_tanh_op(ax_tensor_t *a);
ax_tensor_t *ax_leaky_relu(ax_tensor_t *a, float alpha);
ax_tensor_t *ax_elu(ax_tensor_t *a, float alpha);
ax_tensor_t *ax_swish(ax_tensor_t *a);
ax_tensor_t *ax_softmax(ax_tensor_t *a, int axis);   /* last axis only (-1 or ndim-1), as the reference */
#ifdef __cplusplus
}
#endif
#endif
