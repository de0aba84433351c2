/* axiom/compute.h — backend selection and the ax_compute_* dispatch wrappers of the GEMM path
 * (include/axiom/compute.h:46-317, src/compute/dispatch.c).  Every wrapper initialises the
 * compute layer on first use, returns AX_ERR_BACKEND when no backend is active and
 * AX_ERR_NOT_IMPLEMENTED when the active backend leaves the slot NULL, and bumps
 * out->storage->generation on success. */
#ifndef AX_COMPUTE_H
#define AX_COMPUTE_H

#include "types.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ax_backend_ops ax_backend_ops_t;   /* layout: axiom/internal/backend_ops.h */
typedef struct ax_tensor ax_tensor_t;

typedef struct {            /* conv_gemm slot argument; unused here, kept for the vtable's types */
    const float *input;
    int64_t C_in, H, W;
    int kh, kw, sh, sw, ph, pw;
    int64_t out_h, out_w;
} ax_conv_params_t;

typedef enum {
    AX_BACKEND_CPU_NAIVE = 0,   /* ids kept for numeric compatibility; this build registers */
    AX_BACKEND_CPU_SIMD,        /* no CPU backend: there is no CPU compute path             */
    AX_BACKEND_CPU_BLAS,
    AX_BACKEND_CUDA,
    AX_BACKEND_HIP,             /* ax_hip_ops */
    AX_BACKEND_COUNT
} ax_backend_id_t;

/* fused-epilogue selector of the appended gemm_bias_act slot */
typedef enum { AX_ACT_NONE = 0, AX_ACT_RELU = 1, AX_ACT_GELU = 2 } ax_activation_t;

ax_status_t     ax_compute_init(void);        /* registers ax_hip_ops, fires its init hook, selects it */
void            ax_compute_shutdown(void);
ax_status_t     ax_compute_set_backend(ax_backend_id_t id);
ax_backend_id_t ax_compute_get_backend(void);
const char     *ax_compute_backend_name(void);
ax_status_t     ax_compute_register_backend(ax_backend_id_t id, const ax_backend_ops_t *ops);
const ax_backend_ops_t *ax_compute_get_ops(void);
const ax_backend_ops_t *ax_backend_for_device(ax_device_t device);

ax_status_t ax_compute_gemm(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out);
ax_status_t ax_compute_gemm_nt(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out);
ax_status_t ax_compute_gemm_tn(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out);
ax_status_t ax_compute_gemm_relu(const ax_tensor_t *a, const ax_tensor_t *b, const ax_tensor_t *bias, ax_tensor_t *out);
ax_status_t ax_compute_gemm_ex(const ax_tensor_t *a, const ax_tensor_t *b, float alpha, float beta, ax_tensor_t *out);
ax_status_t ax_compute_bias_add(const ax_tensor_t *in, const ax_tensor_t *bias, int axis, ax_tensor_t *out);
ax_status_t ax_compute_relu(const ax_tensor_t *in, ax_tensor_t *out);
ax_status_t ax_compute_fill(ax_tensor_t *t, double value);
ax_status_t ax_compute_copy(const ax_tensor_t *src, ax_tensor_t *dst);
/* Reduction and accumulation the dense layer's backward pass is made of
 * (src/core/autograd_ops.c:603-757): dA = gemm_nt(dY, W), dW = gemm_tn(X, dY),
 * dBias = sum(dY, 0), and axpy to add into a gradient that already exists. */
ax_status_t ax_compute_sum(const ax_tensor_t *in, int axis, ax_tensor_t *out);
ax_status_t ax_compute_axpy(const ax_tensor_t *x, float alpha, ax_tensor_t *y);
/* The remaining elementwise, reduction and optimizer wrappers (src/compute/dispatch.c:385-412,
 * 657-721, 762-841; include/axiom/compute.h of the reference).  Binary ops broadcast (trailing
 * dimensions aligned, extent 1 repeats); reductions take axis -1 for "everything" and want the
 * output to hold numel(in) / shape[axis] elements; argmax writes int64. */
ax_status_t ax_compute_add(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out);
ax_status_t ax_compute_sub(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out);
ax_status_t ax_compute_mul(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out);
ax_status_t ax_compute_div(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out);
ax_status_t ax_compute_equal(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out);
ax_status_t ax_compute_greater(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out);
ax_status_t ax_compute_add_relu(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out);
ax_status_t ax_compute_neg(const ax_tensor_t *in, ax_tensor_t *out);
ax_status_t ax_compute_abs(const ax_tensor_t *in, ax_tensor_t *out);
ax_status_t ax_compute_exp(const ax_tensor_t *in, ax_tensor_t *out);
ax_status_t ax_compute_log(const ax_tensor_t *in, ax_tensor_t *out);
ax_status_t ax_compute_sqrt(const ax_tensor_t *in, ax_tensor_t *out);
ax_status_t ax_compute_square(const ax_tensor_t *in, ax_tensor_t *out);
ax_status_t ax_compute_sigmoid(const ax_tensor_t *in, ax_tensor_t *out);
ax_status_t ax_compute_tanh(const ax_tensor_t *in, ax_tensor_t *out);
ax_status_t ax_compute_add_scalar(const ax_tensor_t *in, double scalar, ax_tensor_t *out);
ax_status_t ax_compute_mul_scalar(const ax_tensor_t *in, double scalar, ax_tensor_t *out);
ax_status_t ax_compute_softmax_rowwise(const ax_tensor_t *in, ax_tensor_t *out);
ax_status_t ax_compute_mean(const ax_tensor_t *in, int axis, ax_tensor_t *out);
ax_status_t ax_compute_max(const ax_tensor_t *in, int axis, ax_tensor_t *out);
ax_status_t ax_compute_min(const ax_tensor_t *in, int axis, ax_tensor_t *out);
ax_status_t ax_compute_argmax(const ax_tensor_t *in, int axis, ax_tensor_t *out);
ax_status_t ax_compute_adam_update(ax_tensor_t *weight, ax_tensor_t *grad, ax_tensor_t *m, ax_tensor_t *v, float lr,
                                   float beta1, float beta2, float eps, float weight_decay, float bc1, float bc2,
                                   bool decoupled);
ax_status_t ax_compute_sgd_update(ax_tensor_t *weight, ax_tensor_t *grad, ax_tensor_t *momentum_buf, float lr,
                                  float momentum, float weight_decay, bool nesterov);
int ax_compute_has_adam_update(void);
int ax_compute_has_sgd_update(void);
int ax_compute_has_gemm_relu(void);
int ax_compute_has_gemm_nt(void);
int ax_compute_has_gemm_tn(void);
int ax_compute_has_gemm_ex(void);
int ax_compute_has_bias_add(void);

/* Not in the reference: its vtable has a gelu_op slot but no wrapper reaches it
 * (src/core/activations.c:267 always runs on the host pointer), and it has no fused
 * bias+activation GEMM beyond gemm_relu. */
ax_status_t ax_compute_gelu(const ax_tensor_t *in, ax_tensor_t *out);
ax_status_t ax_compute_gemm_bias_act(const ax_tensor_t *a, const ax_tensor_t *b, const ax_tensor_t *bias,
                                     ax_activation_t act, ax_tensor_t *out);
int ax_compute_has_gemm_bias_act(void);
/* Not in the reference: two Dense layers, the second at most 16 wide, in one backend call (the appended
 * gemm_act_head slot).  AX_ERR_NOT_IMPLEMENTED when the backend has no such slot or does not take the shape. */
ax_status_t ax_compute_gemm_act_head(const ax_tensor_t *a, const ax_tensor_t *b, const ax_tensor_t *bias, ax_activation_t act,
                                     const ax_tensor_t *w2, const ax_tensor_t *bias2, ax_activation_t act2, ax_tensor_t *out2);
int ax_compute_has_gemm_act_head(void);
/* The reference's vtable has leaky_relu / elu_op / swish_op slots (filled by its GPU backend,
 * cuda/ops_activations.cu) but no dispatch wrapper: ax_leaky_relu, ax_elu, ax_swish
 * (src/core/activations.c:79,141,363) loop over host pointers. */
ax_status_t ax_compute_leaky_relu(const ax_tensor_t *in, float alpha, ax_tensor_t *out);
ax_status_t ax_compute_elu(const ax_tensor_t *in, float alpha, ax_tensor_t *out);
ax_status_t ax_compute_swish(const ax_tensor_t *in, ax_tensor_t *out);
/* Layer normalisation over the last axis, the device form of the loop in layernorm_forward
 * (src/core/norm.c:1338-1399); x_hat and inv_std (saved for backward) may be NULL. */
ax_status_t ax_compute_layernorm(const ax_tensor_t *x, const ax_tensor_t *gamma, const ax_tensor_t *beta, float eps,
                                 ax_tensor_t *out, ax_tensor_t *x_hat, ax_tensor_t *inv_std);

#ifdef __cplusplus
}
#endif
#endif
