/* axiom/internal/backend_ops.h — the backend vtable: the drop-in boundary.
 *
 * Slot order, names and signatures reproduce struct ax_backend_ops of Axiom 0.10.0
 * (include/axiom/internal/backend_ops.h:30-298) up to and including memcpy_d2d, so that a
 * pointer to ax_hip_ops can be handed to the reference's ax_compute_register_backend()
 * (src/compute/dispatch.c:302-315) unchanged.  tests/golden/abi_layout.json records the
 * reference's offsets and tests/test_host_core.py compares them with this header.
 * Any slot may be NULL; dispatch answers AX_ERR_NOT_IMPLEMENTED for those.
 *
 * Four slots are appended after the reference's last member (gemm_bias_act, layernorm_fwd,
 * storage_alloc_uninit, gemm_act_head); the reference never reads that far, this repository's host core does. */
#ifndef AX_INTERNAL_BACKEND_OPS_H
#define AX_INTERNAL_BACKEND_OPS_H

#include "axiom/compute.h"
#include "axiom/tensor.h"
#include "axiom/types.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef const ax_tensor_t *ax_tin_t;     /* borrowed input  */
typedef ax_tensor_t *ax_tout_t;          /* borrowed output, pre-allocated by the caller */

struct ax_backend_ops {
    const char *name;

    /* broadcasting binary, unary and scalar elementwise slots */
    ax_status_t (*add)(ax_tin_t a, ax_tin_t b, ax_tout_t out);
    ax_status_t (*sub)(ax_tin_t a, ax_tin_t b, ax_tout_t out);
    ax_status_t (*mul)(ax_tin_t a, ax_tin_t b, ax_tout_t out);
    ax_status_t (*div_op)(ax_tin_t a, ax_tin_t b, ax_tout_t out);
    ax_status_t (*neg)(ax_tin_t in, ax_tout_t out);
    ax_status_t (*abs_op)(ax_tin_t in, ax_tout_t out);
    ax_status_t (*exp_op)(ax_tin_t in, ax_tout_t out);
    ax_status_t (*log_op)(ax_tin_t in, ax_tout_t out);
    ax_status_t (*sqrt_op)(ax_tin_t in, ax_tout_t out);
    ax_status_t (*square)(ax_tin_t in, ax_tout_t out);
    ax_status_t (*add_scalar)(ax_tin_t in, double scalar, ax_tout_t out);
    ax_status_t (*mul_scalar)(ax_tin_t in, double scalar, ax_tout_t out);

    /* GEMM family: out fully overwritten, a/b/out 2-D fp32 */
    ax_status_t (*gemm)(ax_tin_t a, ax_tin_t b, ax_tout_t out);        /* [M,K] x [K,N]   */
    ax_status_t (*gemm_nt)(ax_tin_t a, ax_tin_t b, ax_tout_t out);     /* [M,K] x [N,K]^T */
    ax_status_t (*gemm_tn)(ax_tin_t a, ax_tin_t b, ax_tout_t out);     /* [K,M]^T x [K,N] */

    /* fused attention-training slots — out of scope, NULL in ax_hip_ops */
    ax_status_t (*dwqkv_split_acc)(ax_tin_t x_flat, ax_tin_t dQKV, ax_tout_t dWq, ax_tout_t dWk,
                                   ax_tout_t dWv);
    ax_status_t (*dwqkv_split_acc_hm)(ax_tin_t x_flat, ax_tin_t dQh, ax_tin_t dKh, ax_tin_t dVh,
                                      int64_t B, int64_t S, int64_t H, int64_t dk, ax_tout_t dWq,
                                      ax_tout_t dWk, ax_tout_t dWv);
    ax_status_t (*qkv_head_gemm)(ax_tin_t X, ax_tin_t Wqkv, ax_tin_t bqkv, int64_t B, int64_t S,
                                 int64_t H, int64_t dk, ax_tout_t Qh, ax_tout_t Kh, ax_tout_t Vh);
    ax_status_t (*dattn_head_gemm_nt)(ax_tin_t dout, ax_tin_t Wo, int64_t B, int64_t S, int64_t H,
                                      int64_t dk, ax_tout_t dO_head);
    ax_status_t (*mha_output_proj_fused)(ax_tin_t attn_flat, ax_tin_t Wo, ax_tin_t bo, ax_tin_t dout,
                                         ax_tout_t y, ax_tout_t dattn, ax_tout_t dWo_acc,
                                         ax_tout_t dbo_acc);

    ax_status_t (*gemm_relu)(ax_tin_t a, ax_tin_t b, ax_tin_t bias /* [N] or NULL */, ax_tout_t out);
    ax_status_t (*gemm_ex)(ax_tin_t a, ax_tin_t b, float alpha, float beta, ax_tout_t out);

    ax_status_t (*add_relu)(ax_tin_t a, ax_tin_t b, ax_tout_t out);
    ax_status_t (*axpy)(ax_tin_t x, float alpha, ax_tout_t y);
    ax_status_t (*softmax_rowwise)(ax_tin_t in, ax_tout_t out);
    ax_status_t (*bias_add)(ax_tin_t in, ax_tin_t bias, int axis, ax_tout_t out);
    ax_status_t (*conv_gemm)(ax_tin_t weight, const ax_conv_params_t *params, ax_tout_t out);
    ax_status_t (*conv_gemm_nt_dw)(ax_tin_t grad_out, const ax_conv_params_t *params, ax_tout_t dw);

    ax_status_t (*sum)(ax_tin_t in, int axis, ax_tout_t out);
    ax_status_t (*mean)(ax_tin_t in, int axis, ax_tout_t out);
    ax_status_t (*max_op)(ax_tin_t in, int axis, ax_tout_t out);
    ax_status_t (*min_op)(ax_tin_t in, int axis, ax_tout_t out);
    ax_status_t (*argmax)(ax_tin_t in, int axis, ax_tout_t out);
    ax_status_t (*equal)(ax_tin_t a, ax_tin_t b, ax_tout_t out);
    ax_status_t (*greater)(ax_tin_t a, ax_tin_t b, ax_tout_t out);

    ax_status_t (*fill)(ax_tout_t t, double value);
    ax_status_t (*copy)(ax_tin_t src, ax_tout_t dst);

    ax_status_t (*relu)(ax_tin_t in, ax_tout_t out);
    ax_status_t (*sigmoid)(ax_tin_t in, ax_tout_t out);
    ax_status_t (*tanh_op)(ax_tin_t in, ax_tout_t out);
    ax_status_t (*leaky_relu)(ax_tin_t in, float alpha, ax_tout_t out);
    ax_status_t (*elu_op)(ax_tin_t in, float alpha, ax_tout_t out);
    ax_status_t (*gelu_op)(ax_tin_t in, ax_tout_t out);
    ax_status_t (*swish_op)(ax_tin_t in, ax_tout_t out);

    ax_status_t (*adam_update)(ax_tout_t weight, ax_tout_t grad, ax_tout_t m, ax_tout_t v, float lr,
                               float beta1, float beta2, float eps, float weight_decay, float bc1,
                               float bc2, bool decoupled);
    ax_status_t (*sgd_update)(ax_tout_t weight, ax_tout_t grad, ax_tout_t momentum_buf, float lr,
                              float momentum, float weight_decay, bool nesterov);

    /* device-owner hooks: a backend that owns a non-CPU device fills these */
    ax_device_t device;                         /* AX_DEVICE_COUNT: owns none */
    ax_status_t (*init)(void);
    void (*shutdown)(void);
    void (*synchronize)(void);
    int (*device_count)(void);
    void *(*storage_alloc)(size_t size_bytes);  /* zero-filled, or NULL */
    void (*storage_free)(void *ptr);
    ax_status_t (*memcpy_h2d)(void *dst, const void *src, size_t bytes);
    ax_status_t (*memcpy_d2h)(void *dst, const void *src, size_t bytes);
    ax_status_t (*memcpy_d2d)(void *dst, const void *src, size_t bytes);

    /* ---- appended by this repository (absent from the reference's struct) ---- */
    /* out = act(a x b + bias[n]); bias may be NULL; act is an ax_activation_t */
    ax_status_t (*gemm_bias_act)(ax_tin_t a, ax_tin_t b, ax_tin_t bias, int act, ax_tout_t out);
    /* layer normalisation over the last axis (the loop of layernorm_forward, src/core/norm.c:1338-1399,
     * which the reference runs on host pointers): out = gamma * x_hat + beta; x_hat (shape of x) and
     * inv_std (one value per row) are the tensors its backward pass keeps, either may be NULL */
    ax_status_t (*layernorm_fwd)(ax_tin_t x, ax_tin_t gamma, ax_tin_t beta, float eps, ax_tout_t out,
                                 ax_tout_t x_hat, ax_tout_t inv_std);
    /* storage_alloc without the zero fill, for ax_tensor_create, whose contents are undefined by
     * contract (include/axiom/tensor.h of the reference): an operator's result is overwritten in
     * full, and a fill launch per result is a sizeable share of a bs=1 layer's time */
    void *(*storage_alloc_uninit)(size_t size_bytes);
    /* two Dense layers in one call, the second at most 16 wide (a hidden layer and its classifier head):
     * out2 = act2(act(a x b + bias) x w2 + bias2); the wide intermediate is not materialised.  Biases may be
     * NULL, acts are ax_activation_t.  A backend returns AX_ERR_NOT_IMPLEMENTED for shapes it does not
     * take this way (more than a few rows, a wider second layer); the caller then runs the layers one by one. */
    ax_status_t (*gemm_act_head)(ax_tin_t a, ax_tin_t b, ax_tin_t bias, int act, ax_tin_t w2, ax_tin_t bias2, int act2,
                                 ax_tout_t out2);
};

/* The MI355X backend.  `device` is AX_DEVICE_HIP. */
extern const ax_backend_ops_t ax_hip_ops;

/* The same table with `device` set to `as_device`, for hosts whose device enum has no HIP
 * entry (the unmodified reference: pass its AX_DEVICE_CUDA = 1).  Returns a pointer to
 * static storage, rewritten by each call. */
const ax_backend_ops_t *ax_hip_ops_for_device(ax_device_t as_device);

/* Attention forward on device pointers: same arguments as the sdpa_fwd member of the
 * reference's GPU extension table (include/axiom/internal/cuda_extension.h:86-92).  Q, K, V,
 * out are [BH, S, dk] fp32, L is [BH, S] or NULL; P_save must be NULL. */
ax_status_t ax_hip_sdpa_fwd(const float *Q, const float *K, const float *V, float *out, float *L,
                            int64_t BH, int64_t S, int64_t dk, float scale, bool causal, float *P_save);

#ifdef __cplusplus
}
#endif
#endif
