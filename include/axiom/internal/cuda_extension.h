/* axiom/internal/cuda_extension.h — the GPU extension table: device-side operations that do not
 * fit the backend vtable (layout transforms around attention, fused-projection caches, attention
 * forward/backward, batched convolution).
 *
 * Member order, names and signatures reproduce `ax_cuda_extension_t` of Axiom 0.10.0
 * (include/axiom/internal/cuda_extension.h:41-140) — the name is the reference's; nothing in the
 * table is specific to one vendor — so that &ax_hip_extension can be handed to the reference's
 * ax_compute_register_cuda_extension() (src/compute/dispatch.c:290-300) unchanged: its MHA layer
 * (src/core/attention.c:121-430, src/core/attention/cache.c:24-85) then runs its forward pass on
 * the device.  Members may be NULL; callers test before dispatching. */
#ifndef AX_INTERNAL_CUDA_EXTENSION_H
#define AX_INTERNAL_CUDA_EXTENSION_H
#include "axiom/compute.h"
#include "axiom/types.h"
#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    /* qkv [B*S, 3D] -> q, k, v each [B*H, S, dk]; the _bias form adds bqkv [3D] = [bq | bk | bv] */
    void (*head_interleave_qkv_split)(const float *src, float *q, float *k, float *v, int64_t B, int64_t S,
                                      int64_t H, int64_t dk, int64_t D);
    void (*head_interleave_qkv_split_bias)(const float *src, const float *bqkv, float *q, float *k, float *v,
                                           int64_t B, int64_t S, int64_t H, int64_t dk, int64_t D);
    /* [B, S, H, dk] -> [B*H, S, dk] and its inverse */
    void (*head_interleave)(const float *src, float *dst, int64_t B, int64_t S, int64_t H, int64_t dk);
    void (*head_deinterleave)(const float *src, float *dst, int64_t B, int64_t S, int64_t H, int64_t dk);
    /* backward of the split — not provided by ax_hip_extension */
    void (*head_deinterleave_qkv_merge)(const float *dQ, const float *dK, const float *dV, float *dst, int64_t B,
                                        int64_t S, int64_t H, int64_t dk, int64_t D);
    /* fused [D, 3D] weight panel and [3D] bias from the three projections */
    ax_status_t (*qkv_cache_build)(float *dst, const float *wq, const float *wk, const float *wv, int64_t D);
    ax_status_t (*bias_cache_build)(float *dst, const float *bq, const float *bk, const float *bv, int64_t D);
    /* attention forward: out [BH, S, dk], L [BH, S] log-sum-exp; P_save must be NULL here */
    ax_status_t (*sdpa_fwd)(const float *Q, const float *K, const float *V, float *out, float *L, int64_t BH,
                            int64_t S, int64_t dk, float scale, bool causal, float *P_save);
    /* not provided by ax_hip_extension: attention backward and the convolution entries */
    ax_status_t (*sdpa_bwd)(const float *Q, const float *K, const float *V, const float *O, const float *dO,
                            const float *L, float *dQ, float *dK, float *dV, int64_t BH, int64_t S, int64_t dk,
                            float scale, bool causal, const float *P_saved);
    ax_status_t (*conv_gemm_batched)(const ax_tensor_t *weight, const float *in_dev, int64_t N,
                                     const ax_conv_params_t *single, ax_tensor_t *out);
    ax_status_t (*conv_winograd_f23)(const ax_tensor_t *weight, const float *in_dev, int64_t N,
                                     const ax_conv_params_t *single, ax_tensor_t *out);
    bool (*winograd_f23_prefer)(int64_t C_in, int64_t C_out, int64_t H, int64_t W);
    /* Appended after the reference's last member (only tables built against this header carry it):
     * attention straight on the fused projection.  Head (b, h) is the block of rows b*S.., columns
     * h*dk.. of Q, K, V (row pitch ld floats) and of out (pitch ldo), so qkv [B*S, 3D] goes in as
     * (qkv, qkv + D, qkv + 2D, ld = 3D) and out [B*S, D] comes back ready for the output
     * projection, with no split / interleave pass.  AX_ERR_NOT_IMPLEMENTED for a head size it
     * does not cover: the caller then takes the split path. */
    ax_status_t (*sdpa_fwd_rows)(const float *Q, const float *K, const float *V, int64_t ld, float *out,
                                 int64_t ldo, float *L, int64_t B, int64_t H, int64_t S, int64_t dk, float scale,
                                 bool causal);
} ax_cuda_extension_t;

/* The MI355X table: the layout transforms, both cache builders and sdpa_fwd are filled. */
extern const ax_cuda_extension_t ax_hip_extension;

ax_status_t ax_compute_register_cuda_extension(const ax_cuda_extension_t *ext);   /* NULL clears it */
const ax_cuda_extension_t *ax_compute_get_cuda_extension(void);

#ifdef __cplusplus
}
#endif
#endif
