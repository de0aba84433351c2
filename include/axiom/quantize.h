/* axiom/quantize.h — per-channel symmetric int8 weights and the quantized GEMMs
 * (include/axiom/quantize.h, src/core/quantize.c).
 *
 * ax_qweight_t is the reference's public struct.  ax_qweight_create_from_fp32 quantizes on
 * the host exactly as the reference does and leaves the result in host memory;
 * ax_qweight_to_device makes a device-resident copy (same struct, device pointers) for the
 * *_dev entry points.  ax_qgemm_w8a32 keeps the reference's host-pointer signature: it stages
 * its operands through the GPU (there is no CPU compute path). */
#ifndef AX_QUANTIZE_H
#define AX_QUANTIZE_H
#include "error.h"
#include "tensor.h"
#include "types.h"
#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    int8_t *data;      /* [N,K] row-major */
    float *scales;     /* [N]: w_fp32[n,k] ~= data[n,k] * scales[n], scale = absmax/127 (1 for a zero row) */
    int64_t N, K;
} ax_qweight_t;

ax_qweight_t *ax_qweight_create_from_fp32(const float *fp32_w, int64_t N, int64_t K);  /* host */
void          ax_qweight_destroy(ax_qweight_t *qw);                                    /* host copy */
void          ax_qweight_dequantize(const ax_qweight_t *qw, float *out_fp32);          /* host */

ax_qweight_t *ax_qweight_to_device(const ax_qweight_t *host_qw, ax_device_t device);
void          ax_qweight_device_destroy(ax_qweight_t *dev_qw, ax_device_t device);

/* out[M,N] = scales[n] * sum_k a[m,k]*q[n,k]; all pointers are HOST memory (reference signature) */
ax_status_t ax_qgemm_w8a32(const float *a, const ax_qweight_t *qw, float *out, int64_t M);
/* the same on device-resident operands (a, out and qw's buffers are device pointers) */
ax_status_t ax_qgemm_w8a32_dev(const float *a, const ax_qweight_t *qw, float *out, int64_t M);
/* W8A8 on device-resident operands: int32-exact accumulators, then
 * out = act((float)acc * (x_scale*scales[n]) + bias[n]).  bias/out/acc_out may be NULL
 * (not both out and acc_out).  act: 0 none, 1 relu, 2 gelu.  No reference counterpart. */
ax_status_t ax_qgemm_w8a8_dev(const int8_t *x, float x_scale, const ax_qweight_t *qw, const float *bias,
                              int act, float *out, int32_t *acc_out, int64_t M);

#ifdef __cplusplus
}
#endif
#endif
