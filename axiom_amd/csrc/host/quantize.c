/* int8 weights and the quantized GEMM entry points (Axiom's src/core/quantize.c).
 * Quantization is a one-time host step with the reference's exact arithmetic; the GEMMs run
 * on the GPU through libaxhip — there is no host compute path. */
#include <math.h>
#include <stdlib.h>

#include "axhip.h"
#include "axiom/compute.h"
#include "axiom/internal/backend_ops.h"
#include "axiom/quantize.h"

ax_qweight_t *ax_qweight_create_from_fp32(const float *w, int64_t N, int64_t K) {
    if (!w || N <= 0 || K <= 0) return NULL;
    ax_qweight_t *qw = calloc(1, sizeof *qw);
    if (!qw) return NULL;
    const size_t nk = ((size_t)N * (size_t)K + 63) & ~(size_t)63, ns = ((size_t)N * sizeof(float) + 63) & ~(size_t)63;
    qw->data = aligned_alloc(64, nk);
    qw->scales = aligned_alloc(64, ns);
    if (!qw->data || !qw->scales) {
        free(qw->data);
        free(qw->scales);
        free(qw);
        return NULL;
    }
    qw->N = N;
    qw->K = K;
    for (int64_t n = 0; n < N; n++) {              /* quantize.c:36-54 */
        const float *row = w + n * K;
        float top = 0.0f;
        for (int64_t k = 0; k < K; k++) {
            float m = fabsf(row[k]);
            if (m > top) top = m;
        }
        const float scale = top > 0.0f ? top / 127.0f : 1.0f;
        const float inv = 1.0f / scale;
        qw->scales[n] = scale;
        for (int64_t k = 0; k < K; k++) {
            long v = lrintf(row[k] * inv);         /* round-half-to-even under the default mode */
            if (v > 127) v = 127;
            if (v < -127) v = -127;
            qw->data[n * K + k] = (int8_t)v;
        }
    }
    return qw;
}

void ax_qweight_destroy(ax_qweight_t *qw) {
    if (!qw) return;
    free(qw->data);
    free(qw->scales);
    free(qw);
}

void ax_qweight_dequantize(const ax_qweight_t *qw, float *out) {
    if (!qw || !out) return;
    for (int64_t n = 0; n < qw->N; n++)
        for (int64_t k = 0; k < qw->K; k++) out[n * qw->K + k] = (float)qw->data[n * qw->K + k] * qw->scales[n];
}

ax_qweight_t *ax_qweight_to_device(const ax_qweight_t *h, ax_device_t device) {
    if (!h || !h->data || !h->scales) {
        ax_err_set(AX_ERR_NULL_ARG, "qweight_to_device: NULL");
        return NULL;
    }
    const ax_backend_ops_t *ops = ax_backend_for_device(device);
    if (!ops || !ops->storage_alloc || !ops->memcpy_h2d) {
        ax_err_set(AX_ERR_BACKEND, "no backend registered for device %d", (int)device);
        return NULL;
    }
    ax_qweight_t *d = calloc(1, sizeof *d);
    if (!d) {
        ax_err_set(AX_ERR_ALLOC, "qweight_to_device: out of memory");
        return NULL;
    }
    d->N = h->N;
    d->K = h->K;
    d->data = ops->storage_alloc((size_t)h->N * (size_t)h->K);
    d->scales = ops->storage_alloc((size_t)h->N * sizeof(float));
    if (!d->data || !d->scales ||
        ops->memcpy_h2d(d->data, h->data, (size_t)h->N * (size_t)h->K) != AX_OK ||
        ops->memcpy_h2d(d->scales, h->scales, (size_t)h->N * sizeof(float)) != AX_OK) {
        ax_qweight_device_destroy(d, device);
        return NULL;
    }
    return d;
}

void ax_qweight_device_destroy(ax_qweight_t *d, ax_device_t device) {
    if (!d) return;
    const ax_backend_ops_t *ops = ax_backend_for_device(device);
    if (ops && ops->storage_free) {
        if (d->data) ops->storage_free(d->data);
        if (d->scales) ops->storage_free(d->scales);
    }
    free(d);
}

static ax_status_t lift(int rc, const char *who) {
    if (rc == AXHIP_OK) return AX_OK;
    ax_err_set((ax_status_t)rc, "%s: %s", who, axhip_last_error());
    return (ax_status_t)rc;
}

ax_status_t ax_qgemm_w8a32_dev(const float *a, const ax_qweight_t *qw, float *out, int64_t M) {
    if (!a || !qw || !out) {
        ax_err_set(AX_ERR_NULL_ARG, "qgemm_w8a32: NULL");
        return AX_ERR_NULL_ARG;
    }
    return lift(axhip_qgemm_w8a32(a, qw->data, qw->scales, out, M, qw->N, qw->K), "qgemm_w8a32");
}

ax_status_t ax_qgemm_w8a8_dev(const int8_t *x, float x_scale, const ax_qweight_t *qw, const float *bias, int act,
                              float *out, int32_t *acc_out, int64_t M) {
    if (!x || !qw) {
        ax_err_set(AX_ERR_NULL_ARG, "qgemm_w8a8: NULL");
        return AX_ERR_NULL_ARG;
    }
    return lift(axhip_qgemm_w8a8(x, x_scale, qw->data, qw->scales, bias, act, out, acc_out, M, qw->N, qw->K),
                "qgemm_w8a8");
}

/* Reference signature: every pointer is host memory.  Operands are staged to the GPU, the
 * kernel runs there, the result is copied back (the copy waits for the kernel). */
ax_status_t ax_qgemm_w8a32(const float *a, const ax_qweight_t *qw, float *out, int64_t M) {
    if (!a || !qw || !out) {
        ax_err_set(AX_ERR_NULL_ARG, "qgemm_w8a32: NULL");
        return AX_ERR_NULL_ARG;
    }
    if (M <= 0) return AX_OK;
    ax_status_t st = ax_compute_init();
    if (st != AX_OK) return st;
    const size_t abytes = (size_t)M * (size_t)qw->K * sizeof(float), obytes = (size_t)M * (size_t)qw->N * sizeof(float);
    ax_qweight_t *dq = ax_qweight_to_device(qw, AX_DEVICE_HIP);
    float *da = axhip_malloc(abytes), *dout = axhip_malloc(obytes);
    st = AX_ERR_ALLOC;
    if (dq && da && dout) {
        st = lift(axhip_memcpy_h2d(da, a, abytes), "qgemm_w8a32 upload");
        if (st == AX_OK) st = ax_qgemm_w8a32_dev(da, dq, dout, M);
        if (st == AX_OK) st = lift(axhip_memcpy_d2h(out, dout, obytes), "qgemm_w8a32 download");
    } else {
        ax_err_set(AX_ERR_ALLOC, "qgemm_w8a32: device staging buffers: %s", axhip_last_error());
    }
    axhip_free(da);
    axhip_free(dout);
    ax_qweight_device_destroy(dq, AX_DEVICE_HIP);
    return st;
}
