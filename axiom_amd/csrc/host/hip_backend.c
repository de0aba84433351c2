/* ax_hip_ops — the MI355X backend object behind Axiom's vtable.
 *
 * Plain C: it unpacks ax_tensor_t (shape, strides, offset, device) into pointers and sizes and
 * calls the C ABI of libaxhip.so; no HIP header is included here.  It takes the place of
 * ax_cuda_ops (src/compute/backends/cuda/backend.cu:140-192) for the GEMM family, bias_add,
 * relu, gelu_op, fill, copy and the ten device-owner hooks; every other slot stays NULL.
 * Operands are borrowed, never retained.  Errors follow the reference's backend convention
 * (cuda/ops_gemm.cu:16-23): dtype != f32 -> AX_ERR_DTYPE_MISMATCH, rank/shape -> AX_ERR_SHAPE_MISMATCH,
 * plus AX_ERR_BACKEND for a tensor that does not live on this backend's device. */
#include <string.h>

#include "axhip.h"
#include "axiom/error.h"
#include "axiom/internal/backend_ops.h"

static ax_device_t g_my_device = AX_DEVICE_HIP;

static ax_status_t lift(int rc, const char *who) {
    if (rc == AXHIP_OK) return AX_OK;
    ax_err_set((ax_status_t)rc, "%s: %s", who, axhip_last_error());
    return (ax_status_t)rc;
}

/* a dense 2-D (or contiguous n-D) fp32 operand resident on this backend's device */
typedef struct {
    float *p;
    int64_t rows, cols, ld;
} mat_t;

static ax_status_t as_matrix(const ax_tensor_t *t, const char *who, const char *which, mat_t *m) {
    if (!t || !t->storage) {
        ax_err_set(AX_ERR_NULL_ARG, "%s: NULL %s", who, which);
        return AX_ERR_NULL_ARG;
    }
    if (t->dtype != AX_FLOAT32) {
        ax_err_set(AX_ERR_DTYPE_MISMATCH, "%s only supports float32 (%s)", who, which);
        return AX_ERR_DTYPE_MISMATCH;
    }
    if (t->ndim != 2) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s requires 2d tensors (%s has %d dims)", who, which, t->ndim);
        return AX_ERR_SHAPE_MISMATCH;
    }
    if (t->storage->device != g_my_device) {
        ax_err_set(AX_ERR_BACKEND, "%s: %s lives on device %d, not on the hip device", who, which,
                   (int)t->storage->device);
        return AX_ERR_BACKEND;
    }
    if (t->shape[1] > 1 && t->strides[1] != 1) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s: %s must have unit column stride", who, which);
        return AX_ERR_SHAPE_MISMATCH;
    }
    m->p = (float *)t->storage->data + t->offset;
    m->rows = t->shape[0];
    m->cols = t->shape[1];
    m->ld = t->shape[0] > 1 ? t->strides[0] : t->shape[1];
    if (m->ld < m->cols) m->ld = m->cols;
    return AX_OK;
}

static ax_status_t as_vector(const ax_tensor_t *t, const char *who, int64_t want, const float **p) {
    *p = NULL;
    if (!t) return AX_OK;                                   /* optional operand */
    if (!t->storage || t->dtype != AX_FLOAT32) {
        ax_err_set(AX_ERR_DTYPE_MISMATCH, "%s: bias must be float32", who);
        return AX_ERR_DTYPE_MISMATCH;
    }
    if (t->storage->device != g_my_device) {
        ax_err_set(AX_ERR_BACKEND, "%s: bias is not on the hip device", who);
        return AX_ERR_BACKEND;
    }
    if (ax_tensor_numel(t) != want || (t->ndim >= 1 && t->shape[t->ndim - 1] > 1 && t->strides[t->ndim - 1] != 1)) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s: bias must be a contiguous vector of %lld", who, (long long)want);
        return AX_ERR_SHAPE_MISMATCH;
    }
    *p = (const float *)t->storage->data + t->offset;
    return AX_OK;
}

/* out = act(alpha * op(a) op(b) + beta*out + bias) with the reference's shape rules */
static ax_status_t run_gemm(const char *who, int transa, int transb, const ax_tensor_t *a,
                            const ax_tensor_t *b, float alpha, float beta, const ax_tensor_t *bias,
                            int act, ax_tensor_t *out) {
    mat_t A, B, C;
    ax_status_t st;
    if ((st = as_matrix(a, who, "a", &A)) || (st = as_matrix(b, who, "b", &B)) ||
        (st = as_matrix(out, who, "out", &C)))
        return st;
    const int64_t M = transa ? A.cols : A.rows, K = transa ? A.rows : A.cols;
    const int64_t Kb = transb ? B.cols : B.rows, N = transb ? B.rows : B.cols;
    if (K != Kb || C.rows != M || C.cols != N) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s shape mismatch: [%lld,%lld] x [%lld,%lld] -> [%lld,%lld]", who,
                   (long long)M, (long long)K, (long long)Kb, (long long)N, (long long)C.rows, (long long)C.cols);
        return AX_ERR_SHAPE_MISMATCH;
    }
    const float *bp;
    if ((st = as_vector(bias, who, N, &bp))) return st;
    return lift(axhip_sgemm(transa, transb, M, N, K, alpha, A.p, A.ld, B.p, B.ld, beta, C.p, C.ld, bp, act), who);
}

static ax_status_t hip_gemm(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) {
    return run_gemm("hip gemm", 0, 0, a, b, 1.0f, 0.0f, NULL, AXHIP_ACT_NONE, out);
}
static ax_status_t hip_gemm_nt(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) {
    return run_gemm("hip gemm_nt", 0, 1, a, b, 1.0f, 0.0f, NULL, AXHIP_ACT_NONE, out);
}
static ax_status_t hip_gemm_tn(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) {
    return run_gemm("hip gemm_tn", 1, 0, a, b, 1.0f, 0.0f, NULL, AXHIP_ACT_NONE, out);
}
static ax_status_t hip_gemm_relu(const ax_tensor_t *a, const ax_tensor_t *b, const ax_tensor_t *bias, ax_tensor_t *out) {
    return run_gemm("hip gemm_relu", 0, 0, a, b, 1.0f, 0.0f, bias, AXHIP_ACT_RELU, out);
}
static ax_status_t hip_gemm_ex(const ax_tensor_t *a, const ax_tensor_t *b, float alpha, float beta, ax_tensor_t *out) {
    return run_gemm("hip gemm_ex", 0, 0, a, b, alpha, beta, NULL, AXHIP_ACT_NONE, out);
}
static ax_status_t hip_gemm_bias_act(const ax_tensor_t *a, const ax_tensor_t *b, const ax_tensor_t *bias, int act, ax_tensor_t *out) {
    if (act < AXHIP_ACT_NONE || act > AXHIP_ACT_GELU) {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "hip gemm_bias_act: activation %d", act);
        return AX_ERR_NOT_IMPLEMENTED;
    }
    return run_gemm("hip gemm_bias_act", 0, 0, a, b, 1.0f, 0.0f, bias, act, out);
}

/* contiguous fp32 tensor on this device -> pointer + element count */
static ax_status_t as_flat(const ax_tensor_t *t, const char *who, float **p, int64_t *n) {
    if (!t || !t->storage) {
        ax_err_set(AX_ERR_NULL_ARG, "%s: NULL tensor", who);
        return AX_ERR_NULL_ARG;
    }
    if (t->dtype != AX_FLOAT32) {
        ax_err_set(AX_ERR_DTYPE_MISMATCH, "%s only supports float32", who);
        return AX_ERR_DTYPE_MISMATCH;
    }
    if (t->storage->device != g_my_device) {
        ax_err_set(AX_ERR_BACKEND, "%s: tensor is not on the hip device", who);
        return AX_ERR_BACKEND;
    }
    if (!ax_tensor_is_contiguous(t)) {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "%s: non-contiguous tensor", who);
        return AX_ERR_NOT_IMPLEMENTED;
    }
    *p = (float *)t->storage->data + t->offset;
    *n = ax_tensor_numel(t);
    return AX_OK;
}

static ax_status_t same_shape(const ax_tensor_t *a, const ax_tensor_t *b, const char *who) {
    if (a->ndim != b->ndim || memcmp(a->shape, b->shape, sizeof(int64_t) * (size_t)a->ndim)) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s: in/out shapes differ", who);
        return AX_ERR_SHAPE_MISMATCH;
    }
    return AX_OK;
}

static ax_status_t hip_relu(const ax_tensor_t *in, ax_tensor_t *out) {
    float *ip, *op;
    int64_t n, no;
    ax_status_t st;
    if ((st = as_flat(in, "hip relu", &ip, &n)) || (st = as_flat(out, "hip relu", &op, &no)) ||
        (st = same_shape(in, out, "hip relu")))
        return st;
    return lift(axhip_relu(ip, op, n), "hip relu");
}

static ax_status_t hip_gelu(const ax_tensor_t *in, ax_tensor_t *out) {
    float *ip, *op;
    int64_t n, no;
    ax_status_t st;
    if ((st = as_flat(in, "hip gelu", &ip, &n)) || (st = as_flat(out, "hip gelu", &op, &no)) ||
        (st = same_shape(in, out, "hip gelu")))
        return st;
    return lift(axhip_gelu(ip, op, n), "hip gelu");
}

static ax_status_t hip_fill(ax_tensor_t *t, double value) {
    float *p;
    int64_t n;
    ax_status_t st = as_flat(t, "hip fill", &p, &n);
    if (st) return st;
    return lift(axhip_fill_f32(p, (float)value, n), "hip fill");
}

static ax_status_t hip_copy(const ax_tensor_t *src, ax_tensor_t *dst) {
    float *sp, *dp;
    int64_t n, nd;
    ax_status_t st;
    if ((st = as_flat(src, "hip copy", &sp, &n)) || (st = as_flat(dst, "hip copy", &dp, &nd)) ||
        (st = same_shape(src, dst, "hip copy")))
        return st;
    return lift(axhip_memcpy_d2d(dp, sp, (size_t)n * sizeof(float)), "hip copy");
}

/* out[o,a,i] = in[o,a,i] + bias[a]: the contract of the slot (backend_ops.h) and of
 * opt_bias_add (cpu_opt.c:7148-7194), including its error codes. */
static ax_status_t hip_bias_add(const ax_tensor_t *in, const ax_tensor_t *bias, int axis, ax_tensor_t *out) {
    float *ip, *op, *bp;
    int64_t n, no, nb;
    ax_status_t st;
    if (!in || !bias || !out) return AX_ERR_NULL_ARG;
    if ((st = as_flat(in, "hip bias_add", &ip, &n)) || (st = as_flat(out, "hip bias_add", &op, &no)) ||
        (st = as_flat(bias, "hip bias_add", &bp, &nb)))
        return st;
    if (bias->ndim != 1) return AX_ERR_SHAPE_MISMATCH;
    if (axis < 0 || axis >= in->ndim) return AX_ERR_INVALID_AXIS;
    if (bias->shape[0] != in->shape[axis]) return AX_ERR_SHAPE_MISMATCH;
    if ((st = same_shape(in, out, "hip bias_add"))) return st;
    int64_t outer = 1, inner = 1;
    for (int d = 0; d < axis; d++) outer *= in->shape[d];
    for (int d = axis + 1; d < in->ndim; d++) inner *= in->shape[d];
    return lift(axhip_bias_add(ip, bp, outer, in->shape[axis], inner, op), "hip bias_add");
}

/* out = sum of `in` over `axis` (-1: over everything, out holds one element); the output must
 * hold numel(in) / shape[axis] elements (cuda_sum, cuda/ops_reduce.cu:262-295). */
static ax_status_t hip_sum(const ax_tensor_t *in, int axis, ax_tensor_t *out) {
    float *ip, *op;
    int64_t n, no;
    ax_status_t st;
    if (!in || !out) return AX_ERR_NULL_ARG;
    if ((st = as_flat(in, "hip sum", &ip, &n)) || (st = as_flat(out, "hip sum", &op, &no))) return st;
    if (axis == -1) {
        if (no != 1) {
            ax_err_set(AX_ERR_SHAPE_MISMATCH, "hip sum: full reduction needs a one-element output");
            return AX_ERR_SHAPE_MISMATCH;
        }
        return lift(axhip_sum_all(ip, n, op), "hip sum");
    }
    if (axis < 0 || axis >= in->ndim) {
        ax_err_set(AX_ERR_INVALID_AXIS, "axis %d out of range", axis);
        return AX_ERR_INVALID_AXIS;
    }
    int64_t outer = 1, inner = 1;
    for (int d = 0; d < axis; d++) outer *= in->shape[d];
    for (int d = axis + 1; d < in->ndim; d++) inner *= in->shape[d];
    if (no != outer * inner) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "hip sum: output holds %lld elements, expected %lld",
                   (long long)no, (long long)(outer * inner));
        return AX_ERR_SHAPE_MISMATCH;
    }
    return lift(axhip_sum_axis(ip, outer, in->shape[axis], inner, op), "hip sum");
}

/* y += alpha * x over matching element counts (cuda_axpy, cuda/ops_fused.cu:193-211) */
static ax_status_t hip_axpy(const ax_tensor_t *x, float alpha, ax_tensor_t *y) {
    float *xp, *yp;
    int64_t nx, ny;
    ax_status_t st;
    if (!x || !y) return AX_ERR_NULL_ARG;
    if ((st = as_flat(x, "hip axpy", &xp, &nx)) || (st = as_flat(y, "hip axpy", &yp, &ny))) return st;
    if (nx != ny) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "hip axpy requires matching numel");
        return AX_ERR_SHAPE_MISMATCH;
    }
    return lift(axhip_axpy(xp, alpha, yp, nx), "hip axpy");
}

/* ---- device-owner hooks ---- */
static ax_status_t hook_init(void) { return lift(axhip_init(), "hip init"); }
static void hook_shutdown(void) { axhip_shutdown(); }
static void hook_synchronize(void) { (void)axhip_synchronize(); }
static int hook_device_count(void) { return axhip_device_count(); }
static void *hook_alloc(size_t bytes) {
    void *p = axhip_malloc(bytes);
    if (!p) ax_err_set(AX_ERR_ALLOC, "hip storage_alloc(%zu): %s", bytes, axhip_last_error());
    return p;
}
static void hook_free(void *p) { axhip_free(p); }
static ax_status_t hook_h2d(void *d, const void *s, size_t n) { return lift(axhip_memcpy_h2d(d, s, n), "hip memcpy_h2d"); }
static ax_status_t hook_d2h(void *d, const void *s, size_t n) { return lift(axhip_memcpy_d2h(d, s, n), "hip memcpy_d2h"); }
static ax_status_t hook_d2d(void *d, const void *s, size_t n) { return lift(axhip_memcpy_d2d(d, s, n), "hip memcpy_d2d"); }

#define AX_HIP_OPS_INIT(dev)                                                                    \
    {                                                                                           \
        .name = "hip", .gemm = hip_gemm, .gemm_nt = hip_gemm_nt, .gemm_tn = hip_gemm_tn,        \
        .gemm_relu = hip_gemm_relu, .gemm_ex = hip_gemm_ex, .bias_add = hip_bias_add,           \
        .fill = hip_fill, .copy = hip_copy, .relu = hip_relu, .gelu_op = hip_gelu,              \
        .sum = hip_sum, .axpy = hip_axpy,                                                       \
        .device = (dev), .init = hook_init, .shutdown = hook_shutdown,                          \
        .synchronize = hook_synchronize, .device_count = hook_device_count,                     \
        .storage_alloc = hook_alloc, .storage_free = hook_free, .memcpy_h2d = hook_h2d,         \
        .memcpy_d2h = hook_d2h, .memcpy_d2d = hook_d2d, .gemm_bias_act = hip_gemm_bias_act,     \
    }

const ax_backend_ops_t ax_hip_ops = AX_HIP_OPS_INIT(AX_DEVICE_HIP);

/* Attention forward on device pointers, with the signature of the `sdpa_fwd` member of the
 * reference's GPU extension table (include/axiom/internal/cuda_extension.h:86-92; its CUDA
 * implementation is ax_cuda_sdpa_fwd, cuda/ops_attention.cu:299-392).  P_save (a copy of the
 * probabilities for the save-aware backward) is not produced: the fused kernel never forms them. */
ax_status_t ax_hip_sdpa_fwd(const float *Q, const float *K, const float *V, float *out, float *L,
                            int64_t BH, int64_t S, int64_t dk, float scale, bool causal, float *P_save) {
    if (P_save) {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "hip sdpa_fwd: P_save is not supported");
        return AX_ERR_NOT_IMPLEMENTED;
    }
    return lift(axhip_sdpa_fwd(Q, K, V, out, L, BH, S, dk, scale, causal ? 1 : 0), "hip sdpa_fwd");
}

const ax_backend_ops_t *ax_hip_ops_for_device(ax_device_t as_device) {
    static ax_backend_ops_t alias = AX_HIP_OPS_INIT(AX_DEVICE_HIP);
    alias.device = as_device;
    g_my_device = as_device;     /* tensors of the host library carry this id */
    return &alias;
}
