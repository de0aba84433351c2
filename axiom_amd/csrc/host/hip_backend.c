/* ax_hip_ops — the MI355X backend object behind Axiom's vtable.
 *
 * Plain C: it unpacks ax_tensor_t (shape, strides, offset, device) into pointers and sizes and
 * calls the C ABI of libaxhip.so; no HIP header is included here.  It takes the place of
 * ax_cuda_ops (src/compute/backends/cuda/backend.cu:140-192): every slot that object fills
 * except conv_gemm, plus gemm_relu and argmax, and the ten device-owner hooks; the attention
 * training slots and the convolution slots stay NULL.
 * Operands are borrowed, never retained.  Errors follow the reference's backend convention
 * (cuda/ops_gemm.cu:16-23): dtype != f32 -> AX_ERR_DTYPE_MISMATCH, rank/shape -> AX_ERR_SHAPE_MISMATCH,
 * plus AX_ERR_BACKEND for a tensor that does not live on this backend's device. */
#include <string.h>

#include "axhip.h"
#include "axiom/error.h"
#include "axiom/internal/backend_ops.h"
#include "axiom/internal/cuda_extension.h"

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
    /* a view whose rows overlap or repeat (a stride-0 expanded row, say) is not a dense matrix with a pitch */
    if (t->shape[0] > 1 && t->strides[0] < t->shape[1]) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s: rows of %s overlap (row stride %lld < %lld columns)", who, which,
                   (long long)t->strides[0], (long long)t->shape[1]);
        return AX_ERR_SHAPE_MISMATCH;
    }
    m->ld = t->shape[0] > 1 ? t->strides[0] : t->shape[1];
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

/* Dense -> narrow Dense on the skinny route (at most 16 rows, second layer at most 16 wide, dense weights);
 * anything else is left to the caller's layer-by-layer path */
static ax_status_t hip_gemm_act_head(const ax_tensor_t *a, const ax_tensor_t *b, const ax_tensor_t *bias, int act,
                                     const ax_tensor_t *w2, const ax_tensor_t *bias2, int act2, ax_tensor_t *out2) {
    const char *who = "hip gemm_act_head";
    mat_t A, B, W, O;
    ax_status_t st;
    if ((st = as_matrix(a, who, "a", &A)) || (st = as_matrix(b, who, "b", &B)) || (st = as_matrix(w2, who, "w2", &W)) ||
        (st = as_matrix(out2, who, "out2", &O)))
        return st;
    if (A.cols != B.rows || B.cols != W.rows || O.rows != A.rows || O.cols != W.cols) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s shape mismatch: [%lld,%lld] x [%lld,%lld] x [%lld,%lld] -> [%lld,%lld]", who,
                   (long long)A.rows, (long long)A.cols, (long long)B.rows, (long long)B.cols, (long long)W.rows,
                   (long long)W.cols, (long long)O.rows, (long long)O.cols);
        return AX_ERR_SHAPE_MISMATCH;
    }
    if (A.rows < 1 || A.rows > 16 || W.cols < 1 || W.cols > 16 || W.ld != W.cols || O.ld != O.cols ||
        act < AXHIP_ACT_NONE || act > AXHIP_ACT_GELU || act2 < AXHIP_ACT_NONE || act2 > AXHIP_ACT_GELU) {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "%s: %lld rows into a head of %lld is not taken in one launch", who,
                   (long long)A.rows, (long long)W.cols);
        return AX_ERR_NOT_IMPLEMENTED;
    }
    const float *bp, *bp2;
    if ((st = as_vector(bias, who, B.cols, &bp)) || (st = as_vector(bias2, who, W.cols, &bp2))) return st;
    return lift(axhip_sgemm_skinny_head(A.rows, B.cols, A.cols, A.p, A.ld, B.p, B.ld, NULL, B.cols, bp, act, W.cols, W.p, bp2,
                                        act2, O.p), who);
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

/* ---- broadcasting binary slots ---------------------------------------------------------
 * Operands may be any strided views; the output is contiguous.  Each operand's stride per
 * OUTPUT dimension follows broadcast_index (cpu_naive.c:48-62): trailing dimensions aligned,
 * an operand extent of 1 contributes stride 0. */
static ax_status_t on_device_f32(const ax_tensor_t *t, const char *who) {
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
    return AX_OK;
}

static ax_status_t operand_strides(const ax_tensor_t *t, const ax_tensor_t *out, const char *who, int64_t *st) {
    for (int d = 0; d < out->ndim; d++) {
        const int td = d - (out->ndim - t->ndim);
        st[d] = 0;
        if (td < 0 || t->shape[td] == 1) continue;
        if (t->shape[td] != out->shape[d]) {
            ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s: extent %lld does not broadcast to %lld", who,
                       (long long)t->shape[td], (long long)out->shape[d]);
            return AX_ERR_SHAPE_MISMATCH;
        }
        st[d] = t->strides[td];
    }
    return AX_OK;
}

static ax_status_t run_binary(const char *who, int op, const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) {
    ax_status_t st;
    float *op_;
    int64_t no, sa[AX_MAX_DIMS], sb[AX_MAX_DIMS];
    if ((st = on_device_f32(a, who)) || (st = on_device_f32(b, who)) || (st = as_flat(out, who, &op_, &no))) return st;
    if (a->ndim > out->ndim || b->ndim > out->ndim) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s: operand has more dimensions than the output", who);
        return AX_ERR_SHAPE_MISMATCH;
    }
    if ((st = operand_strides(a, out, who, sa)) || (st = operand_strides(b, out, who, sb))) return st;
    return lift(axhip_binary(op, (const float *)a->storage->data + a->offset, (const float *)b->storage->data + b->offset,
                             op_, out->ndim, out->shape, sa, sb), who);
}

static ax_status_t hip_add(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { return run_binary("hip add", AXHIP_BIN_ADD, a, b, out); }
static ax_status_t hip_sub(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { return run_binary("hip sub", AXHIP_BIN_SUB, a, b, out); }
static ax_status_t hip_mul(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { return run_binary("hip mul", AXHIP_BIN_MUL, a, b, out); }
static ax_status_t hip_div(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { return run_binary("hip div", AXHIP_BIN_DIV, a, b, out); }
static ax_status_t hip_equal(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { return run_binary("hip equal", AXHIP_BIN_EQUAL, a, b, out); }
static ax_status_t hip_greater(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { return run_binary("hip greater", AXHIP_BIN_GREATER, a, b, out); }

/* same element counts only, as cuda_add_relu (cuda/ops_fused.cu:168-190) */
static ax_status_t hip_add_relu(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) {
    float *ap, *bp, *op;
    int64_t na, nb, no;
    ax_status_t st;
    if ((st = as_flat(a, "hip add_relu", &ap, &na)) || (st = as_flat(b, "hip add_relu", &bp, &nb)) ||
        (st = as_flat(out, "hip add_relu", &op, &no)))
        return st;
    if (na != no || nb != no) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "hip add_relu requires matching shapes");
        return AX_ERR_SHAPE_MISMATCH;
    }
    const int64_t one = 1;
    return lift(axhip_binary(AXHIP_BIN_ADD_RELU, ap, bp, op, 1, &no, &one, &one), "hip add_relu");
}

/* ---- unary, scalar and activation slots (contiguous, element count of the output) ---- */
static ax_status_t run_unary(const char *who, int op, const ax_tensor_t *in, float param, ax_tensor_t *out) {
    float *ip, *op_;
    int64_t n, no;
    ax_status_t st;
    if ((st = as_flat(in, who, &ip, &n)) || (st = as_flat(out, who, &op_, &no))) return st;
    if (n != no) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s: in/out element counts differ", who);
        return AX_ERR_SHAPE_MISMATCH;
    }
    return lift(axhip_unary(op, ip, op_, n, param), who);
}

static ax_status_t hip_neg(const ax_tensor_t *in, ax_tensor_t *out) { return run_unary("hip neg", AXHIP_UN_NEG, in, 0.0f, out); }
static ax_status_t hip_abs(const ax_tensor_t *in, ax_tensor_t *out) { return run_unary("hip abs", AXHIP_UN_ABS, in, 0.0f, out); }
static ax_status_t hip_exp(const ax_tensor_t *in, ax_tensor_t *out) { return run_unary("hip exp", AXHIP_UN_EXP, in, 0.0f, out); }
static ax_status_t hip_log(const ax_tensor_t *in, ax_tensor_t *out) { return run_unary("hip log", AXHIP_UN_LOG, in, 0.0f, out); }
static ax_status_t hip_sqrt(const ax_tensor_t *in, ax_tensor_t *out) { return run_unary("hip sqrt", AXHIP_UN_SQRT, in, 0.0f, out); }
static ax_status_t hip_square(const ax_tensor_t *in, ax_tensor_t *out) { return run_unary("hip square", AXHIP_UN_SQUARE, in, 0.0f, out); }
static ax_status_t hip_sigmoid(const ax_tensor_t *in, ax_tensor_t *out) { return run_unary("hip sigmoid", AXHIP_UN_SIGMOID, in, 0.0f, out); }
static ax_status_t hip_tanh(const ax_tensor_t *in, ax_tensor_t *out) { return run_unary("hip tanh", AXHIP_UN_TANH, in, 0.0f, out); }
static ax_status_t hip_swish(const ax_tensor_t *in, ax_tensor_t *out) { return run_unary("hip swish", AXHIP_UN_SWISH, in, 0.0f, out); }
static ax_status_t hip_leaky_relu(const ax_tensor_t *in, float alpha, ax_tensor_t *out) { return run_unary("hip leaky_relu", AXHIP_UN_LEAKY_RELU, in, alpha, out); }
static ax_status_t hip_elu(const ax_tensor_t *in, float alpha, ax_tensor_t *out) { return run_unary("hip elu", AXHIP_UN_ELU, in, alpha, out); }
static ax_status_t hip_add_scalar(const ax_tensor_t *in, double s, ax_tensor_t *out) { return run_unary("hip add_scalar", AXHIP_UN_ADD_SCALAR, in, (float)s, out); }
static ax_status_t hip_mul_scalar(const ax_tensor_t *in, double s, ax_tensor_t *out) { return run_unary("hip mul_scalar", AXHIP_UN_MUL_SCALAR, in, (float)s, out); }

/* ---- mean / max / min / argmax: the shape rules of hip_sum ---- */
static ax_status_t reduction_extents(const char *who, const ax_tensor_t *in, int axis, int64_t n_out, int64_t *outer,
                                     int64_t *axis_len, int64_t *inner) {
    if (axis == -1) {
        *outer = 1;
        *inner = 1;
        *axis_len = ax_tensor_numel(in);
    } else {
        if (axis < 0 || axis >= in->ndim) {
            ax_err_set(AX_ERR_INVALID_AXIS, "axis %d out of range", axis);
            return AX_ERR_INVALID_AXIS;
        }
        *outer = *inner = 1;
        for (int d = 0; d < axis; d++) *outer *= in->shape[d];
        for (int d = axis + 1; d < in->ndim; d++) *inner *= in->shape[d];
        *axis_len = in->shape[axis];
    }
    if (n_out != *outer * *inner) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s: output holds %lld elements, expected %lld", who, (long long)n_out,
                   (long long)(*outer * *inner));
        return AX_ERR_SHAPE_MISMATCH;
    }
    return AX_OK;
}

static ax_status_t run_reduce(const char *who, int op, const ax_tensor_t *in, int axis, ax_tensor_t *out) {
    float *ip, *op_;
    int64_t n, no, outer, axis_len, inner;
    ax_status_t st;
    if (!in || !out) return AX_ERR_NULL_ARG;
    if ((st = as_flat(in, who, &ip, &n)) || (st = as_flat(out, who, &op_, &no)) ||
        (st = reduction_extents(who, in, axis, no, &outer, &axis_len, &inner)))
        return st;
    if (axis == -1) return lift(axhip_reduce_all(op, ip, n, op_), who);
    return lift(axhip_reduce_axis(op, ip, outer, axis_len, inner, op_), who);
}

static ax_status_t hip_mean(const ax_tensor_t *in, int axis, ax_tensor_t *out) { return run_reduce("hip mean", AXHIP_RED_MEAN, in, axis, out); }
static ax_status_t hip_max(const ax_tensor_t *in, int axis, ax_tensor_t *out) { return run_reduce("hip max", AXHIP_RED_MAX, in, axis, out); }
static ax_status_t hip_min(const ax_tensor_t *in, int axis, ax_tensor_t *out) { return run_reduce("hip min", AXHIP_RED_MIN, in, axis, out); }

/* int64 output (opt_argmax, cpu_opt.c:7202-7249) */
static ax_status_t hip_argmax(const ax_tensor_t *in, int axis, ax_tensor_t *out) {
    float *ip;
    int64_t n, outer, axis_len, inner;
    ax_status_t st;
    if (!in || !out) return AX_ERR_NULL_ARG;
    if ((st = as_flat(in, "hip argmax", &ip, &n))) return st;
    if (out->dtype != AX_INT64) return AX_ERR_DTYPE_MISMATCH;
    if (!out->storage || !out->storage->data || out->storage->device != g_my_device || !ax_tensor_is_contiguous(out))
        return AX_ERR_BACKEND;
    if ((st = reduction_extents("hip argmax", in, axis, ax_tensor_numel(out), &outer, &axis_len, &inner))) return st;
    return lift(axhip_argmax_axis(ip, outer, axis_len, inner, (int64_t *)out->storage->data + out->offset), "hip argmax");
}

/* 2-D, matching shapes (cuda_softmax_rowwise, cuda/ops_fused.cu:213-229) */
static ax_status_t hip_softmax_rowwise(const ax_tensor_t *in, ax_tensor_t *out) {
    float *ip, *op;
    int64_t n, no;
    ax_status_t st;
    if ((st = as_flat(in, "hip softmax_rowwise", &ip, &n)) || (st = as_flat(out, "hip softmax_rowwise", &op, &no))) return st;
    if (in->ndim != 2 || out->ndim != 2 || in->shape[0] != out->shape[0] || in->shape[1] != out->shape[1]) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "hip softmax_rowwise shape mismatch");
        return AX_ERR_SHAPE_MISMATCH;
    }
    return lift(axhip_softmax_rows(ip, op, in->shape[0], in->shape[1]), "hip softmax_rowwise");
}

/* ---- optimizer slots (cuda_adam_update / cuda_sgd_update, cuda/ops_optim.cu:66-110) ---- */
static ax_status_t hip_adam_update(ax_tensor_t *weight, ax_tensor_t *grad, ax_tensor_t *m, ax_tensor_t *v, float lr,
                                   float beta1, float beta2, float eps, float weight_decay, float bc1, float bc2,
                                   bool decoupled) {
    float *wp, *gp, *mp, *vp;
    int64_t n, ng, nm, nv;
    ax_status_t st;
    if (!weight || !grad || !m || !v) return AX_ERR_NULL_ARG;
    if ((st = as_flat(weight, "hip adam_update", &wp, &n)) || (st = as_flat(grad, "hip adam_update", &gp, &ng)) ||
        (st = as_flat(m, "hip adam_update", &mp, &nm)) || (st = as_flat(v, "hip adam_update", &vp, &nv)))
        return st;
    if (ng != n || nm != n || nv != n) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "hip adam_update: element counts differ");
        return AX_ERR_SHAPE_MISMATCH;
    }
    return lift(axhip_adam_update(wp, gp, mp, vp, n, lr, beta1, beta2, eps, weight_decay, bc1, bc2, decoupled ? 1 : 0),
                "hip adam_update");
}

static ax_status_t hip_sgd_update(ax_tensor_t *weight, ax_tensor_t *grad, ax_tensor_t *momentum_buf, float lr,
                                  float momentum, float weight_decay, bool nesterov) {
    float *wp, *gp, *mp = NULL;
    int64_t n, ng, nm = 0;
    ax_status_t st;
    if (!weight || !grad) return AX_ERR_NULL_ARG;
    if ((st = as_flat(weight, "hip sgd_update", &wp, &n)) || (st = as_flat(grad, "hip sgd_update", &gp, &ng))) return st;
    if (momentum_buf && (st = as_flat(momentum_buf, "hip sgd_update", &mp, &nm))) return st;
    if (ng != n || (momentum_buf && nm != n)) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "hip sgd_update: element counts differ");
        return AX_ERR_SHAPE_MISMATCH;
    }
    return lift(axhip_sgd_update(wp, gp, mp, n, lr, momentum, weight_decay, nesterov ? 1 : 0), "hip sgd_update");
}

/* x is [rows..., D] contiguous; gamma, beta are [D] */
static ax_status_t hip_layernorm_fwd(const ax_tensor_t *x, const ax_tensor_t *gamma, const ax_tensor_t *beta, float eps,
                                     ax_tensor_t *out, ax_tensor_t *x_hat, ax_tensor_t *inv_std) {
    float *xp, *op, *gp, *bp, *hp = NULL, *sp = NULL;
    int64_t n, no, ng, nb, nh = 0, ns = 0;
    ax_status_t st;
    if (!x || !gamma || !beta || !out) return AX_ERR_NULL_ARG;
    if ((st = as_flat(x, "hip layernorm", &xp, &n)) || (st = as_flat(out, "hip layernorm", &op, &no)) ||
        (st = as_flat(gamma, "hip layernorm", &gp, &ng)) || (st = as_flat(beta, "hip layernorm", &bp, &nb)))
        return st;
    if (x_hat && (st = as_flat(x_hat, "hip layernorm", &hp, &nh))) return st;
    if (inv_std && (st = as_flat(inv_std, "hip layernorm", &sp, &ns))) return st;
    if (x->ndim < 1 || x->shape[x->ndim - 1] < 1) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "hip layernorm: input needs a non-empty feature axis");
        return AX_ERR_SHAPE_MISMATCH;
    }
    const int64_t cols = x->shape[x->ndim - 1], rows = n / cols;
    if (no != n || ng != cols || nb != cols || (x_hat && nh != n) || (inv_std && ns != rows)) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "hip layernorm: operand sizes do not match [%lld, %lld]", (long long)rows,
                   (long long)cols);
        return AX_ERR_SHAPE_MISMATCH;
    }
    return lift(axhip_layernorm_fwd(xp, gp, bp, op, hp, sp, rows, cols, eps), "hip layernorm");
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
static void *hook_alloc_uninit(size_t bytes) {
    void *p = axhip_malloc_uninit(bytes);
    if (!p) ax_err_set(AX_ERR_ALLOC, "hip storage_alloc(%zu): %s", bytes, axhip_last_error());
    return p;
}
static void hook_free(void *p) { axhip_free(p); }
static ax_status_t hook_h2d(void *d, const void *s, size_t n) { return lift(axhip_memcpy_h2d(d, s, n), "hip memcpy_h2d"); }
static ax_status_t hook_d2h(void *d, const void *s, size_t n) { return lift(axhip_memcpy_d2h(d, s, n), "hip memcpy_d2h"); }
static ax_status_t hook_d2d(void *d, const void *s, size_t n) { return lift(axhip_memcpy_d2d(d, s, n), "hip memcpy_d2d"); }

#define AX_HIP_OPS_INIT(dev)                                                                    \
    {                                                                                           \
        .name = "hip", .add = hip_add, .sub = hip_sub, .mul = hip_mul, .div_op = hip_div,       \
        .neg = hip_neg, .abs_op = hip_abs, .exp_op = hip_exp, .log_op = hip_log,                \
        .sqrt_op = hip_sqrt, .square = hip_square, .add_scalar = hip_add_scalar,                \
        .mul_scalar = hip_mul_scalar, .add_relu = hip_add_relu,                                 \
        .softmax_rowwise = hip_softmax_rowwise, .mean = hip_mean, .max_op = hip_max,            \
        .min_op = hip_min, .argmax = hip_argmax, .equal = hip_equal, .greater = hip_greater,    \
        .sigmoid = hip_sigmoid, .tanh_op = hip_tanh, .leaky_relu = hip_leaky_relu,              \
        .elu_op = hip_elu, .swish_op = hip_swish, .adam_update = hip_adam_update,               \
        .sgd_update = hip_sgd_update,                                                           \
        .gemm = hip_gemm, .gemm_nt = hip_gemm_nt, .gemm_tn = hip_gemm_tn,                       \
        .gemm_relu = hip_gemm_relu, .gemm_ex = hip_gemm_ex, .bias_add = hip_bias_add,           \
        .fill = hip_fill, .copy = hip_copy, .relu = hip_relu, .gelu_op = hip_gelu,              \
        .sum = hip_sum, .axpy = hip_axpy,                                                       \
        .device = (dev), .init = hook_init, .shutdown = hook_shutdown,                          \
        .synchronize = hook_synchronize, .device_count = hook_device_count,                     \
        .storage_alloc = hook_alloc, .storage_free = hook_free, .memcpy_h2d = hook_h2d,         \
        .memcpy_d2h = hook_d2h, .memcpy_d2d = hook_d2d, .gemm_bias_act = hip_gemm_bias_act,     \
        .gemm_act_head = hip_gemm_act_head,                                                     \
        .layernorm_fwd = hip_layernorm_fwd, .storage_alloc_uninit = hook_alloc_uninit,          \
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

static ax_status_t ext_sdpa_fwd_rows(const float *Q, const float *K, const float *V, int64_t ld, float *out, int64_t ldo,
                                     float *L, int64_t B, int64_t H, int64_t S, int64_t dk, float scale, bool causal) {
    return lift(axhip_sdpa_fwd_rows(Q, K, V, ld, out, ldo, L, B, H, S, dk, scale, causal ? 1 : 0), "hip sdpa_fwd_rows");
}

/* ---- the extension table (include/axiom/internal/cuda_extension.h).  The layout members return
 * nothing in the reference's table; a failure is left for ax_err_last_message(). ---- */
static void ext_split(const float *src, float *q, float *k, float *v, int64_t B, int64_t S, int64_t H, int64_t dk, int64_t D) {
    (void)lift(axhip_head_split_qkv(src, NULL, q, k, v, B, S, H, dk, D), "hip head_interleave_qkv_split");
}
static void ext_split_bias(const float *src, const float *bqkv, float *q, float *k, float *v, int64_t B, int64_t S,
                           int64_t H, int64_t dk, int64_t D) {
    (void)lift(axhip_head_split_qkv(src, bqkv, q, k, v, B, S, H, dk, D), "hip head_interleave_qkv_split_bias");
}
static void ext_interleave(const float *src, float *dst, int64_t B, int64_t S, int64_t H, int64_t dk) {
    (void)lift(axhip_head_interleave(src, dst, B, S, H, dk), "hip head_interleave");
}
static void ext_deinterleave(const float *src, float *dst, int64_t B, int64_t S, int64_t H, int64_t dk) {
    (void)lift(axhip_head_deinterleave(src, dst, B, S, H, dk), "hip head_deinterleave");
}
static ax_status_t ext_qkv_cache(float *dst, const float *wq, const float *wk, const float *wv, int64_t D) {
    return lift(axhip_concat3_rows(dst, wq, wk, wv, D, D), "hip qkv_cache_build");
}
static ax_status_t ext_bias_cache(float *dst, const float *bq, const float *bk, const float *bv, int64_t D) {
    return lift(axhip_concat3_rows(dst, bq, bk, bv, 1, D), "hip bias_cache_build");
}

const ax_cuda_extension_t ax_hip_extension = {
    .head_interleave_qkv_split = ext_split, .head_interleave_qkv_split_bias = ext_split_bias,
    .head_interleave = ext_interleave, .head_deinterleave = ext_deinterleave,
    .qkv_cache_build = ext_qkv_cache, .bias_cache_build = ext_bias_cache, .sdpa_fwd = ax_hip_sdpa_fwd,
    .sdpa_fwd_rows = ext_sdpa_fwd_rows,
};

const ax_backend_ops_t *ax_hip_ops_for_device(ax_device_t as_device) {
    static ax_backend_ops_t alias = AX_HIP_OPS_INIT(AX_DEVICE_HIP);
    alias.device = as_device;
    g_my_device = as_device;     /* tensors of the host library carry this id */
    return &alias;
}
