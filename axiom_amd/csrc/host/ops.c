/* Tensor-level matmul family and activations, inference half of Axiom's src/core/ops.c:285-440
 * and activations.c: validate, allocate an uninitialised output on the inputs' device, dispatch.
 * The bias is added to columns (see axiom/ops.h for how this departs from ops.c:357). */
#include <inttypes.h>

#include "axiom/compute.h"
#include "axiom/ops.h"

static ax_tensor_t *alloc_like_device(const ax_tensor_t *like, const int64_t *shape, int ndim) {
    ax_device_t prev = ax_get_default_device();
    ax_set_default_device(like->storage->device);
    ax_tensor_t *t = ax_tensor_create(shape, ndim, like->dtype);
    ax_set_default_device(prev);
    return t;
}

static ax_tensor_t *matmul_impl(ax_tensor_t *a, ax_tensor_t *b, ax_tensor_t *bias, ax_activation_t act,
                                bool allow_3d, const char *who) {
    if (!a || !b) {
        ax_err_set(AX_ERR_NULL_ARG, "%s: NULL tensor", who);
        return NULL;
    }
    if (!((a->ndim == 2) || (allow_3d && a->ndim == 3)) || b->ndim != 2) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s needs a:[M,K]%s and b:[K,N]", who, allow_3d ? " or [B,S,K]" : "");
        return NULL;
    }
    const int64_t inner = a->shape[a->ndim - 1];
    if (inner != b->shape[0]) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "%s: inner dims don't match (a_inner=%" PRId64 " b_outer=%" PRId64 ")",
                   who, inner, b->shape[0]);
        return NULL;
    }
    /* a [B,S,K] input is viewed as [B*S,K] for the GEMM and the result viewed back (ops.c:330-342) */
    ax_tensor_t *a2 = a;
    if (a->ndim == 3) {
        int64_t flat[2] = {a->shape[0] * a->shape[1], a->shape[2]};
        a2 = ax_tensor_reshape(a, flat, 2);
        if (!a2) return NULL;
    }
    int64_t oshape[2] = {a2->shape[0], b->shape[1]};
    ax_tensor_t *out = alloc_like_device(a, oshape, 2);
    ax_status_t st = AX_ERR_ALLOC;
    if (out) {
        if (ax_compute_has_gemm_bias_act()) {
            st = ax_compute_gemm_bias_act(a2, b, bias, act, out);
        } else if (act == AX_ACT_RELU && ax_compute_has_gemm_relu()) {
            st = ax_compute_gemm_relu(a2, b, bias, out);
        } else {                                            /* unfused: gemm, column bias, activation */
            st = ax_compute_gemm(a2, b, out);
            if (st == AX_OK && bias) st = ax_compute_bias_add(out, bias, 1, out);
            if (st == AX_OK && act == AX_ACT_RELU) st = ax_compute_relu(out, out);
            if (st == AX_OK && act == AX_ACT_GELU) st = ax_compute_gelu(out, out);
        }
    }
    if (a2 != a) ax_tensor_destroy(a2);
    if (st != AX_OK) {
        ax_tensor_destroy(out);
        return NULL;
    }
    if (a->ndim == 3) {
        int64_t s3[3] = {a->shape[0], a->shape[1], b->shape[1]};
        ax_tensor_t *view = ax_tensor_reshape(out, s3, 3);
        ax_tensor_destroy(out);
        return view;
    }
    return out;
}

ax_tensor_t *ax_matmul(ax_tensor_t *a, ax_tensor_t *b) { return matmul_impl(a, b, NULL, AX_ACT_NONE, true, "matmul"); }
ax_tensor_t *ax_matmul_bias(ax_tensor_t *a, ax_tensor_t *b, ax_tensor_t *bias) {
    return matmul_impl(a, b, bias, AX_ACT_NONE, true, "matmul");
}
ax_tensor_t *ax_matmul_bias_relu(ax_tensor_t *a, ax_tensor_t *b, ax_tensor_t *bias) {
    return matmul_impl(a, b, bias, AX_ACT_RELU, false, "matmul_bias_relu");
}
ax_tensor_t *ax_matmul_bias_gelu(ax_tensor_t *a, ax_tensor_t *b, ax_tensor_t *bias) {
    return matmul_impl(a, b, bias, AX_ACT_GELU, true, "matmul_bias_gelu");
}

ax_tensor_t *ax_matmul_bias_act_head(ax_tensor_t *a, ax_tensor_t *b, ax_tensor_t *bias, int act, ax_tensor_t *w2,
                                     ax_tensor_t *bias2, int act2) {
    if (!a || !b || !w2) {
        ax_err_set(AX_ERR_NULL_ARG, "matmul_bias_act_head: NULL tensor");
        return NULL;
    }
    if (a->ndim != 2 || b->ndim != 2 || w2->ndim != 2 || a->shape[1] != b->shape[0] || b->shape[1] != w2->shape[0]) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "matmul_bias_act_head needs a:[M,K], b:[K,N], w2:[N,H]");
        return NULL;
    }
    if (!ax_compute_has_gemm_act_head()) {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "matmul_bias_act_head: the active backend has no such operation");
        return NULL;
    }
    int64_t oshape[2] = {a->shape[0], w2->shape[1]};
    ax_tensor_t *out = alloc_like_device(a, oshape, 2);
    if (!out) return NULL;
    if (ax_compute_gemm_act_head(a, b, bias, (ax_activation_t)act, w2, bias2, (ax_activation_t)act2, out) != AX_OK) {
        ax_tensor_destroy(out);
        return NULL;
    }
    return out;
}

static ax_tensor_t *unary(ax_tensor_t *a, ax_status_t (*op)(const ax_tensor_t *, ax_tensor_t *), const char *who) {
    if (!a) {
        ax_err_set(AX_ERR_NULL_ARG, "%s: NULL tensor", who);
        return NULL;
    }
    if (a->dtype != AX_FLOAT32) {
        ax_err_set(AX_ERR_DTYPE_MISMATCH, "%s only supports float32", who);
        return NULL;
    }
    ax_tensor_t *out = alloc_like_device(a, a->shape, a->ndim);
    if (!out) return NULL;
    if (op(a, out) != AX_OK) {
        ax_tensor_destroy(out);
        return NULL;
    }
    return out;
}

ax_tensor_t *ax_relu(ax_tensor_t *a) { return unary(a, ax_compute_relu, "relu"); }
ax_tensor_t *ax_gelu(ax_tensor_t *a) { return unary(a, ax_compute_gelu, "gelu"); }
ax_tensor_t *ax_sigmoid(ax_tensor_t *a) { return unary(a, ax_compute_sigmoid, "sigmoid"); }
ax_tensor_t *ax_tanh_op(ax_tensor_t *a) { return unary(a, ax_compute_tanh, "tanh"); }
ax_tensor_t *ax_swish(ax_tensor_t *a) { return unary(a, ax_compute_swish, "swish"); }

static ax_tensor_t *unary_alpha(ax_tensor_t *a, float alpha,
                                ax_status_t (*op)(const ax_tensor_t *, float, ax_tensor_t *), const char *who) {
    if (!a) {
        ax_err_set(AX_ERR_NULL_ARG, "%s: NULL tensor", who);
        return NULL;
    }
    if (a->dtype != AX_FLOAT32) {
        ax_err_set(AX_ERR_DTYPE_MISMATCH, "%s only supports float32", who);
        return NULL;
    }
    ax_tensor_t *out = alloc_like_device(a, a->shape, a->ndim);
    if (!out) return NULL;
    if (op(a, alpha, out) != AX_OK) {
        ax_tensor_destroy(out);
        return NULL;
    }
    return out;
}

ax_tensor_t *ax_leaky_relu(ax_tensor_t *a, float alpha) { return unary_alpha(a, alpha, ax_compute_leaky_relu, "leaky_relu"); }
ax_tensor_t *ax_elu(ax_tensor_t *a, float alpha) { return unary_alpha(a, alpha, ax_compute_elu, "elu"); }

/* softmax over the last axis: the rows of the tensor viewed as [numel / last, last] */
ax_tensor_t *ax_softmax(ax_tensor_t *a, int axis) {
    if (!a || a->dtype != AX_FLOAT32 || a->ndim < 1) {
        ax_err_set(AX_ERR_NULL_ARG, "softmax: needs a float32 tensor");
        return NULL;
    }
    if (axis == -1) axis = a->ndim - 1;
    if (axis != a->ndim - 1) {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "softmax: only the last axis is supported");
        return NULL;
    }
    const int64_t cols = a->shape[a->ndim - 1];
    int64_t flat[2] = {cols ? ax_tensor_numel(a) / cols : 0, cols};
    ax_tensor_t *a2 = ax_tensor_reshape(a, flat, 2);
    ax_tensor_t *out = a2 ? alloc_like_device(a, flat, 2) : NULL;
    ax_status_t st = out ? ax_compute_softmax_rowwise(a2, out) : AX_ERR_ALLOC;
    if (a2) ax_tensor_destroy(a2);
    if (st != AX_OK) {
        ax_tensor_destroy(out);
        return NULL;
    }
    ax_tensor_t *view = ax_tensor_reshape(out, a->shape, a->ndim);
    ax_tensor_destroy(out);
    return view;
}
