/* Backend registry and the ax_compute_* wrappers of the GEMM path (Axiom's
 * src/compute/dispatch.c:61-143, 251-315, 347-454).  Process-global, unsynchronised state:
 * ops are issued from one host thread at a time, as in the reference.  The only backend this
 * build registers is ax_hip_ops; with no usable GPU nothing is active and every wrapper
 * returns AX_ERR_BACKEND — there is no CPU compute path to fall back to. */
#include "axiom/axiom.h"
#include "axiom/internal/backend_ops.h"
#include "axiom/internal/cuda_extension.h"

static const ax_backend_ops_t *g_backends[AX_BACKEND_COUNT];
static const ax_backend_ops_t *g_device_owner[AX_DEVICE_COUNT];
static int g_device_inited[AX_DEVICE_COUNT];
static ax_backend_id_t g_active_id = AX_BACKEND_HIP;
static const ax_backend_ops_t *g_active;
static int g_initialised;

static void claim_device(const ax_backend_ops_t *ops) {
    if (!ops) return;
    const int d = (int)ops->device;
    if (d <= AX_DEVICE_CPU || d >= AX_DEVICE_COUNT || g_device_owner[d]) return;
    g_device_owner[d] = ops;
    if (!g_device_inited[d] && ops->init) ops->init();
    g_device_inited[d] = 1;
}

const ax_backend_ops_t *ax_backend_for_device(ax_device_t device) {
    if ((int)device < 0 || (int)device >= AX_DEVICE_COUNT) return NULL;
    return g_device_owner[device];
}

/* the GPU extension table (src/compute/dispatch.c:286-300) */
static const ax_cuda_extension_t *g_extension;

ax_status_t ax_compute_register_cuda_extension(const ax_cuda_extension_t *ext) {
    g_extension = ext;
    return AX_OK;
}

const ax_cuda_extension_t *ax_compute_get_cuda_extension(void) { return g_extension; }

ax_status_t ax_compute_init(void) {
    if (g_initialised) {
        if (g_active) return AX_OK;
        ax_err_set(AX_ERR_BACKEND, "no MI355X visible: the hip backend is the only compute path");
        return AX_ERR_BACKEND;
    }
    g_initialised = 1;
    g_backends[AX_BACKEND_HIP] = &ax_hip_ops;
    claim_device(&ax_hip_ops);
    g_extension = &ax_hip_extension;
    if (ax_hip_ops.device_count && ax_hip_ops.device_count() > 0) {
        g_active_id = AX_BACKEND_HIP;
        g_active = &ax_hip_ops;
        return AX_OK;
    }
    g_active = NULL;
    ax_err_set(AX_ERR_BACKEND, "no MI355X visible: the hip backend is the only compute path");
    return AX_ERR_BACKEND;
}

static void ensure_init(void) {
    if (!g_initialised) ax_compute_init();
}

void ax_compute_shutdown(void) {
    for (int d = AX_DEVICE_COUNT - 1; d >= 0; d--) {
        const ax_backend_ops_t *ops = g_device_owner[d];
        if (ops && ops->shutdown && g_device_inited[d]) ops->shutdown();
        g_device_owner[d] = NULL;
        g_device_inited[d] = 0;
    }
    g_active = NULL;
    g_extension = NULL;
    g_initialised = 0;
}

ax_status_t ax_init(void) { return ax_compute_init(); }
void ax_shutdown(void) { ax_compute_shutdown(); }

ax_status_t ax_compute_set_backend(ax_backend_id_t id) {
    ensure_init();
    if ((int)id < 0 || id >= AX_BACKEND_COUNT || !g_backends[id]) {
        ax_err_set(AX_ERR_BACKEND, "backend %d not available", (int)id);
        return AX_ERR_BACKEND;
    }
    g_active_id = id;
    g_active = g_backends[id];
    return AX_OK;
}

ax_backend_id_t ax_compute_get_backend(void) { return g_active_id; }
const ax_backend_ops_t *ax_compute_get_ops(void) { return g_active; }
const char *ax_compute_backend_name(void) { return g_active ? g_active->name : NULL; }

ax_status_t ax_compute_register_backend(ax_backend_id_t id, const ax_backend_ops_t *ops) {
    if ((int)id < 0 || id >= AX_BACKEND_COUNT) {
        ax_err_set(AX_ERR_BACKEND, "invalid backend id %d", (int)id);
        return AX_ERR_BACKEND;
    }
    if (!ops) {
        ax_err_set(AX_ERR_NULL_ARG, "null ops table");
        return AX_ERR_NULL_ARG;
    }
    g_backends[id] = ops;
    claim_device(ops);
    return AX_OK;
}

int ax_device_count(ax_device_t device) {
    if (device == AX_DEVICE_CPU) return 1;
    ensure_init();
    const ax_backend_ops_t *ops = ax_backend_for_device(device);
    return (ops && ops->device_count) ? ops->device_count() : 0;
}

void ax_device_synchronize(ax_device_t device) {
    if (device == AX_DEVICE_CPU) return;
    ensure_init();
    const ax_backend_ops_t *ops = ax_backend_for_device(device);
    if (ops && ops->synchronize) ops->synchronize();
}

int ax_device_is_available(ax_device_t device) {
    if (device == AX_DEVICE_CPU) return 1;
    ensure_init();
    return ax_backend_for_device(device) != NULL && ax_device_count(device) > 0;
}

/* Common prologue/epilogue of a wrapper: lazy init, active-backend and slot checks, then the
 * generation bump that lets caches keyed on a storage pointer notice in-place writes. */
#define AX_DISPATCH(slot, out_tensor, call)                                                     \
    do {                                                                                        \
        ensure_init();                                                                          \
        if (!g_active) {                                                                        \
            ax_err_set(AX_ERR_BACKEND, "compute not initialized (no usable backend)");          \
            return AX_ERR_BACKEND;                                                              \
        }                                                                                       \
        if (!g_active->slot) {                                                                  \
            ax_err_set(AX_ERR_NOT_IMPLEMENTED, #slot " not implemented in %s", g_active->name); \
            return AX_ERR_NOT_IMPLEMENTED;                                                      \
        }                                                                                       \
        ax_status_t st_ = g_active->call;                                                       \
        if (st_ == AX_OK && (out_tensor) && (out_tensor)->storage) (out_tensor)->storage->generation++; \
        return st_;                                                                             \
    } while (0)

ax_status_t ax_compute_gemm(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { AX_DISPATCH(gemm, out, gemm(a, b, out)); }
ax_status_t ax_compute_gemm_nt(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { AX_DISPATCH(gemm_nt, out, gemm_nt(a, b, out)); }
ax_status_t ax_compute_gemm_tn(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { AX_DISPATCH(gemm_tn, out, gemm_tn(a, b, out)); }
ax_status_t ax_compute_gemm_relu(const ax_tensor_t *a, const ax_tensor_t *b, const ax_tensor_t *bias, ax_tensor_t *out) { AX_DISPATCH(gemm_relu, out, gemm_relu(a, b, bias, out)); }
ax_status_t ax_compute_gemm_ex(const ax_tensor_t *a, const ax_tensor_t *b, float alpha, float beta, ax_tensor_t *out) { AX_DISPATCH(gemm_ex, out, gemm_ex(a, b, alpha, beta, out)); }
ax_status_t ax_compute_bias_add(const ax_tensor_t *in, const ax_tensor_t *bias, int axis, ax_tensor_t *out) { AX_DISPATCH(bias_add, out, bias_add(in, bias, axis, out)); }
ax_status_t ax_compute_relu(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(relu, out, relu(in, out)); }
ax_status_t ax_compute_gelu(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(gelu_op, out, gelu_op(in, out)); }
ax_status_t ax_compute_fill(ax_tensor_t *t, double value) { AX_DISPATCH(fill, t, fill(t, value)); }
ax_status_t ax_compute_copy(const ax_tensor_t *src, ax_tensor_t *dst) { AX_DISPATCH(copy, dst, copy(src, dst)); }
ax_status_t ax_compute_sum(const ax_tensor_t *in, int axis, ax_tensor_t *out) { AX_DISPATCH(sum, out, sum(in, axis, out)); }
ax_status_t ax_compute_axpy(const ax_tensor_t *x, float alpha, ax_tensor_t *y) { AX_DISPATCH(axpy, y, axpy(x, alpha, y)); }
/* the remaining wrappers of src/compute/dispatch.c:385-412, 657-721, 762-841 */
ax_status_t ax_compute_add(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { AX_DISPATCH(add, out, add(a, b, out)); }
ax_status_t ax_compute_sub(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { AX_DISPATCH(sub, out, sub(a, b, out)); }
ax_status_t ax_compute_mul(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { AX_DISPATCH(mul, out, mul(a, b, out)); }
ax_status_t ax_compute_div(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { AX_DISPATCH(div_op, out, div_op(a, b, out)); }
ax_status_t ax_compute_equal(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { AX_DISPATCH(equal, out, equal(a, b, out)); }
ax_status_t ax_compute_greater(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { AX_DISPATCH(greater, out, greater(a, b, out)); }
ax_status_t ax_compute_add_relu(const ax_tensor_t *a, const ax_tensor_t *b, ax_tensor_t *out) { AX_DISPATCH(add_relu, out, add_relu(a, b, out)); }
ax_status_t ax_compute_neg(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(neg, out, neg(in, out)); }
ax_status_t ax_compute_abs(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(abs_op, out, abs_op(in, out)); }
ax_status_t ax_compute_exp(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(exp_op, out, exp_op(in, out)); }
ax_status_t ax_compute_log(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(log_op, out, log_op(in, out)); }
ax_status_t ax_compute_sqrt(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(sqrt_op, out, sqrt_op(in, out)); }
ax_status_t ax_compute_square(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(square, out, square(in, out)); }
ax_status_t ax_compute_sigmoid(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(sigmoid, out, sigmoid(in, out)); }
ax_status_t ax_compute_tanh(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(tanh_op, out, tanh_op(in, out)); }
ax_status_t ax_compute_add_scalar(const ax_tensor_t *in, double scalar, ax_tensor_t *out) { AX_DISPATCH(add_scalar, out, add_scalar(in, scalar, out)); }
ax_status_t ax_compute_mul_scalar(const ax_tensor_t *in, double scalar, ax_tensor_t *out) { AX_DISPATCH(mul_scalar, out, mul_scalar(in, scalar, out)); }
ax_status_t ax_compute_softmax_rowwise(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(softmax_rowwise, out, softmax_rowwise(in, out)); }
ax_status_t ax_compute_mean(const ax_tensor_t *in, int axis, ax_tensor_t *out) { AX_DISPATCH(mean, out, mean(in, axis, out)); }
ax_status_t ax_compute_max(const ax_tensor_t *in, int axis, ax_tensor_t *out) { AX_DISPATCH(max_op, out, max_op(in, axis, out)); }
ax_status_t ax_compute_min(const ax_tensor_t *in, int axis, ax_tensor_t *out) { AX_DISPATCH(min_op, out, min_op(in, axis, out)); }
ax_status_t ax_compute_argmax(const ax_tensor_t *in, int axis, ax_tensor_t *out) { AX_DISPATCH(argmax, out, argmax(in, axis, out)); }
ax_status_t ax_compute_adam_update(ax_tensor_t *weight, ax_tensor_t *grad, ax_tensor_t *m, ax_tensor_t *v, float lr,
                                   float beta1, float beta2, float eps, float weight_decay, float bc1, float bc2,
                                   bool decoupled) {
    AX_DISPATCH(adam_update, weight, adam_update(weight, grad, m, v, lr, beta1, beta2, eps, weight_decay, bc1, bc2, decoupled));
}
ax_status_t ax_compute_sgd_update(ax_tensor_t *weight, ax_tensor_t *grad, ax_tensor_t *momentum_buf, float lr,
                                  float momentum, float weight_decay, bool nesterov) {
    AX_DISPATCH(sgd_update, weight, sgd_update(weight, grad, momentum_buf, lr, momentum, weight_decay, nesterov));
}
/* the three activation slots the reference's dispatch layer has no wrapper for */
ax_status_t ax_compute_leaky_relu(const ax_tensor_t *in, float alpha, ax_tensor_t *out) { AX_DISPATCH(leaky_relu, out, leaky_relu(in, alpha, out)); }
ax_status_t ax_compute_elu(const ax_tensor_t *in, float alpha, ax_tensor_t *out) { AX_DISPATCH(elu_op, out, elu_op(in, alpha, out)); }
ax_status_t ax_compute_swish(const ax_tensor_t *in, ax_tensor_t *out) { AX_DISPATCH(swish_op, out, swish_op(in, out)); }
ax_status_t ax_compute_gemm_bias_act(const ax_tensor_t *a, const ax_tensor_t *b, const ax_tensor_t *bias,
                                     ax_activation_t act, ax_tensor_t *out) {
    AX_DISPATCH(gemm_bias_act, out, gemm_bias_act(a, b, bias, (int)act, out));
}

ax_status_t ax_compute_gemm_act_head(const ax_tensor_t *a, const ax_tensor_t *b, const ax_tensor_t *bias, ax_activation_t act,
                                     const ax_tensor_t *w2, const ax_tensor_t *bias2, ax_activation_t act2, ax_tensor_t *out2) {
    AX_DISPATCH(gemm_act_head, out2, gemm_act_head(a, b, bias, (int)act, w2, bias2, (int)act2, out2));
}

ax_status_t ax_compute_layernorm(const ax_tensor_t *x, const ax_tensor_t *gamma, const ax_tensor_t *beta, float eps,
                                 ax_tensor_t *out, ax_tensor_t *x_hat, ax_tensor_t *inv_std) {
    AX_DISPATCH(layernorm_fwd, out, layernorm_fwd(x, gamma, beta, eps, out, x_hat, inv_std));
}

#define AX_HAS(slot) (ensure_init(), (g_active && g_active->slot) ? 1 : 0)
int ax_compute_has_gemm_relu(void) { return AX_HAS(gemm_relu); }
int ax_compute_has_gemm_nt(void) { return AX_HAS(gemm_nt); }
int ax_compute_has_gemm_tn(void) { return AX_HAS(gemm_tn); }
int ax_compute_has_gemm_ex(void) { return AX_HAS(gemm_ex); }
int ax_compute_has_bias_add(void) { return AX_HAS(bias_add); }
int ax_compute_has_gemm_bias_act(void) { return AX_HAS(gemm_bias_act); }
int ax_compute_has_gemm_act_head(void) { return AX_HAS(gemm_act_head); }
int ax_compute_has_adam_update(void) { return AX_HAS(adam_update); }
int ax_compute_has_sgd_update(void) { return AX_HAS(sgd_update); }
