/* Multi-head self-attention layer, forward pass (Axiom's src/core/attention.c:121-430 for a tensor
 * on a GPU device): fused QKV projection as one GEMM, head split (+ bias) through the extension
 * table, attention forward through its sdpa_fwd member, head merge, output projection with the
 * column bias.  Every step runs on the device that holds the input. */
#include <math.h>
#include <stdlib.h>

#include "axiom/attention.h"
#include "axiom/compute.h"
#include "axiom/error.h"
#include "axiom/init.h"
#include "axiom/internal/cuda_extension.h"

static float *dev_ptr(const ax_tensor_t *t) { return (float *)t->storage->data + t->offset; }

static ax_tensor_t *on_device_of(const ax_tensor_t *like, const int64_t *shape, int ndim) {
    ax_device_t prev = ax_get_default_device();
    ax_set_default_device(like->storage->device);
    ax_tensor_t *t = ax_tensor_create(shape, ndim, AX_FLOAT32);
    ax_set_default_device(prev);
    return t;
}

/* src/core/attention/cache.c:24-85 */
static ax_status_t refresh_fused_qkv(ax_mha_t *m, const ax_cuda_extension_t *ext) {
    const int64_t D = m->d_model;
    const uint64_t gq = m->Wq->storage->generation, gk = m->Wk->storage->generation, gv = m->Wv->storage->generation;
    if (!m->Wqkv_cache || gq != m->Wq_gen || gk != m->Wk_gen || gv != m->Wv_gen) {
        if (!m->Wqkv_cache) {
            int64_t sh[2] = {D, 3 * D};
            if (!(m->Wqkv_cache = on_device_of(m->Wq, sh, 2))) return AX_ERR_ALLOC;
        }
        ax_status_t st = ext->qkv_cache_build(dev_ptr(m->Wqkv_cache), dev_ptr(m->Wq), dev_ptr(m->Wk), dev_ptr(m->Wv), D);
        if (st != AX_OK) return st;
        m->Wqkv_cache->storage->generation++;
        m->Wq_gen = gq;
        m->Wk_gen = gk;
        m->Wv_gen = gv;
    }
    if (m->use_bias) {
        /* the reference rebuilds the bias on every call (cache.c:67-84: "cheap"); here that is a
         * kernel launch, so it follows the generations like the weights */
        const uint64_t bq = m->bq->storage->generation, bk = m->bk->storage->generation, bv = m->bv->storage->generation;
        if (!m->bqkv_cache || bq != m->bq_gen || bk != m->bk_gen || bv != m->bv_gen) {
            if (!m->bqkv_cache) {
                int64_t sh[1] = {3 * D};
                if (!(m->bqkv_cache = on_device_of(m->Wq, sh, 1))) return AX_ERR_ALLOC;
            }
            ax_status_t st = ext->bias_cache_build(dev_ptr(m->bqkv_cache), dev_ptr(m->bq), dev_ptr(m->bk), dev_ptr(m->bv), D);
            if (st != AX_OK) return st;
            m->bqkv_cache->storage->generation++;
            m->bq_gen = bq;
            m->bk_gen = bk;
            m->bv_gen = bv;
        }
    }
    return AX_OK;
}

/* Head sizes the fused kernel covers (multiples of 4 up to 128): attention reads the heads where the
 * projection wrote them (columns h*dk.. of the q, k and v thirds of qkv) and writes them where the
 * output projection reads them, so the three layout passes of attention.c:211-262, 391-400 and their
 * four [B*H, S, dk] temporaries fall away; the projection bias moves into the GEMM write-back. */
static ax_status_t attend_on_projection(ax_mha_t *m, const ax_cuda_extension_t *ext, ax_tensor_t *x_flat, ax_tensor_t *qkv,
                                        ax_tensor_t *attn, int64_t B, int64_t S) {
    const int64_t D = m->d_model;
    ax_status_t st = m->use_bias ? ax_compute_gemm_bias_act(x_flat, m->Wqkv_cache, m->bqkv_cache, AX_ACT_NONE, qkv)
                                 : ax_compute_gemm(x_flat, m->Wqkv_cache, qkv);
    if (st != AX_OK) return st;
    return ext->sdpa_fwd_rows(dev_ptr(qkv), dev_ptr(qkv) + D, dev_ptr(qkv) + 2 * D, 3 * D, dev_ptr(attn), D, NULL, B, m->n_heads,
                              S, m->d_k, 1.0f / sqrtf((float)m->d_k), m->causal);
}

/* The reference's own sequence (attention.c:211-262, 391-400): projection, split into one matrix per head
 * (adding the fused bias), attention per head, merge back to [B*S, D]. */
static ax_status_t attend_per_head(ax_mha_t *m, const ax_cuda_extension_t *ext, ax_tensor_t *x_flat, ax_tensor_t *qkv,
                                   ax_tensor_t *attn, int64_t B, int64_t S) {
    const int64_t D = m->d_model, H = m->n_heads, dk = m->d_k;
    int64_t head_sh[3] = {B * H, S, dk};
    ax_tensor_t *heads[4] = {NULL, NULL, NULL, NULL};         /* Q, K, V, O as [B*H, S, dk] */
    ax_status_t st = AX_OK;
    for (int i = 0; i < 4 && st == AX_OK; i++)
        if (!(heads[i] = on_device_of(x_flat, head_sh, 3))) st = AX_ERR_ALLOC;
    if (st == AX_OK) st = ax_compute_gemm(x_flat, m->Wqkv_cache, qkv);
    if (st == AX_OK) {
        ax_err_clear();                                      /* the layout members return nothing: read the error state */
        if (m->use_bias)
            ext->head_interleave_qkv_split_bias(dev_ptr(qkv), dev_ptr(m->bqkv_cache), dev_ptr(heads[0]), dev_ptr(heads[1]),
                                                dev_ptr(heads[2]), B, S, H, dk, D);
        else
            ext->head_interleave_qkv_split(dev_ptr(qkv), dev_ptr(heads[0]), dev_ptr(heads[1]), dev_ptr(heads[2]), B, S, H, dk, D);
        st = ax_err_last_status();
    }
    if (st == AX_OK)
        st = ext->sdpa_fwd(dev_ptr(heads[0]), dev_ptr(heads[1]), dev_ptr(heads[2]), dev_ptr(heads[3]), NULL, B * H, S, dk,
                           1.0f / sqrtf((float)dk), m->causal, NULL);
    if (st == AX_OK) {
        ext->head_deinterleave(dev_ptr(heads[3]), dev_ptr(attn), B, S, H, dk);
        st = ax_err_last_status();
    }
    for (int i = 0; i < 4; i++) ax_tensor_destroy(heads[i]);
    return st;
}

static ax_tensor_t *mha_forward(ax_layer_t *self, ax_tensor_t *x) {
    ax_mha_t *m = (ax_mha_t *)self;
    if (!x || x->ndim != 3 || x->dtype != AX_FLOAT32 || x->shape[2] != m->d_model) {
        ax_err_set(AX_ERR_SHAPE_MISMATCH, "mha: input must be float32 [B, S, %lld]", (long long)m->d_model);
        return NULL;
    }
    const ax_cuda_extension_t *ext = ax_compute_get_cuda_extension();
    if (x->storage->device == AX_DEVICE_CPU || !ext || !ext->sdpa_fwd || !ext->head_interleave_qkv_split ||
        !ext->head_interleave_qkv_split_bias || !ext->head_deinterleave || !ext->qkv_cache_build || !ext->bias_cache_build) {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "mha: needs a device tensor and a registered GPU extension table");
        return NULL;
    }
    if (!ax_tensor_is_contiguous(x) || m->Wq->storage->device != x->storage->device) {
        ax_err_set(AX_ERR_BACKEND, "mha: input must be contiguous and on the device that holds the weights");
        return NULL;
    }
    const int64_t B = x->shape[0], S = x->shape[1], D = m->d_model, dk = m->d_k, rows = B * S;
    ax_tensor_t *x_flat = NULL, *qkv = NULL, *attn = NULL, *out_flat = NULL, *out = NULL;
    int64_t flat_sh[2] = {rows, D}, qkv_sh[2] = {rows, 3 * D};
    ax_status_t st = refresh_fused_qkv(m, ext);
    if (st == AX_OK && (!(x_flat = ax_tensor_reshape(x, flat_sh, 2)) || !(qkv = on_device_of(x, qkv_sh, 2)) ||
                        !(attn = on_device_of(x, flat_sh, 2)) || !(out_flat = on_device_of(x, flat_sh, 2))))
        st = AX_ERR_ALLOC;
    if (st == AX_OK) {
        const bool on_projection = ext->sdpa_fwd_rows && dk % 4 == 0 && dk <= 128 &&
                                   (!m->use_bias || ax_compute_has_gemm_bias_act());
        st = on_projection ? attend_on_projection(m, ext, x_flat, qkv, attn, B, S)
                           : attend_per_head(m, ext, x_flat, qkv, attn, B, S);
    }
    if (st == AX_OK) {                                       /* attention.c:402-417: gemm, then bias along axis 1 */
        if (m->use_bias && ax_compute_has_gemm_bias_act()) st = ax_compute_gemm_bias_act(attn, m->Wo, m->bo, AX_ACT_NONE, out_flat);
        else {
            st = ax_compute_gemm(attn, m->Wo, out_flat);
            if (st == AX_OK && m->use_bias) st = ax_compute_bias_add(out_flat, m->bo, 1, out_flat);
        }
    }
    if (st == AX_OK) out = ax_tensor_reshape(out_flat, x->shape, 3);
    ax_tensor_destroy(x_flat);
    ax_tensor_destroy(qkv);
    ax_tensor_destroy(attn);
    ax_tensor_destroy(out_flat);
    return out;
}

static void mha_destroy(ax_layer_t *self) {
    ax_mha_t *m = (ax_mha_t *)self;
    ax_tensor_t *all[10] = {m->Wq, m->Wk, m->Wv, m->Wo, m->bq, m->bk, m->bv, m->bo, m->Wqkv_cache, m->bqkv_cache};
    for (int i = 0; i < 10; i++) ax_tensor_destroy(all[i]);
    free(m);
}

ax_layer_t *ax_mha_create(int64_t d_model, int n_heads, bool use_bias, bool causal) {
    if (d_model <= 0 || n_heads <= 0) return NULL;
    if (d_model % n_heads != 0) {
        ax_err_set(AX_ERR_INVALID_SHAPE, "ax_mha_create: d_model=%lld must be divisible by n_heads=%d", (long long)d_model,
                   n_heads);
        return NULL;
    }
    ax_mha_t *m = calloc(1, sizeof *m);
    if (!m) {
        ax_err_set(AX_ERR_ALLOC, "ax_mha_create: out of memory");
        return NULL;
    }
    m->base.ops.forward = mha_forward;
    m->base.ops.destroy = mha_destroy;
    m->base.type = AX_LAYER_MHA;
    m->base.training = true;
    m->base.input_features = m->base.output_features = d_model;
    m->d_model = d_model;
    m->n_heads = n_heads;
    m->d_k = d_model / n_heads;
    m->use_bias = use_bias;
    m->causal = causal;
    int64_t ws[2] = {d_model, d_model};
    ax_tensor_t **w[4] = {&m->Wq, &m->Wk, &m->Wv, &m->Wo};
    for (int i = 0; i < 4; i++) {                            /* drawn in this order: attention.c:980-992 */
        if (!(*w[i] = ax_tensor_create(ws, 2, AX_FLOAT32))) {
            mha_destroy(&m->base);
            return NULL;
        }
    }
    for (int i = 0; i < 4; i++) {
        ax_init_xavier_uniform(*w[i], d_model, d_model);
        (*w[i])->requires_grad = true;
        m->base.params[i] = *w[i];
    }
    m->base.n_params = 4;
    if (use_bias) {
        ax_tensor_t **b[4] = {&m->bq, &m->bk, &m->bv, &m->bo};
        for (int i = 0; i < 4; i++) {
            if (!(*b[i] = ax_tensor_zeros(&d_model, 1, AX_FLOAT32))) {
                mha_destroy(&m->base);
                return NULL;
            }
            (*b[i])->requires_grad = true;
            m->base.params[4 + i] = *b[i];
        }
        m->base.n_params = 8;
    }
    return &m->base;
}
