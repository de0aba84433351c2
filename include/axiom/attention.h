/* axiom/attention.h — the multi-head self-attention layer, forward only (include/axiom/attention.h:59-98,
 * src/core/attention.c:121-430, 952-1030).  Struct layout, parameter order (Wq, Wk, Wv, Wo, then
 * bq, bk, bv, bo when use_bias) and initialisation (Xavier-uniform weights, zero biases) are the
 * reference's, so its model files load into this layer.  Input and output are [B, S, d_model]. */
#ifndef AX_ATTENTION_H
#define AX_ATTENTION_H
#include "layer.h"
#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    ax_layer_t base;
    int64_t d_model;
    int n_heads;
    int64_t d_k;                       /* d_model / n_heads */
    bool use_bias;
    bool causal;
    ax_tensor_t *Wq, *Wk, *Wv, *Wo;    /* each [d_model, d_model] */
    ax_tensor_t *bq, *bk, *bv, *bo;    /* each [d_model], NULL without bias */
    /* fused [d_model, 3 d_model] projection and [3 d_model] bias, rebuilt when a projection's
     * storage generation has moved (src/core/attention/cache.c:24-85) */
    ax_tensor_t *Wqkv_cache, *bqkv_cache;
    uint64_t Wq_gen, Wk_gen, Wv_gen;
    /* appended after the reference's last member: the generations the fused bias was built from
     * (the reference rebuilds it on every forward, which on a device is a kernel launch) */
    uint64_t bq_gen, bk_gen, bv_gen;
} ax_mha_t;

ax_layer_t *ax_mha_create(int64_t d_model, int n_heads, bool use_bias, bool causal);

#ifdef __cplusplus
}
#endif
#endif
