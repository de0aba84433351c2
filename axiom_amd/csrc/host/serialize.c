/* Model, tensor and quantized-weight files (Axiom's src/core/serialize.c; formats in
 * axiom/serialize.h).  Reading treats the file as untrusted: counts, extents and sizes are
 * checked before use, a tensor is capped at 2 GiB (serialize.c:56), the trailing CRC-32 must
 * match.  Parameters pass through a host staging buffer to and from the device that holds them. */
#include <inttypes.h>
#include <limits.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "axiom/attention.h"
#include "axiom/error.h"
#include "axiom/serialize.h"

#define TENSOR_MAGIC 0x41585430u                 /* "AXT0" */
#define QWEIGHT_MAGIC 0x41585130u                /* "AXQ0" */
#define MAX_TENSOR_BYTES ((size_t)2u * 1024u * 1024u * 1024u)

/* ---- CRC-32, reflected polynomial 0xEDB88320 (serialize.c:60-90) ---- */
static uint32_t crc_table[256];
static int crc_table_ready;

static uint32_t crc32_update(uint32_t crc, const void *data, size_t len) {
    if (!crc_table_ready) {
        for (uint32_t i = 0; i < 256; i++) {
            uint32_t c = i;
            for (int j = 0; j < 8; j++) c = (c & 1) ? (0xEDB88320u ^ (c >> 1)) : (c >> 1);
            crc_table[i] = c;
        }
        crc_table_ready = 1;
    }
    const uint8_t *p = data;
    crc = ~crc;
    for (size_t i = 0; i < len; i++) crc = crc_table[(crc ^ p[i]) & 0xFF] ^ (crc >> 8);
    return ~crc;
}

/* a file being read or written with a running checksum of the bytes that passed */
typedef struct {
    FILE *f;
    uint32_t crc;
    bool ok;
} stream_t;

static void put(stream_t *s, const void *data, size_t len) {
    if (!s->ok) return;
    if (len && fwrite(data, 1, len, s->f) != len) s->ok = false;
    else s->crc = crc32_update(s->crc, data, len);
}
static void put_u32(stream_t *s, uint32_t v) { put(s, &v, 4); }
static void put_i64(stream_t *s, int64_t v) { put(s, &v, 8); }
static void put_f32(stream_t *s, float v) { put(s, &v, 4); }
static void put_u8(stream_t *s, uint8_t v) { put(s, &v, 1); }

static bool get(stream_t *s, void *data, size_t len) {
    if (!s->ok) return false;
    if (len && fread(data, 1, len, s->f) != len) return s->ok = false;
    s->crc = crc32_update(s->crc, data, len);
    return true;
}
static bool get_u32(stream_t *s, uint32_t *v) { return get(s, v, 4); }
static bool get_i64(stream_t *s, int64_t *v) { return get(s, v, 8); }
static bool get_f32(stream_t *s, float *v) { return get(s, v, 4); }
static bool get_u8(stream_t *s, uint8_t *v) { return get(s, v, 1); }

/* ---- tensor records ---- */
static void put_tensor(stream_t *s, const ax_tensor_t *t) {
    put_u32(s, (uint32_t)t->dtype);
    put_u32(s, (uint32_t)t->ndim);
    for (int i = 0; i < t->ndim; i++) put_i64(s, t->shape[i]);
    const size_t bytes = (size_t)ax_tensor_numel(t) * ax_dtype_size(t->dtype);
    if (!s->ok || !bytes) return;
    if (!ax_tensor_is_contiguous(t)) {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "saving a non-contiguous tensor");
        s->ok = false;
        return;
    }
    if (t->storage->device == AX_DEVICE_CPU) {
        put(s, (const char *)t->storage->data + (size_t)t->offset * ax_dtype_size(t->dtype), bytes);
        return;
    }
    void *host = malloc(bytes);
    if (!host || ax_tensor_read(t, host, bytes) != AX_OK) s->ok = false;
    else put(s, host, bytes);
    free(host);
}

/* header of a tensor record, validated (serialize.c:189-245); returns the payload size */
static bool get_tensor_header(stream_t *s, ax_dtype_t *dtype, int *ndim, int64_t *shape, size_t *bytes) {
    uint32_t dt, nd;
    if (!get_u32(s, &dt) || !get_u32(s, &nd)) return false;
    if (dt >= AX_DTYPE_COUNT) {
        ax_err_set(AX_ERR_INVALID_DTYPE, "invalid dtype %u in file (max %d)", dt, AX_DTYPE_COUNT - 1);
        return false;
    }
    if (nd > AX_MAX_DIMS) {
        ax_err_set(AX_ERR_INVALID_SHAPE, "ndim %u exceeds AX_MAX_DIMS (%d)", nd, AX_MAX_DIMS);
        return false;
    }
    uint64_t numel = 1;
    const size_t esz = ax_dtype_size((ax_dtype_t)dt);
    for (uint32_t i = 0; i < nd; i++) {
        if (!get_i64(s, &shape[i])) return false;
        if (shape[i] <= 0) {
            ax_err_set(AX_ERR_INVALID_SHAPE, "shape[%u] = %" PRId64 " is non-positive in file", i, shape[i]);
            return false;
        }
        if ((uint64_t)shape[i] > MAX_TENSOR_BYTES || numel * (uint64_t)shape[i] * esz > MAX_TENSOR_BYTES) {
            ax_err_set(AX_ERR_INVALID_SHAPE, "tensor too large for deserialization (max %zu bytes)", MAX_TENSOR_BYTES);
            return false;
        }
        numel *= (uint64_t)shape[i];
    }
    *dtype = (ax_dtype_t)dt;
    *ndim = (int)nd;
    *bytes = (size_t)numel * esz;
    return true;
}

/* reads one record's payload into a fresh host buffer (caller frees) */
static void *get_payload(stream_t *s, size_t bytes) {
    void *host = malloc(bytes ? bytes : 1);
    if (!host) {
        ax_err_set(AX_ERR_ALLOC, "out of memory reading %zu bytes", bytes);
        s->ok = false;
        return NULL;
    }
    if (!get(s, host, bytes)) {
        free(host);
        return NULL;
    }
    return host;
}

ax_status_t ax_tensor_save(ax_tensor_t *t, const char *path) {
    if (!t || !path) {
        ax_err_set(AX_ERR_NULL_ARG, "null tensor or path");
        return AX_ERR_NULL_ARG;
    }
    stream_t s = {fopen(path, "wb"), 0, true};
    if (!s.f) {
        ax_err_set(AX_ERR_INTERNAL, "cannot open %s for writing", path);
        return AX_ERR_INTERNAL;
    }
    put_u32(&s, TENSOR_MAGIC);
    put_tensor(&s, t);
    if (fclose(s.f) != 0) s.ok = false;
    if (!s.ok) {
        ax_err_set(AX_ERR_INTERNAL, "write failed");
        return AX_ERR_INTERNAL;
    }
    return AX_OK;
}

ax_tensor_t *ax_tensor_load(const char *path) {
    if (!path) return NULL;
    stream_t s = {fopen(path, "rb"), 0, true};
    if (!s.f) {
        ax_err_set(AX_ERR_INTERNAL, "cannot open %s for reading", path);
        return NULL;
    }
    uint32_t magic;
    ax_tensor_t *t = NULL;
    if (!get_u32(&s, &magic) || magic != TENSOR_MAGIC) {
        ax_err_set(AX_ERR_INTERNAL, "not a valid axiom tensor file");
    } else {
        ax_dtype_t dtype;
        int ndim;
        int64_t shape[AX_MAX_DIMS];
        size_t bytes;
        void *host = NULL;
        if (get_tensor_header(&s, &dtype, &ndim, shape, &bytes) && (host = get_payload(&s, bytes))) {
            t = ax_tensor_from_array(host, shape, ndim, dtype);
            free(host);
        }
    }
    fclose(s.f);
    return t;
}

/* ---- model files ---- */
static ax_status_t refuse_layer(ax_layer_type_t type, int index) {
    ax_err_set(AX_ERR_NOT_IMPLEMENTED, "layer %d: layer type %d has no forward pass in this library", index, (int)type);
    return AX_ERR_NOT_IMPLEMENTED;
}

ax_status_t ax_model_save(ax_model_t *model, const char *path) {
    if (!model || !model->net || !path) {
        ax_err_set(AX_ERR_NULL_ARG, "null model or path");
        return AX_ERR_NULL_ARG;
    }
    if (model->net->type != AX_LAYER_SEQUENTIAL) {
        ax_err_set(AX_ERR_NOT_IMPLEMENTED, "only sequential models can be saved");
        return AX_ERR_NOT_IMPLEMENTED;
    }
    ax_sequential_t *seq = (ax_sequential_t *)model->net;
    for (int i = 0; i < seq->n_layers; i++) {
        switch (seq->layers[i]->type) {
            case AX_LAYER_DENSE: case AX_LAYER_RELU: case AX_LAYER_SIGMOID: case AX_LAYER_TANH:
            case AX_LAYER_LEAKY_RELU: case AX_LAYER_ELU: case AX_LAYER_GELU: case AX_LAYER_SWISH:
            case AX_LAYER_SOFTMAX: case AX_LAYER_LAYERNORM: case AX_LAYER_MHA: break;
            default: return refuse_layer(seq->layers[i]->type, i);
        }
    }
    stream_t s = {fopen(path, "wb"), 0, true};
    if (!s.f) {
        ax_err_set(AX_ERR_INTERNAL, "cannot open %s for writing", path);
        return AX_ERR_INTERNAL;
    }
    put_u32(&s, AX_MAGIC);
    put_u32(&s, AX_FORMAT_VERSION);
    put_u32(&s, (uint32_t)seq->n_layers);
    for (int i = 0; i < seq->n_layers; i++) {                 /* descriptors: serialize.c:350-430 */
        ax_layer_t *l = seq->layers[i];
        put_u32(&s, (uint32_t)l->type);
        put_u32(&s, (uint32_t)l->n_params);
        put_u32(&s, (uint32_t)l->n_buffers);
        switch (l->type) {
            case AX_LAYER_DENSE:
                put_i64(&s, l->input_features);
                put_i64(&s, l->output_features);
                put_u8(&s, ((ax_dense_t *)l)->use_bias ? 1 : 0);
                break;
            case AX_LAYER_LAYERNORM:
                put_i64(&s, ((ax_layernorm_t *)l)->num_features);
                put_f32(&s, ((ax_layernorm_t *)l)->eps);
                break;
            case AX_LAYER_LEAKY_RELU: case AX_LAYER_ELU:
                put_f32(&s, ((ax_activation_layer_t *)l)->alpha);
                break;
            case AX_LAYER_SOFTMAX:
                put_u32(&s, 1);                               /* the reference writes a constant 1 here */
                break;
            case AX_LAYER_MHA: {
                const ax_mha_t *mh = (const ax_mha_t *)l;
                put_i64(&s, mh->d_model);
                put_u32(&s, (uint32_t)mh->n_heads);
                put_u8(&s, mh->use_bias ? 1 : 0);
                put_u8(&s, mh->causal ? 1 : 0);
                break;
            }
            default: break;
        }
    }
    for (int i = 0; i < seq->n_layers && s.ok; i++) {
        ax_layer_t *l = seq->layers[i];
        for (int p = 0; p < l->n_params; p++) put_tensor(&s, l->params[p]);
        for (int p = 0; p < l->n_buffers; p++) put_tensor(&s, l->buffers[p]);
    }
    const uint32_t crc = s.crc;
    put_u32(&s, crc);                                         /* not part of the checksum itself */
    if (fclose(s.f) != 0) s.ok = false;
    if (!s.ok) {
        if (ax_err_last_status() == AX_OK) ax_err_set(AX_ERR_INTERNAL, "failed writing %s", path);
        return AX_ERR_INTERNAL;
    }
    return AX_OK;
}

/* rows x cols floats stay under the per-tensor cap; each factor is bounded first so the product
 * cannot wrap (extents come straight from the file) */
static bool floats_fit(int64_t rows, int64_t cols) {
    const uint64_t cap = MAX_TENSOR_BYTES / 4;
    return rows > 0 && cols > 0 && (uint64_t)rows <= cap && (uint64_t)cols <= cap && (uint64_t)rows * (uint64_t)cols <= cap;
}

/* one layer from its descriptor (serialize.c:540-660); NULL with the error set */
static ax_layer_t *read_layer(stream_t *s, uint32_t type, uint32_t index) {
    switch (type) {
        case AX_LAYER_DENSE: {
            int64_t in_f, out_f;
            uint8_t bias;
            if (!get_i64(s, &in_f) || !get_i64(s, &out_f) || !get_u8(s, &bias)) return NULL;
            if (!floats_fit(in_f, out_f)) {
                ax_err_set(AX_ERR_INVALID_SHAPE, "layer %u: dense %" PRId64 " x %" PRId64 " is not acceptable", index, in_f, out_f);
                return NULL;
            }
            return ax_dense_create(in_f, out_f, bias & 1);
        }
        case AX_LAYER_LAYERNORM: {
            int64_t nf;
            float eps;
            if (!get_i64(s, &nf) || !get_f32(s, &eps)) return NULL;
            if (!floats_fit(nf, 1)) {
                ax_err_set(AX_ERR_INVALID_SHAPE, "layer %u: layernorm over %" PRId64 " features", index, nf);
                return NULL;
            }
            return ax_layernorm_create(nf, eps);
        }
        case AX_LAYER_LEAKY_RELU: case AX_LAYER_ELU: {
            float alpha;
            if (!get_f32(s, &alpha)) return NULL;
            return type == AX_LAYER_LEAKY_RELU ? ax_leaky_relu_layer_create(alpha) : ax_elu_layer_create(alpha);
        }
        case AX_LAYER_SOFTMAX: {
            uint32_t axis;
            if (!get_u32(s, &axis)) return NULL;
            return ax_softmax_layer_create((int)axis);
        }
        case AX_LAYER_MHA: {
            int64_t d_model;
            uint32_t n_heads;
            uint8_t use_bias, causal;
            if (!get_i64(s, &d_model) || !get_u32(s, &n_heads) || !get_u8(s, &use_bias) || !get_u8(s, &causal)) return NULL;
            if (!floats_fit(d_model, d_model) || n_heads == 0 || n_heads > (uint32_t)INT_MAX ||
                d_model % (int64_t)n_heads != 0) {
                ax_err_set(AX_ERR_INVALID_SHAPE, "layer %u: attention with d_model %" PRId64 " and %u heads", index, d_model, n_heads);
                return NULL;
            }
            return ax_mha_create(d_model, (int)n_heads, use_bias & 1, causal & 1);
        }
        case AX_LAYER_RELU: return ax_relu_layer_create();
        case AX_LAYER_SIGMOID: return ax_sigmoid_layer_create();
        case AX_LAYER_TANH: return ax_tanh_layer_create();
        case AX_LAYER_GELU: return ax_gelu_layer_create();
        case AX_LAYER_SWISH: return ax_swish_layer_create();
        default:
            if (type < AX_LAYER_TYPE_COUNT) refuse_layer((ax_layer_type_t)type, (int)index);
            else ax_err_set(AX_ERR_INTERNAL, "unknown layer type %u at layer %u", type, index);
            return NULL;
    }
}

ax_model_t *ax_model_load(const char *path) {
    if (!path) return NULL;
    stream_t s = {fopen(path, "rb"), 0, true};
    if (!s.f) {
        ax_err_set(AX_ERR_INTERNAL, "cannot open %s", path);
        return NULL;
    }
    ax_layer_t *seq = NULL;
    uint32_t magic, version, n_layers;
    uint32_t n_buffers[AX_SEQ_MAX_LAYERS] = {0};
    ax_err_clear();
    if (!get_u32(&s, &magic) || !get_u32(&s, &version) || !get_u32(&s, &n_layers)) {
        ax_err_set(AX_ERR_INTERNAL, "truncated model file header");
        goto fail;
    }
    if (magic != AX_MAGIC) {
        ax_err_set(AX_ERR_INTERNAL, "not a valid axiom model file");
        goto fail;
    }
    if (version > AX_FORMAT_VERSION) {
        ax_err_set(AX_ERR_INTERNAL, "model version %u newer than supported %u", version, AX_FORMAT_VERSION);
        goto fail;
    }
    if (n_layers == 0 || n_layers > AX_SEQ_MAX_LAYERS) {
        ax_err_set(AX_ERR_INVALID_SHAPE, "n_layers %u invalid (max %d)", n_layers, AX_SEQ_MAX_LAYERS);
        goto fail;
    }
    if (!(seq = ax_sequential_create())) goto fail;
    for (uint32_t i = 0; i < n_layers; i++) {
        uint32_t type, n_params;
        if (!get_u32(&s, &type) || !get_u32(&s, &n_params) || (version >= 3 && !get_u32(&s, &n_buffers[i]))) {
            ax_err_set(AX_ERR_INTERNAL, "truncated layer header at layer %u", i);
            goto fail;
        }
        if (n_params > AX_LAYER_MAX_PARAMS || n_buffers[i] > AX_LAYER_MAX_BUFFERS) {
            ax_err_set(AX_ERR_INVALID_SHAPE, "layer %u: %u params / %u buffers exceed the maximum", i, n_params, n_buffers[i]);
            goto fail;
        }
        ax_layer_t *layer = read_layer(&s, type, i);
        if (!layer) {
            if (ax_err_last_status() == AX_OK) ax_err_set(AX_ERR_INTERNAL, "truncated descriptor at layer %u", i);
            goto fail;
        }
        if (!ax_sequential_add(seq, layer)) {
            ax_layer_destroy(layer);
            goto fail;
        }
    }
    for (uint32_t i = 0; i < n_layers; i++) {                 /* parameter data: serialize.c:664-716 */
        ax_layer_t *layer = ((ax_sequential_t *)seq)->layers[i];
        const uint32_t records = (uint32_t)layer->n_params + n_buffers[i];
        for (uint32_t r = 0; r < records; r++) {
            ax_dtype_t dtype;
            int ndim;
            int64_t shape[AX_MAX_DIMS];
            size_t bytes;
            void *host;
            if (!get_tensor_header(&s, &dtype, &ndim, shape, &bytes) || !(host = get_payload(&s, bytes))) {
                if (ax_err_last_status() == AX_OK) ax_err_set(AX_ERR_INTERNAL, "failed reading tensor %u of layer %u", r, i);
                goto fail;
            }
            /* buffers beyond what the layer owns are read and dropped, as the reference does */
            ax_tensor_t *dst = r < (uint32_t)layer->n_params ? layer->params[r]
                               : (int)(r - (uint32_t)layer->n_params) < layer->n_buffers ? layer->buffers[r - layer->n_params] : NULL;
            ax_status_t st = AX_OK;
            if (dst) {
                const size_t want = (size_t)ax_tensor_numel(dst) * ax_dtype_size(dst->dtype);
                if (want != bytes || dtype != dst->dtype) {
                    ax_err_set(AX_ERR_SHAPE_MISMATCH, "layer %u tensor %u: expected %zu bytes, file has %zu", i, r, want, bytes);
                    st = AX_ERR_SHAPE_MISMATCH;
                } else {
                    st = ax_tensor_write(dst, host, bytes);
                }
            }
            free(host);
            if (st != AX_OK) goto fail;
        }
    }
    if (version >= 4) {
        const uint32_t computed = s.crc;
        uint32_t stored;
        if (!get_u32(&s, &stored)) {
            ax_err_set(AX_ERR_INTERNAL, "missing checksum in model file");
            goto fail;
        }
        if (stored != computed) {
            ax_err_set(AX_ERR_INTERNAL, "model file corrupted: checksum mismatch (stored 0x%08x, computed 0x%08x)", stored, computed);
            goto fail;
        }
    }
    fclose(s.f);
    ax_model_t *model = ax_model_create(seq);
    if (!model) ax_layer_destroy(seq);
    return model;
fail:
    if (seq) ax_layer_destroy(seq);
    fclose(s.f);
    return NULL;
}

/* ---- quantized weights ---- */
ax_status_t ax_qweight_save(const ax_qweight_t *qw, const char *path) {
    if (!qw || !qw->data || !qw->scales || !path || qw->N <= 0 || qw->K <= 0) {
        ax_err_set(AX_ERR_NULL_ARG, "ax_qweight_save: incomplete weights or NULL path");
        return AX_ERR_NULL_ARG;
    }
    stream_t s = {fopen(path, "wb"), 0, true};
    if (!s.f) {
        ax_err_set(AX_ERR_INTERNAL, "cannot open %s for writing", path);
        return AX_ERR_INTERNAL;
    }
    put_u32(&s, QWEIGHT_MAGIC);
    put_i64(&s, qw->N);
    put_i64(&s, qw->K);
    put(&s, qw->scales, (size_t)qw->N * sizeof(float));
    put(&s, qw->data, (size_t)qw->N * (size_t)qw->K);
    const uint32_t crc = s.crc;
    put_u32(&s, crc);
    if (fclose(s.f) != 0) s.ok = false;
    if (!s.ok) {
        ax_err_set(AX_ERR_INTERNAL, "failed writing %s", path);
        return AX_ERR_INTERNAL;
    }
    return AX_OK;
}

ax_qweight_t *ax_qweight_load(const char *path) {
    if (!path) return NULL;
    stream_t s = {fopen(path, "rb"), 0, true};
    if (!s.f) {
        ax_err_set(AX_ERR_INTERNAL, "cannot open %s", path);
        return NULL;
    }
    uint32_t magic, stored;
    int64_t N, K;
    ax_qweight_t *qw = NULL;
    if (!get_u32(&s, &magic) || magic != QWEIGHT_MAGIC || !get_i64(&s, &N) || !get_i64(&s, &K)) {
        ax_err_set(AX_ERR_INTERNAL, "not a valid quantized-weight file");
    } else if (N <= 0 || K <= 0 || (uint64_t)N > MAX_TENSOR_BYTES || (uint64_t)K > MAX_TENSOR_BYTES ||
               (uint64_t)N * (uint64_t)K > MAX_TENSOR_BYTES) {
        ax_err_set(AX_ERR_INVALID_SHAPE, "quantized weights %" PRId64 " x %" PRId64 " are not acceptable", N, K);
    } else if ((qw = calloc(1, sizeof *qw))) {
        qw->N = N;
        qw->K = K;
        qw->scales = aligned_alloc(64, ((size_t)N * sizeof(float) + 63) / 64 * 64);
        qw->data = aligned_alloc(64, ((size_t)N * (size_t)K + 63) / 64 * 64);
        if (!qw->scales || !qw->data || !get(&s, qw->scales, (size_t)N * sizeof(float)) ||
            !get(&s, qw->data, (size_t)N * (size_t)K)) {
            ax_err_set(AX_ERR_INTERNAL, "truncated quantized-weight file");
            ax_qweight_destroy(qw);
            qw = NULL;
        } else {
            const uint32_t computed = s.crc;
            if (!get_u32(&s, &stored) || stored != computed) {
                ax_err_set(AX_ERR_INTERNAL, "quantized-weight file corrupted: checksum mismatch");
                ax_qweight_destroy(qw);
                qw = NULL;
            }
        }
    }
    fclose(s.f);
    return qw;
}
