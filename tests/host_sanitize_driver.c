/* Host-side file and tensor code under AddressSanitizer + UndefinedBehaviorSanitizer (the reference's
 * CI builds its C with the same pair, CMakeLists.txt:46-65).  No GPU: everything stays on the CPU
 * device.  For every file named on the command line: load it, save it again and compare the bytes;
 * then feed the loader truncations in steps of 37 bytes (211 for files above 20 kB) and the file with one
 * bit flipped every 101 (499) bytes (each must be refused or load cleanly — never touch memory it does not own), and the
 * crafted headers of the reference's tests/test_fuzz_serialize.c.  Exit status 0 = no finding. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "axiom/axiom.h"

static unsigned char *slurp(const char *path, size_t *n) {
    FILE *f = fopen(path, "rb");
    if (!f) return NULL;
    fseek(f, 0, SEEK_END);
    long sz = ftell(f);
    fseek(f, 0, SEEK_SET);
    unsigned char *b = malloc((size_t)sz + 1);
    if (b && fread(b, 1, (size_t)sz, f) != (size_t)sz) { free(b); b = NULL; }
    fclose(f);
    *n = (size_t)sz;
    return b;
}

/* CRC-32 of zlib (reflected 0xEDB88320), bit by bit: the trailer of a model file */
static uint32_t crc32_of(const unsigned char *b, size_t n) {
    uint32_t c = 0xffffffffu;
    for (size_t i = 0; i < n; i++) {
        c ^= b[i];
        for (int k = 0; k < 8; k++) c = (c >> 1) ^ (0xedb88320u & (0u - (c & 1u)));
    }
    return ~c;
}

static int spit(const char *path, const unsigned char *b, size_t n) {
    FILE *f = fopen(path, "wb");
    if (!f) return -1;
    size_t w = fwrite(b, 1, n, f);
    fclose(f);
    return w == n ? 0 : -1;
}

static int try_load(const char *path, int is_model) {
    if (is_model) {
        ax_model_t *m = ax_model_load(path);
        if (!m) return 0;
        ax_model_destroy(m);
        return 1;
    }
    ax_tensor_t *t = ax_tensor_load(path);
    if (!t) return 0;
    ax_tensor_destroy(t);
    return 1;
}

#define EXPECT(cond)                                                              \
    do {                                                                          \
        if (!(cond)) { fprintf(stderr, "line %d: %s\n", __LINE__, #cond); bad++; } \
    } while (0)

/* Tensors, layers, model container and quantized weights on the CPU device: object lifetimes,
 * refused arguments, capacity limits.  Nothing here computes on a device; a forward pass on a host
 * tensor must come back as an error, not as a result. */
static int api_section(const char *tmp) {
    int bad = 0;
    int64_t sh2[2] = {3, 4}, sh9[9] = {1, 1, 1, 1, 1, 1, 1, 1, 1}, neg[2] = {3, -4};
    int64_t huge[3] = {INT64_MAX / 2, 4, 4}, wrap[2] = {(int64_t)1 << 62, 2}, flat[1] = {12}, wrong[1] = {13};
    EXPECT(!ax_tensor_create(NULL, 2, AX_FLOAT32));
    EXPECT(!ax_tensor_create(sh9, 9, AX_FLOAT32));
    EXPECT(!ax_tensor_create(neg, 2, AX_FLOAT32));
    EXPECT(!ax_tensor_create(huge, 3, AX_FLOAT32));
    EXPECT(!ax_tensor_create(wrap, 2, AX_FLOAT32));
    EXPECT(!ax_tensor_zeros(sh2, 2, (ax_dtype_t)99));
    EXPECT(ax_tensor_numel(NULL) == 0);
    ax_tensor_destroy(NULL);
    float vals[12];
    for (int i = 0; i < 12; i++) vals[i] = (float)i;
    ax_tensor_t *t = ax_tensor_from_array(vals, sh2, 2, AX_FLOAT32);
    EXPECT(t && ax_tensor_numel(t) == 12 && ax_tensor_is_contiguous(t));
    ax_tensor_t *v = ax_tensor_reshape(t, flat, 1);
    EXPECT(v && !ax_tensor_reshape(t, wrong, 1));
    ax_tensor_destroy(t);                                   /* the view keeps the storage alive */
    float back[12] = {0};
    EXPECT(v && ax_tensor_read(v, back, sizeof back) == AX_OK && back[11] == 11.0f);
    EXPECT(v && ax_tensor_read(v, back, sizeof back + 4) != AX_OK);
    EXPECT(v && ax_tensor_write(v, vals, sizeof vals + 4) != AX_OK);
    ax_tensor_t *copy = v ? ax_tensor_to_device(v, AX_DEVICE_CPU) : NULL;
    EXPECT(copy != NULL);
    ax_tensor_destroy(copy);
    ax_tensor_destroy(v);
    ax_set_seed(3);
    ax_tensor_t *r = ax_tensor_rand(sh2, 2, -1.0f, 1.0f);
    EXPECT(r && ax_tensor_read(r, back, sizeof back) == AX_OK && back[0] >= -1.0f && back[0] < 1.0f);

    /* layers: refused extents, a full container, a parameter list shorter than the model */
    EXPECT(!ax_dense_create(0, 5, true) && !ax_dense_create(5, -1, true) && !ax_layernorm_create(0, 1e-5f));
    EXPECT(!ax_mha_create(10, 3, true, false) && !ax_mha_create(0, 1, true, false) && !ax_mha_create(8, 0, false, false));
    ax_layer_t *seq = ax_sequential_create();
    EXPECT(seq && !ax_sequential_add(seq, NULL) && !ax_sequential_add(NULL, NULL));
    EXPECT(ax_sequential_add(seq, ax_dense_create(4, 6, true)) && ax_sequential_add(seq, ax_relu_layer_create()));
    EXPECT(ax_sequential_add(seq, ax_mha_create(6, 2, true, true)) && ax_sequential_add(seq, ax_layernorm_create(6, 1e-5f)));
    ax_layer_t *nested = ax_sequential_create();              /* a container inside a container: held, never saved */
    EXPECT(ax_sequential_add(nested, ax_dense_create(2, 2, false)) != NULL);
    ax_layer_t *(*acts[])(void) = {ax_relu_layer_create, ax_sigmoid_layer_create, ax_tanh_layer_create, ax_gelu_layer_create,
                                   ax_swish_layer_create};
    int added = 4;
    for (int i = 0; i < 100; i++) {
        ax_layer_t *l = i % 7 == 0 ? ax_leaky_relu_layer_create(0.1f) : i % 7 == 1 ? ax_elu_layer_create(1.0f)
                      : i % 7 == 2 ? ax_softmax_layer_create(-1) : acts[i % 5]();
        if (ax_sequential_add(seq, l)) added++;
        else ax_layer_destroy(l);                           /* a refused layer stays the caller's */
    }
    EXPECT(added == AX_SEQ_MAX_LAYERS);
    ax_tensor_t *few[3], *all[64];
    EXPECT(ax_layer_get_params(seq, few, 3) == 3);
    EXPECT(ax_layer_get_params(seq, all, 64) == 2 + 8 + 2 && ax_layer_get_params(NULL, all, 64) == 0);
    EXPECT(r && !ax_layer_forward(seq, r) && ax_err_last_message()[0] != 0);     /* host tensor: refused */
    EXPECT(!ax_layer_forward(NULL, r));
    ax_tensor_destroy(r);

    /* model container: owns the net; save to a directory that does not exist; load of nothing */
    ax_layer_t *outer = ax_sequential_create();
    EXPECT(ax_sequential_add(outer, nested) != NULL);
    ax_model_t *unsaveable = ax_model_create(outer);
    EXPECT(unsaveable && ax_model_save(unsaveable, tmp) != AX_OK);
    ax_model_destroy(unsaveable);
    ax_model_t *model = ax_model_create(seq);
    EXPECT(model && !ax_model_create(NULL));
    EXPECT(model && ax_model_save(model, "/nonexistent-dir/x.axm") != AX_OK);
    EXPECT(!ax_model_load("/nonexistent-dir/x.axm") && !ax_model_load(NULL));
    EXPECT(model && ax_model_save(model, tmp) == AX_OK);
    ax_model_t *again = ax_model_load(tmp);
    EXPECT(again != NULL);
    if (again) {
        ax_tensor_t *p2[64];
        ax_layer_t *net2 = *(ax_layer_t **)again;            /* ax_model_t.net is the first member */
        EXPECT(ax_layer_get_params(net2, p2, 64) == 12);
        float a[24], b[24];
        EXPECT(ax_tensor_read(all[0], a, sizeof a) == AX_OK && ax_tensor_read(p2[0], b, sizeof b) == AX_OK && !memcmp(a, b, sizeof a));
        ax_model_destroy(again);
    }
    ax_model_destroy(model);
    ax_model_destroy(NULL);

    /* quantized weights: quantize, save, load, dequantize; every truncation and a bit flip every 7 bytes */
    float w[5 * 16];
    for (int i = 0; i < 80; i++) w[i] = (float)((i * 37) % 41 - 20) / 7.0f;
    EXPECT(!ax_qweight_create_from_fp32(NULL, 5, 16) && !ax_qweight_create_from_fp32(w, 0, 16));
    ax_qweight_t *qw = ax_qweight_create_from_fp32(w, 5, 16);
    EXPECT(qw && ax_qweight_save(qw, tmp) == AX_OK && ax_qweight_save(NULL, tmp) != AX_OK);
    ax_qweight_t *q2 = ax_qweight_load(tmp);
    EXPECT(q2 && q2->N == 5 && q2->K == 16 && !memcmp(q2->data, qw->data, 80) && !memcmp(q2->scales, qw->scales, 20));
    float deq[80];
    if (q2) ax_qweight_dequantize(q2, deq);
    for (int i = 0; q2 && i < 80; i++) EXPECT(deq[i] - w[i] <= 1.5f * q2->scales[i / 16] && w[i] - deq[i] <= 1.5f * q2->scales[i / 16]);
    ax_qweight_destroy(q2);
    size_t n = 0;
    unsigned char *blob = slurp(tmp, &n), *mut = malloc(n ? n : 1);
    for (size_t cut = 0; blob && cut < n; cut++) {
        if (spit(tmp, blob, cut)) break;
        ax_qweight_t *q = ax_qweight_load(tmp);
        EXPECT(q == NULL);
        ax_qweight_destroy(q);
    }
    for (size_t pos = 0; blob && pos < n; pos += 7) {
        memcpy(mut, blob, n);
        mut[pos] ^= 0x80;
        if (spit(tmp, mut, n)) break;
        ax_qweight_destroy(ax_qweight_load(tmp));              /* refused by its checksum or loaded: either way clean */
    }
    free(blob);
    free(mut);
    ax_qweight_destroy(qw);
    ax_qweight_destroy(NULL);
    printf("api section: %d findings\n", bad);
    return bad;
}

int main(int argc, char **argv) {
    if (argc < 3) { fprintf(stderr, "usage: %s scratch-file file...\n", argv[0]); return 2; }
    const char *tmp = argv[1];
    ax_set_default_device(AX_DEVICE_CPU);
    int bad = api_section(tmp);
    for (int a = 2; a < argc; a++) {
        const char *path = argv[a];
        const size_t plen = strlen(path);
        const int is_model = plen > 4 && strcmp(path + plen - 4, ".axm") == 0;
        size_t n = 0;
        unsigned char *blob = slurp(path, &n);
        if (!blob) { fprintf(stderr, "cannot read %s\n", path); return 2; }
        /* round trip */
        if (is_model) {
            ax_model_t *m = ax_model_load(path);
            if (!m || ax_model_save(m, tmp) != AX_OK) { fprintf(stderr, "%s: load/save failed: %s\n", path, ax_err_last_message()); bad++; }
            if (m) ax_model_destroy(m);
        } else {
            ax_tensor_t *t = ax_tensor_load(path);
            if (!t || ax_tensor_save(t, tmp) != AX_OK) { fprintf(stderr, "%s: load/save failed: %s\n", path, ax_err_last_message()); bad++; }
            if (t) ax_tensor_destroy(t);
        }
        size_t n2 = 0;
        unsigned char *again = slurp(tmp, &n2);
        if (!again || n2 != n || memcmp(again, blob, n) != 0) { fprintf(stderr, "%s: round trip differs\n", path); bad++; }
        free(again);
        /* truncations: all must be refused */
        int loaded = 0, tried = 0;
        for (size_t cut = 0; cut < n; cut += (n > 20000 ? 211 : 37)) {
            if (spit(tmp, blob, cut)) return 2;
            tried++;
            if (try_load(tmp, is_model)) { fprintf(stderr, "%s: truncation to %zu bytes loaded\n", path, cut); bad++; }
        }
        /* bit flips: refused (a model's checksum catches every one) or, for a tensor file, loaded cleanly */
        unsigned char *mut = malloc(n);
        for (size_t pos = 0; pos < n; pos += (n > 20000 ? 499 : 101)) {
            memcpy(mut, blob, n);
            mut[pos] ^= (unsigned char)(1u << (pos % 8));
            if (spit(tmp, mut, n)) return 2;
            tried++;
            const int ok = try_load(tmp, is_model);
            loaded += ok;
            if (ok && is_model) { fprintf(stderr, "%s: flipped bit at %zu not detected\n", path, pos); bad++; }
        }
        /* crafted counts and extents (tests/test_fuzz_serialize.c): every third byte offset of the first 128
         * bytes overwritten with a huge, a negative and a tiny value, the model's trailing checksum
         * recomputed so that the parser, not the checksum, has to refuse what does not fit */
        for (size_t off = 4; off + 4 <= n && off < 128; off += 3) {
            static const unsigned char pat[4][4] = {{0xff, 0xff, 0xff, 0xff}, {0xff, 0xff, 0xff, 0x7f}, {0x00, 0x00, 0x00, 0x80},
                                                    {0x01, 0x00, 0x00, 0x00}};
            for (int p = 0; p < 4; p++) {
                memcpy(mut, blob, n);
                memcpy(mut + off, pat[p], 4);
                if (is_model && n >= 4) {
                    const uint32_t c = crc32_of(mut, n - 4);
                    mut[n - 4] = (unsigned char)c; mut[n - 3] = (unsigned char)(c >> 8);
                    mut[n - 2] = (unsigned char)(c >> 16); mut[n - 1] = (unsigned char)(c >> 24);
                }
                if (spit(tmp, mut, n)) return 2;
                tried++;
                loaded += try_load(tmp, is_model);
            }
        }
        free(mut);
        free(blob);
        printf("%s: %d mutated inputs, %d loaded, round trip ok\n", path, tried, loaded);
    }
    remove(tmp);
    return bad ? 1 : 0;
}
