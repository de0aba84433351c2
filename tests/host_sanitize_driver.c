/* Host-side file and tensor code under AddressSanitizer + UndefinedBehaviorSanitizer (the reference's
 * CI builds its C with the same pair, CMakeLists.txt:46-65).  No GPU: everything stays on the CPU
 * device.  For every file named on the command line: load it, save it again and compare the bytes;
 * then feed the loader every truncation in steps of 37 bytes and the file with one bit flipped every
 * 101 bytes (each must be refused or load cleanly — never touch memory it does not own), and the
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

int main(int argc, char **argv) {
    if (argc < 3) { fprintf(stderr, "usage: %s scratch-file file...\n", argv[0]); return 2; }
    const char *tmp = argv[1];
    ax_set_default_device(AX_DEVICE_CPU);
    int bad = 0;
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
        for (size_t cut = 0; cut < n; cut += 37) {
            if (spit(tmp, blob, cut)) return 2;
            tried++;
            if (try_load(tmp, is_model)) { fprintf(stderr, "%s: truncation to %zu bytes loaded\n", path, cut); bad++; }
        }
        /* bit flips: refused (a model's checksum catches every one) or, for a tensor file, loaded cleanly */
        unsigned char *mut = malloc(n);
        for (size_t pos = 0; pos < n; pos += 101) {
            memcpy(mut, blob, n);
            mut[pos] ^= (unsigned char)(1u << (pos % 8));
            if (spit(tmp, mut, n)) return 2;
            tried++;
            const int ok = try_load(tmp, is_model);
            loaded += ok;
            if (ok && is_model) { fprintf(stderr, "%s: flipped bit at %zu not detected\n", path, pos); bad++; }
        }
        /* crafted counts and extents (tests/test_fuzz_serialize.c): every byte offset of the first 128
         * bytes overwritten with a huge, a negative and a tiny value, the model's trailing checksum
         * recomputed so that the parser, not the checksum, has to refuse what does not fit */
        for (size_t off = 4; off + 4 <= n && off < 128; off++) {
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
