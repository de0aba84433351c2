/* ax_oracle.c — CPU restatement of Axiom's GEMM hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * The checker for the GPU path and the timed CPU leg of the benchmark; never linked,
 * loaded or called by the shipped libraries.  See ax_oracle.h for what pins each
 * function.  Built with -ffp-contract=off: every fused multiply-add below is written
 * out with fmaf()/_mm256_fmadd_ps exactly where the reference's AVX2+FMA build has one.
 */
#include "ax_oracle.h"

#include <float.h>
#include <immintrin.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ======================================================================== */
/* RNG — src/core/rng.c                                                     */
/* ======================================================================== */

static uint64_t g_state[4];
static int      g_have_spare = 0;
static float    g_spare = 0.0f;

static inline uint64_t rol64(uint64_t v, int r) { return (v << r) | (v >> (64 - r)); }

/* rng.c:21-26 */
static uint64_t splitmix_next(uint64_t *ctr) {
    uint64_t z = (*ctr += 0x9e3779b97f4a7c15ULL);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}

void axo_rng_seed(uint64_t seed) {
    uint64_t ctr = seed;
    for (int i = 0; i < 4; i++) g_state[i] = splitmix_next(&ctr);
    /* the reference does not clear its cached normal on reseed (rng.c:33-40,84-85) */
}

void axo_rng_drop_spare(void) { g_have_spare = 0; }

uint64_t axo_rng_uint64(void) {
    const uint64_t out = rol64(g_state[1] * 5, 7) * 9;
    const uint64_t sh = g_state[1] << 17;
    g_state[2] ^= g_state[0];
    g_state[3] ^= g_state[1];
    g_state[1] ^= g_state[2];
    g_state[0] ^= g_state[3];
    g_state[2] ^= sh;
    g_state[3] = rol64(g_state[3], 45);
    return out;
}

float axo_rng_float(void) { return (float)(axo_rng_uint64() >> 40) * 0x1.0p-24f; }

float axo_rng_uniform(float lo, float hi) { return lo + axo_rng_float() * (hi - lo); }

float axo_rng_normal(void) {
    if (g_have_spare) { g_have_spare = 0; return g_spare; }
    float u, v, r2;
    do {
        u = axo_rng_float() * 2.0f - 1.0f;
        v = axo_rng_float() * 2.0f - 1.0f;
        r2 = u * u + v * v;
    } while (r2 >= 1.0f || r2 == 0.0f);
    float f = sqrtf(-2.0f * logf(r2) / r2);
    g_spare = v * f;
    g_have_spare = 1;
    return u * f;
}

uint64_t axo_rng_bounded(uint64_t n) {
    if (n <= 1) return 0;
    uint64_t reject_below = (0 - n) % n;
    for (;;) {
        uint64_t r = axo_rng_uint64();
        if (r >= reject_below) return r % n;
    }
}

void axo_fill_uniform(float *dst, int64_t n, float lo, float hi) {
    for (int64_t i = 0; i < n; i++) dst[i] = axo_rng_uniform(lo, hi);
}

void axo_fill_normal(float *dst, int64_t n, float mean, float std) {
    for (int64_t i = 0; i < n; i++) dst[i] = mean + std * axo_rng_normal();
}

void axo_fill_kaiming_uniform(float *dst, int64_t n, int64_t fan_in) {
    float lim = sqrtf(6.0f / (float)fan_in);
    for (int64_t i = 0; i < n; i++) dst[i] = axo_rng_uniform(-lim, lim);
}

void axo_fill_int8(int8_t *dst, int64_t n) {
    for (int64_t i = 0; i < n; i++) dst[i] = (int8_t)((int)axo_rng_bounded(255) - 127);
}

/* ======================================================================== */
/* fp32 GEMM                                                                */
/* ======================================================================== */

void axo_gemm_f64(const float *a, const float *b, double *c, int64_t M, int64_t N, int64_t K,
                  int transb) {
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; i++) {
        double *ci = c + i * N;
        if (transb) {
            for (int64_t j = 0; j < N; j++) {
                double s = 0.0;
                for (int64_t p = 0; p < K; p++) s += (double)a[i * K + p] * (double)b[j * K + p];
                ci[j] = s;
            }
        } else {
            for (int64_t j = 0; j < N; j++) ci[j] = 0.0;
            for (int64_t p = 0; p < K; p++) {
                double av = (double)a[i * K + p];
                const float *bp = b + p * N;
                for (int64_t j = 0; j < N; j++) ci[j] += av * (double)bp[j];
            }
        }
    }
}

void axo_gemm_abs_f64(const float *a, const float *b, double *c, int64_t M, int64_t N,
                      int64_t K, int transb) {
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; i++) {
        double *ci = c + i * N;
        for (int64_t j = 0; j < N; j++) ci[j] = 0.0;
        if (transb) {
            for (int64_t j = 0; j < N; j++) {
                double s = 0.0;
                for (int64_t p = 0; p < K; p++)
                    s += fabs((double)a[i * K + p]) * fabs((double)b[j * K + p]);
                ci[j] = s;
            }
        } else {
            for (int64_t p = 0; p < K; p++) {
                double av = fabs((double)a[i * K + p]);
                const float *bp = b + p * N;
                for (int64_t j = 0; j < N; j++) ci[j] += av * fabs((double)bp[j]);
            }
        }
    }
}

/* cpu_naive.c:176-185.  That translation unit is built without -mfma in the reference,
   so the multiply and the add round separately. */
void axo_gemm_naive(const float *a, const float *b, float *c, int64_t M, int64_t N, int64_t K) {
    for (int64_t i = 0; i < M; i++)
        for (int64_t j = 0; j < N; j++) {
            float s = 0.0f;
            for (int64_t p = 0; p < K; p++) {
                float prod = a[i * K + p] * b[p * N + j];
                s = s + prod;
            }
            c[i * N + j] = s;
        }
}

enum { MR = 6, NR = 16, MC_DEFAULT = 72, NC_DEFAULT = 256, KC_DEFAULT = 256, KC_CEIL = 512 };

int axo_gemm_takes_small_route(int64_t m, int64_t n, int64_t k) {
    int64_t work = m * n * k;
    return (work < 100000) || (m < MR && work < 5000000);
}

/* cpu_opt.c:3546-3564: C zeroed, then for each row i and each p the row B[p,:] is scaled
   by a[i,p] and fused-multiply-added into C[i,:].  Every output element therefore sees
   k ascending with one FMA per step; the 8-wide body and the scalar tail are the same
   arithmetic because the reference's scalar tail contracts to an FMA under -mfma. */
static void gemm_small_route(const float *a, const float *b, float *c,
                             int64_t M, int64_t N, int64_t K) {
    memset(c, 0, (size_t)(M * N) * sizeof(float));
    for (int64_t i = 0; i < M; i++) {
        float *ci = c + i * N;
        for (int64_t p = 0; p < K; p++) {
            float av = a[i * K + p];
            const float *bp = b + p * N;
            __m256 va = _mm256_set1_ps(av);
            int64_t j = 0;
            for (; j + 8 <= N; j += 8)
                _mm256_storeu_ps(ci + j, _mm256_fmadd_ps(va, _mm256_loadu_ps(bp + j),
                                                         _mm256_loadu_ps(ci + j)));
            for (; j < N; j++) ci[j] = fmaf(av, bp[j], ci[j]);
        }
    }
}

/* cpu_opt.c:1833-1848: rows [0,rows) x k [0,kc) of A -> strips of MR rows,
   element (strip s, k p, row r) at s*kc*MR + p*MR + r, missing rows zero. */
static void pack_rows_mr(const float *a, int64_t lda, int64_t rows, int64_t kc, float *dst) {
    for (int64_t r0 = 0; r0 < rows; r0 += MR) {
        int64_t live = rows - r0 < MR ? rows - r0 : MR;
        for (int64_t p = 0; p < kc; p++) {
            for (int64_t r = 0; r < MR; r++)
                dst[r] = (r < live) ? a[(r0 + r) * lda + p] : 0.0f;
            dst += MR;
        }
    }
}

/* cpu_opt.c:2123-2143: k [0,kc) x cols [0,cols) of row-major B -> strips of NR columns,
   element (strip s, k p, col q) at s*kc*NR + p*NR + q, missing columns zero. */
static void pack_cols_nr(const float *b, int64_t ldb, int64_t kc, int64_t cols, float *dst) {
    for (int64_t c0 = 0; c0 < cols; c0 += NR) {
        int64_t live = cols - c0 < NR ? cols - c0 : NR;
        for (int64_t p = 0; p < kc; p++) {
            const float *src = b + p * ldb + c0;
            for (int64_t q = 0; q < NR; q++) dst[q] = (q < live) ? src[q] : 0.0f;
            dst += NR;
        }
    }
}

/* cpu_opt.c:1912-2043 (layout only): the same NR-strip panel, from B stored [N,K]. */
static void pack_cols_nr_from_nk(const float *b, int64_t ldb, int64_t kc, int64_t cols,
                                 float *dst) {
    for (int64_t c0 = 0; c0 < cols; c0 += NR) {
        int64_t live = cols - c0 < NR ? cols - c0 : NR;
        for (int64_t p = 0; p < kc; p++) {
            for (int64_t q = 0; q < NR; q++) dst[q] = (q < live) ? b[(c0 + q) * ldb + p] : 0.0f;
            dst += NR;
        }
    }
}

/* cpu_opt.c:2436-2521: 6x16 tile, twelve 8-lane accumulators started at zero, one FMA per
   (row, half, k) with k ascending, then the tile is added into C. */
static void tile_6x16(int64_t kc, const float *ap, const float *bp, float *c, int64_t ldc,
                      int64_t mr, int64_t nr) {
    __m256 acc[MR][2];
    for (int r = 0; r < MR; r++) acc[r][0] = acc[r][1] = _mm256_setzero_ps();
    for (int64_t p = 0; p < kc; p++) {
        __m256 b0 = _mm256_loadu_ps(bp);
        __m256 b1 = _mm256_loadu_ps(bp + 8);
        for (int r = 0; r < MR; r++) {
            __m256 av = _mm256_broadcast_ss(ap + r);
            acc[r][0] = _mm256_fmadd_ps(av, b0, acc[r][0]);
            acc[r][1] = _mm256_fmadd_ps(av, b1, acc[r][1]);
        }
        ap += MR;
        bp += NR;
    }
    if (mr == MR && nr == NR) {
        for (int r = 0; r < MR; r++) {
            float *cr = c + r * ldc;
            _mm256_storeu_ps(cr, _mm256_add_ps(acc[r][0], _mm256_loadu_ps(cr)));
            _mm256_storeu_ps(cr + 8, _mm256_add_ps(acc[r][1], _mm256_loadu_ps(cr + 8)));
        }
    } else {
        float tmp[MR * NR];
        for (int r = 0; r < MR; r++) {
            _mm256_storeu_ps(tmp + r * NR, acc[r][0]);
            _mm256_storeu_ps(tmp + r * NR + 8, acc[r][1]);
        }
        for (int64_t r = 0; r < mr; r++)
            for (int64_t q = 0; q < nr; q++) c[r * ldc + q] += tmp[r * NR + q];
    }
}

static int64_t round_up(int64_t v, int64_t to) { return (v + to - 1) / to * to; }

/* The BLIS loop nest of cpu_opt.c:3795-3833 (JC variant): column tiles are the parallel
   dimension (NC shrunk so there is at least one tile per thread, cpu_opt.c:3250-3259),
   pc steps of kc (kc = K when K <= 512, cpu_opt.c:3583), ic steps of MC. */
static void gemm_packed(const float *a, const float *b, float *c, int64_t M, int64_t N,
                        int64_t K, int b_is_nk) {
    memset(c, 0, (size_t)(M * N) * sizeof(float));
    int threads = 1;
#ifdef _OPENMP
    threads = omp_get_max_threads();
#endif
    if (2 * M * N * K < 10000000) threads = 1;          /* cpu_opt.c:711-767: <10 MFLOP serial */
    const int64_t kc_step = (K <= KC_CEIL) ? K : KC_DEFAULT;
    int64_t nc = NC_DEFAULT;
    if ((N + nc - 1) / nc < threads) {
        nc = round_up((N + threads - 1) / threads, NR);
        if (nc < NR) nc = NR;
    }
    const int64_t n_jc = (N + nc - 1) / nc;
    const int64_t mc = MC_DEFAULT;

    #pragma omp parallel num_threads(threads)
    {
        float *pa = aligned_alloc(64, (size_t)(round_up(mc, MR) * kc_step) * sizeof(float));
        float *pb = aligned_alloc(64, (size_t)(round_up(nc, NR) * kc_step) * sizeof(float));
        #pragma omp for schedule(static)
        for (int64_t jt = 0; jt < n_jc; jt++) {
            int64_t jc = jt * nc;
            int64_t ncur = N - jc < nc ? N - jc : nc;
            for (int64_t pc = 0; pc < K; pc += kc_step) {
                int64_t kc = K - pc < kc_step ? K - pc : kc_step;
                if (b_is_nk) pack_cols_nr_from_nk(b + jc * K + pc, K, kc, ncur, pb);
                else         pack_cols_nr(b + pc * N + jc, N, kc, ncur, pb);
                for (int64_t ic = 0; ic < M; ic += mc) {
                    int64_t mcur = M - ic < mc ? M - ic : mc;
                    pack_rows_mr(a + ic * K + pc, K, mcur, kc, pa);
                    for (int64_t jr = 0; jr < ncur; jr += NR) {
                        int64_t nr = ncur - jr < NR ? ncur - jr : NR;
                        for (int64_t ir = 0; ir < mcur; ir += MR) {
                            int64_t mr = mcur - ir < MR ? mcur - ir : MR;
                            tile_6x16(kc, pa + (ir / MR) * kc * MR, pb + (jr / NR) * kc * NR,
                                      c + (ic + ir) * N + jc + jr, N, mr, nr);
                        }
                    }
                }
            }
        }
        free(pa);
        free(pb);
    }
}

void axo_gemm_opt(const float *a, const float *b, float *c, int64_t M, int64_t N, int64_t K) {
    if (axo_gemm_takes_small_route(M, N, K)) gemm_small_route(a, b, c, M, N, K);
    else gemm_packed(a, b, c, M, N, K, 0);
}

void axo_gemm_opt_nt(const float *a, const float *b, float *c, int64_t M, int64_t N, int64_t K) {
    if (M * N * K < 100000) {                           /* cpu_opt.c:4842-4914: dot products */
        for (int64_t i = 0; i < M; i++)
            for (int64_t j = 0; j < N; j++) {
                float s = 0.0f;
                for (int64_t p = 0; p < K; p++) s = fmaf(a[i * K + p], b[j * K + p], s);
                c[i * N + j] = s;
            }
        return;
    }
    gemm_packed(a, b, c, M, N, K, 1);
}

void axo_bias_add_cols(float *c, const float *bias, int64_t M, int64_t N) {
    for (int64_t i = 0; i < M; i++)
        for (int64_t j = 0; j < N; j++) c[i * N + j] = c[i * N + j] + bias[j];
}

void axo_bias_relu(float *c, const float *bias, int64_t M, int64_t N) {
    for (int64_t i = 0; i < M; i++)
        for (int64_t j = 0; j < N; j++) {
            float v = c[i * N + j];
            if (bias) v = v + bias[j];
            c[i * N + j] = v > 0.0f ? v : 0.0f;
        }
}

float axo_gelu_tanh(float x) {
    const float k0 = 0.7978845608028654f, k1 = 0.044715f;
    float inner = k0 * (x + k1 * x * x * x);
    return 0.5f * x * (1.0f + tanhf(inner));
}

double axo_gelu_f64(double x) {
    return 0.5 * x * (1.0 + tanh(0.7978845608028654 * (x + 0.044715 * x * x * x)));
}

void axo_gelu(float *x, int64_t n) {
    #pragma omp parallel for schedule(static) if (n > 65536)
    for (int64_t i = 0; i < n; i++) x[i] = axo_gelu_tanh(x[i]);
}

/* ======================================================================== */
/* int8                                                                     */
/* ======================================================================== */

void axo_quantize_rows(const float *w, int64_t N, int64_t K, int8_t *q, float *scales) {
    for (int64_t n = 0; n < N; n++) {
        const float *row = w + n * K;
        float top = 0.0f;
        for (int64_t k = 0; k < K; k++) {
            float m = fabsf(row[k]);
            if (m > top) top = m;
        }
        float scale = (top > 0.0f) ? (top / 127.0f) : 1.0f;
        float inv = 1.0f / scale;
        scales[n] = scale;
        for (int64_t k = 0; k < K; k++) {
            long v = lrintf(row[k] * inv);
            if (v > 127) v = 127;
            if (v < -127) v = -127;
            q[n * K + k] = (int8_t)v;
        }
    }
}

void axo_dequantize_rows(const int8_t *q, const float *scales, int64_t N, int64_t K, float *out) {
    for (int64_t n = 0; n < N; n++)
        for (int64_t k = 0; k < K; k++) out[n * K + k] = (float)q[n * K + k] * scales[n];
}

/* quantize.c:115-175 restated lane by lane.  lane[g][l] is lane l of the reference's
   g-th 8-wide accumulator: blocks of 32 k feed all four, the 8-wide tail feeds the first. */
void axo_qgemm_w8a32(const float *a, const int8_t *q, const float *scales, float *out,
                     int64_t M, int64_t N, int64_t K) {
    #pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        const int8_t *wn = q + n * K;
        for (int64_t m = 0; m < M; m++) {
            const float *am = a + m * K;
            float lane[4][8];
            memset(lane, 0, sizeof lane);
            int64_t k = 0;
            for (; k + 32 <= K; k += 32)
                for (int g = 0; g < 4; g++)
                    for (int l = 0; l < 8; l++)
                        lane[g][l] = fmaf(am[k + 8 * g + l], (float)wn[k + 8 * g + l], lane[g][l]);
            for (; k + 8 <= K; k += 8)
                for (int l = 0; l < 8; l++)
                    lane[0][l] = fmaf(am[k + l], (float)wn[k + l], lane[0][l]);
            float v[8];
            for (int l = 0; l < 8; l++)
                v[l] = (lane[0][l] + lane[1][l]) + (lane[2][l] + lane[3][l]);
            float h0 = v[0] + v[4], h1 = v[1] + v[5], h2 = v[2] + v[6], h3 = v[3] + v[7];
            float s = (h0 + h1) + (h2 + h3);
            for (; k < K; k++) s = fmaf(am[k], (float)wn[k], s);
            out[m * N + n] = s * scales[n];
        }
    }
}

void axo_qgemm_w8a8_acc(const int8_t *x, const int8_t *w, int32_t *acc,
                        int64_t M, int64_t N, int64_t K) {
    #pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        const int8_t *wn = w + n * K;
        for (int64_t m = 0; m < M; m++) {
            const int8_t *xm = x + m * K;
            int32_t s = 0;
            for (int64_t k = 0; k < K; k++) s += (int32_t)xm[k] * (int32_t)wn[k];
            acc[m * N + n] = s;
        }
    }
}

void axo_w8a8_epilogue(const int32_t *acc, float x_scale, const float *w_scales,
                       const float *bias, int act, float *out, int64_t M, int64_t N) {
    #pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            float s = x_scale * w_scales[n];
            float f = (float)acc[m * N + n];
            float v = bias ? fmaf(f, s, bias[n]) : f * s;
            if (act == 1) v = v > 0.0f ? v : 0.0f;
            else if (act == 2) v = axo_gelu_tanh(v);
            out[m * N + n] = v;
        }
}

/* ---- reductions / accumulation of the dense backward pass ------------------------------ */
void axo_sum_axis0(const float *in, int64_t rows, int64_t cols, float *out) {
    for (int64_t j = 0; j < cols; j++) {
        float s = 0.0f;
        for (int64_t i = 0; i < rows; i++) s += in[i * cols + j];
        out[j] = s;
    }
}

void axo_sum_axis_f64(const float *in, int64_t outer, int64_t axis_len, int64_t inner, double *out,
                      double *out_abs) {
    for (int64_t o = 0; o < outer; o++)
        for (int64_t i = 0; i < inner; i++) {
            double s = 0.0, sa = 0.0;
            for (int64_t a = 0; a < axis_len; a++) {
                const double v = (double)in[(o * axis_len + a) * inner + i];
                s += v;
                sa += fabs(v);
            }
            out[o * inner + i] = s;
            if (out_abs) out_abs[o * inner + i] = sa;
        }
}

void axo_axpy(const float *x, float alpha, float *y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = fmaf(alpha, x[i], y[i]);
}

/* ---- scaled dot-product attention forward ---------------------------------------------- */
void axo_sdpa_fwd(const float *Q, const float *K, const float *V, float *O, float *L, int64_t BH,
                  int64_t S, int64_t dk, float scale, int causal) {
#pragma omp parallel for schedule(dynamic)
    for (int64_t h = 0; h < BH; h++) {
        const float *q = Q + h * S * dk, *k = K + h * S * dk, *v = V + h * S * dk;
        float *scores = (float *)malloc((size_t)S * sizeof(float));
        for (int64_t i = 0; i < S; i++) {
            const int64_t n = causal ? i + 1 : S;
            float mx = -INFINITY;
            for (int64_t j = 0; j < n; j++) {
                float dot = 0.0f;
                for (int64_t d = 0; d < dk; d++) dot += q[i * dk + d] * k[j * dk + d];
                dot *= scale;
                scores[j] = dot;
                if (dot > mx) mx = dot;
            }
            float sum = 0.0f;
            for (int64_t j = 0; j < n; j++) {
                scores[j] = expf(scores[j] - mx);
                sum += scores[j];
            }
            const float inv = 1.0f / sum;
            for (int64_t d = 0; d < dk; d++) {
                float acc = 0.0f;
                for (int64_t j = 0; j < n; j++) acc += scores[j] * inv * v[j * dk + d];
                O[(h * S + i) * dk + d] = acc;
            }
            if (L) L[h * S + i] = mx + logf(sum);
        }
        free(scores);
    }
}

void axo_sdpa_fwd_f64(const float *Q, const float *K, const float *V, double *O, double *L, int64_t BH,
                      int64_t S, int64_t dk, float scale, int causal) {
#pragma omp parallel for schedule(dynamic)
    for (int64_t h = 0; h < BH; h++) {
        const float *q = Q + h * S * dk, *k = K + h * S * dk, *v = V + h * S * dk;
        double *scores = (double *)malloc((size_t)S * sizeof(double));
        for (int64_t i = 0; i < S; i++) {
            const int64_t n = causal ? i + 1 : S;
            double mx = -INFINITY;
            for (int64_t j = 0; j < n; j++) {
                double dot = 0.0;
                for (int64_t d = 0; d < dk; d++) dot += (double)q[i * dk + d] * (double)k[j * dk + d];
                dot *= (double)scale;
                scores[j] = dot;
                if (dot > mx) mx = dot;
            }
            double sum = 0.0;
            for (int64_t j = 0; j < n; j++) {
                scores[j] = exp(scores[j] - mx);
                sum += scores[j];
            }
            for (int64_t d = 0; d < dk; d++) {
                double acc = 0.0;
                for (int64_t j = 0; j < n; j++) acc += scores[j] * (double)v[j * dk + d];
                O[(h * S + i) * dk + d] = acc / sum;
            }
            if (L) L[h * S + i] = mx + log(sum);
        }
        free(scores);
    }
}

/* ---- remaining elementwise / reduction / optimizer slots -------------------------------- */
static int64_t bcast_offset(const int64_t *t_shape, int t_ndim, const int64_t *out_shape, int out_ndim,
                            int64_t out_flat) {
    int64_t t_strides[8], st = 1;
    for (int d = t_ndim - 1; d >= 0; d--) {
        t_strides[d] = st;
        st *= t_shape[d];
    }
    int64_t remaining = out_flat, off = 0;
    for (int d = out_ndim - 1; d >= 0; d--) {
        const int64_t idx = remaining % out_shape[d];
        remaining /= out_shape[d];
        const int td = d - (out_ndim - t_ndim);
        if (td >= 0 && t_shape[td] > 1) off += idx * t_strides[td];
    }
    return off;
}

void axo_binary(int op, const float *a, const int64_t *a_shape, int a_ndim, const float *b,
                const int64_t *b_shape, int b_ndim, float *out, const int64_t *out_shape, int out_ndim) {
    int64_t n = 1;
    for (int d = 0; d < out_ndim; d++) n *= out_shape[d];
    for (int64_t i = 0; i < n; i++) {
        const float va = a[bcast_offset(a_shape, a_ndim, out_shape, out_ndim, i)];
        const float vb = b[bcast_offset(b_shape, b_ndim, out_shape, out_ndim, i)];
        float r;
        switch (op) {
            case 0: r = va + vb; break;
            case 1: r = va - vb; break;
            case 2: r = va * vb; break;
            case 3: r = va / vb; break;
            case 4: r = (va == vb) ? 1.0f : 0.0f; break;
            case 5: r = (va > vb) ? 1.0f : 0.0f; break;
            default: r = va + vb; r = r > 0.0f ? r : 0.0f; break;
        }
        out[i] = r;
    }
}

void axo_unary(int op, const float *in, float *out, int64_t n, float p) {
    for (int64_t i = 0; i < n; i++) {
        const float v = in[i];
        float r;
        switch (op) {
            case 0: r = -v; break;
            case 1: r = fabsf(v); break;
            case 2: r = expf(v); break;
            case 3: r = v > 0.0f ? logf(v) : -FLT_MAX; break;
            case 4: r = v >= 0.0f ? sqrtf(v) : 0.0f; break;
            case 5: r = v * v; break;
            case 6: r = 1.0f / (1.0f + expf(-v)); break;
            case 7: r = tanhf(v); break;
            case 8: r = v > 0.0f ? v : p * v; break;
            case 9: r = v > 0.0f ? v : p * (expf(v) - 1.0f); break;
            case 10: r = v / (1.0f + expf(-v)); break;
            case 11: r = v + p; break;
            default: r = v * p; break;
        }
        out[i] = r;
    }
}

void axo_reduce_axis(int op, const float *in, int64_t outer, int64_t axis_len, int64_t inner, float *out) {
    for (int64_t o = 0; o < outer; o++)
        for (int64_t i = 0; i < inner; i++) {
            float acc = op == 2 ? -FLT_MAX : op == 3 ? FLT_MAX : 0.0f;
            for (int64_t a = 0; a < axis_len; a++) {
                const float v = in[(o * axis_len + a) * inner + i];
                if (op == 2) { if (v > acc) acc = v; }
                else if (op == 3) { if (v < acc) acc = v; }
                else acc += v;
            }
            if (op == 1) acc *= 1.0f / (float)axis_len;
            out[o * inner + i] = acc;
        }
}

void axo_argmax_axis(const float *in, int64_t outer, int64_t axis_len, int64_t inner, int64_t *out) {
    for (int64_t oi = 0; oi < outer * inner; oi++) {
        const int64_t o = oi / inner, i = oi - o * inner;
        const float *base = in + o * axis_len * inner + i;
        int64_t best = 0;
        float bestv = base[0];
        for (int64_t a = 1; a < axis_len; a++) {
            const float v = base[a * inner];
            if (v > bestv) { bestv = v; best = a; }
        }
        out[oi] = best;
    }
}

void axo_softmax_rows(const float *in, float *out, int64_t rows, int64_t cols) {
    for (int64_t r = 0; r < rows; r++) {
        const float *x = in + r * cols;
        float *y = out + r * cols;
        float mx = x[0];
        for (int64_t c = 1; c < cols; c++) if (x[c] > mx) mx = x[c];
        float sum = 0.0f;
        for (int64_t c = 0; c < cols; c++) {
            const float e = expf(x[c] - mx);
            y[c] = e;
            sum += e;
        }
        const float inv = 1.0f / sum;
        for (int64_t c = 0; c < cols; c++) y[c] *= inv;
    }
}

void axo_layernorm_fwd(const float *x, const float *gamma, const float *beta, float *out, float *x_hat,
                       float *inv_std_out, int64_t rows, int64_t cols, float eps) {
    for (int64_t r = 0; r < rows; r++) {
        const float *ip = x + r * cols;
        float sum = 0.0f, sum2 = 0.0f;
        for (int64_t f = 0; f < cols; f++) {
            sum += ip[f];
            sum2 += ip[f] * ip[f];
        }
        const float mean = sum / (float)cols;
        float var = sum2 / (float)cols - mean * mean;
        if (var < 0.0f) var = 0.0f;
        const float inv_std = 1.0f / sqrtf(var + eps);
        if (inv_std_out) inv_std_out[r] = inv_std;
        for (int64_t f = 0; f < cols; f++) {
            const float xh = (ip[f] - mean) * inv_std;
            out[r * cols + f] = gamma[f] * xh + beta[f];
            if (x_hat) x_hat[r * cols + f] = xh;
        }
    }
}

void axo_adam_update(float *w, const float *g, float *m, float *v, int64_t n, float lr, float beta1,
                     float beta2, float eps, float weight_decay, float bc1, float bc2, int decoupled) {
    float decay_scale = decoupled ? (1.0f - lr * weight_decay) : 1.0f;
    if (decay_scale < 0.0f) decay_scale = 0.0f;
    const float wd_grad = (!decoupled && weight_decay > 0.0f) ? weight_decay : 0.0f;
    for (int64_t i = 0; i < n; i++) {
        const float wi = w[i] * decay_scale;
        const float gi = g[i] + wd_grad * wi;
        const float mi = beta1 * m[i] + (1.0f - beta1) * gi;
        const float vi = beta2 * v[i] + (1.0f - beta2) * gi * gi;
        const float mh = mi / bc1, vh = vi / bc2;
        w[i] = wi - lr * mh / (sqrtf(vh) + eps);
        m[i] = mi;
        v[i] = vi;
    }
}

void axo_sgd_update(float *w, const float *g, float *mom, int64_t n, float lr, float momentum,
                    float weight_decay, int nesterov) {
    for (int64_t i = 0; i < n; i++) {
        float gi = g[i];
        if (weight_decay > 0.0f) gi += weight_decay * w[i];
        if (mom && momentum > 0.0f) {
            const float vi = momentum * mom[i] + gi;
            mom[i] = vi;
            w[i] -= nesterov ? lr * (gi + momentum * vi) : lr * vi;
        } else {
            w[i] -= lr * gi;
        }
    }
}
