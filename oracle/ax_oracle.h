/* ax_oracle.h — CPU restatement of Axiom's GEMM hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This library is the checker the GPU results are compared against (and the timed CPU
 * leg of the benchmark).  Nothing in the product links, loads or calls it: the shipped
 * libraries fail with an error when the HIP path is unavailable instead of coming here.
 *
 * Each function names the reference source it follows (paths relative to the Axiom tree).
 * Pinning status (what each function has been checked against):
 *   rng_*            reference known answers + the compiled reference, bit-exact
 *   quantize_rows    compiled reference, bit-exact; hand-derived vectors (ties, zero row)
 *   qgemm_w8a32      compiled reference, bit-exact (same lane order and FMA placement)
 *   gemm_naive       compiled reference cpu_naive backend, bit-exact
 *   gemm_opt/_nt     fp64 ground truth bound + compiled reference cpu_opt within 1e-4
 *                    (bit-exact on the skinny/small route, whose order is fully specified)
 *   gemm_f64         the mathematics: known answers 58/64/139/154, 19/22/43/50, A*I=A
 *   qgemm_w8a8_acc   exact integer closed form; brute force; the reference's W8A32
 *                    routine with unit scales for K <= 1040 (partial sums < 2^24)
 *   gelu_tanh        closed form in fp64 + the compiled reference's ax_gelu within 2e-6
 *   w8a8 epilogue    defined by this build (no reference counterpart): checked against
 *                    an fp64 evaluation of the same formula
 */
#ifndef AX_ORACLE_H
#define AX_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- RNG: src/core/rng.c ------------------------------------------------ */
void     axo_rng_seed(uint64_t seed);                 /* rng.c:33-40 (splitmix64 x4) */
uint64_t axo_rng_uint64(void);                        /* rng.c:56-71 (xoshiro256**)  */
float    axo_rng_float(void);                         /* rng.c:73-76 (top 24 bits)   */
float    axo_rng_uniform(float lo, float hi);         /* rng.c:78-80                 */
float    axo_rng_normal(void);                        /* rng.c:87-105 (polar, cached spare) */
uint64_t axo_rng_bounded(uint64_t n);                 /* rng.c:111-121 (rejection)   */
void     axo_rng_drop_spare(void);                    /* forget the cached normal    */
void     axo_fill_uniform(float *dst, int64_t n, float lo, float hi);   /* tensor.c:520-531 */
void     axo_fill_normal(float *dst, int64_t n, float mean, float std); /* rng.c:107-109   */
void     axo_fill_kaiming_uniform(float *dst, int64_t n, int64_t fan_in); /* init.c:84-94  */
void     axo_fill_int8(int8_t *dst, int64_t n);       /* (int8)(bounded(255) - 127)  */

/* ---- fp32 GEMM ---------------------------------------------------------- */
/* ground truth: fp64 accumulation, fp64 result.  transb: B stored [N,K]. */
void axo_gemm_f64(const float *a, const float *b, double *c, int64_t M, int64_t N, int64_t K,
                  int transb);
/* sum_k |a_ik|*|b_kj| in fp64: the scale of the rounding-error bound. */
void axo_gemm_abs_f64(const float *a, const float *b, double *c, int64_t M, int64_t N,
                      int64_t K, int transb);
/* cpu_naive.c:150-187: fp32 running sum, k ascending, separate multiply and add. */
void axo_gemm_naive(const float *a, const float *b, float *c, int64_t M, int64_t N, int64_t K);
/* cpu_opt.c:3509: 1 when (m,n,k) takes the serial small/skinny-M AXPY route (MR = 6). */
int  axo_gemm_takes_small_route(int64_t m, int64_t n, int64_t k);
/* cpu_opt.c:3446-3956: small route, else packed 6x16 BLIS loops (JC-parallel). */
void axo_gemm_opt(const float *a, const float *b, float *c, int64_t M, int64_t N, int64_t K);
/* cpu_opt.c:4842-5258: C = A[M,K] * B[N,K]^T through the same packed kernel. */
void axo_gemm_opt_nt(const float *a, const float *b, float *c, int64_t M, int64_t N, int64_t K);
/* cpu_opt.c:7148-7194 with the mathematically intended axis: c[m,n] += bias[n]. */
void axo_bias_add_cols(float *c, const float *bias, int64_t M, int64_t N);
/* Bias gradient: out[j] = sum_i in[i*cols + j], each column added row by row in fp32 — the
 * order of both the scalar loop in autograd_ops.c:740-752 and the per-lane accumulators of
 * simd_axis0_sum (cpu_opt.c opt_sum, axis 0), so this restatement is bit-exact with them.
 * Pinned against oracle/_ref (ax_compute_sum) in tests/test_oracle.py. */
void axo_sum_axis0(const float *in, int64_t rows, int64_t cols, float *out);
/* fp64 ground truth of any axis: out[o,i] = sum_a in[o,a,i], and the sum of |in| for the bound. */
void axo_sum_axis_f64(const float *in, int64_t outer, int64_t axis_len, int64_t inner, double *out, double *out_abs);
/* cpu_opt.c:7287-7307 (vector body): y[i] = fma(alpha, x[i], y[i]). */
void axo_axpy(const float *x, float alpha, float *y, int64_t n);
/* Scaled dot-product attention forward, per head: O = softmax(scale * Q K^T [causal]) V,
 * L = row max + log(row sum) or NULL.  The textbook evaluation the reference's own test uses as
 * its yardstick (tests/test_attention.c:17-48, gate 1e-4); the reference's fused kernel
 * (src/core/fused_attention.c:559-573) is pinned against it through oracle/_ref and the
 * golden vectors in tests/test_oracle.py.  The _f64 form is the ground truth. */
void axo_sdpa_fwd(const float *Q, const float *K, const float *V, float *O, float *L, int64_t BH,
                  int64_t S, int64_t dk, float scale, int causal);
void axo_sdpa_fwd_f64(const float *Q, const float *K, const float *V, double *O, double *L, int64_t BH,
                      int64_t S, int64_t dk, float scale, int causal);
/* cpu_opt.c:7401-7440: c = max(c + bias[n], 0); bias may be NULL. */
void axo_bias_relu(float *c, const float *bias, int64_t M, int64_t N);
/* activations.c:24-25,267-316 (scalar tail form): 0.5x(1+tanh(0.79788456(x+0.044715x^3))). */
float axo_gelu_tanh(float x);
void  axo_gelu(float *x, int64_t n);
double axo_gelu_f64(double x);

/* ---- remaining elementwise / reduction / optimizer slots ----------------------------------
 * Pinned in tests/test_oracle.py against oracle/_ref through the golden vectors (the reference's
 * naive and optimised CPU backends, its activation functions, its layer-norm layer and its
 * optimizers) and against numpy closed forms. */
/* Broadcasting binary op, element by element as cpu_naive.c:48-62,70-97,482-507: trailing
 * dimensions are aligned, an operand dimension of extent 1 is broadcast.  op: 0 add, 1 sub,
 * 2 mul, 3 div, 4 equal, 5 greater, 6 add_relu (cpu_naive.c:192-216).  Operands are contiguous. */
void axo_binary(int op, const float *a, const int64_t *a_shape, int a_ndim, const float *b,
                const int64_t *b_shape, int b_ndim, float *out, const int64_t *out_shape, int out_ndim);
/* cpu_naive.c:112-147,552-576 and the parametrised activations of src/core/activations.c
 * (leaky_relu :79-93, elu :141-155, swish :363-376): op numbering of axhip_unary. */
void axo_unary(int op, const float *in, float *out, int64_t n, float param);
/* cpu_naive.c:311-479: op 0 sum, 1 mean (sum * (1/count)), 2 max, 3 min over [outer, axis, inner];
 * sums add in ascending axis order. */
void axo_reduce_axis(int op, const float *in, int64_t outer, int64_t axis_len, int64_t inner, float *out);
/* cpu_opt.c:7236-7247 */
void axo_argmax_axis(const float *in, int64_t outer, int64_t axis_len, int64_t inner, int64_t *out);
/* cpu_naive.c:235-270 */
void axo_softmax_rows(const float *in, float *out, int64_t rows, int64_t cols);
/* src/core/norm.c:1338-1399, scalar form; x_hat / inv_std may be NULL. */
void axo_layernorm_fwd(const float *x, const float *gamma, const float *beta, float *out, float *x_hat,
                       float *inv_std, int64_t rows, int64_t cols, float eps);
/* cuda/ops_optim.cu:17-35,66-77 (the per-element form of adam_step, src/core/optim.c:262-330) */
void axo_adam_update(float *w, const float *g, float *m, float *v, int64_t n, float lr, float beta1,
                     float beta2, float eps, float weight_decay, float bc1, float bc2, int decoupled);
/* cuda/ops_optim.cu:40-62 (sgd_step, src/core/optim.c:100-205); mom may be NULL */
void axo_sgd_update(float *w, const float *g, float *mom, int64_t n, float lr, float momentum,
                    float weight_decay, int nesterov);

/* ---- int8 --------------------------------------------------------------- */
/* quantize.c:21-57: per-row absmax/127, zero row -> 1, lrintf, clamp +-127. */
void axo_quantize_rows(const float *w, int64_t N, int64_t K, int8_t *q, float *scales);
/* quantize.c:66-76 */
void axo_dequantize_rows(const int8_t *q, const float *scales, int64_t N, int64_t K, float *out);
/* quantize.c:100-177, AVX2 build: 4x8 lane partial sums, 8-wide tail, pairwise reduce. */
void axo_qgemm_w8a32(const float *a, const int8_t *q, const float *scales, float *out,
                     int64_t M, int64_t N, int64_t K);
/* exact: acc[m,n] = sum_k (int32)x[m,k]*(int32)w[n,k]  (no reference counterpart). */
void axo_qgemm_w8a8_acc(const int8_t *x, const int8_t *w, int32_t *acc,
                        int64_t M, int64_t N, int64_t K);
/* out = act((float)acc * (x_scale*w_scale[n]) + bias[n]); act: 0 none, 1 relu, 2 gelu.
   Evaluated as one fp32 product of the scales, one int->float convert, one fused
   multiply-add (plain multiply when bias is NULL). */
void axo_w8a8_epilogue(const int32_t *acc, float x_scale, const float *w_scales,
                       const float *bias, int act, float *out, int64_t M, int64_t N);

#ifdef __cplusplus
}
#endif
#endif
