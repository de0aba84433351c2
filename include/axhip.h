/* axhip.h — C ABI of libaxhip.so, the MI355X (gfx950) GEMM kernels for Axiom.
 *
 * Plain pointers and sizes only.  Every pointer named "device" is HIP device memory
 * obtained from axhip_malloc (or any hipMalloc in the same process).  All matrices are
 * row-major.  Work is queued on the HIP null stream and is asynchronous with respect to
 * the host unless stated; axhip_memcpy_d2h and axhip_synchronize wait for it.
 *
 * Return value: 0 (AXHIP_OK) on success, otherwise one of the AXHIP_ERR_* codes, whose
 * numeric values equal Axiom's ax_status_t (include/axiom/types.h:89-103) so the host
 * adapter can return them unchanged.  axhip_last_error() holds a description.
 * There is no CPU fallback anywhere in this library: without a usable GPU every compute
 * entry point fails with AXHIP_ERR_BACKEND.
 *
 * Each entry point cites the reference interface it stands in for (paths relative to the
 * Axiom tree).
 */
#ifndef AXHIP_H
#define AXHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    AXHIP_OK = 0,
    AXHIP_ERR_NULL_ARG = 1,
    AXHIP_ERR_ALLOC = 2,
    AXHIP_ERR_SHAPE = 3,          /* AX_ERR_SHAPE_MISMATCH */
    AXHIP_ERR_INVALID_AXIS = 5,
    AXHIP_ERR_BACKEND = 9,
    AXHIP_ERR_NOT_IMPLEMENTED = 10
};

/* fused epilogue activation */
enum { AXHIP_ACT_NONE = 0, AXHIP_ACT_RELU = 1, AXHIP_ACT_GELU = 2 };

/* ---- lifecycle: the device-owner hooks of struct ax_backend_ops
 *      (include/axiom/internal/backend_ops.h:267-296; CUDA versions in
 *      src/compute/backends/cuda/backend.cu:56-116) ------------------------------ */
int         axhip_init(void);                 /* .init          */
void        axhip_shutdown(void);             /* .shutdown      */
int         axhip_synchronize(void);          /* .synchronize   */
int         axhip_device_count(void);         /* .device_count  */
const char *axhip_last_error(void);           /* thread-local message of the last failure */
const char *axhip_device_name(void);          /* gcnArchName of device 0, "" without a GPU */

/* Tile-selection overrides, for re-measuring the dispatch thresholds without recompiling — the
 * counterpart of AX_GEMM_MC / AX_GEMM_NC / AX_GEMM_KC (src/compute/backends/cpu_opt.c:512-539).
 * Read from the environment by axhip_init and again by axhip_tuning_reload (which needs no GPU and
 * returns how many variables were recognised); unset, empty or invalid values mean "choose by shape".
 * A forced choice applies only where the shape permits that kernel; results do not depend on it.
 *   AX_HIP_I8_TILE       64x64 | 64x64k2 | 128x64 | 128x128 | 256x256   W8A8 tile (256x256: M, N multiples of 256;
 *                        k2: two wave sets split each K slab)
 *   AX_HIP_I8_SPLITK     1..16      workgroups over K per W8A8 tile of 64x64 / 128x128 (1: never split)
 *   AX_HIP_I8_MFMA       16 | 32    matrix-core instruction of the persistent 256x256 W8A8 kernel: v_mfma_i32_16x16x64_i8 (what
 *                        runs by default) or v_mfma_i32_32x32x32_i8; the results are the same bits
 *   AX_HIP_F32_TILE      64x64 | 64x64k2 | 128x128   fp32 tile on the aligned fast path (k2: two wave sets split each K slab)
 *   AX_HIP_F32_SPLITK    1..4096    K ranges of the fp32 few-tile route (1: never split)
 *   AX_HIP_NT_WALK       1 | 2      batched A B^T with K <= 128: 1, a 128-row block of A stays in LDS and the column blocks of B^T
 *                        are walked; 2, 256 rows of B stay in registers and A is walked in blocks of 32 rows (N a multiple of 256)
 *   AX_HIP_SKINNY_BLOCKS 1..65535   workgroups the skinny-M route aims for
 *   AX_HIP_SKINNY_KPS    16..8192   most rows of K one skinny-M workgroup takes (rounded down to a multiple of 16)
 *   AX_HIP_SKINNY_FORM   1..3       form of the skinny-M kernel for M <= 8: 1, workgroups of 256 threads; 2, the same with the
 *                        four lane groups of a wave added before LDS; 3, workgroups of 512 threads
 *   AX_HIP_W8A32_TILE    128x256 | 128x128 | 64x128 | 32x128 | 32x64   W8A32 matrix-core tile where K > 128 and a multiple of 32
 *                        (edge form off the tile grid)
 * axhip_tuning_get returns the value in effect (0: automatic; tiles as their first number, 64x64k2 as
 * 642, 128x64 as 1264; AX_HIP_W8A32_TILE as the position in its list, 1..5), or -1 for an unknown name. */
int axhip_tuning_reload(void);
int axhip_tuning_get(const char *name);

/* Threading: compute entry points must be called from one host thread at a time.  They share a
 * device workspace, arrival counters and a vector of ones that several of them keep data in across
 * two or more launches (split-K partial sums, reduction partials, padded operand copies), all on the
 * HIP null stream; a second thread issuing such a call in between would overwrite them.  This is the
 * contract of the reference's backends (include/axiom/ops.h:17-19, cuda/internal.h:70-74).  Only
 * axhip_malloc / axhip_free / axhip_alloc_stats may be called concurrently with anything. */

/* ---- memory: .storage_alloc/.storage_free/.memcpy_* hooks
 *      (src/compute/backends/cuda/memory.cu:78-140).  axhip_malloc returns zero-filled
 *      memory like the reference's allocator (memory.cu:90), or NULL.  Blocks are pooled: axhip_free
 *      keeps a block (up to 1 GiB each, 16 GiB in all) for the next request of its size class, and
 *      neither call waits for the device; axhip_shutdown returns everything to the driver. ------ */
void *axhip_malloc(size_t bytes);
void *axhip_malloc_uninit(size_t bytes);   /* contents undefined: for results that are fully overwritten */
void  axhip_free(void *device_ptr);             /* NULL, foreign and already-freed pointers are ignored */
/* Allocation counters for leak diagnosis (ax_cuda_alloc_stats / ax_cuda_reset_alloc_stats,
 * cuda/memory.cu:13-29): requests served and blocks given back, in calls and in bytes of their size
 * classes, so allocs == frees and bytes_alloc == bytes_free once every tensor is destroyed; plus
 * how many of the requests needed the driver (the rest were pool hits) and the bytes the pool holds
 * back now.  Any pointer may be NULL. */
void  axhip_alloc_stats(int64_t *allocs, int64_t *frees, int64_t *bytes_alloc, int64_t *bytes_free,
                        int64_t *driver_allocs, int64_t *bytes_cached);
void  axhip_reset_alloc_stats(void);
/* Bytes of device memory the driver reports free on the current device (hipMemGetInfo), or -1 without
 * a device.  The counterpart of what cudaMemGetInfo gives a caller of the reference's CUDA backend. */
int64_t axhip_device_free_bytes(void);
/* The shared device workspace (split-K partial sums, reduction partials, padded operand copies) is 64 MiB
 * from axhip_init on and grows when a call needs more; growing waits for the device, frees the old block and asks the
 * driver for a new one, which costs the first call at a larger shape some tens of microseconds that later
 * calls do not pay.  axhip_workspace_reserve grows it ahead of time (at model load, before a timed or
 * latency-bound loop) to at least `bytes` and reports the size it then has in *have (may be NULL); bytes = 0
 * only reports.  It never shrinks.  No counterpart in the reference, whose CUDA backend grows its score
 * buffer on demand in the same way (cuda/ops_attention.cu:305-318) and offers no call to do it ahead of
 * time.  Same threading rule as the compute entry points. */
int   axhip_workspace_reserve(size_t bytes, size_t *have);
int   axhip_memset(void *device_ptr, int byte_value, size_t bytes);
int   axhip_memcpy_h2d(void *device_dst, const void *host_src, size_t bytes);
int   axhip_memcpy_d2h(void *host_dst, const void *device_src, size_t bytes);   /* blocking */
int   axhip_memcpy_d2d(void *device_dst, const void *device_src, size_t bytes);

/* ---- fp32 GEMM.  Replaces cuda_gemm / cuda_gemm_ex / cuda_gemm_nt / cuda_gemm_tn
 *      (src/compute/backends/cuda/ops_gemm.cu:15-126) and the cpu_opt drivers
 *      opt_gemm / opt_gemm_nt / opt_gemm_relu / opt_gemm_ex
 *      (src/compute/backends/cpu_opt.c:3446, 4842, 7401, 7442), with the bias add of
 *      k_bias_add (cuda/ops_fused.cu:260-297) and the GELU of k_gelu
 *      (cuda/ops_activations.cu:22) folded into the write-back.
 *
 *      C[M,N] = act( alpha * op(A) * op(B) + beta * C + bias[n] )
 *      transa = 0: A is [M,K] (lda >= K);  1: A is [K,M] (lda >= M)
 *      transb = 0: B is [K,N] (ldb >= N);  1: B is [N,K] (ldb >= K)
 *      bias may be NULL; beta == 0 never reads C (C may be uninitialised).
 *      True fp32 MFMA arithmetic; M <= 16 with transa = transb = 0, alpha = 1, beta = 0 takes
 *      the weight-streaming route below. ------------------------------------------------- */
int axhip_sgemm(int transa, int transb, int64_t M, int64_t N, int64_t K, float alpha,
                const float *A, int64_t lda, const float *B, int64_t ldb, float beta,
                float *C, int64_t ldc, const float *bias, int act);

/* Strided-batched form.  Replaces cublasSgemmStridedBatched as used for the per-head
 * products in src/compute/backends/cuda/ops_attention.cu:326-334 (score = scale*Q*K^T)
 * and :378-386 (O = P*V).  Matrix i of each operand starts at ptr + i*stride (elements). */
int axhip_sgemm_strided_batched(int transa, int transb, int64_t M, int64_t N, int64_t K,
                                float alpha, const float *A, int64_t lda, int64_t stride_a,
                                const float *B, int64_t ldb, int64_t stride_b, float beta,
                                float *C, int64_t ldc, int64_t stride_c, int64_t batch);

/* Skinny-M route (1 <= M <= 16): C[M,N] = act(A[M,K] * B[K,N] + bias[n]), B streamed once
 * for all M rows.  The GPU counterpart of the small/skinny-M AXPY route of opt_gemm
 * (src/compute/backends/cpu_opt.c:3499-3567).  Results are deterministic run to run. */
int axhip_sgemm_skinny(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                       const float *B, int64_t ldb, float *C, int64_t ldc,
                       const float *bias, int act);

/* The skinny-M route with a narrow layer riding on it, in one launch:
 *   C[M,N]     = act(A[M,K] * B[K,N] + bias[n])                 (C may be NULL: then it is never written)
 *   out2[M,NH] = act2(C[M,N] * W2[N,NH] + bias2[j]),   1 <= NH <= 16, W2 and out2 dense
 * i.e. a Dense(+activation) layer followed by a Dense layer of at most 16 outputs — the hidden layer and
 * classifier head that end the 784-4096-4096-10 network of the reference's benchmarks — as Sequential runs
 * them at batch sizes of a few rows (src/core/layer.c:181-230 over opt_gemm's skinny route,
 * src/compute/backends/cpu_opt.c:3499-3567).  Whoever finishes a strip of C multiplies it by the head's rows
 * for that strip; the strips' partial vectors are added in strip order, so results are deterministic.  C is
 * bit-identical to axhip_sgemm_skinny; out2 is the same sum in another order. */
int axhip_sgemm_skinny_head(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B,
                            int64_t ldb, float *C, int64_t ldc, const float *bias, int act, int64_t NH,
                            const float *W2, const float *bias2, int act2, float *out2);

/* The same route for callers that cannot allocate device memory (tight serving loops, harnesses that
 * forbid hipMalloc).  It has no counterpart in the reference.  Arguments, results and kernels are those of
 * axhip_sgemm_skinny — outputs are bit-identical — but what the K ranges of a launch are joined through
 * (8 MiB of exchange slots, 8 MiB for partial tiles, 4096 strip counters) lives in a 16 MiB + 16 KiB
 * array that is part of the library's device code (one copy per GPU, held until the process ends), and
 * the call makes no hipMalloc / hipFree and grows no workspace.  Like every entry point here it launches
 * on the HIP null stream, so it cannot itself be recorded into a HIP graph.  axhip_init must have run on
 * the current device.  A plan that needs more than 8 MiB of either kind ((K ranges - 1) * M * N * 4 bytes
 * of slots, or K ranges * M * N * 4 bytes of tiles for M >= 5 with more than four ranges) or more than
 * 4096 strips of 64 columns with tiles is refused with AXHIP_ERR_SHAPE.  All calls on one GPU share the
 * array: calls that overlap in time on one GPU (two streams, two host threads) race; calls issued one
 * after another do not.  Slots must read "empty" and counters zero when a launch starts: axhip_init
 * leaves them so and every launch that runs to its end does too; after a launch that did not (a device
 * error reported by this or a later call), call axhip_sgemm_skinny_reset before the next one. */
int axhip_sgemm_skinny_static(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                              const float *B, int64_t ldb, float *C, int64_t ldc,
                              const float *bias, int act);

/* Empties the join slots and zeroes the arrival counters of the skinny-M route again (those of
 * axhip_sgemm_skinny_static and those the allocating entry points own): fills queued on the null stream,
 * no allocation.  Only needed after a skinny-M launch was cut short by a device error; without that, a
 * later launch would take the stale sums or arrivals of the dead one for its own and leave outputs
 * unwritten. */
int axhip_sgemm_skinny_reset(void);

/* ---- measurement probe --------------------------------------------------------------- */
/* Not a compute path: one launch does the int8 matrix-core work of axhip_qgemm_w8a8 at M = N = K = 8192 on
 * a 256-CU device (8192 blocks of 262144 multiply-adds per CU-resident wave) with nothing around it but LDS
 * fragment reads, so that a committed command (bench.py --sustain S --operands probe...) can show what the
 * matrix cores of the GPU at hand sustain, and at what clock, on operands that change from instruction to
 * instruction.  mfma_shape: 32 (v_mfma_i32_32x32x32_i8) or 16 (v_mfma_i32_16x16x64_i8, twice as many
 * instructions for the same multiply-adds); lds_reads: 16-byte fragment reads per block, 0..6 (6 = the
 * 128x64 wave tile of the GEMM kernel, 4 = what a 128x128 wave tile would need, 0 = operands that never
 * change); operand_bytes: 128 KiB of device memory that every workgroup copies into LDS (random bytes, or
 * zeros for a loop without switching activity); sink: 512 ints per CU, receives checksums.  It has no
 * counterpart in the reference. */
int axhip_probe_int8_matrix_core(int mfma_shape, int lds_reads, const int8_t *operand_bytes, int32_t *sink);
/* The fp32 counterpart (bench.py --sustain S --operands fprobe...): per launch 1024 blocks of 16384 multiply-adds per
 * wave, eight waves per CU, as v_mfma_f32_32x32x2_f32 (mfma_shape 32) or v_mfma_f32_16x16x4_f32 (16), with lds_reads
 * (0..3) 16-byte fragment reads per block (3 = the 64x32 wave tile of the batched attention kernels); operand_floats:
 * 128 KiB of device memory, sink: 512 floats per CU. */
int axhip_probe_fp32_matrix_core(int mfma_shape, int lds_reads, const float *operand_floats, float *sink);

/* ---- int8 -------------------------------------------------------------------------- */
/* W8A8: acc[m,n] = sum_k (int32)x[m,k] * (int32)w[n,k]   (exact, int32 MFMA)
 *       out[m,n] = act( (float)acc * (x_scale * w_scales[n]) + bias[n] )
 * x is [M,K] int8, w is [N,K] int8 — the data/scales layout of ax_qweight_t
 * (include/axiom/quantize.h:50-55).  bias, out and acc_out may each be NULL (at least one
 * of out / acc_out must be given).  Extends ax_qgemm_w8a32 (src/core/quantize.c:100-177)
 * to int8 activations with int32 accumulation; there is no reference counterpart. */
int axhip_qgemm_w8a8(const int8_t *x, float x_scale, const int8_t *w, const float *w_scales,
                     const float *bias, int act, float *out, int32_t *acc_out,
                     int64_t M, int64_t N, int64_t K);

/* W8A32: out[m,n] = w_scales[n] * sum_k a[m,k] * (float)w[n,k], fp32 accumulation.
 * Device-memory form of ax_qgemm_w8a32 (src/core/quantize.c:100-177).  Every product
 * a[m,k] * w[n,k] enters the sum exactly (up to M = 6 as a fused multiply-add; above, as three
 * bf16 terms of a[m,k] that add up to it exactly, times the int8 weight as a bf16, on the bf16
 * matrix core); only the order of the fp32 additions differs from the reference's loop.
 * +-inf and NaN among the activations give what that loop gives.  The bf16 matrix core flushes
 * denormal operands: the low-order terms of activations below 2^-110 in magnitude are dropped, an
 * absolute error of less than K * 2^-118 * w_scales[n] per output on top of the accumulation's. */
int axhip_qgemm_w8a32(const float *a, const int8_t *w, const float *w_scales, float *out,
                      int64_t M, int64_t N, int64_t K);

/* Per-row symmetric int8 quantization on the device: the arithmetic of
 * ax_qweight_create_from_fp32 (src/core/quantize.c:36-54). w is [N,K] fp32. */
int axhip_quantize_rows(const float *w, int64_t N, int64_t K, int8_t *q, float *scales);

/* ---- elementwise vtable slots ------------------------------------------------------- */
/* .bias_add: out[o,a,i] = in[o,a,i] + bias[a]   (cuda/ops_fused.cu:260-297,
 * cpu_opt.c:7148-7194); in/out may alias. */
int axhip_bias_add(const float *in, const float *bias, int64_t outer, int64_t axis_len,
                   int64_t inner, float *out);
int axhip_relu(const float *in, float *out, int64_t n);       /* .relu    */
int axhip_gelu(const float *in, float *out, int64_t n);       /* .gelu_op (tanh form) */
int axhip_fill_f32(float *dst, float value, int64_t n);       /* .fill    */

/* ---- reductions and accumulation used by the dense layer's backward pass -------------- */
/* .sum over one axis of a contiguous fp32 tensor viewed as [outer, axis_len, inner]:
 * out[o,i] = sum_a in[o,a,i]  (cuda_sum, cuda/ops_reduce.cu:262-295; opt_sum,
 * cpu_opt.c:4614-4660).  outer = 1 gives the bias gradient sum(grad_out, axis=0)
 * (src/core/autograd_ops.c:724-757). */
int axhip_sum_axis(const float *in, int64_t outer, int64_t axis_len, int64_t inner, float *out);
/* .sum with axis = -1: out[0] = sum of all n elements (cuda/ops_reduce.cu:268-275). */
int axhip_sum_all(const float *in, int64_t n, float *out);
/* .axpy: y[i] = fma(alpha, x[i], y[i])  (cuda_axpy, cuda/ops_fused.cu:193-211; opt_axpy,
 * cpu_opt.c:7287-7307). */
int axhip_axpy(const float *x, float alpha, float *y, int64_t n);

/* ---- the remaining elementwise, reduction and optimizer vtable slots ------------------- */
/* Broadcasting binary ops (.add .sub .mul .div_op .equal .greater .add_relu): out is contiguous
 * with shape out_shape[ndim] (ndim <= 8); a_strides / b_strides are the operands' element
 * strides per OUTPUT dimension, 0 where the operand is broadcast along it — the mapping of
 * bcast_offset (cuda/ops_elementwise.cu:20-35) / broadcast_index (cpu_naive.c:48-62) resolved by
 * the caller.  equal/greater write 1.0f / 0.0f (cuda/ops_elementwise.cu:64-65); add_relu is
 * max(a + b, 0) (cuda/ops_fused.cu:13-21).  out may alias an operand that is not broadcast. */
enum {
    AXHIP_BIN_ADD = 0, AXHIP_BIN_SUB, AXHIP_BIN_MUL, AXHIP_BIN_DIV, AXHIP_BIN_EQUAL, AXHIP_BIN_GREATER,
    AXHIP_BIN_ADD_RELU
};
int axhip_binary(int op, const float *a, const float *b, float *out, int ndim, const int64_t *out_shape,
                 const int64_t *a_strides, const int64_t *b_strides);

/* Unary and scalar ops over n contiguous elements; in/out may alias.  Definitions:
 * cuda/ops_elementwise.cu:147-155 (neg, abs, exp, log: v > 0 ? logf(v) : -FLT_MAX, sqrt:
 * v >= 0 ? sqrtf(v) : 0, square, sigmoid, tanh), :195-208 (add_scalar, mul_scalar with the
 * scalar in `param`), cuda/ops_activations.cu:23-52 (swish = v / (1 + exp(-v)), leaky_relu and
 * elu with alpha in `param`). */
enum {
    AXHIP_UN_NEG = 0, AXHIP_UN_ABS, AXHIP_UN_EXP, AXHIP_UN_LOG, AXHIP_UN_SQRT, AXHIP_UN_SQUARE,
    AXHIP_UN_SIGMOID, AXHIP_UN_TANH, AXHIP_UN_LEAKY_RELU, AXHIP_UN_ELU, AXHIP_UN_SWISH,
    AXHIP_UN_ADD_SCALAR, AXHIP_UN_MUL_SCALAR
};
int axhip_unary(int op, const float *in, float *out, int64_t n, float param);

/* .sum .mean .max_op .min_op over one axis of [outer, axis_len, inner], or over everything
 * (cuda/ops_reduce.cu:262-378; cpu_naive.c:311-479).  mean = sum * (1 / count); max / min start
 * from -FLT_MAX / FLT_MAX and pass over NaNs, as the reference's compare-and-replace loops do. */
enum { AXHIP_RED_SUM = 0, AXHIP_RED_MEAN, AXHIP_RED_MAX, AXHIP_RED_MIN };
int axhip_reduce_axis(int op, const float *in, int64_t outer, int64_t axis_len, int64_t inner, float *out);
int axhip_reduce_all(int op, const float *in, int64_t n, float *out);
/* .argmax: index (int64) of the first largest element along the axis (opt_argmax,
 * cpu_opt.c:7202-7249). */
int axhip_argmax_axis(const float *in, int64_t outer, int64_t axis_len, int64_t inner, int64_t *out);

/* .softmax_rowwise over contiguous [rows, cols]: exp(x - rowmax) / sum (cuda/ops_fused.cu:44-91,
 * cpu_naive.c:235-270); in/out may alias. */
int axhip_softmax_rows(const float *in, float *out, int64_t rows, int64_t cols);

/* Layer normalisation forward over the last axis of contiguous [rows, cols]
 * (layernorm_forward, src/core/norm.c:1338-1399): mean and E[x^2] in one pass, var clamped at 0,
 * inv_std = 1 / sqrt(var + eps), out = gamma * x_hat + beta.  x_hat [rows, cols] and inv_std
 * [rows] are the tensors the reference saves for its backward pass; either may be NULL. */
int axhip_layernorm_fwd(const float *x, const float *gamma, const float *beta, float *out, float *x_hat,
                        float *inv_std, int64_t rows, int64_t cols, float eps);

/* .adam_update / .sgd_update: one fused pass per parameter tensor, w (and m, v / the momentum
 * buffer) updated in place (cuda_adam_update / cuda_sgd_update, cuda/ops_optim.cu:17-110, which
 * follow adam_step / sgd_step of src/core/optim.c).  bc1 = 1 - beta1^t, bc2 = 1 - beta2^t;
 * momentum_buf may be NULL. */
int axhip_adam_update(float *w, const float *g, float *m, float *v, int64_t n, float lr, float beta1,
                      float beta2, float eps, float weight_decay, float bc1, float bc2, int decoupled);
int axhip_sgd_update(float *w, const float *g, float *momentum_buf, int64_t n, float lr, float momentum,
                     float weight_decay, int nesterov);

/* ---- scaled dot-product attention forward --------------------------------------------- */
/* O[h] = softmax(scale * Q[h] K[h]^T) V[h] for BH heads; Q, K, V, O are [BH, S, dk] row-major
 * fp32 in device memory, L is [BH, S] (log-sum-exp of each score row, natural log) or NULL;
 * causal != 0: query i sees keys j <= i.  Replaces ax_cuda_sdpa_fwd
 * (cuda/ops_attention.cu:299-392) and the device form of ax_fused_attention_fwd /
 * ax_fused_attention_fwd_causal (include/axiom/attention.h:273-283,
 * src/core/fused_attention.c:559-573).  dk a multiple of 4 up to 128 (16-byte aligned tensors, any S)
 * runs fused, with no score matrix in memory, on the kernel of the next size among 32, 64 and 128;
 * other head sizes go through batched GEMMs and a row softmax. */
int axhip_sdpa_fwd(const float *Q, const float *K, const float *V, float *O, float *L,
                   int64_t BH, int64_t S, int64_t dk, float scale, int causal);
/* The same attention on heads that lie side by side in the rows of wider matrices: head (b, h)
 * reads rows b*S .. b*S+S-1, columns h*dk .. h*dk+dk-1 of Q, K and V (row pitch ld floats) and
 * writes the same block of O (row pitch ldo); L is [B*H, S] or NULL.  With Q = qkv, K = qkv + D,
 * V = qkv + 2D, ld = 3D, ldo = D this consumes the fused projection [B*S, 3D] and produces the
 * [B*S, D] input of the output projection directly, i.e. it stands for the sequence
 * head_interleave_qkv_split -> sdpa_fwd -> head_deinterleave of the reference's MHA forward
 * (src/core/attention.c:211-262, 391-400) without the three layout passes.  dk must be a multiple
 * of 4 up to 128, pitches multiples of 4 floats, tensors 16-byte aligned (AXHIP_ERR_NOT_IMPLEMENTED /
 * AXHIP_ERR_SHAPE otherwise). */
int axhip_sdpa_fwd_rows(const float *Q, const float *K, const float *V, int64_t ld, float *O, int64_t ldo,
                        float *L, int64_t B, int64_t H, int64_t S, int64_t dk, float scale, int causal);

/* ---- layout transforms around attention (the layout members of the reference's GPU extension
 * table, include/axiom/internal/cuda_extension.h:45-84) ------------------------------------- */
/* qkv [B*S, 3D] (row = [q | k | v], D = H*dk) -> q, k, v each [B*H, S, dk]; bqkv [3D] is added
 * when not NULL (ax_attn_head_interleave_qkv_split[_bias], src/core/attention/layout.c:215-262). */
int axhip_head_split_qkv(const float *qkv, const float *bqkv, float *q, float *k, float *v, int64_t B, int64_t S,
                         int64_t H, int64_t dk, int64_t D);
/* [B, S, H, dk] -> [B*H, S, dk] and back (ax_attn_head_interleave / ax_attn_head_deinterleave,
 * src/core/attention/layout.c:84-152). */
int axhip_head_interleave(const float *src, float *dst, int64_t B, int64_t S, int64_t H, int64_t dk);
int axhip_head_deinterleave(const float *src, float *dst, int64_t B, int64_t S, int64_t H, int64_t dk);
/* dst [rows, 3*cols]: row i = [a[i,:] | b[i,:] | c[i,:]] — the fused projection weight [D, 3D] from
 * Wq, Wk, Wv, and with rows = 1 the fused bias (src/core/attention/cache.c:49-57, 79-81). */
int axhip_concat3_rows(float *dst, const float *a, const float *b, const float *c, int64_t rows, int64_t cols);

/* ---- timing on the library's stream (for benchmarks) -------------------------------- */
void *axhip_event_create(void);
void  axhip_event_destroy(void *ev);
int   axhip_event_record(void *ev);
int   axhip_event_elapsed_ms(void *start, void *stop, float *ms);   /* waits for stop */

/* Name of the kernel variant the last GEMM-type call launched (for profiles/tests). */
const char *axhip_last_kernel(void);

#ifdef __cplusplus
}
#endif
#endif /* AXHIP_H */
