// Measurement probe, not a compute path: the int8 matrix-core work of one W8A8 GEMM at M = N = K = 8192
// (8192 MFMAs of 32x32x32 per wave, eight waves on each of 256 CUs) with nothing around it but LDS
// fragment reads.  It answers, with a committed command (bench.py --sustain ... --operands probe...),
// what the matrix cores of a given GPU sustain on operands that change from instruction to instruction,
// how that depends on the MFMA shape (32x32x32 against 16x16x64, same multiply-adds per block) and on
// the number of 16-byte fragment reads per 262144 multiply-adds (6 in k_qgemm_w8a8_256, whose wave tile
// is 128x64; 4 for a 128x128 wave tile; 0 = registers that never change).  Nothing in the library calls
// it; its output is a checksum nobody interprets.
#include "common.h"

namespace {
using namespace axhip;

#define AXP_DS_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off))
#define AXP_LGKM0() __builtin_amdgcn_s_waitcnt(0x3F | (3 << 14) | (7 << 4) | (0 << 8))

constexpr int kLdsBytes = 128 * 1024;       // the two operand stages of the GEMM kernel
constexpr int kBlocksPerLaunch = 1024;      // blocks of 262144 multiply-adds per wave: 4 tiles x 64 slabs x 4 k-steps

// One block = the multiply-adds of one k-step of the GEMM kernel's wave tile (128x64x32).
//   SHAPE 32: 8 MFMAs 32x32x32 on fragments fx[4] (rows) and fw[2] (columns)
//   SHAPE 16: 16 MFMAs 16x16x64 on fragments fx[4] and fw[4] (half a 128x64x64 step)
// READS of the fragments are re-read from LDS for the next block, at addresses that move through 48 KiB,
// between the MFMAs; the others keep their values.
template <int SHAPE, int READS>
__global__ void __launch_bounds__(512)
k_probe_i8(const int8_t *__restrict__ src, int blocks, int *__restrict__ sink) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    for (int i = tid; i < kLdsBytes / 16; i += 512)
        reinterpret_cast<v4i *>(lds)[i] = reinterpret_cast<const v4i *>(src)[i];
    __syncthreads();
    const unsigned base = (unsigned)(uintptr_t)lds + ((tid >> 6) & 7) * 8192 + lane * 16;
    constexpr int NF = SHAPE == 32 ? 6 : 8;
    v4i f[2][NF];
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
        for (int r = 0; r < NF; r++) f[b][r] = *reinterpret_cast<const v4i *>(lds + ((tid >> 6) & 7) * 8192 + lane * 16 + r * 1024);

    if constexpr (SHAPE == 32) {
        v16i acc[8];
#pragma unroll
        for (int m = 0; m < 8; m++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[m][v] = 0;
#define AXP_BLOCK32(cur, off)                                                                                    \
    do {                                                                                                         \
        AXP_LGKM0();                                                                                             \
        __builtin_amdgcn_sched_barrier(0);                                                                       \
        _Pragma("unroll") for (int m = 0; m < 8; m++) {                                                          \
            acc[m] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f[cur][4 + (m & 1)], f[cur][m >> 1], acc[m], 0, 0, 0); \
            __builtin_amdgcn_sched_barrier(0);                                                                   \
            if (m == 0 && READS > 0) AXP_DS_READ(f[1 - (cur)][0], base, (off) + 0 * 1024);                       \
            if (m == 1 && READS > 1) AXP_DS_READ(f[1 - (cur)][4], base, (off) + 1 * 1024);                       \
            if (m == 2 && READS > 2) AXP_DS_READ(f[1 - (cur)][1], base, (off) + 2 * 1024);                       \
            if (m == 3 && READS > 3) AXP_DS_READ(f[1 - (cur)][5], base, (off) + 3 * 1024);                       \
            if (m == 4 && READS > 4) AXP_DS_READ(f[1 - (cur)][2], base, (off) + 4 * 1024);                       \
            if (m == 5 && READS > 5) AXP_DS_READ(f[1 - (cur)][3], base, (off) + 5 * 1024);                       \
            __builtin_amdgcn_sched_barrier(0);                                                                   \
        }                                                                                                        \
    } while (0)
        for (int s = 0; s < blocks; s += 8) {
            AXP_BLOCK32(0, 0 * 6144 + 16);
            AXP_BLOCK32(1, 1 * 6144 + 32);
            AXP_BLOCK32(0, 2 * 6144 + 48);
            AXP_BLOCK32(1, 3 * 6144 + 64);
            AXP_BLOCK32(0, 4 * 6144 + 80);
            AXP_BLOCK32(1, 5 * 6144 + 96);
            AXP_BLOCK32(0, 6 * 6144 + 112);
            AXP_BLOCK32(1, 7 * 6144 + 0);
        }
#undef AXP_BLOCK32
        AXP_LGKM0();
        int sum = 0;
#pragma unroll
        for (int m = 0; m < 8; m++)
#pragma unroll
            for (int v = 0; v < 16; v++) sum += acc[m][v];
        sink[(int64_t)blockIdx.x * 512 + tid] = sum;
    } else {
        v4i acc[16];
#pragma unroll
        for (int m = 0; m < 16; m++) acc[m] = v4i{0, 0, 0, 0};
#define AXP_BLOCK16(cur, off)                                                                                      \
    do {                                                                                                           \
        AXP_LGKM0();                                                                                               \
        __builtin_amdgcn_sched_barrier(0);                                                                         \
        _Pragma("unroll") for (int m = 0; m < 16; m++) {                                                           \
            acc[m] = __builtin_amdgcn_mfma_i32_16x16x64_i8(f[cur][4 + (m & 3)], f[cur][m >> 2], acc[m], 0, 0, 0);   \
            __builtin_amdgcn_sched_barrier(0);                                                                     \
            if (m == 0 && READS > 0) AXP_DS_READ(f[1 - (cur)][0], base, (off) + 0 * 1024);                         \
            if (m == 2 && READS > 1) AXP_DS_READ(f[1 - (cur)][4], base, (off) + 1 * 1024);                         \
            if (m == 4 && READS > 2) AXP_DS_READ(f[1 - (cur)][1], base, (off) + 2 * 1024);                         \
            if (m == 6 && READS > 3) AXP_DS_READ(f[1 - (cur)][5], base, (off) + 3 * 1024);                         \
            if (m == 8 && READS > 4) AXP_DS_READ(f[1 - (cur)][2], base, (off) + 4 * 1024);                         \
            if (m == 10 && READS > 5) AXP_DS_READ(f[1 - (cur)][6], base, (off) + 5 * 1024);                        \
            __builtin_amdgcn_sched_barrier(0);                                                                     \
        }                                                                                                          \
    } while (0)
        for (int s = 0; s < blocks; s += 8) {
            AXP_BLOCK16(0, 0 * 6144 + 16);
            AXP_BLOCK16(1, 1 * 6144 + 32);
            AXP_BLOCK16(0, 2 * 6144 + 48);
            AXP_BLOCK16(1, 3 * 6144 + 64);
            AXP_BLOCK16(0, 4 * 6144 + 80);
            AXP_BLOCK16(1, 5 * 6144 + 96);
            AXP_BLOCK16(0, 6 * 6144 + 112);
            AXP_BLOCK16(1, 7 * 6144 + 0);
        }
#undef AXP_BLOCK16
        AXP_LGKM0();
        int sum = 0;
#pragma unroll
        for (int m = 0; m < 16; m++)
#pragma unroll
            for (int v = 0; v < 4; v++) sum += acc[m][v];
        sink[(int64_t)blockIdx.x * 512 + tid] = sum;
    }
}

template <int SHAPE>
int launch_probe(int reads, const int8_t *src, int *sink) {
    typedef void (*kern_t)(const int8_t *, int, int *);
    static const kern_t kerns[7] = {k_probe_i8<SHAPE, 0>, k_probe_i8<SHAPE, 1>, k_probe_i8<SHAPE, 2>, k_probe_i8<SHAPE, 3>,
                                    k_probe_i8<SHAPE, 4>, k_probe_i8<SHAPE, 5>, k_probe_i8<SHAPE, 6>};
    static bool raised[7] = {};
    if (!raised[reads]) {
        AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kerns[reads]), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes),
                      "hipFuncSetAttribute");
        raised[reads] = true;
    }
    hipLaunchKernelGGL(kerns[reads], dim3((unsigned)cu_count()), dim3(512), kLdsBytes, kStream, src, kBlocksPerLaunch, sink);
    return check_launch("probe_int8_matrix_core");
}

// The fp32 counterpart: the MFMAs of a 64x32 wave tile (the batched attention products' kernels) per block of 16384
// multiply-adds, as 8 x v_mfma_f32_32x32x2_f32 (fragments fa[2], fb[1], four k each) or 16 x v_mfma_f32_16x16x4_f32
// (half of fa[4], fb[2]), with READS (0..3) 16-byte fragment reads per block.
template <int SHAPE, int READS>
__global__ void __launch_bounds__(512)
k_probe_f32(const float *__restrict__ src, int blocks, float *__restrict__ sink) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    for (int i = tid; i < kLdsBytes / 16; i += 512)
        reinterpret_cast<v4f *>(lds)[i] = reinterpret_cast<const v4f *>(src)[i];
    __syncthreads();
    const unsigned base = (unsigned)(uintptr_t)lds + ((tid >> 6) & 7) * 8192 + lane * 16;
    v4f f[2][3];
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
        for (int r = 0; r < 3; r++) f[b][r] = *reinterpret_cast<const v4f *>(lds + ((tid >> 6) & 7) * 8192 + lane * 16 + r * 1024);
    float sum = 0.0f;
    if constexpr (SHAPE == 32) {
        v16f acc[2];
#pragma unroll
        for (int m = 0; m < 2; m++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[m][v] = 0.0f;
#define AXP_FBLOCK32(cur, off)                                                                                   \
    do {                                                                                                         \
        AXP_LGKM0();                                                                                             \
        __builtin_amdgcn_sched_barrier(0);                                                                       \
        _Pragma("unroll") for (int m = 0; m < 8; m++) {                                                          \
            acc[m & 1] = __builtin_amdgcn_mfma_f32_32x32x2f32(f[cur][2][m >> 1], f[cur][m & 1][m >> 1], acc[m & 1], 0, 0, 0); \
            __builtin_amdgcn_sched_barrier(0);                                                                   \
            if (m == 0 && READS > 0) AXP_DS_READ(f[1 - (cur)][0], base, (off) + 0 * 1024);                       \
            if (m == 2 && READS > 1) AXP_DS_READ(f[1 - (cur)][1], base, (off) + 1 * 1024);                       \
            if (m == 4 && READS > 2) AXP_DS_READ(f[1 - (cur)][2], base, (off) + 2 * 1024);                       \
            __builtin_amdgcn_sched_barrier(0);                                                                   \
        }                                                                                                        \
    } while (0)
        for (int s = 0; s < blocks; s += 8) {
            AXP_FBLOCK32(0, 0 * 3072 + 16);
            AXP_FBLOCK32(1, 1 * 3072 + 32);
            AXP_FBLOCK32(0, 2 * 3072 + 48);
            AXP_FBLOCK32(1, 3 * 3072 + 64);
            AXP_FBLOCK32(0, 4 * 3072 + 80);
            AXP_FBLOCK32(1, 5 * 3072 + 96);
            AXP_FBLOCK32(0, 6 * 3072 + 112);
            AXP_FBLOCK32(1, 7 * 3072 + 0);
        }
#undef AXP_FBLOCK32
        AXP_LGKM0();
#pragma unroll
        for (int m = 0; m < 2; m++)
#pragma unroll
            for (int v = 0; v < 16; v++) sum += acc[m][v];
    } else {
        v4f acc[4];
#pragma unroll
        for (int m = 0; m < 4; m++) acc[m] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#define AXP_FBLOCK16(cur, off)                                                                                   \
    do {                                                                                                         \
        AXP_LGKM0();                                                                                             \
        __builtin_amdgcn_sched_barrier(0);                                                                       \
        _Pragma("unroll") for (int m = 0; m < 16; m++) {                                                         \
            acc[m & 3] = __builtin_amdgcn_mfma_f32_16x16x4f32(f[cur][2][m >> 2], f[cur][m & 1][m >> 2], acc[m & 3], 0, 0, 0); \
            __builtin_amdgcn_sched_barrier(0);                                                                   \
            if (m == 0 && READS > 0) AXP_DS_READ(f[1 - (cur)][0], base, (off) + 0 * 1024);                       \
            if (m == 4 && READS > 1) AXP_DS_READ(f[1 - (cur)][1], base, (off) + 1 * 1024);                       \
            if (m == 8 && READS > 2) AXP_DS_READ(f[1 - (cur)][2], base, (off) + 2 * 1024);                       \
            __builtin_amdgcn_sched_barrier(0);                                                                   \
        }                                                                                                        \
    } while (0)
        for (int s = 0; s < blocks; s += 8) {
            AXP_FBLOCK16(0, 0 * 3072 + 16);
            AXP_FBLOCK16(1, 1 * 3072 + 32);
            AXP_FBLOCK16(0, 2 * 3072 + 48);
            AXP_FBLOCK16(1, 3 * 3072 + 64);
            AXP_FBLOCK16(0, 4 * 3072 + 80);
            AXP_FBLOCK16(1, 5 * 3072 + 96);
            AXP_FBLOCK16(0, 6 * 3072 + 112);
            AXP_FBLOCK16(1, 7 * 3072 + 0);
        }
#undef AXP_FBLOCK16
        AXP_LGKM0();
#pragma unroll
        for (int m = 0; m < 4; m++)
#pragma unroll
            for (int v = 0; v < 4; v++) sum += acc[m][v];
    }
    sink[(int64_t)blockIdx.x * 512 + tid] = sum;
}

constexpr int kF32BlocksPerLaunch = 1024;   // blocks of 16384 multiply-adds per wave: 70 GFLOP per launch on 256 CUs

template <int SHAPE>
int launch_probe_f32(int reads, const float *src, float *sink) {
    typedef void (*kern_t)(const float *, int, float *);
    static const kern_t kerns[4] = {k_probe_f32<SHAPE, 0>, k_probe_f32<SHAPE, 1>, k_probe_f32<SHAPE, 2>, k_probe_f32<SHAPE, 3>};
    static bool raised[4] = {};
    if (!raised[reads]) {
        AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kerns[reads]), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes),
                      "hipFuncSetAttribute");
        raised[reads] = true;
    }
    hipLaunchKernelGGL(kerns[reads], dim3((unsigned)cu_count()), dim3(512), kLdsBytes, kStream, src, kF32BlocksPerLaunch, sink);
    return check_launch("probe_fp32_matrix_core");
}
}  // namespace

extern "C" int axhip_probe_int8_matrix_core(int mfma_shape, int lds_reads, const int8_t *operand_bytes, int32_t *sink) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!operand_bytes || !sink) return axhip::fail(AXHIP_ERR_NULL_ARG, "probe_int8_matrix_core: NULL buffer");
    if ((mfma_shape != 32 && mfma_shape != 16) || lds_reads < 0 || lds_reads > 6)
        return axhip::fail(AXHIP_ERR_SHAPE, "probe_int8_matrix_core: shape %d (32 or 16), reads %d (0..6)", mfma_shape, lds_reads);
    axhip::note_kernel(mfma_shape == 32 ? "probe_i8_mfma_32x32x32" : "probe_i8_mfma_16x16x64");
    return mfma_shape == 32 ? launch_probe<32>(lds_reads, operand_bytes, sink) : launch_probe<16>(lds_reads, operand_bytes, sink);
}

extern "C" int axhip_probe_fp32_matrix_core(int mfma_shape, int lds_reads, const float *operand_floats, float *sink) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!operand_floats || !sink) return axhip::fail(AXHIP_ERR_NULL_ARG, "probe_fp32_matrix_core: NULL buffer");
    if ((mfma_shape != 32 && mfma_shape != 16) || lds_reads < 0 || lds_reads > 3)
        return axhip::fail(AXHIP_ERR_SHAPE, "probe_fp32_matrix_core: shape %d (32 or 16), reads %d (0..3)", mfma_shape, lds_reads);
    axhip::note_kernel(mfma_shape == 32 ? "probe_f32_mfma_32x32x2" : "probe_f32_mfma_16x16x4");
    return mfma_shape == 32 ? launch_probe_f32<32>(lds_reads, operand_floats, sink) : launch_probe_f32<16>(lds_reads, operand_floats, sink);
}
