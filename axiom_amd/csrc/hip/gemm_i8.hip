// int8 x int8 -> int32 GEMM (W8A8) with fused dequantize + bias + activation write-back.
//
//   acc[m,n] = sum_k x[m,k] * w[n,k]          x: [M,K] int8, w: [N,K] int8 (both K-contiguous)
//   out[m,n] = act((float)acc * (x_scale*w_scale[n]) + bias[n])
//
// Two kernels.  k_qgemm_w8a8_256 (further down) serves large aligned shapes; the template
// below serves everything else, including ragged and unaligned shapes through its guarded form.
//
// Template kernel: one workgroup owns a BM x BN tile of the output and walks K in slabs of 128
// bytes.  Slabs are fetched with 16-byte global loads (8 consecutive lanes cover one 128-byte row
// segment), staged through registers into a double-buffered LDS tile, and consumed by
// v_mfma_i32_32x32x32_i8: lane l supplies row (l & 31), bytes [16*(l>>5), +16) of each
// 32-byte k-step.  Because A and B fragments use the same byte placement the integer dot
// product is exact whatever order the matrix core sums in.
//
// LDS rows are 128 bytes = 32 banks, so the 16-byte chunk index is XOR-swizzled with
// (row >> 1) & 7: the 16 lanes served together by a ds_read_b128 (16 consecutive rows, one
// chunk) and the 16 lanes of a ds_write_b128 (2 rows x 8 chunks) then touch 64 distinct banks.
#include <cstring>

#include "common.h"

namespace {
using namespace axhip;

constexpr int BK = 128;   // bytes of K per slab

__device__ __forceinline__ int swz(int row, int chunk) {
    return row * BK + ((chunk ^ ((row >> 1) & 7)) << 4);
}

template <bool GUARD>
__device__ __forceinline__ v4i load_chunk(const int8_t *base, int64_t row, int64_t rows,
                                          int64_t k, int64_t K) {
    if (!GUARD) return *reinterpret_cast<const v4i *>(base + row * K + k);
    v4i r = {0, 0, 0, 0};
    if (row >= rows || k >= K) return r;
    const int8_t *p = base + row * K + k;
    if (k + 16 <= K) {
        // a whole chunk inside the row: one 16-byte load at whatever alignment K leaves the row
        // (global memory takes unaligned vector loads; byte loads made K % 16 != 0 24x slower)
        __builtin_memcpy(&r, p, 16);
        return r;
    }
    int64_t left = K - k;
    unsigned w[4] = {0, 0, 0, 0};
    for (int b = 0; b < 16; b++)
        if (b < left) w[b >> 2] |= (unsigned)(unsigned char)p[b] << ((b & 3) * 8);
    r.x = (int)w[0]; r.y = (int)w[1]; r.z = (int)w[2]; r.w = (int)w[3];
    return r;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool GUARD>
__global__ void __launch_bounds__(WAVES_M *WAVES_N * 64)
k_qgemm_w8a8(const int8_t *__restrict__ X, const int8_t *__restrict__ W, int64_t M, int64_t N,
             int64_t K, float x_scale, const float *__restrict__ w_scales,
             const float *__restrict__ bias, int act, float *__restrict__ out,
             int32_t *__restrict__ acc_out, int64_t ldc) {
    constexpr int T = WAVES_M * WAVES_N * 64;
    constexpr int CA = BM * 8 / T, CB = BN * 8 / T;       // 16-byte chunks per thread per slab
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N; // wave tile
    constexpr int TM = WTM / 32, TN = WTN / 32;           // 32x32 MFMA tiles per wave
    static_assert(CA * T == BM * 8 && CB * T == BN * 8, "slab must divide over the workgroup");
    static_assert(TM * 32 * WAVES_M == BM && TN * 32 * WAVES_N == BN, "wave tiling");
    constexpr int STAGE = (BM + BN) * BK;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
    int tm, tn;
    tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

    const int64_t slabs = (K + BK - 1) / BK;

    v4i ra[CA], rb[CB];
    auto fetch = [&](int64_t slab) {
        const int64_t k0 = slab * BK;
#pragma unroll
        for (int i = 0; i < CA; i++) {
            int c = tid + i * T;
            ra[i] = load_chunk<GUARD>(X, m0 + (c >> 3), M, k0 + ((c & 7) << 4), K);
        }
#pragma unroll
        for (int i = 0; i < CB; i++) {
            int c = tid + i * T;
            rb[i] = load_chunk<GUARD>(W, n0 + (c >> 3), N, k0 + ((c & 7) << 4), K);
        }
    };
    auto stash = [&](int stage) {
        unsigned char *sa = lds + stage * STAGE, *sb = sa + BM * BK;
#pragma unroll
        for (int i = 0; i < CA; i++) {
            int c = tid + i * T;
            *reinterpret_cast<v4i *>(sa + swz(c >> 3, c & 7)) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < CB; i++) {
            int c = tid + i * T;
            *reinterpret_cast<v4i *>(sb + swz(c >> 3, c & 7)) = rb[i];
        }
    };

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0;

    fetch(0);
    stash(0);
    __syncthreads();

    const int frow = lane & 31, fhalf = lane >> 5;
    for (int64_t s = 0; s < slabs; s++) {
        const int cur = (int)(s & 1);
        if (s + 1 < slabs) fetch(s + 1);
        const unsigned char *sa = lds + cur * STAGE + (wm * WTM) * BK;
        const unsigned char *sb = lds + cur * STAGE + BM * BK + (wn * WTN) * BK;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            v4i fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; i++)
                fa[i] = *reinterpret_cast<const v4i *>(sa + swz(i * 32 + frow, ks * 2 + fhalf));
#pragma unroll
            for (int j = 0; j < TN; j++)
                fb[j] = *reinterpret_cast<const v4i *>(sb + swz(j * 32 + frow, ks * 2 + fhalf));
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (s + 1 < slabs) stash(cur ^ 1);
        __syncthreads();
    }

    // Write-back.  Accumulator register v of lane l holds row (v&3) + 8*(v>>2) + 4*(l>>5),
    // column (l & 31) of its 32x32 tile: 32 lanes store 128 contiguous bytes of one row.
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int64_t col = n0 + wn * WTN + j * 32 + frow;
        const bool col_ok = !GUARD || col < N;
        float scale = 0.0f, bv = 0.0f;
        if (out && col_ok) {
            scale = x_scale * w_scales[col];
            if (bias) bv = bias[col];
        }
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int64_t row = m0 + wm * WTM + i * 32 + (v & 3) + 8 * (v >> 2) + 4 * fhalf;
                if (GUARD && (row >= M || !col_ok)) continue;
                const int a = acc[i][j][v];
                if (acc_out) acc_out[row * ldc + col] = a;
                if (out) {
                    float f = (float)a;
                    float r = bias ? __builtin_fmaf(f, scale, bv) : f * scale;
                    out[row * ldc + col] = apply_act(r, act);
                }
            }
        }
    }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool GUARD>
int launch(const char *name, const int8_t *x, float x_scale, const int8_t *w,
           const float *w_scales, const float *bias, int act, float *out, int32_t *acc_out,
           int64_t M, int64_t N, int64_t K, int64_t ldc) {
    auto kern = k_qgemm_w8a8<BM, BN, WAVES_M, WAVES_N, GUARD>;
    constexpr int smem = 2 * (BM + BN) * BK;
    static bool attr_set = false;
    if (!attr_set) {
        AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, smem),
                      "hipFuncSetAttribute");
        attr_set = true;
    }
    const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    if (tiles > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "qgemm_w8a8: too many tiles");
    note_kernel(name);
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(WAVES_M * WAVES_N * 64), smem, kStream, x,
                       w, M, N, K, x_scale, w_scales, bias, act, out, acc_out, ldc);
    return check_launch(name);
}


// ---------------------------------------------------------------------------------------
// Large aligned shapes (M, N multiples of 256, K a multiple of 128): 256x256 tile, 8 waves as
// 2 (M) x 4 (N), wave tile 128x64, K slabs of 128 bytes, two LDS stages laid out
// [X stage0][X stage1][W stage0][W stage1] (32 KiB each).
//
// The inner loop holds no vector-ALU instruction other than the MFMAs.  On gfx950 a VALU
// instruction issued by any wave of a SIMD while that SIMD streams MFMAs costs about a
// whole MFMA slot, so pointer arithmetic inside the loop serialises memory traffic with
// the matrix core.  Therefore:
//   * global -> LDS copies are global_load_lds_dwordx4 (no register staging) addressed by a
//     scalar base pointer, advanced with scalar adds, plus a per-lane byte offset computed once;
//   * LDS -> register fragment reads use per-lane addresses computed once plus immediate offsets;
//   * waits and barriers are scalar.
// Each load instruction of a wave fills 1 KiB of LDS = 8 rows x 128 bytes, so every row
// segment is one full 128-byte cache line (half-line segments run the texture path at
// about 60% of that rate).  Lane l of the instruction writes LDS row (l>>3), physical 16-byte
// chunk (l&7); it fetches logical chunk (l&7) ^ ((row>>1)&7) so that the XOR swizzle, which
// keeps ds_read_b128 conflict-free, is applied on the global side.
// Fragments are double-buffered in registers: the reads of k-step ks+1 are issued one by one
// between the 8 MFMAs of k-step ks, and so are the loads of the slab after next.
//
// The MFMA takes the W fragment as its first operand: a lane then holds 4 consecutive n of
// one output row m, and the write-back is 16-byte stores with the per-channel scale and bias
// fetched as float4.
#define AXI8_LGKM(n) __builtin_amdgcn_s_waitcnt(0x3F | (3 << 14) | (7 << 4) | ((n) << 8))
#define AXI8_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))
#define AXI8_VM0() AXI8_VM(0)
#define AXI8_DS_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off))
#define AXI8_LOAD_LDS(m0val, voff, base)                                                     \
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0val), \
                 "v"(voff), "s"(base)                                                        \
                 : "memory")
// the same for an operand that is read once and is too large to be met again in the caches (non-temporal)
#define AXI8_LOAD_LDS_NT(m0val, voff, base)                                                  \
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(m0val), \
                 "v"(voff), "s"(base)                                                        \
                 : "memory")

template <int ACT>
__global__ void __launch_bounds__(512)
k_qgemm_w8a8_256(const int8_t *__restrict__ X, const int8_t *__restrict__ W, int64_t M, int64_t N,
                 int64_t K, float x_scale, const float *__restrict__ w_scales,
                 const float *__restrict__ bias, float *__restrict__ out,
                 int32_t *__restrict__ acc_out, int64_t ldc) {
    constexpr int BM = 256, BN = 256, BKB = 128, WAVES_N = 4, WTM = 128, WTN = 64, TM = 4, TN = 2;
    constexpr int OPER = BM * BKB;   // bytes of one operand in one stage
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int tiles_m = (int)(M / BM), tiles_n = (int)(N / BN), total = tiles_m * tiles_n;
    const int slabs = (int)(K / BKB);

    // Loads and stores retire in issue order within a wave, so a wave that has stores in flight
    // cannot see its later loads complete before them.  The two are therefore kept on different
    // waves: waves 0-3 issue every global->LDS load of the workgroup (and never store), waves
    // 4-7 issue every global store (and never load), and the write-back of one tile drains to
    // HBM underneath the next tile's slabs instead of stalling them.
    const bool loader = wave < 4;
    // load instruction j (0..7) of loader wave w fills rows (j*4+w)*8 .. +8 of an operand stage
    unsigned voff[8];
    {
        const int sw = (wave & 1) * 4 + (lane >> 4);      // (row >> 1) & 7 of this lane's row
#pragma unroll
        for (int j = 0; j < 8; j++)
            voff[j] = (unsigned)(((j * 4 + (wave & 3)) * 8 + (lane >> 3)) * K + (((lane & 7) ^ sw) << 4));
    }
    const int8_t *gx = X, *gw = W;
    const unsigned lds_w = (unsigned)(uintptr_t)lds + (wave & 3) * 1024;

    // fragment reads: lane (frow, fhalf) of tile i takes row i*32+frow, logical chunk ks*2+fhalf
    const int frow = lane & 31, fhalf = lane >> 5;
    unsigned rx[4], rw[4];
    {
        const int sw = (frow >> 1) & 7;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const unsigned inrow = (unsigned)(frow * BKB + (((ks * 2 + fhalf) ^ sw) << 4));
            rx[ks] = (unsigned)(uintptr_t)lds + wm * WTM * BKB + inrow;
            rw[ks] = (unsigned)(uintptr_t)lds + 2 * OPER + wn * WTN * BKB + inrow;
        }
    }

    typedef float v4f_t __attribute__((ext_vector_type(4)));
    float *lds_scale = reinterpret_cast<float *>(lds + 4 * OPER);     // [2 slots][scale 256 | bias 256]
    v16i acc[TM][TN];

#define AXI8_LOAD_X(stage, j) AXI8_LOAD_LDS(lds_w + (stage) * OPER + (j) * 4096, voff[j], gx)
#define AXI8_LOAD_W(stage, j) AXI8_LOAD_LDS(lds_w + 2 * OPER + (stage) * OPER + (j) * 4096, voff[j], gw)
// a loader wave's 16 loads of the next unfetched slab
#define AXI8_ISSUE(stage)                                                                 \
    do {                                                                                  \
        AXI8_LOAD_X(stage, 0); AXI8_LOAD_X(stage, 1); AXI8_LOAD_X(stage, 2); AXI8_LOAD_X(stage, 3); \
        AXI8_LOAD_X(stage, 4); AXI8_LOAD_X(stage, 5); AXI8_LOAD_X(stage, 6); AXI8_LOAD_X(stage, 7); \
        AXI8_LOAD_W(stage, 0); AXI8_LOAD_W(stage, 1); AXI8_LOAD_W(stage, 2); AXI8_LOAD_W(stage, 3); \
        AXI8_LOAD_W(stage, 4); AXI8_LOAD_W(stage, 5); AXI8_LOAD_W(stage, 6); AXI8_LOAD_W(stage, 7); \
        gx += BKB;                                                                        \
        gw += BKB;                                                                        \
    } while (0)

#define AXI8_FRAGS(buf, stage, ks)                                          \
    do {                                                                    \
        AXI8_DS_READ(fx[buf][0], rx[ks], (stage) * OPER + 0 * 4096);        \
        AXI8_DS_READ(fx[buf][1], rx[ks], (stage) * OPER + 1 * 4096);        \
        AXI8_DS_READ(fw[buf][0], rw[ks], (stage) * OPER + 0 * 4096);        \
        AXI8_DS_READ(fw[buf][1], rw[ks], (stage) * OPER + 1 * 4096);        \
        AXI8_DS_READ(fx[buf][2], rx[ks], (stage) * OPER + 2 * 4096);        \
        AXI8_DS_READ(fx[buf][3], rx[ks], (stage) * OPER + 3 * 4096);        \
    } while (0)

// MFMA m (0..7) of a k-step: tile row m>>1, tile column m&1
#define AXI8_M(buf, m)                                                                          \
    do {                                                                                        \
        acc[(m) >> 1][(m) & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(                         \
            fw[buf][(m) & 1], fx[buf][(m) >> 1], acc[(m) >> 1][(m) & 1], 0, 0, 0);              \
        __builtin_amdgcn_sched_barrier(0);                                                      \
    } while (0)

// The 8 MFMAs of the k-step held in fragment buffer `buf`.  Between them, so that their issue
// falls into the shadow of the MFMA before: (RD) the 6 fragment reads of k-step rks of stage
// rstage into the other buffer, in the order the next block consumes them; (LD, loader waves
// only) the 16 loads of the next unfetched slab into stage lstage.
#define AXI8_BLOCK(buf, RD, rstage, rks, LD, lstage)                                            \
    do {                                                                                        \
        AXI8_M(buf, 0);                                                                         \
        if (RD) AXI8_DS_READ(fx[1 - (buf)][0], rx[rks], (rstage) * OPER + 0 * 4096);            \
        if (LD) { AXI8_LOAD_X(lstage, 0); AXI8_LOAD_W(lstage, 0); }                             \
        AXI8_M(buf, 1);                                                                         \
        if (RD) AXI8_DS_READ(fw[1 - (buf)][0], rw[rks], (rstage) * OPER + 0 * 4096);            \
        if (LD) { AXI8_LOAD_X(lstage, 1); AXI8_LOAD_W(lstage, 1); }                             \
        AXI8_M(buf, 2);                                                                         \
        if (RD) AXI8_DS_READ(fw[1 - (buf)][1], rw[rks], (rstage) * OPER + 1 * 4096);            \
        if (LD) { AXI8_LOAD_X(lstage, 2); AXI8_LOAD_W(lstage, 2); }                             \
        AXI8_M(buf, 3);                                                                         \
        if (RD) AXI8_DS_READ(fx[1 - (buf)][1], rx[rks], (rstage) * OPER + 1 * 4096);            \
        if (LD) { AXI8_LOAD_X(lstage, 3); AXI8_LOAD_W(lstage, 3); }                             \
        AXI8_M(buf, 4);                                                                         \
        if (RD) AXI8_DS_READ(fx[1 - (buf)][2], rx[rks], (rstage) * OPER + 2 * 4096);            \
        if (LD) { AXI8_LOAD_X(lstage, 4); AXI8_LOAD_W(lstage, 4); }                             \
        AXI8_M(buf, 5);                                                                         \
        if (RD) AXI8_DS_READ(fx[1 - (buf)][3], rx[rks], (rstage) * OPER + 3 * 4096);            \
        if (LD) { AXI8_LOAD_X(lstage, 5); AXI8_LOAD_W(lstage, 5); }                             \
        AXI8_M(buf, 6);                                                                         \
        if (LD) { AXI8_LOAD_X(lstage, 6); AXI8_LOAD_W(lstage, 6); }                             \
        AXI8_M(buf, 7);                                                                         \
        if (LD) { AXI8_LOAD_X(lstage, 7); AXI8_LOAD_W(lstage, 7); gx += BKB; gw += BKB; }       \
        __builtin_amdgcn_sched_barrier(0);                                                      \
    } while (0)

#define AXI8_WAIT_FRAGS() do { AXI8_LGKM(0); __builtin_amdgcn_sched_barrier(0); } while (0)

    // One slab resident in `stage`, its k-step 0 already (being) read into buffer 0.  After the
    // third k-step every wave has read all it needs of this stage and waits for its own loads
    // of the next slab; past the barrier the stage is free, so the last k-step's MFMAs cover
    // the first fragment reads of the next slab (after the last slab they fetch stale bytes
    // nobody uses) and, when more2, the loads of the slab after.
#define AXI8_SLAB(stage, more2)                                              \
    do {                                                                     \
        AXI8_WAIT_FRAGS();                                                   \
        AXI8_BLOCK(0, 1, stage, 1, 0, 0);                                    \
        AXI8_WAIT_FRAGS();                                                   \
        AXI8_BLOCK(1, 1, stage, 2, 0, 0);                                    \
        AXI8_WAIT_FRAGS();                                                   \
        AXI8_BLOCK(0, 1, stage, 3, 0, 0);                                    \
        AXI8_WAIT_FRAGS();                                                   \
        if (loader) AXI8_VM0();                                              \
        __builtin_amdgcn_s_barrier();                                        \
        __builtin_amdgcn_sched_barrier(0);                                   \
        AXI8_BLOCK(1, 1, 1 - (stage), 0, (more2) && loader, stage);          \
    } while (0)

    // Persistent: one workgroup per CU walks tiles t = blockIdx.x, + gridDim.x, ... (the same
    // tile a non-persistent launch would hand that CU next).  With an even slab count the last
    // slab of a tile sits in stage 1, so the loader waves fetch the first slab of the next tile
    // into stage 0 before the write-back starts.
    const bool carry = (slabs & 1) == 0;
    bool fetched = false;
    // Per-channel scale (premultiplied by x_scale) and bias of a tile's 256 columns go to LDS
    // ahead of its write-back, into one of two slots so the coming tile's can be staged while
    // the current tile's are still being read.  Wave 0 only, behind one scalar branch: the
    // waits the compiler places around these loads must stay out of the storer waves' path,
    // where they would wait for the stores in flight.
    v4f_t col_s = {0.f, 0.f, 0.f, 0.f}, col_b = {0.f, 0.f, 0.f, 0.f};
    auto load_cols = [&](int64_t n0) {            // issued a whole tile ahead of store_cols
        if (out && wave == 0) {
            col_s = *reinterpret_cast<const v4f_t *>(w_scales + n0 + lane * 4);
            if (bias) col_b = *reinterpret_cast<const v4f_t *>(bias + n0 + lane * 4);
        }
    };
    auto store_cols = [&](int slot) {
        if (out && wave == 0) {
            v4f_t v = col_s;
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = x_scale * v[e];
            float *dst = lds_scale + slot * 2 * BN + lane * 4;
            *reinterpret_cast<v4f_t *>(dst) = v;
            *reinterpret_cast<v4f_t *>(dst + BN) = col_b;
        }
    };
    int slot = 0;
    v4i fx[2][TM], fw[2][TN];

    // Write-back of one 32x32 sub-tile per wave and round.  With W as the MFMA's first operand,
    // register v of lane l holds m = (l&31), n = 8*(v>>2) + 4*(l>>5) + (v&3) of the sub-tile:
    // four consecutive n per lane.  Every wave writes its sub-tile (16-byte chunk c of row r at
    // chunk c ^ ((r>>1)&7), conflict-free both ways) into its 4 KiB of a turn buffer; after the
    // barrier storer wave 4+s reads the sub-tiles of waves 2s and 2s+1 back row-major and stores
    // whole 128-byte rows.  The two turn buffers (stage 1 of X and of W, dead after the loop's
    // last barrier) alternate, so one barrier per round is enough: a buffer is rewritten two
    // rounds later, after every storer has passed the barrier in between.
    int round = 0;
    auto emit = [&](const auto (&r)[4], auto *base, int64_t m0, int64_t n0, int i, int j) {
        typedef typename std::remove_const<typename std::remove_reference<decltype(r[0])>::type>::type V4;
        unsigned char *buf = lds + ((round & 1) ? 3 * OPER : OPER);
        round++;
#pragma unroll
        for (int g = 0; g < 4; g++)
            *reinterpret_cast<V4 *>(buf + wave * 4096 + frow * 128 + (((2 * g + fhalf) ^ ((frow >> 1) & 7)) << 4)) = r[g];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
        if (!loader) {
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const int src = 2 * (wave - 4) + q;                     // wave whose sub-tile this is
                auto *dst = base + (m0 + (src / WAVES_N) * WTM + i * 32) * ldc + n0 + (src % WAVES_N) * WTN + j * 32;
#pragma unroll
                for (int p = 0; p < 4; p++) {
                    const int row = p * 8 + (lane >> 3);
                    const V4 v = *reinterpret_cast<const V4 *>(buf + src * 4096 + row * 128 +
                                                               (((lane & 7) ^ ((row >> 1) & 7)) << 4));
                    // streaming store: the 256 KB a tile writes must not evict the operand panels the
                    // XCD's other workgroups are re-reading from its 4 MB L2 (plain stores: +30 us)
                    __builtin_nontemporal_store(v, reinterpret_cast<V4 *>(dst + (int64_t)row * ldc + (lane & 7) * 4));
                }
            }
        }
    };

    for (int t = blockIdx.x; t < total; t += gridDim.x) {
        int tm, tn;
        tile_of_block(t, tiles_m, tiles_n, tm, tn);
        const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
        if (!fetched) {
            gx = X + m0 * K;
            gw = W + n0 * K;
            if (loader) AXI8_ISSUE(0);
            load_cols(n0);
            store_cols(slot);
        }
        const int t_next = t + (int)gridDim.x;
        const bool will_fetch = carry && t_next < total;
        int tm2 = 0, tn2 = 0;
        if (will_fetch) {
            tile_of_block(t_next, tiles_m, tiles_n, tm2, tn2);
            load_cols((int64_t)tn2 * BN);
        }
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[i][j][v] = 0;

        if (loader) AXI8_VM0();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        if (slabs > 1 && loader) AXI8_ISSUE(1);
        AXI8_FRAGS(0, 0, 0);

        for (int s = 0; s < slabs; s += 2) {       // the flags are wave-uniform: scalar branches only
            AXI8_SLAB(0, s + 2 < slabs);
            if (s + 1 < slabs) AXI8_SLAB(1, s + 3 < slabs);
        }
        AXI8_WAIT_FRAGS();      // the stale reads must land before their registers are reused

        fetched = will_fetch;
        if (fetched) {
            store_cols(slot ^ 1);
            gx = X + (int64_t)tm2 * BM * K;
            gw = W + (int64_t)tn2 * BN * K;
            if (loader) AXI8_ISSUE(0);
        }

        if (acc_out) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    v4i r[4];
#pragma unroll
                    for (int g = 0; g < 4; g++)
                        r[g] = v4i{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                    emit(r, acc_out, m0, n0, i, j);
                }
        }
        if (out) {
            const float *sp = lds_scale + slot * 2 * BN + wn * WTN + 4 * fhalf, *bp = sp + BN;
            const bool has_bias = bias != nullptr;
#pragma unroll
            for (int j = 0; j < TN; j++) {
                v4f_t sc[4], bv[4];
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    sc[g] = *reinterpret_cast<const v4f_t *>(sp + j * 32 + 8 * g);
                    bv[g] = *reinterpret_cast<const v4f_t *>(bp + j * 32 + 8 * g);
                }
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    v4f_t r[4];
#pragma unroll
                    for (int g = 0; g < 4; g++)
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float f = (float)acc[i][j][4 * g + e];
                            // a fused multiply-add with bias = 0 would round differently from the plain product
                            r[g][e] = apply_act(has_bias ? __builtin_fmaf(f, sc[g][e], bv[g][e]) : f * sc[g][e], ACT);
                        }
                    emit(r, out, m0, n0, i, j);
                }
            }
        }
        slot ^= 1;
        // Every wave is done with the turn buffers and this tile's scale/bias slot before the next
        // tile overwrites them.  Only LDS traffic is ordered here, never the stores.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    }
}
#undef AXI8_ISSUE
#undef AXI8_FRAGS
#undef AXI8_M
#undef AXI8_BLOCK
#undef AXI8_WAIT_FRAGS
#undef AXI8_LOAD_X
#undef AXI8_LOAD_W
#undef AXI8_SLAB

// ---------------------------------------------------------------------------------------
// The same kernel on v_mfma_i32_16x16x64_i8.  The instruction does half the multiply-adds of
// the 32x32x32 one with a quarter of its accumulator registers, so every accumulator is read
// and written half as often per multiply-add.  On operands that change from instruction to
// instruction the matrix cores run into the GPU's power limit; with that traffic halved the same
// multiply-adds and LDS fragment reads take 13 % less time at a clock 13 % higher (measured with
// axhip_probe_int8_matrix_core: 352.7 us at 1646 MHz against 305.7 us at 1858 MHz).  Everything
// outside the inner loop is as above: tile, waves, stages, direct-to-LDS loads, loader and storer
// waves, persistent walk over the tiles, write-back through LDS.
//
// A slab of 128 bytes is two k-steps of 64.  Per k-step a wave multiplies its 128x64 tile as 8 x 4
// tiles of 16x16: lane (r = l & 15, q = l >> 4) of a fragment holds row r, bytes 16 q .. of the
// k-step, i.e. logical chunk 4 ks + q of the LDS row, kept at chunk ^ ((row >> 1) & 7) like above
// (16 lanes read 16 rows at one logical chunk: 8 physical chunks on even and odd rows, every
// bank once).  With W as the first operand lane l then holds, for tile (i, j), the outputs m =
// 16 i + (l & 15), n = 16 j + 4 (l >> 4) + v: four consecutive n, as above.
#define AXK_LOAD_X(stage, j) AXI8_LOAD_LDS(lds_w + (stage) * OPER + (j) * 4096, voff[j], gx)
#define AXK_LOAD_W(stage, j) AXI8_LOAD_LDS(lds_w + 2 * OPER + (stage) * OPER + (j) * 4096, voff[j], gw)
#define AXK_ISSUE(stage)                                                                          \
    do {                                                                                          \
        AXK_LOAD_X(stage, 0); AXK_LOAD_X(stage, 1); AXK_LOAD_X(stage, 2); AXK_LOAD_X(stage, 3);   \
        AXK_LOAD_X(stage, 4); AXK_LOAD_X(stage, 5); AXK_LOAD_X(stage, 6); AXK_LOAD_X(stage, 7);   \
        AXK_LOAD_W(stage, 0); AXK_LOAD_W(stage, 1); AXK_LOAD_W(stage, 2); AXK_LOAD_W(stage, 3);   \
        AXK_LOAD_W(stage, 4); AXK_LOAD_W(stage, 5); AXK_LOAD_W(stage, 6); AXK_LOAD_W(stage, 7);   \
        gx += BKB;                                                                                \
        gw += BKB;                                                                                \
    } while (0)
// fragment reads of k-step ks of a stage: X tile i at rows 16 i .. (2 KiB apart), W tile j likewise
#define AXK_RX(buf, stage, ks, i) AXI8_DS_READ(fx[buf][i], rx[ks], (stage) * OPER + (i) * 2048)
#define AXK_RW(buf, stage, ks, j) AXI8_DS_READ(fw[buf][j], rw[ks], (stage) * OPER + (j) * 2048)
#define AXK_FRAGS(buf, stage, ks)                                                                 \
    do {                                                                                          \
        AXK_RW(buf, stage, ks, 0); AXK_RX(buf, stage, ks, 0); AXK_RW(buf, stage, ks, 1);          \
        AXK_RW(buf, stage, ks, 2); AXK_RW(buf, stage, ks, 3); AXK_RX(buf, stage, ks, 1);          \
        AXK_RX(buf, stage, ks, 2); AXK_RX(buf, stage, ks, 3); AXK_RX(buf, stage, ks, 4);          \
        AXK_RX(buf, stage, ks, 5); AXK_RX(buf, stage, ks, 6); AXK_RX(buf, stage, ks, 7);          \
    } while (0)
#define AXK_M(buf, i, j)                                                                          \
    do {                                                                                          \
        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fw[buf][j], fx[buf][i], acc[i][j], 0, 0, 0); \
        __builtin_amdgcn_sched_barrier(0);                                                        \
    } while (0)
// The 32 MFMAs of the k-step held in fragment buffer `buf`, tile row by tile row.  Behind the even ones
// of the first 24: (RD) the 12 fragment reads of k-step rks of stage rstage into the other buffer, in
// the order the next block consumes them; behind the odd ones: (LD, loader waves only) the 16 loads of
// the next unfetched slab into stage lstage.
#define AXK_ROW(buf, i, RD, r0, r1, LD, l0, l1, l2, l3)                                           \
    do {                                                                                          \
        AXK_M(buf, i, 0);                                                                         \
        if (RD) { r0; }                                                                           \
        AXK_M(buf, i, 1);                                                                         \
        if (LD) { l0; l1; }                                                                       \
        AXK_M(buf, i, 2);                                                                         \
        if (RD) { r1; }                                                                           \
        AXK_M(buf, i, 3);                                                                         \
        if (LD) { l2; l3; }                                                                       \
    } while (0)
// the same with the tile columns walked backwards: between one row of tiles and the next only the X fragment changes
#define AXK_ROW_REV(buf, i, RD, r0, r1, LD, l0, l1, l2, l3)                                       \
    do {                                                                                          \
        AXK_M(buf, i, 3);                                                                         \
        if (RD) { r0; }                                                                           \
        AXK_M(buf, i, 2);                                                                         \
        if (LD) { l0; l1; }                                                                       \
        AXK_M(buf, i, 1);                                                                         \
        if (RD) { r1; }                                                                           \
        AXK_M(buf, i, 0);                                                                         \
        if (LD) { l2; l3; }                                                                       \
    } while (0)
#define AXK_BLOCK(buf, RD, rstage, rks, LD, lstage)                                                                      \
    do {                                                                                                                 \
        AXK_ROW(buf, 0, RD, AXK_RW(1 - (buf), rstage, rks, 0), AXK_RX(1 - (buf), rstage, rks, 0), LD,                    \
                AXK_LOAD_X(lstage, 0), AXK_LOAD_W(lstage, 0), (void)0, (void)0);                                         \
        AXK_ROW_REV(buf, 1, RD, AXK_RW(1 - (buf), rstage, rks, 1), AXK_RW(1 - (buf), rstage, rks, 2), LD,                    \
                AXK_LOAD_X(lstage, 1), AXK_LOAD_W(lstage, 1), (void)0, (void)0);                                         \
        AXK_ROW(buf, 2, RD, AXK_RW(1 - (buf), rstage, rks, 3), AXK_RX(1 - (buf), rstage, rks, 1), LD,                    \
                AXK_LOAD_X(lstage, 2), AXK_LOAD_W(lstage, 2), (void)0, (void)0);                                         \
        AXK_ROW_REV(buf, 3, RD, AXK_RX(1 - (buf), rstage, rks, 2), AXK_RX(1 - (buf), rstage, rks, 3), LD,                    \
                AXK_LOAD_X(lstage, 3), AXK_LOAD_W(lstage, 3), (void)0, (void)0);                                         \
        AXK_ROW(buf, 4, RD, AXK_RX(1 - (buf), rstage, rks, 4), AXK_RX(1 - (buf), rstage, rks, 5), LD,                    \
                AXK_LOAD_X(lstage, 4), AXK_LOAD_W(lstage, 4), (void)0, (void)0);                                         \
        AXK_ROW_REV(buf, 5, RD, AXK_RX(1 - (buf), rstage, rks, 6), AXK_RX(1 - (buf), rstage, rks, 7), LD,                    \
                AXK_LOAD_X(lstage, 5), AXK_LOAD_W(lstage, 5), (void)0, (void)0);                                         \
        AXK_ROW(buf, 6, 0, (void)0, (void)0, LD, AXK_LOAD_X(lstage, 6), AXK_LOAD_W(lstage, 6), (void)0, (void)0);        \
        AXK_ROW_REV(buf, 7, 0, (void)0, (void)0, LD, AXK_LOAD_X(lstage, 7), AXK_LOAD_W(lstage, 7), gx += BKB, gw += BKB);    \
        __builtin_amdgcn_sched_barrier(0);                                                                               \
    } while (0)
#define AXK_WAIT_FRAGS() do { AXI8_LGKM(0); __builtin_amdgcn_sched_barrier(0); } while (0)
// One slab resident in `stage`, its k-step 0 already (being) read into buffer 0.  After the first
// k-step every wave has read all it needs of this stage and waits for its own loads of the next
// slab; past the barrier the stage is free, so the second k-step's MFMAs cover the first fragment
// reads of the next slab (after the last slab they fetch stale bytes nobody uses) and, when more2,
// the loads of the slab after.
#define AXK_SLAB(stage, more2)                                               \
    do {                                                                     \
        AXK_WAIT_FRAGS();                                                    \
        AXK_BLOCK(0, 1, stage, 1, 0, 0);                                     \
        AXK_WAIT_FRAGS();                                                    \
        if (loader) AXI8_VM0();                                              \
        __builtin_amdgcn_s_barrier();                                        \
        __builtin_amdgcn_sched_barrier(0);                                   \
        AXK_BLOCK(1, 1, 1 - (stage), 0, (more2) && loader, stage);           \
    } while (0)

template <int ACT>
__global__ void __launch_bounds__(512)
k_qgemm_w8a8_256_k64(const int8_t *__restrict__ X, const int8_t *__restrict__ W, int64_t M, int64_t N,
                     int64_t K, float x_scale, const float *__restrict__ w_scales,
                     const float *__restrict__ bias, float *__restrict__ out,
                     int32_t *__restrict__ acc_out, int64_t ldc) {
    constexpr int BM = 256, BN = 256, BKB = 128, WAVES_N = 4, WTM = 128, WTN = 64, TM = 8, TN = 4;
    constexpr int OPER = BM * BKB;   // bytes of one operand in one stage
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int tiles_m = (int)(M / BM), tiles_n = (int)(N / BN), total = tiles_m * tiles_n;
    const int slabs = (int)(K / BKB);
    const bool loader = wave < 4;         // waves 0-3 load and never store, waves 4-7 store and never load
    // load instruction j (0..7) of loader wave w fills rows (j*4+w)*8 .. +8 of an operand stage
    unsigned voff[8];
    {
        const int sw = (wave & 1) * 4 + (lane >> 4);      // (row >> 1) & 7 of this lane's row
#pragma unroll
        for (int j = 0; j < 8; j++)
            voff[j] = (unsigned)(((j * 4 + (wave & 3)) * 8 + (lane >> 3)) * K + (((lane & 7) ^ sw) << 4));
    }
    const int8_t *gx = X, *gw = W;
    const unsigned lds_w = (unsigned)(uintptr_t)lds + (wave & 3) * 1024;

    // fragment reads: lane (frow, fq) of tile i takes row i*16 + frow, logical chunk ks*4 + fq
    const int frow = lane & 15, fq = lane >> 4;
    unsigned rx[2], rw[2];
    {
        const int sw = (frow >> 1) & 7;
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            const unsigned inrow = (unsigned)(frow * BKB + (((ks * 4 + fq) ^ sw) << 4));
            rx[ks] = (unsigned)(uintptr_t)lds + wm * WTM * BKB + inrow;
            rw[ks] = (unsigned)(uintptr_t)lds + 2 * OPER + wn * WTN * BKB + inrow;
        }
    }

    typedef float v4f_t __attribute__((ext_vector_type(4)));
    float *lds_scale = reinterpret_cast<float *>(lds + 4 * OPER);     // [2 slots][scale 256 | bias 256]
    v4i acc[TM][TN];

    const bool carry = (slabs & 1) == 0;
    bool fetched = false;
    v4f_t col_s = {0.f, 0.f, 0.f, 0.f}, col_b = {0.f, 0.f, 0.f, 0.f};
    auto load_cols = [&](int64_t n0) {            // issued a whole tile ahead of store_cols
        if (out && wave == 0) {
            col_s = *reinterpret_cast<const v4f_t *>(w_scales + n0 + lane * 4);
            if (bias) col_b = *reinterpret_cast<const v4f_t *>(bias + n0 + lane * 4);
        }
    };
    auto store_cols = [&](int slot) {
        if (out && wave == 0) {
            v4f_t v = col_s;
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = x_scale * v[e];
            float *dst = lds_scale + slot * 2 * BN + lane * 4;
            *reinterpret_cast<v4f_t *>(dst) = v;
            *reinterpret_cast<v4f_t *>(dst + BN) = col_b;
        }
    };
    int slot = 0;
    v4i fx[2][TM], fw[2][TN];

    // Write-back of one 32x32 sub-tile (2 x 2 tiles of 16x16) per wave and round.  r[2a + b] is tile (a, b)
    // of the sub-tile: lane l holds its row 16 a + (l & 15) and the four columns of 16-byte chunk
    // 4 b + (l >> 4).  Every wave writes its sub-tile (chunk c of row r at chunk c ^ ((r>>1)&7), conflict-free
    // both ways) into its 4 KiB of a turn buffer; after the barrier storer wave 4+s reads the sub-tiles of
    // waves 2s and 2s+1 back row-major and stores whole 128-byte rows, as in the kernel above.
    int round = 0;
    auto emit = [&](const auto (&r)[4], auto *base, int64_t m0, int64_t n0, int i, int j) {
        typedef typename std::remove_const<typename std::remove_reference<decltype(r[0])>::type>::type V4;
        unsigned char *buf = lds + ((round & 1) ? 3 * OPER : OPER);
        round++;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int row = (g >> 1) * 16 + frow, chunk = 4 * (g & 1) + fq;
            *reinterpret_cast<V4 *>(buf + wave * 4096 + row * 128 + ((chunk ^ ((frow >> 1) & 7)) << 4)) = r[g];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
        if (!loader) {
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const int src = 2 * (wave - 4) + q;                     // wave whose sub-tile this is
                auto *dst = base + (m0 + (src / WAVES_N) * WTM + i * 32) * ldc + n0 + (src % WAVES_N) * WTN + j * 32;
#pragma unroll
                for (int p = 0; p < 4; p++) {
                    const int row = p * 8 + (lane >> 3);
                    const V4 v = *reinterpret_cast<const V4 *>(buf + src * 4096 + row * 128 +
                                                               (((lane & 7) ^ ((row >> 1) & 7)) << 4));
                    __builtin_nontemporal_store(v, reinterpret_cast<V4 *>(dst + (int64_t)row * ldc + (lane & 7) * 4));
                }
            }
        }
    };

    for (int t = blockIdx.x; t < total; t += gridDim.x) {
        int tm, tn;
        tile_of_block(t, tiles_m, tiles_n, tm, tn);
        const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
        if (!fetched) {
            gx = X + m0 * K;
            gw = W + n0 * K;
            if (loader) AXK_ISSUE(0);
            load_cols(n0);
            store_cols(slot);
        }
        const int t_next = t + (int)gridDim.x;
        const bool will_fetch = carry && t_next < total;
        int tm2 = 0, tn2 = 0;
        if (will_fetch) {
            tile_of_block(t_next, tiles_m, tiles_n, tm2, tn2);
            load_cols((int64_t)tn2 * BN);
        }
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) acc[i][j] = v4i{0, 0, 0, 0};

        if (loader) AXI8_VM0();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        if (slabs > 1 && loader) AXK_ISSUE(1);
        AXK_FRAGS(0, 0, 0);

        for (int s = 0; s < slabs; s += 2) {       // the flags are wave-uniform: scalar branches only
            AXK_SLAB(0, s + 2 < slabs);
            if (s + 1 < slabs) AXK_SLAB(1, s + 3 < slabs);
        }
        AXK_WAIT_FRAGS();      // the stale reads must land before their registers are reused

        fetched = will_fetch;
        if (fetched) {
            store_cols(slot ^ 1);
            gx = X + (int64_t)tm2 * BM * K;
            gw = W + (int64_t)tn2 * BN * K;
            if (loader) AXK_ISSUE(0);
        }

        if (acc_out) {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const v4i r[4] = {acc[2 * i][2 * j], acc[2 * i][2 * j + 1], acc[2 * i + 1][2 * j], acc[2 * i + 1][2 * j + 1]};
                    emit(r, acc_out, m0, n0, i, j);
                }
        }
        if (out) {
            const float *sp = lds_scale + slot * 2 * BN + wn * WTN + 4 * fq, *bp = sp + BN;
            const bool has_bias = bias != nullptr;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                v4f_t sc[2], bv[2];
#pragma unroll
                for (int b = 0; b < 2; b++) {
                    sc[b] = *reinterpret_cast<const v4f_t *>(sp + j * 32 + 16 * b);
                    bv[b] = *reinterpret_cast<const v4f_t *>(bp + j * 32 + 16 * b);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    v4f_t r[4];
#pragma unroll
                    for (int g = 0; g < 4; g++)
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float f = (float)acc[2 * i + (g >> 1)][2 * j + (g & 1)][e];
                            // a fused multiply-add with bias = 0 would round differently from the plain product
                            r[g][e] = apply_act(has_bias ? __builtin_fmaf(f, sc[g & 1][e], bv[g & 1][e]) : f * sc[g & 1][e], ACT);
                        }
                    emit(r, out, m0, n0, i, j);
                }
            }
        }
        slot ^= 1;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    }
}
#undef AXK_LOAD_X
#undef AXK_LOAD_W
#undef AXK_ISSUE
#undef AXK_RX
#undef AXK_RW
#undef AXK_FRAGS
#undef AXK_M
#undef AXK_ROW
#undef AXK_ROW_REV
#undef AXK_BLOCK
#undef AXK_WAIT_FRAGS
#undef AXK_SLAB

// ---------------------------------------------------------------------------------------
// Mid-size aligned shapes (M, N multiples of the tile, K a multiple of 128) that cannot fill
// the chip with 256x256 tiles: the same direct-to-LDS, VALU-free loop over smaller tiles with
// NST LDS stages, so NST-1 slabs of loads are in flight per workgroup (a 64x64 tile has only
// 128 MFMA cycles of work per slab and wave: the loop is bound by load latency and by the
// CU's L1 bandwidth, not by the matrix core).  LDS: NST stages of X (BM rows x 128 B), NST
// stages of W, then BN scales and BN biases.  Not persistent.
// EDGE: M and N need not be multiples of the tile.  A row past the end of X or W is fetched from
// the last row instead (its products land in outputs that are not stored), and the write-back
// keeps to rows below M and 4-column groups below N (N a multiple of 4).
// WAVES_K = 2: a second set of WAVES_M x WAVES_N waves takes k-steps 2 and 3 of every slab (the first
// set keeps 0 and 1) and hands its accumulators over through LDS at the end.  A tile then has two
// waves on every SIMD with no more global traffic, so one wave's waits for LDS and for the slab
// barrier are covered by the other's MFMAs: for a launch of at most one small tile per CU, whose
// time is the chain of those waits rather than memory or matrix-core throughput.
// STREAM_W: the weights are read once and are large, their loads are non-temporal (a template parameter: a run-time
// test in front of every load costs the launches that do not stream 3-5 %).
template <int BM, int BN, int WAVES_M, int WAVES_N, int NST, int ACT, bool EDGE = false, int WAVES_K = 1, int SPB = 1,
          bool STREAM_W = false>
__global__ void __launch_bounds__(WAVES_M *WAVES_N *WAVES_K * 64)
k_qgemm_w8a8_dma(const int8_t *__restrict__ X, const int8_t *__restrict__ W, int64_t M, int64_t N,
                 int64_t K, float x_scale, const float *__restrict__ w_scales,
                 const float *__restrict__ bias, float *__restrict__ out,
                 int32_t *__restrict__ acc_out, int64_t ldc, int splits, int32_t *partials,
                 int *__restrict__ counters, int phases) {
    constexpr int NWO = WAVES_M * WAVES_N, NW = NWO * WAVES_K, BKB = 128;      // waves that own outputs / all waves
    constexpr int KSTEPS = 4 / WAVES_K;                                        // k-steps of a slab per wave
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N, TM = WTM / 32, TN = WTN / 32;
    // SPB = 2: a stage holds two slabs and the loop synchronises once per two (half the barriers and
    // waits, for tiles whose slab is only a few dozen MFMA cycles); K is then a multiple of 256, no
    // EDGE and no split.  XS / WS stay the bytes of ONE slab; a stage is SPB of them.
    constexpr int XS = BM * BKB, WS = BN * BKB;          // bytes of one slab of each operand
    constexpr int W_BASE = NST * SPB * XS;
    constexpr int IPW_X = BM / 8 / NW, IPW_W = BN / 8 / NW;   // load instructions per wave and slab
    constexpr int NREADS = TM + TN;
    constexpr int VM_KEEP = (NST - 2) * SPB * (IPW_X + IPW_W);
    static_assert(IPW_X * 8 * NW == BM && IPW_W * 8 * NW == BN, "slab must divide over the waves");
    static_assert(NST >= 2 && NST <= 4 && VM_KEEP < 64, "stage count");
    static_assert(SPB == 1 || (SPB == 2 && !EDGE), "one or two slabs per stage");
    static_assert((NST * SPB - 1) * XS + (TM - 1) * 4096 < 65536 && (NST * SPB - 1) * WS + (TN - 1) * 4096 < 65536,
                  "ds_read immediates are 16 bits");
    static_assert(WAVES_K == 1 || WAVES_K == 2, "one or two wave sets over k");
    static_assert(NWO * 4096 + (WAVES_K - 1) * NWO * TM * TN * 4096 <= NST * SPB * XS, "write-back turn area and k hand-over");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = wave / NWO, wo = wave % NWO;          // wave set over k, output wave inside the set
    const int wm = wo / WAVES_N, wn = wo % WAVES_N;
    int tm, tn;
    tile_of_block(blockIdx.x, (int)((M + BM - 1) / BM), (int)((N + BN - 1) / BN), tm, tn);
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    // EDGE also takes a K that ends inside a slab (K a multiple of 16): in the last slab the lanes
    // whose 16 bytes lie past K load nothing and write zeros to their LDS place instead
    const int slabs_all = EDGE ? (int)((K + BKB - 1) / BKB) : (int)(K / BKB);
    // Split over K (gridDim.y = splits > 1): workgroup y of a tile multiplies slabs [slab0, slab0 + slabs);
    // the host picks splits so that none is empty.  The int32 partial tiles are added by whichever
    // workgroup of the tile finishes last: integer sums are exact in any order.
    const int per_split = (slabs_all + splits - 1) / splits, slab0 = (int)blockIdx.y * per_split;
    const int slabs = slabs_all - slab0 < per_split ? slabs_all - slab0 : per_split;
    const int ktail = EDGE && slab0 + slabs == slabs_all ? (int)(K - (int64_t)(slabs_all - 1) * BKB) : BKB;   // bytes of K in this range's last slab
    int left = slabs;                                                          // slabs not yet requested
    // rows of this tile that exist (EDGE; the last tile row / column may hang over)
    const int mrows = EDGE && M - m0 < BM ? (int)(M - m0) : BM, nrows = EDGE && N - n0 < BN ? (int)(N - n0) : BN;

    // load instruction q fills rows q*8 .. q*8+7 of an operand stage; wave w issues q = j*NW + w.
    // The LDS place (and so the swizzle) is that of the nominal row; the source row is clamped.
    unsigned vx[IPW_X], vw[IPW_W];
    bool tx[IPW_X], tw[IPW_W];                   // is this lane's chunk inside K in the last slab
#pragma unroll
    for (int j = 0; j < IPW_X; j++) {
        const int row = (j * NW + wave) * 8 + (lane >> 3);
        vx[j] = (unsigned)((row < mrows ? row : mrows - 1) * K + (((lane & 7) ^ ((row >> 1) & 7)) << 4));
        tx[j] = (((lane & 7) ^ ((row >> 1) & 7)) << 4) < ktail;
    }
#pragma unroll
    for (int j = 0; j < IPW_W; j++) {
        const int row = (j * NW + wave) * 8 + (lane >> 3);
        vw[j] = (unsigned)((row < nrows ? row : nrows - 1) * K + (((lane & 7) ^ ((row >> 1) & 7)) << 4));
        tw[j] = (((lane & 7) ^ ((row >> 1) & 7)) << 4) < ktail;
    }
    // phases > 1 (K on the slab grid): the workgroups that share a block of W rows (same tn) or of X rows (same
    // tm) start their walk over K at different slabs and wrap around, so they miss on different lines at any
    // moment and find the others' lines in L2 later.  Integer sums are exact in any order.
    int first = 0;
    if (phases > 1 && slabs >= phases) first = ((tm * 7 + tn * 3) % phases) * (slabs / phases);
    int wrap_in = slabs - first;                                               // slabs to request before the walk wraps to this range's start
    const int8_t *gx = X + m0 * K + (int64_t)(slab0 + first) * BKB, *gw = W + n0 * K + (int64_t)(slab0 + first) * BKB;
    const unsigned lds0 = (unsigned)(uintptr_t)lds, lds_w = lds0 + wave * 1024;

    const int frow = lane & 31, fhalf = lane >> 5;
    unsigned rx[KSTEPS], rw[KSTEPS];                     // this wave's k-steps: wk * KSTEPS + 0 ..
#pragma unroll
    for (int i = 0; i < KSTEPS; i++) {
        const int ks = wk * KSTEPS + i;
        const unsigned inrow = (unsigned)(frow * BKB + (((ks * 2 + fhalf) ^ ((frow >> 1) & 7)) << 4));
        rx[i] = lds0 + wm * WTM * BKB + inrow;
        rw[i] = lds0 + W_BASE + wn * WTN * BKB + inrow;
    }

    typedef float v4f_t __attribute__((ext_vector_type(4)));
    float *lds_scale = reinterpret_cast<float *>(lds + NST * SPB * (XS + WS)), *lds_bias = lds_scale + BN;
    if (out) {
        for (int c = tid; c < BN; c += NW * 64) {
            const bool live = c < nrows;
            lds_scale[c] = live ? x_scale * w_scales[n0 + c] : 0.0f;
            lds_bias[c] = live && bias ? bias[n0 + c] : 0.0f;
        }
    }

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0;
    v4i fx[2][TM], fw[2][TN];

#define AXI8G_ISSUE1(ST)                                                                         \
    do {                                                                                         \
        --left;                                                                                  \
        if (EDGE && left == 0 && ktail < BKB) {                                                  \
            _Pragma("unroll") for (int j = 0; j < IPW_X; j++) {                                  \
                const unsigned at = wave * 1024 + (ST) * XS + j * NW * 1024;                     \
                if (tx[j]) AXI8_LOAD_LDS(lds0 + at, vx[j], gx);                                  \
                else *reinterpret_cast<v4i *>(lds + at + lane * 16) = v4i{0, 0, 0, 0};           \
            }                                                                                    \
            _Pragma("unroll") for (int j = 0; j < IPW_W; j++) {                                  \
                const unsigned at = wave * 1024 + W_BASE + (ST) * WS + j * NW * 1024;            \
                if (!tw[j]) *reinterpret_cast<v4i *>(lds + at + lane * 16) = v4i{0, 0, 0, 0};    \
                else if (STREAM_W) AXI8_LOAD_LDS_NT(lds0 + at, vw[j], gw);                       \
                else AXI8_LOAD_LDS(lds0 + at, vw[j], gw);                                        \
            }                                                                                    \
        } else {                                                                                 \
            _Pragma("unroll") for (int j = 0; j < IPW_X; j++)                                    \
                AXI8_LOAD_LDS(lds_w + (ST) * XS + j * NW * 1024, vx[j], gx);                     \
            _Pragma("unroll") for (int j = 0; j < IPW_W; j++) {                                  \
                if (STREAM_W) AXI8_LOAD_LDS_NT(lds_w + W_BASE + (ST) * WS + j * NW * 1024, vw[j], gw); \
                else AXI8_LOAD_LDS(lds_w + W_BASE + (ST) * WS + j * NW * 1024, vw[j], gw);       \
            }                                                                                    \
        }                                                                                        \
        gx += BKB;                                                                               \
        gw += BKB;                                                                               \
        if (--wrap_in == 0) {                                                                    \
            gx -= (int64_t)slabs * BKB;                                                          \
            gw -= (int64_t)slabs * BKB;                                                          \
        }                                                                                        \
    } while (0)
// a stage: SPB slabs into consecutive slab places
#define AXI8G_ISSUE(ST)                                                                          \
    do {                                                                                         \
        AXI8G_ISSUE1((ST) * SPB);                                                                \
        if constexpr (SPB == 2) AXI8G_ISSUE1((ST) * SPB + 1);                                    \
    } while (0)
#define AXI8G_FRAGS(buf, ST, ks)                                                                 \
    do {                                                                                         \
        _Pragma("unroll") for (int t = 0; t < TM; t++)                                           \
            AXI8_DS_READ(fx[buf][t], rx[ks], (ST) * XS + t * 4096);                              \
        _Pragma("unroll") for (int t = 0; t < TN; t++)                                           \
            AXI8_DS_READ(fw[buf][t], rw[ks], (ST) * WS + t * 4096);                              \
    } while (0)
#define AXI8G_MFMAS(buf)                                                                         \
    do {                                                                                         \
        __builtin_amdgcn_sched_barrier(0);                                                       \
        _Pragma("unroll") for (int i = 0; i < TM; i++)                                           \
            _Pragma("unroll") for (int j = 0; j < TN; j++)                                       \
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[buf][j], fx[buf][i],        \
                                                                  acc[i][j], 0, 0, 0);           \
        __builtin_amdgcn_sched_barrier(0);                                                       \
    } while (0)
    // one slab out of stage ST; `more`: slab s+NST-1 exists and is fetched into the stage read last
#define AXI8G_COMPUTE(SS)                                                                        \
    do {                                                                                         \
        AXI8G_FRAGS(0, SS, 0);                                                                   \
        AXI8G_FRAGS(1, SS, 1);                                                                   \
        AXI8_LGKM(NREADS);                                                                       \
        AXI8G_MFMAS(0);                                                                          \
        if constexpr (KSTEPS == 4) {                                                             \
            AXI8G_FRAGS(0, SS, 2);                                                               \
            AXI8_LGKM(NREADS);                                                                   \
            AXI8G_MFMAS(1);                                                                      \
            AXI8G_FRAGS(1, SS, 3);                                                               \
            AXI8_LGKM(NREADS);                                                                   \
            AXI8G_MFMAS(0);                                                                      \
        }                                                                                        \
        AXI8_LGKM(0);                                                                            \
        AXI8G_MFMAS(1);                                                                          \
    } while (0)
#define AXI8G_SLAB(ST, more)                                                                     \
    do {                                                                                         \
        if (more) AXI8G_ISSUE(((ST) + NST - 1) % NST);                                           \
        AXI8G_COMPUTE((ST) * SPB);                                                               \
        if constexpr (SPB == 2) AXI8G_COMPUTE((ST) * SPB + 1);                                   \
        if (VM_KEEP > 0 && (more)) AXI8_VM(VM_KEEP); else AXI8_VM(0);                            \
        __builtin_amdgcn_s_barrier();                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                       \
    } while (0)

    // prologue: the first NST-1 slabs are requested; compute starts as soon as the first has landed
    const int rounds = slabs / SPB;              // stages' worth of slabs (SPB == 2: the host guarantees an even count)
    AXI8G_ISSUE(0);
    if constexpr (NST > 2) { if (rounds > 1) AXI8G_ISSUE(1); }
    if constexpr (NST > 3) { if (rounds > 2) AXI8G_ISSUE(2); }
    if (VM_KEEP > 0 && rounds >= NST - 1) AXI8_VM(VM_KEEP); else AXI8_VM(0);
    if constexpr (EDGE) AXI8_LGKM(0);            // zeros written for a K tail that is already in the first slabs
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    // whole rounds of the ring in a loop with one way out, then the slabs % NST that remain (nothing is
    // left to fetch by then): an exit between two slabs of the loop body makes the compiler copy the
    // accumulators from one register set to another every round
    int s = 0;
    for (; s + NST <= rounds; s += NST) {
        AXI8G_SLAB(0, s + NST - 1 < rounds);
        AXI8G_SLAB(1, s + NST < rounds);
        if constexpr (NST > 2) AXI8G_SLAB(2, s + NST + 1 < rounds);
        if constexpr (NST > 3) AXI8G_SLAB(3, s + NST + 2 < rounds);
    }
    if (s < rounds) AXI8G_SLAB(0, false);
    if (s + 1 < rounds) AXI8G_SLAB(1, false);
    if constexpr (NST > 3) { if (s + 2 < rounds) AXI8G_SLAB(2, false); }
#undef AXI8G_ISSUE1
#undef AXI8G_ISSUE
#undef AXI8G_FRAGS
#undef AXI8G_MFMAS
#undef AXI8G_COMPUTE
#undef AXI8G_SLAB

    if constexpr (WAVES_K == 2) {
        // the second wave set hands its sums to the first through the dead stages, register by register
        // ([wave][16-byte group][lane], past the turn area), and is done
        v4i *hand = reinterpret_cast<v4i *>(lds + NWO * 4096) + wo * (TM * TN * 4 * 64) + lane;
        if (wk == 1) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int g = 0; g < 4; g++)
                        hand[((i * TN + j) * 4 + g) * 64] =
                            v4i{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
        }
        __syncthreads();
        if (wk == 1) return;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const v4i t = hand[((i * TN + j) * 4 + g) * 64];
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[i][j][4 * g + e] += t[e];
                }
    }
    // from here on only the NWO output waves are alive (a finished wave no longer counts at barriers)
    if (splits > 1) {
        // Partial tiles are kept register by register, [tile][split][wave][register][lane]: whoever reads
        // them back has the same wave / lane / register roles, so the layout never has to mean rows and
        // columns.  Partials, the arrival counter and the reads below are device-scope accesses (the
        // workgroups of one tile run on different XCDs, each with its own L2); the wait makes this thread's
        // stores complete before the barrier, the barrier orders them before thread 0's increment.
        constexpr int REGS = TM * TN * 16;
        int32_t *tile_part = partials + (int64_t)blockIdx.x * splits * (NWO * REGS * 64);
        int32_t *mine = tile_part + ((int64_t)blockIdx.y * NWO + wave) * (REGS * 64);
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int v = 0; v < 16; v++)
                    __hip_atomic_store(mine + ((i * TN + j) * 16 + v) * 64 + lane, acc[i][j][v], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        int *last_flag = reinterpret_cast<int *>(lds_bias + BN);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (tid == 0) {
            const int arrived = __hip_atomic_fetch_add(counters + blockIdx.x, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *last_flag = (arrived == splits - 1);
        }
        __syncthreads();
        if (!*last_flag) return;
        for (int p = 0; p < splits; p++) {
            if (p == (int)blockIdx.y) continue;
            const int32_t *theirs = tile_part + ((int64_t)p * NWO + wave) * (REGS * 64);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int v = 0; v < 16; v++)
                        acc[i][j][v] += __hip_atomic_load(theirs + ((i * TN + j) * 16 + v) * 64 + lane, __ATOMIC_RELAXED,
                                                          __HIP_MEMORY_SCOPE_AGENT);
        }
        if (tid == 0)                                   // ready for the next launch
            __hip_atomic_store(counters + blockIdx.x, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // write-back as in the 256x256 kernel: through 4 KiB of dead stage per wave
    unsigned char *turn = lds + wave * 4096;
    const int64_t trow = m0 + wm * WTM, tcol = n0 + wn * WTN;
    if (acc_out) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                v4i r[4];
#pragma unroll
                for (int g = 0; g < 4; g++)
                    r[g] = v4i{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                if (EDGE)
                    turn_tile_and_store_edge(turn, lane, r, acc_out + (trow + i * 32) * ldc + tcol + j * 32, ldc,
                                             M - trow - i * 32, N - tcol - j * 32);
                else
                    turn_tile_and_store(turn, lane, r, acc_out + (trow + i * 32) * ldc + tcol + j * 32, ldc);
            }
    }
    if (out) {
        const float *sp = lds_scale + wn * WTN + 4 * fhalf, *bp = lds_bias + wn * WTN + 4 * fhalf;
        const bool has_bias = bias != nullptr;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            v4f_t sc[4], bv[4];
#pragma unroll
            for (int g = 0; g < 4; g++) {
                sc[g] = *reinterpret_cast<const v4f_t *>(sp + j * 32 + 8 * g);
                bv[g] = *reinterpret_cast<const v4f_t *>(bp + j * 32 + 8 * g);
            }
#pragma unroll
            for (int i = 0; i < TM; i++) {
                v4f_t r[4];
#pragma unroll
                for (int g = 0; g < 4; g++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float f = (float)acc[i][j][4 * g + e];
                        r[g][e] = apply_act(has_bias ? __builtin_fmaf(f, sc[g][e], bv[g][e]) : f * sc[g][e], ACT);
                    }
                if (EDGE)
                    turn_tile_and_store_edge(turn, lane, r, out + (trow + i * 32) * ldc + tcol + j * 32, ldc,
                                             M - trow - i * 32, N - tcol - j * 32);
                else
                    turn_tile_and_store(turn, lane, r, out + (trow + i * 32) * ldc + tcol + j * 32, ldc);
            }
        }
    }
}

// Workgroups over K for a launch of `tiles` output tiles and `slabs` slabs of 128 bytes.  The join
// costs a store, an atomic and a load in a row at the end of every workgroup, about 4 us, so a split
// pays only when the tiles leave at least half the CUs idle and K is long: up to one workgroup per CU,
// at most 8, each with at least 8 slabs (64 x 1024 x 4096: 8.6 -> 6.4 us with 4; 256 x 2048 x 8192:
// 14.8 -> 12.3 with 2; M = 256, N = K = 4096, one tile per CU already: 9.8 -> 12.8 with 2).
int pick_splits(int64_t tiles, int64_t slabs) {
    const Tuning &tune = tuning();
    int64_t splits = 1;
    if (tune.i8_splitk > 0) splits = tune.i8_splitk;
    else if (tiles * 2 <= cu_count() && slabs >= 16) {
        splits = cu_count() / tiles;
        if (splits > slabs / 8) splits = slabs / 8;
        if (splits > 8) splits = 8;
    }
    if (splits > slabs) splits = slabs;
    if (splits < 1) splits = 1;
    const int64_t per = (slabs + splits - 1) / splits;
    return (int)((slabs + per - 1) / per);          // drop ranges that would be empty
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int NST, bool EDGE = false, int WAVES_K = 1, int SPB = 1>
int launch_dma(const char *name, const char *split_name, const int8_t *x, float x_scale, const int8_t *w,
               const float *w_scales, const float *bias, int act, float *out, int32_t *acc_out, int64_t M, int64_t N,
               int64_t K, int64_t ldc) {
    constexpr int smem = NST * SPB * (BM + BN) * 128 + 2 * BN * 4 + 16;      // stages, scale and bias rows, the split join's flag
    typedef void (*kern_t)(const int8_t *, const int8_t *, int64_t, int64_t, int64_t, float, const float *,
                           const float *, float *, int32_t *, int64_t, int, int32_t *, int *, int);
    // the streaming forms are built for the tiles of at most 64 rows, which are the ones few rows get
    constexpr bool CAN_STREAM = BM <= 64;
    static const kern_t kerns[6] = {k_qgemm_w8a8_dma<BM, BN, WAVES_M, WAVES_N, NST, AXHIP_ACT_NONE, EDGE, WAVES_K, SPB>,
                                    k_qgemm_w8a8_dma<BM, BN, WAVES_M, WAVES_N, NST, AXHIP_ACT_RELU, EDGE, WAVES_K, SPB>,
                                    k_qgemm_w8a8_dma<BM, BN, WAVES_M, WAVES_N, NST, AXHIP_ACT_GELU, EDGE, WAVES_K, SPB>,
                                    k_qgemm_w8a8_dma<BM, BN, WAVES_M, WAVES_N, NST, AXHIP_ACT_NONE, EDGE, WAVES_K, SPB, CAN_STREAM>,
                                    k_qgemm_w8a8_dma<BM, BN, WAVES_M, WAVES_N, NST, AXHIP_ACT_RELU, EDGE, WAVES_K, SPB, CAN_STREAM>,
                                    k_qgemm_w8a8_dma<BM, BN, WAVES_M, WAVES_N, NST, AXHIP_ACT_GELU, EDGE, WAVES_K, SPB, CAN_STREAM>};
    static bool attr_set = false;
    if (!attr_set) {
        for (kern_t kf : kerns)
            AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kf),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, smem),
                          "hipFuncSetAttribute");
        attr_set = true;
    }
    const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    if (tiles > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "qgemm_w8a8: too many tiles");
    const int splits = SPB == 2 ? 1 : pick_splits(tiles, (K + 127) / 128);     // two slabs per stage: the caller checked that no split is wanted
    int32_t *partials = nullptr;
    int *counters = nullptr;
    if (splits > 1) {
        partials = static_cast<int32_t *>(workspace((size_t)tiles * splits * BM * BN * sizeof(int32_t)));
        counters = strip_counters((size_t)tiles);
        if (!partials || !counters) return AXHIP_ERR_ALLOC;
    }
    // Staggered walks over K (kernel comment) pay when the weights come from HBM: a CU sustains only about 31 GB/s
    // of misses, so workgroups that miss on the same lines together divide the rate at which new bytes arrive
    // (M = 256, N = K = 4096, weights in rotation: 13.0 -> 10.8 us; the same weights cached: 8.5 -> 8.7).  They need
    // an XCD's share of the operands to stay in its 4 MiB of L2 until the last sharer has passed, or every line
    // is fetched once per sharer (512 x 4096 x 11008: 31.6 -> 52.2 us): one round of tiles, all of X and an eighth
    // of W within 3 MiB (at 4 MiB, 512 x 4096 x 4096 on 128x64 tiles: 18.0 -> 16.6 us from HBM but 14.0 -> 15.1 cached).
    const int phases = (K % 128 == 0 && tiles <= cu_count() && (M + N / 8) * K <= (int64_t(3) << 20)) ? 4 : 0;
    // one row of tiles reads every byte of W once: 40 MiB of weights and more then arrive faster through non-temporal
    // loads (a slab here is a whole 128-byte line of every weight row, so nothing is fetched twice)
    // (weights in rotation: 8 x 11008 x 4096 13.9 -> 13.2 us, 64 x 8192 x 8192 20.1 -> 18.8, 16 x 4096 x 11008 14.6 -> 13.5)
    const int stream_w = (CAN_STREAM && M <= BM && N * K >= (int64_t(40) << 20)) ? 3 : 0;
    note_kernel(splits > 1 ? split_name : name);
    hipLaunchKernelGGL(kerns[act + stream_w], dim3((unsigned)tiles, (unsigned)splits), dim3(WAVES_M * WAVES_N * WAVES_K * 64), smem, kStream,
                       x, w, M, N, K, x_scale, w_scales, bias, out, acc_out, ldc, splits, partials, counters, phases);
    return check_launch(name);
}

int launch_256(const int8_t *x, float x_scale, const int8_t *w, const float *w_scales,
               const float *bias, int act, float *out, int32_t *acc_out, int64_t M, int64_t N,
               int64_t K, int64_t ldc) {
    constexpr int smem = 4 * 256 * 128 + 2 * 2 * 256 * 4;   // two stages of both operands + two slots of scale and bias
    typedef void (*kern_t)(const int8_t *, const int8_t *, int64_t, int64_t, int64_t, float, const float *,
                           const float *, float *, int32_t *, int64_t);
    static const kern_t kerns[6] = {k_qgemm_w8a8_256<AXHIP_ACT_NONE>, k_qgemm_w8a8_256<AXHIP_ACT_RELU>,
                                    k_qgemm_w8a8_256<AXHIP_ACT_GELU>, k_qgemm_w8a8_256_k64<AXHIP_ACT_NONE>,
                                    k_qgemm_w8a8_256_k64<AXHIP_ACT_RELU>, k_qgemm_w8a8_256_k64<AXHIP_ACT_GELU>};
    static bool attr_set = false;
    if (!attr_set) {
        for (kern_t kf : kerns)
            AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kf),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, smem),
                          "hipFuncSetAttribute");
        attr_set = true;
    }
    const int64_t tiles = (M / 256) * (N / 256);
    if (tiles > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "qgemm_w8a8: too many tiles");
    // AX_HIP_I8_MFMA: 32 = v_mfma_i32_32x32x32_i8, 16 (and by default) = v_mfma_i32_16x16x64_i8
    const bool k64 = tuning().i8_mfma != 32;
    note_kernel(k64 ? "qgemm_w8a8_256x256_dma" : "qgemm_w8a8_256x256_dma_mfma32x32x32");
    const int64_t grid = tiles < cu_count() ? tiles : cu_count();     // one persistent workgroup per CU
    hipLaunchKernelGGL(kerns[act + (k64 ? 3 : 0)], dim3((unsigned)grid), dim3(512), smem, kStream, x, w, M, N, K,
                       x_scale, w_scales, bias, out, acc_out, ldc);
    return check_launch("qgemm_w8a8_256x256_dma");
}

// ---- M <= 4: bandwidth-bound, no matrix cores ---------------------------------------------
// One wave owns 4 weight rows.  Lanes walk K in 16-byte steps (a wave-wide load covers 1 KiB of a
// row), keep the activation bytes of their k positions in registers across the 4 rows, and feed
// four-byte integer dot products; the per-lane int32 sums are added over the wave, all 4 * M at
// once, and end up one per lane for the write-back.  Integer
// addition is exact in any order, so the accumulators equal the matrix-core kernels' bit for bit,
// and the write-back applies the same expression to them.
constexpr int GEMV_ROWS = 4;

template <int MR>
__global__ void __launch_bounds__(64)
k_w8a8_gemv(const int8_t *__restrict__ X, const int8_t *__restrict__ W, int64_t N, int64_t K, float x_scale,
            const float *__restrict__ w_scales, const float *__restrict__ bias, int act,
            float *__restrict__ out, int32_t *__restrict__ acc_out) {
    const int lane = threadIdx.x;
    const int64_t n0 = (int64_t)blockIdx.x * GEMV_ROWS;
    int acc[GEMV_ROWS][MR];
#pragma unroll
    for (int r = 0; r < GEMV_ROWS; r++)
#pragma unroll
        for (int m = 0; m < MR; m++) acc[r][m] = 0;
    for (int64_t k = (int64_t)lane * 16; k < K; k += 64 * 16) {
        v4i xa[MR];
#pragma unroll
        for (int m = 0; m < MR; m++) xa[m] = *reinterpret_cast<const v4i *>(X + m * K + k);
#pragma unroll
        for (int r = 0; r < GEMV_ROWS; r++) {
            const int64_t n = n0 + r < N ? n0 + r : N - 1;   // the last wave re-reads a row it does not store
            const v4i wv = __builtin_nontemporal_load(reinterpret_cast<const v4i *>(W + n * K + k));
#pragma unroll
            for (int m = 0; m < MR; m++)
#pragma unroll
                for (int q = 0; q < 4; q++) acc[r][m] = __builtin_amdgcn_sdot4(xa[m][q], wv[q], acc[r][m], false);
        }
    }
    constexpr int NV = GEMV_ROWS * MR <= 4 ? 4 : GEMV_ROWS * MR <= 8 ? 8 : GEMV_ROWS * MR <= 16 ? 16 : 32;
    int v[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) v[i] = i < GEMV_ROWS * MR ? acc[i / MR][i % MR] : 0;
    wave_sum_spread(v, lane);
    const int idx = lane / (64 / NV), r = idx / MR, m = idx % MR;
    const int64_t n = n0 + r;
    if (lane % (64 / NV) != 0 || idx >= GEMV_ROWS * MR || n >= N) return;
    const int a = v[0];
    if (acc_out) acc_out[m * N + n] = a;
    if (out) {
        const float f = (float)a, scale = x_scale * w_scales[n];
        const float o = bias ? __builtin_fmaf(f, scale, bias[n]) : f * scale;
        out[m * N + n] = apply_act(o, act);
    }
}

template <int MR>
int launch_gemv(const int8_t *x, float x_scale, const int8_t *w, const float *w_scales, const float *bias,
                int act, float *out, int32_t *acc_out, int64_t N, int64_t K) {
    note_kernel("qgemm_w8a8_gemv");
    hipLaunchKernelGGL(k_w8a8_gemv<MR>, dim3((unsigned)((N + GEMV_ROWS - 1) / GEMV_ROWS)), dim3(64), 0, kStream, x, w,
                       N, K, x_scale, w_scales, bias, act, out, acc_out);
    return check_launch("qgemm_w8a8_gemv");
}


// rows of K bytes -> rows of Kp >= K bytes (Kp a multiple of 16), the tail of each row zero
__global__ void __launch_bounds__(256)
k_pad_rows_i8(const int8_t *__restrict__ src, int8_t *__restrict__ dst, int64_t rows, int64_t K, int64_t Kp) {
    const int64_t per_row = Kp / 16, items = rows * per_row, stride = (int64_t)gridDim.x * 256;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < items; t += stride) {
        const int64_t r = t / per_row, k = (t - r * per_row) * 16;
        *reinterpret_cast<v4i *>(dst + r * Kp + k) = load_chunk<true>(src, r, rows, k, K);
    }
}

// One block of the output, rows of pitch ldc: picks the kernel for its shape and alignment.
int qgemm_block(const int8_t *x, float x_scale, const int8_t *w, const float *w_scales, const float *bias, int act,
                float *out, int32_t *acc_out, int64_t M, int64_t N, int64_t K, int64_t ldc) {
    const bool aligned = ((((uintptr_t)x | (uintptr_t)w) & 15) == 0) && (K % BK == 0) && K > 0;
    const bool vec_out = (!out || (((uintptr_t)out | (uintptr_t)w_scales | (uintptr_t)bias) & 15) == 0) &&
                         (((uintptr_t)acc_out & 15) == 0) && ldc % 4 == 0;
    // the persistent 256x256 kernel from about 80 tiles on (81 tiles, 2304^2 x 8192: 72 us against 82 on
    // 128x128 tiles; 64 tiles, 2048^2 x 4096: 40 against 26)
    if (aligned && vec_out && M % 256 == 0 && N % 256 == 0 && K < (int64_t(1) << 24) &&   // per-lane 32-bit byte offsets span 256 rows
        (tuning().i8_tile == 256 || (tuning().i8_tile == 0 && (M / 256) * (N / 256) >= 80))) {
        // When the 256x256 tiles leave CUs idle or make a short last round, 256x128 tiles (eight waves, one
        // workgroup per CU) spread the work better: a half tile costs about 0.6 of a whole one, so they win
        // when their rounds are fewer than 1.6 times as many and K is long (same box: 2048 x 4096 x 4096, 128
        // whole tiles, 43.1 -> 41.0 us; 2048 x 10752 x 4096, 344: 111.5 -> 105.3; 2304^2 x 8192, 81: 72.2 -> 56.4;
        // but 2048 x 4096 x 1024 17.4 against 20.1 and 4096^3, 256 tiles, 63.2 against 71.8: those stay).
        const int64_t whole = (M / 256) * (N / 256), cus = cu_count();
        const int64_t rounds_whole = (whole + cus - 1) / cus, rounds_half = (2 * whole + cus - 1) / cus;
        if (tuning().i8_tile == 0 && K % 128 == 0 && K >= 2048 && rounds_half * 60 < rounds_whole * 95)
            return launch_dma<256, 128, 4, 2, 2>("qgemm_w8a8_256x128_dma", "qgemm_w8a8_256x128_dma_splitk", x, x_scale, w, w_scales,
                                                 bias, act, out, acc_out, M, N, K, ldc);
        return launch_256(x, x_scale, w, w_scales, bias, act, out, acc_out, M, N, K, ldc);
    }
    // aligned but too few 256x256 tiles: direct-to-LDS kernel over smaller tiles
    const int force = tuning().i8_tile;             // 0 = by shape, else 64 / 128 where the shape permits
    if (aligned && vec_out && K % 128 == 0 && M % 64 == 0 && N % 64 == 0 && K < (int64_t(1) << 24)) {
        // 128x128 tiles once there is one for every CU (2048^2 x 4096: 26.2 us against 30.7 on 64x64); eight waves
        // (2 x 4, wave tile 64x32), two on every SIMD: 25.0 -> 24.2 us against four waves of 64x64
        const bool fits128 = M % 128 == 0 && N % 128 == 0;
        // Between one 64x64 tile per CU and a 128x128 tile per CU, 128x64 tiles on eight waves (4 x 2, wave tile
        // 32x32; 72 KiB of stages, two workgroups per CU): a quarter less operand traffic into LDS per output
        // than 64x64 (same box: 512 x 4096 x 4096 17.5 -> 14.8 us, 896 x 4096 x 4096 28.8 -> 23.4,
        // 512 x 4096 x 11008 39.2 -> 33.3, 256 x 6144 x 4096 14.1 -> 12.5).  One row of tiles (M = 128) stays on
        // 64x64, whose 512 workgroups keep more of W's only pass in flight (128 x 16384 x 4096: 17.6 against 20.0).
        // With 256 to 511 128x128 tiles they also win for K of 2048 to 4096 (2048^3 21.8 -> 17.6,
        // 1024 x 4096 x 4096 29.6 -> 25.3, 1536 x 3072 x 3072 29.2 -> 26.0), not for shorter or longer K
        // (1024 x 4096 x 1024 13.0 against 14.7; 2048^2 x 8192 40.6 against 47.4).
        const int64_t t64 = (M / 64) * (N / 64), t128 = (M / 128) * (N / 128);
        const bool mid_k = K >= 2048 && K <= 4096;
        if (M % 128 == 0 && (force == 1264 || (force == 0 && M >= 256 && t64 > cu_count() &&
                                               (!fits128 || t128 < 256 || (t128 < 512 && mid_k)))))
            return launch_dma<128, 64, 4, 2, 3>("qgemm_w8a8_128x64_dma", "qgemm_w8a8_128x64_dma_splitk", x, x_scale, w,
                                                w_scales, bias, act, out, acc_out, M, N, K, ldc);
        if (fits128 && (force == 128 || (force == 0 && (M / 128) * (N / 128) >= 256)))
            return launch_dma<128, 128, 2, 4, 3>("qgemm_w8a8_128x128_dma", "qgemm_w8a8_128x128_dma_splitk", x, x_scale, w,
                                                 w_scales, bias, act, out, acc_out, M, N, K, ldc);
        // at most one 64x64 tile per CU: two wave sets share each slab's k-steps (M = 256, N = K = 4096: 9.8 us
        // against 10.5; 256 x 2048 x 8192: 14.8 against 17.7).  Such a launch is bound by what one CU can pull
        // out of L2: 512 KiB of operand rows per workgroup at the 115 GB/s a lone workgroup reaches on L2 hits
        // is 4.5 us, and more stages in flight (six, eight) change nothing.
        if (force == 642 || (force == 0 && (M / 64) * (N / 64) <= cu_count())) {
            // a slab of such a tile is 64 MFMA cycles per wave: with K on the 256 grid and no split, two slabs
            // per stage and barrier (three stages of 32 KiB; M = 256, N = K = 4096: 8.6 us against 8.9)
            if (K % 256 == 0 && K >= 1024 && pick_splits((M / 64) * (N / 64), K / 128) == 1)
                return launch_dma<64, 64, 2, 2, 3, false, 2, 2>("qgemm_w8a8_64x64k2_dma", "qgemm_w8a8_64x64k2_dma_splitk", x, x_scale,
                                                                w, w_scales, bias, act, out, acc_out, M, N, K, ldc);
            return launch_dma<64, 64, 2, 2, 4, false, 2>("qgemm_w8a8_64x64k2_dma", "qgemm_w8a8_64x64k2_dma_splitk", x, x_scale, w,
                                                         w_scales, bias, act, out, acc_out, M, N, K, ldc);
        }
        return launch_dma<64, 64, 2, 2, 4>("qgemm_w8a8_64x64_dma", "qgemm_w8a8_64x64_dma_splitk", x, x_scale, w, w_scales,
                                           bias, act, out, acc_out, M, N, K, ldc);
    }
    // the same kernel for M or N off the 64 grid: edge tiles clamp their loads and guard their stores
    const bool aligned16 = ((((uintptr_t)x | (uintptr_t)w) & 15) == 0) && K % 16 == 0 && K > 0;
    if (aligned16 && vec_out && N % 4 == 0 && K < (int64_t(1) << 24)) {
        if (force == 128 || (force == 0 && ((M + 127) / 128) * ((N + 127) / 128) >= 256))
            return launch_dma<128, 128, 2, 4, 3, true>("qgemm_w8a8_128x128_dma_edge", "qgemm_w8a8_128x128_dma_edge_splitk", x,
                                                       x_scale, w, w_scales, bias, act, out, acc_out, M, N, K, ldc);
        // 128x64 tiles as on the grid, unless the last 128-row tile would be mostly padding (same box: 500 x 4096 x 4096
        // 16.5 -> 13.9 us, 520 x 4100 x 4096 35.7 -> 25.9, 900 x 3000 x 3072 22.0 -> 17.0; but M = 260: 6.9 against 8.3)
        const int64_t padded_m = (M + 127) / 128 * 128;
        if (force == 1264 || (force == 0 && M >= 256 && padded_m * 4 <= M * 5 && ((M + 63) / 64) * ((N + 63) / 64) > cu_count()))
            return launch_dma<128, 64, 4, 2, 3, true>("qgemm_w8a8_128x64_dma_edge", "qgemm_w8a8_128x64_dma_edge_splitk", x,
                                                      x_scale, w, w_scales, bias, act, out, acc_out, M, N, K, ldc);
        if (force == 642 || (force == 0 && ((M + 63) / 64) * ((N + 63) / 64) <= cu_count()))
            return launch_dma<64, 64, 2, 2, 4, true, 2>("qgemm_w8a8_64x64k2_dma_edge", "qgemm_w8a8_64x64k2_dma_edge_splitk", x,
                                                        x_scale, w, w_scales, bias, act, out, acc_out, M, N, K, ldc);
        return launch_dma<64, 64, 2, 2, 4, true>("qgemm_w8a8_64x64_dma_edge", "qgemm_w8a8_64x64_dma_edge_splitk", x, x_scale, w,
                                                 w_scales, bias, act, out, acc_out, M, N, K, ldc);
    }
    // fewer than ~3/4 of the 256 CUs busy with 128x128 tiles: quarter the tile instead
    if (aligned && M % 128 == 0 && N % 128 == 0 && (M / 128) * (N / 128) >= 192)
        return launch<128, 128, 2, 2, false>("qgemm_w8a8_128x128", x, x_scale, w, w_scales, bias,
                                             act, out, acc_out, M, N, K, ldc);
    if (aligned && M % 64 == 0 && N % 64 == 0)
        return launch<64, 64, 2, 2, false>("qgemm_w8a8_64x64", x, x_scale, w, w_scales, bias, act,
                                           out, acc_out, M, N, K, ldc);
    return launch<64, 64, 2, 2, true>("qgemm_w8a8_64x64_guarded", x, x_scale, w, w_scales, bias,
                                      act, out, acc_out, M, N, K, ldc);
}
}  // namespace

extern "C" int axhip_qgemm_w8a8(const int8_t *x, float x_scale, const int8_t *w,
                                const float *w_scales, const float *bias, int act, float *out,
                                int32_t *acc_out, int64_t M, int64_t N, int64_t K) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!x || !w) return fail(AXHIP_ERR_NULL_ARG, "qgemm_w8a8: NULL operand");
    if (!out && !acc_out) return fail(AXHIP_ERR_NULL_ARG, "qgemm_w8a8: no output buffer");
    if (out && !w_scales) return fail(AXHIP_ERR_NULL_ARG, "qgemm_w8a8: NULL w_scales");
    if (M < 0 || N < 0 || K < 0) return fail(AXHIP_ERR_SHAPE, "qgemm_w8a8: negative dimension");
    if (act < AXHIP_ACT_NONE || act > AXHIP_ACT_GELU)
        return fail(AXHIP_ERR_SHAPE, "qgemm_w8a8: unknown activation %d", act);
    if (M == 0 || N == 0) return AXHIP_OK;
    // up to four rows stream the weights on the vector ALU; from five on the tiles are ahead (M = 8, same box:
    // 4096 x 4096 10.3 against 8.1 us, 11008 x 4096 16.1 against 9.9, 32000 x 4096 36.4 against 20.2; M = 5: 9.3 against 8.1)
    if (M <= 4 && K % 16 == 0 && K > 0 && ((((uintptr_t)x | (uintptr_t)w) & 15) == 0) &&
        (N + GEMV_ROWS - 1) / GEMV_ROWS <= 0x7fffffff) {
        switch (M) {
            case 1: return launch_gemv<1>(x, x_scale, w, w_scales, bias, act, out, acc_out, N, K);
            case 2: return launch_gemv<2>(x, x_scale, w, w_scales, bias, act, out, acc_out, N, K);
            case 3: return launch_gemv<3>(x, x_scale, w, w_scales, bias, act, out, acc_out, N, K);
            default: return launch_gemv<4>(x, x_scale, w, w_scales, bias, act, out, acc_out, N, K);
        }
    }
    // K off the 128 grid would keep a large product off the direct-to-LDS kernels (8192^2 x 8200:
    // 0.85 POP/s).  Both operands are copied once into rows padded with zeros to the next multiple
    // of 128 — zeros add nothing to an integer sum — and the product runs on the copies.
    const int64_t Kp = (K + BK - 1) / BK * BK;
    if (K % BK != 0 && K >= 512 && (M / 256) * (N / 256) >= 80 && (uint64_t)(M + N) * (uint64_t)Kp <= (uint64_t(1) << 30)) {
        int8_t *xp = static_cast<int8_t *>(workspace((size_t)(M + N) * (size_t)Kp));
        if (!xp) return AXHIP_ERR_ALLOC;
        int8_t *wp = xp + M * Kp;
        const int64_t bx = (M * (Kp / 16) + 255) / 256, bw = (N * (Kp / 16) + 255) / 256;
        hipLaunchKernelGGL(k_pad_rows_i8, dim3((unsigned)(bx < 65536 ? bx : 65536)), dim3(256), 0, kStream, x, xp, M, K, Kp);
        hipLaunchKernelGGL(k_pad_rows_i8, dim3((unsigned)(bw < 65536 ? bw : 65536)), dim3(256), 0, kStream, w, wp, N, K, Kp);
        if (int rc = check_launch("qgemm_w8a8 row padding")) return rc;
        const int rc = axhip_qgemm_w8a8(xp, x_scale, wp, w_scales, bias, act, out, acc_out, M, N, Kp);
        note_kernel(strstr(axhip_last_kernel(), "fringes") ? "qgemm_w8a8_256x256_dma+fringes+k_padded"
                                                           : "qgemm_w8a8_256x256_dma+k_padded");
        return rc;
    }
    const bool fast = ((((uintptr_t)x | (uintptr_t)w) & 15) == 0) && K % BK == 0 && K > 0 && K < (int64_t(1) << 24) &&
                      N % 4 == 0 && (!out || (((uintptr_t)out | (uintptr_t)w_scales | (uintptr_t)bias) & 15) == 0) &&
                      (((uintptr_t)acc_out & 15) == 0);
    // A large shape off the 256 grid: the 256-aligned interior goes to the persistent kernel and
    // the right and bottom fringes to the smaller tiles, each block addressed inside the full
    // output through its row pitch (whole shape on 64x64 tiles: 8000^2 x 8192 at 0.93 POP/s).
    const int64_t Mi = M / 256 * 256, Ni = N / 256 * 256;
    if (fast && (Mi != M || Ni != N) && (Mi / 256) * (Ni / 256) >= 80) {
        int rc = qgemm_block(x, x_scale, w, w_scales, bias, act, out, acc_out, Mi, Ni, K, N);
        if (rc == AXHIP_OK && Ni < N)
            rc = qgemm_block(x, x_scale, w + Ni * K, w_scales ? w_scales + Ni : nullptr, bias ? bias + Ni : nullptr, act,
                             out ? out + Ni : nullptr, acc_out ? acc_out + Ni : nullptr, Mi, N - Ni, K, N);
        if (rc == AXHIP_OK && Mi < M)
            rc = qgemm_block(x + Mi * K, x_scale, w, w_scales, bias, act, out ? out + Mi * N : nullptr,
                             acc_out ? acc_out + Mi * N : nullptr, M - Mi, N, K, N);
        note_kernel("qgemm_w8a8_256x256_dma+fringes");
        return rc;
    }
    return qgemm_block(x, x_scale, w, w_scales, bias, act, out, acc_out, M, N, K, N);
}

