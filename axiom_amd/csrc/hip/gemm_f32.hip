// fp32 GEMM on the fp32 matrix cores (v_mfma_f32_32x32x2_f32), NN / NT / TN, optionally
// strided-batched, with alpha/beta, per-column scale, bias and activation fused into the
// write-back.  True fp32 multiply-accumulate throughout.
//
// One workgroup owns a BM x BN tile of C and walks K in slabs of 32.  An operand whose
// K index is contiguous in memory (A of NN/NT, B of NT) is staged as rows of 32 floats padded
// to 36, and read back with one ds_read_b128 per 8-wide k-block: lane l takes row (l & 31),
// floats [4*(l>>5), +4) of the block.  An operand whose M/N index is contiguous (B of NN, A of
// TN) is staged k-major with the row length padded by 8 floats and read with four
// ds_read_b32: lane l takes column (l & 31) of k = 4*(l>>5) + j.  Either way MFMA j of a k-block
// multiplies the k = 4*(l>>5) + j elements of both operands, so A and B always pair up.
// The pads make the 16 lanes a b128 read serves together, the two lane halves of a b32 read,
// and the staging writes all fall on distinct banks (64 banks x 4 bytes).
#include "common.h"

namespace {
using namespace axhip;

constexpr int BK = 32;
constexpr int KC_STRIDE = BK + 4;          // floats per staged row of a K-contiguous operand

struct SgemmArgs {
    const void *A, *B;
    float *C;
    int64_t M, N, K, lda, ldb, ldc;
    int64_t stride_a, stride_b, stride_c;  // elements between batch members
    float alpha, beta;
    const float *col_scale;                // multiplies column n after alpha (W8A32), or NULL
    const float *bias;
    int act;
};

// One operand's slab: R rows (M or N extent of the tile) x BK.
template <int R, bool KCONTIG, int T, bool GUARD, typename SRC>
struct Operand {
    static constexpr int STRIDE = KCONTIG ? KC_STRIDE : (R + 8);
    static constexpr int FLOATS = KCONTIG ? R * KC_STRIDE : BK * (R + 8);
    static constexpr int CHUNKS = R * BK / 4 / T;          // float4 chunks per thread
    static_assert(CHUNKS * T * 4 == R * BK, "slab must divide over the workgroup");

    v4f reg[CHUNKS];

    // element (r, k) of the logical [R, K] operand lives at src[r*ld + k] (KCONTIG) or
    // src[k*ld + r]
    __device__ __forceinline__ void fetch(const SRC *src, int64_t ld, int64_t r0, int64_t rows,
                                          int64_t k0, int64_t K, int tid) {
#pragma unroll
        for (int i = 0; i < CHUNKS; i++) {
            const int c = tid + i * T;
            int64_t r, k;
            if (KCONTIG) { r = r0 + (c >> 3); k = k0 + ((c & 7) << 2); }
            else         { k = k0 + c / (R / 4); r = r0 + ((c % (R / 4)) << 2); }
            const SRC *p = KCONTIG ? src + r * ld + k : src + k * ld + r;
            v4f v = {0.f, 0.f, 0.f, 0.f};
            if (sizeof(SRC) == 1) {                        // int8 source, K-contiguous only
                // four elements wholly inside the row: one load at whatever alignment the row has
                // (global memory takes unaligned vector loads)
                const bool whole = !GUARD || (r < rows && k + 4 <= K);
                if (whole) {
                    int w;
                    __builtin_memcpy(&w, p, 4);
                    v.x = (float)(signed char)(w & 0xff);
                    v.y = (float)(signed char)((w >> 8) & 0xff);
                    v.z = (float)(signed char)((w >> 16) & 0xff);
                    v.w = (float)(signed char)((w >> 24) & 0xff);
                } else if (r < rows) {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (k + e < K) v[e] = (float)p[e];
                }
            } else if (!GUARD) {
                v = *reinterpret_cast<const v4f *>(p);
            } else if (KCONTIG) {
                if (r < rows) {
                    if (k + 4 <= K) __builtin_memcpy(&v, p, 16);
                    else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (k + e < K) v[e] = (float)p[e];
                    }
                }
            } else {
                if (k < K) {
                    if (r + 4 <= rows) __builtin_memcpy(&v, p, 16);
                    else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (r + e < rows) v[e] = (float)p[e];
                    }
                }
            }
            reg[i] = v;
        }
    }

    __device__ __forceinline__ void stash(float *s, int tid) const {
#pragma unroll
        for (int i = 0; i < CHUNKS; i++) {
            const int c = tid + i * T;
            if (KCONTIG) *reinterpret_cast<v4f *>(s + (c >> 3) * KC_STRIDE + ((c & 7) << 2)) = reg[i];
            else *reinterpret_cast<v4f *>(s + (c / (R / 4)) * STRIDE + ((c % (R / 4)) << 2)) = reg[i];
        }
    }

    // the 4 values lane (row r, half h) feeds to MFMAs j = 0..3 of k-block kb
    __device__ __forceinline__ static v4f frag(const float *s, int r, int h, int kb) {
        if (KCONTIG) return *reinterpret_cast<const v4f *>(s + r * KC_STRIDE + kb + 4 * h);
        v4f v;
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = s[(kb + 4 * h + j) * STRIDE + r];
        return v;
    }
};

template <int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, bool GUARD, typename BSRC>
__global__ void __launch_bounds__(WAVES_M *WAVES_N * 64) k_sgemm(SgemmArgs g) {
    constexpr int T = WAVES_M * WAVES_N * 64;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(TM * 32 * WAVES_M == BM && TN * 32 * WAVES_N == BN, "wave tiling");
    using OpA = Operand<BM, A_KC, T, GUARD, float>;
    using OpB = Operand<BN, B_KC, T, GUARD, BSRC>;
    constexpr int STAGE = OpA::FLOATS + OpB::FLOATS;

    extern __shared__ __attribute__((aligned(16))) float lds_f[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int tiles_m = (int)((g.M + BM - 1) / BM), tiles_n = (int)((g.N + BN - 1) / BN);
    int tm, tn;
    int64_t batch = 0;
    if (gridDim.y == 1) tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
    else tile_of_batched_block(tiles_m, tiles_n, tm, tn, batch);
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const float *A = static_cast<const float *>(g.A) + batch * g.stride_a;
    const BSRC *B = static_cast<const BSRC *>(g.B) + batch * g.stride_b;
    float *C = g.C + batch * g.stride_c;

    OpA opa;
    OpB opb;
    const int64_t slabs = (g.K + BK - 1) / BK;
    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    opa.fetch(A, g.lda, m0, g.M, 0, g.K, tid);
    opb.fetch(B, g.ldb, n0, g.N, 0, g.K, tid);
    opa.stash(lds_f, tid);
    opb.stash(lds_f + OpA::FLOATS, tid);
    __syncthreads();

    const int frow = lane & 31, fhalf = lane >> 5;
    for (int64_t s = 0; s < slabs; s++) {
        const int cur = (int)(s & 1);
        if (s + 1 < slabs) {
            opa.fetch(A, g.lda, m0, g.M, (s + 1) * BK, g.K, tid);
            opb.fetch(B, g.ldb, n0, g.N, (s + 1) * BK, g.K, tid);
        }
        const float *sa = lds_f + cur * STAGE;
        const float *sb = sa + OpA::FLOATS;
#pragma unroll
        for (int kb = 0; kb < BK; kb += 8) {
            v4f fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) fa[i] = OpA::frag(sa, wm * WTM + i * 32 + frow, fhalf, kb);
#pragma unroll
            for (int j = 0; j < TN; j++) fb[j] = OpB::frag(sb, wn * WTN + j * 32 + frow, fhalf, kb);
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][e], fb[j][e],
                                                                         acc[i][j], 0, 0, 0);
        }
        if (s + 1 < slabs) {
            float *na = lds_f + (cur ^ 1) * STAGE;
            opa.stash(na, tid);
            opb.stash(na + OpA::FLOATS, tid);
        }
        __syncthreads();
    }

    // accumulator register v of lane l: row (v&3) + 8*(v>>2) + 4*(l>>5), column (l & 31)
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int64_t col = n0 + wn * WTN + j * 32 + frow;
        const bool col_ok = !GUARD || col < g.N;
        float cs = 1.0f, bv = 0.0f;
        if (col_ok) {
            if (g.col_scale) cs = g.col_scale[col];
            if (g.bias) bv = g.bias[col];
        }
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int64_t row = m0 + wm * WTM + i * 32 + (v & 3) + 8 * (v >> 2) + 4 * fhalf;
                if (GUARD && (row >= g.M || !col_ok)) continue;
                float r = acc[i][j][v];
                if (g.alpha != 1.0f) r *= g.alpha;
                if (g.col_scale) r *= cs;
                float *cp = C + row * g.ldc + col;
                if (g.beta != 0.0f) r += g.beta * *cp;
                if (g.bias) r += bv;
                *cp = apply_act(r, g.act);
            }
        }
    }
}

template <int BM, int BN, bool A_KC, bool B_KC, bool GUARD, typename BSRC>
int launch(const char *name, const SgemmArgs &g, int64_t batch) {
    auto kern = k_sgemm<BM, BN, 2, 2, A_KC, B_KC, GUARD, BSRC>;
    using OpA = Operand<BM, A_KC, 256, GUARD, float>;
    using OpB = Operand<BN, B_KC, 256, GUARD, BSRC>;
    constexpr int smem = 2 * (OpA::FLOATS + OpB::FLOATS) * (int)sizeof(float);
    static bool attr_set = false;
    if (!attr_set) {
        AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, smem),
                      "hipFuncSetAttribute");
        attr_set = true;
    }
    const int64_t tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
    if (tiles > 0x7fffffff || batch > 65535)
        return fail(AXHIP_ERR_SHAPE, "sgemm: grid too large (tiles=%lld batch=%lld)",
                    (long long)tiles, (long long)batch);
    note_kernel(name);
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles, (unsigned)batch), dim3(256), smem, kStream, g);
    return check_launch(name);
}

template <bool A_KC, bool B_KC, typename BSRC>
int pick_tile(const char *const names[3], const SgemmArgs &g, int64_t batch) {
    const int esz_b = (int)sizeof(BSRC);
    bool aligned = (g.K % BK == 0) && g.K > 0 && ((uintptr_t)g.A % 16 == 0) &&
                   ((uintptr_t)g.B % (esz_b == 1 ? 4 : 16) == 0) && (g.lda % 4 == 0) &&
                   (g.ldb % 4 == 0) && (g.stride_a % 4 == 0) && (g.stride_b % 4 == 0);
    if (aligned && g.M % 128 == 0 && g.N % 128 == 0 && (g.M / 128) * (g.N / 128) * batch >= 192)
        return launch<128, 128, A_KC, B_KC, false, BSRC>(names[0], g, batch);
    if (aligned && g.M % 64 == 0 && g.N % 64 == 0)
        return launch<64, 64, A_KC, B_KC, false, BSRC>(names[1], g, batch);
    return launch<64, 64, A_KC, B_KC, true, BSRC>(names[2], g, batch);
}

int validate(const char *who, int transa, int transb, int64_t M, int64_t N, int64_t K,
             const void *A, int64_t lda, const void *B, int64_t ldb, const void *C, int64_t ldc,
             int act) {
    if (!A || !B || !C) return fail(AXHIP_ERR_NULL_ARG, "%s: NULL matrix", who);
    if (M < 0 || N < 0 || K < 0) return fail(AXHIP_ERR_SHAPE, "%s: negative dimension", who);
    if ((transa & ~1) || (transb & ~1)) return fail(AXHIP_ERR_SHAPE, "%s: trans flag must be 0/1", who);
    if (lda < (transa ? M : K) || ldb < (transb ? K : N) || ldc < N)
        return fail(AXHIP_ERR_SHAPE, "%s: leading dimension smaller than the row length", who);
    if (act < AXHIP_ACT_NONE || act > AXHIP_ACT_GELU)
        return fail(AXHIP_ERR_SHAPE, "%s: unknown activation %d", who, act);
    return AXHIP_OK;
}


// =====================================================================================
// Fast path for aligned shapes: direct-to-LDS loads and an inner loop with no vector-ALU
// instruction other than the MFMAs (a VALU instruction issued on a SIMD that is streaming MFMAs
// costs about one MFMA slot, so address arithmetic in the loop serialises with the matrix core).
//
// K slabs of 32 floats, two to four LDS stages.  An operand whose K index is contiguous in memory is
// staged as rows of 128 bytes (one full cache line per row per slab); a wave's load
// instruction fills 1 KiB = 8 rows, lane l -> row (l>>3), physical 16-byte chunk (l&7), and
// fetches logical chunk (l&7) ^ ((row>>1)&7): the bank swizzle is applied on the global side.
// A fragment read is one ds_read_b128 (4 consecutive k).  An operand whose M/N index is
// contiguous is staged k-row by k-row: one load instruction carries RPI = 256/R k-rows of R
// floats (1 KiB), groups are spaced 1024 + 32*RPI bytes apart so that the two lane halves of a
// fragment read (k and k+4) land 128 bytes apart modulo 256 and never share a bank; a fragment
// is four ds_read_b32.  Global addresses are a scalar base (advanced by scalar adds) plus a
// per-lane byte offset computed once; LDS addresses are per-lane constants plus immediates.
// The MFMA takes the B fragment first, so a lane owns four consecutive n of one row m and the
// write-back moves 16 bytes per lane.
#define AXF_LGKM(n) __builtin_amdgcn_s_waitcnt(0x3F | (3 << 14) | (7 << 4) | (((n) > 15 ? 15 : (n)) << 8))
#define AXF_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))
// the same for an operand that is read once and is too large to be met again in the caches (non-temporal)
#define AXF_LOAD_LDS_NT(m0val, voff, base)                                                    \
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(m0val), \
                 "v"(voff), "s"(base)                                                         \
                 : "memory")
#define AXF_LOAD_LDS(m0val, voff, base)                                                       \
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0val), \
                 "v"(voff), "s"(base)                                                         \
                 : "memory")

template <int R, bool KC, int NW>
struct DmaOperand {
    static constexpr int RPI = KC ? 0 : 256 / R;                       // k-rows per load instruction
    static constexpr int PITCH = KC ? 1024 : 1024 + 32 * (256 / R);    // LDS bytes per load instruction
    static constexpr int NINSTR = KC ? R / 8 : 32 / (256 / R);         // load instructions per slab
    static constexpr int IPW = NINSTR / NW;                            // ... per wave
    static constexpr int BYTES = NINSTR * PITCH;                       // one stage
    static constexpr int READS = KC ? 1 : 4;                           // ds_reads per 32-wide tile per k-block
    static_assert(IPW * NW == NINSTR && IPW >= 1, "slab must divide over the waves");

    // byte offset, from the operand's slab origin, of what lane `lane` of instruction q fetches.
    // `valid` (<= R; a multiple of 4 for an M/N-contiguous operand) is how many of the tile's R
    // rows / columns exist: a lane whose row or 4-column group lies past them fetches the last
    // existing one instead, into its own LDS place (swizzle of the nominal row).
    __device__ static unsigned lane_offset(int q, int lane, int64_t ld, int valid = R) {
        if (KC) {
            const int row = q * 8 + (lane >> 3);
            return (unsigned)((row < valid ? row : valid - 1) * ld * 4 + (((lane & 7) ^ ((row >> 1) & 7)) << 4));
        }
        constexpr int LPR = 64 / (256 / R);                            // lanes per k-row
        const int chunk = lane % LPR;
        return (unsigned)((q * (256 / R) + lane / LPR) * ld * 4 + (chunk * 4 < valid ? chunk : valid / 4 - 1) * 16);
    }
    // LDS byte address (within a stage) a lane reads its fragments from, for k-block index kbi
    // (KC) or for all k-blocks (MC, kbi ignored); `first` = first row/column of the wave's tile
    __device__ static unsigned frag_base(int first, int frow, int fhalf, int kbi) {
        if (KC) return (unsigned)((first + frow) * 128 + (((kbi * 2 + fhalf) ^ ((frow >> 1) & 7)) << 4));
        return (unsigned)(fhalf * (4 / (256 / R)) * PITCH + (first + frow) * 4);
    }
    // immediate offset of k = kbi*8 + j (MC only)
    static constexpr int k_imm(int k) { return KC ? 0 : (k / (256 / R)) * PITCH + (k % (256 / R)) * R * 4; }
};

// An int8 operand stored [rows, K] (K contiguous; the weights of the W8A32 product): a slab is 32 bytes
// per row, one load instruction carries 32 rows (lane l -> row l >> 1, 16-byte half l & 1), and only the
// first NINSTR waves have one to issue.  A fragment is one ds_read_b64 per pair of k-blocks — the lane's
// eight consecutive k values, which is exactly one bf16 MFMA operand — converted to bf16 in registers right
// before use (bf16_of_i8 below), so LDS and the loads carry a quarter of the bytes of an fp32 operand; the
// fp32 operand is read to match (two 16-byte chunks side by side).  Reading the eight bytes at once instead
// of four per k-block halves the LDS instructions of this operand: 4096^3 342 -> 331 us, 1024 x 4096 x 4096
// 104.6 -> 96.8.  (Rows 32 bytes apart put the 32 lanes of a read on 8 banks: a 4-way conflict.)
template <int R, int NW>
struct DmaOperandI8 {
    static constexpr int PITCH = 1024;
    static constexpr int NINSTR = R / 32;
    static constexpr int IPW = (NINSTR + NW - 1) / NW;
    static constexpr int BYTES = NINSTR * PITCH;
    static constexpr int READS = 1;
    static_assert(R % 32 == 0, "whole load instructions");
    __device__ static unsigned lane_offset(int q, int lane, int64_t ld, int valid = R) {
        const int row = q * 32 + (lane >> 1);
        return (unsigned)((row < valid ? row : valid - 1) * ld + (lane & 1) * 16);
    }
    // a lane's 8 bytes of the pair of k-blocks kbi belongs to: k = 16 (kbi / 2) + 8 fhalf ..
    __device__ static unsigned frag_base(int first, int frow, int fhalf, int kbi) {
        return (unsigned)((first + frow) * 32 + (kbi >> 1) * 16 + fhalf * 8);
    }
    static constexpr int k_imm(int) { return 0; }
};

struct FragI8 {
    int2 raw;      // the lane's 8 consecutive k values of a pair of k-blocks (16 k): k = 8 * (lane >> 5) + byte index; held in
                   // the even k-block's buffer, the odd one's stays unused
    __device__ __forceinline__ float get(int e) const { return (float)(signed char)(raw.x >> (8 * e)); }   // fp32 form, unused by the bf16 products
};

// fp32 x int8 products on the bf16 matrix core, with fp32 accuracy.  Every int8 value is a bf16 exactly.  An fp32
// value a is cut into three bf16 terms: hi = a with its low 16 bits cleared, mid = (a - hi) with its low 16 bits
// cleared, lo = a - hi - mid; both subtractions are exact and lo has at most 8 significant bits, so
// a = hi + mid + lo exactly, every term times an int8 value is exact in fp32, and only the accumulation rounds —
// as in the fp32 product, at a sixteenth of its matrix-core time per term.  An infinite a keeps hi = a and
// mid = lo = 0 (a - hi would be NaN), so infinities and NaNs come out as the fp32 product gives them.
// Cost per fp32 value: and, subtract, median (the NaN filter), and, subtract, and half of each of three packs:
// 6.5 vector instructions; per int8 value one conversion and half a pack.
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
struct Bf16x3 {
    v4i hi, mid, lo;     // 8 k values each: a k-block's four, then the next k-block's four
};
__device__ __forceinline__ unsigned top_halves(unsigned second, unsigned first) {   // bf16 of two fp32, by truncation
    return __builtin_amdgcn_perm(second, first, 0x07060302);
}
__device__ __forceinline__ Bf16x3 bf16x3_of(const v4f &p, const v4f &q) {
    unsigned h[8], m[8], l[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float a = e < 4 ? p[e] : q[e - 4];
        h[e] = __float_as_uint(a);
        // a NaN whose payload sits in the low 16 bits only would be cut to an infinity: give it a quiet bit the cut keeps
        if ((h[e] & 0x7fffffffu) > 0x7f800000u) h[e] |= 0x00400000u;
        float r = a - __uint_as_float(h[e] & 0xffff0000u);
        r = __builtin_amdgcn_fmed3f(r, r, 0.0f);     // NaN (a infinite or NaN) -> 0, anything else unchanged
        m[e] = __float_as_uint(r);
        l[e] = __float_as_uint(r - __uint_as_float(m[e] & 0xffff0000u));
    }
    Bf16x3 o;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        o.hi[e] = (int)top_halves(h[2 * e + 1], h[2 * e]);
        o.mid[e] = (int)top_halves(m[2 * e + 1], m[2 * e]);
        o.lo[e] = (int)top_halves(l[2 * e + 1], l[2 * e]);
    }
    return o;
}
__device__ __forceinline__ v4i bf16_of_i8(int first, int second) {   // two k-blocks of four int8 -> 8 bf16
    unsigned f[8];
#pragma unroll
    for (int e = 0; e < 8; e++) f[e] = __float_as_uint((float)(signed char)((e < 4 ? first : second) >> (8 * (e & 3))));
    v4i o;
#pragma unroll
    for (int e = 0; e < 4; e++) o[e] = (int)top_halves(f[2 * e + 1], f[2 * e]);
    return o;
}

template <bool KC> struct Frag;
template <> struct Frag<true> {
    v4f q;
    __device__ __forceinline__ float get(int j) const { return q[j]; }
};
template <> struct Frag<false> {
    float s0, s1, s2, s3;
    __device__ __forceinline__ float get(int j) const { return j == 0 ? s0 : j == 1 ? s1 : j == 2 ? s2 : s3; }
};

#define AXF_DS128(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off))
#define AXF_DS32(dst, addr, off) asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off))
#define AXF_DS64(dst, addr, off) asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off))

// EDGE: M and N need not be multiples of the tile (N a multiple of 4, and M too when A is stored
// M-contiguous) nor K of the slab (K a multiple of 4).  Edge tiles fetch the last existing row /
// column group in place of the missing ones — their products land in outputs that are not stored —
// and guard the write-back; in the last slab, lanes whose k values lie past K write zeros to
// their LDS place instead of loading, in both operands, so the tail adds exact zeros.
template <int BM, int BN, int WAVES_M, int WAVES_N, int NST, bool A_KC, bool B_KC, int EPI, int WAVES_K,
          bool EDGE = false, typename BSRC = float, int SPS = 1, bool STREAM_B = false>
__global__ void __launch_bounds__(WAVES_M *WAVES_N *WAVES_K * 64) k_sgemm_dma(SgemmArgs g) {
    // STREAM_B: B is read once and is large, its loads are non-temporal (a template parameter: a run-time test in
    // front of every load costs the tiles that do not stream 3-11 %)
    // SPS == 2: a stage holds two slabs (64 k) and the loop's barrier comes once per stage — for tiles whose slab is
    // only a few MFMAs per wave, where the barrier is a visible share of the slab (K a multiple of 64, no edge form)
    // WAVES_K == 2: a second set of waves shares each tile; set 0 multiplies k-blocks 0 and 1 of
    // every slab, set 1 k-blocks 2 and 3, and the two accumulators are added through LDS at the
    // end.  For 64x64 tiles with one workgroup per CU this puts two waves on every SIMD, so one
    // wave's LDS and barrier waits are covered by the other's MFMAs.
    constexpr int NW = WAVES_M * WAVES_N * WAVES_K;
    static_assert(WAVES_K == 1 || WAVES_K == 2, "k split");
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N, TM = WTM / 32, TN = WTN / 32;
    constexpr bool B_I8 = sizeof(BSRC) == 1;     // int8 B, [N, K]: W8A32 (K a multiple of 32, so no K tail)
    static_assert(!B_I8 || (B_KC && EPI == 1), "int8 B is K-contiguous, turned write-back");
    using OA = DmaOperand<BM, A_KC, NW>;
    using OB = typename std::conditional<B_I8, DmaOperandI8<BN, NW>, DmaOperand<BN, B_KC, NW>>::type;
    // LDS: NST stages of A, then NST stages of B
    static_assert(SPS == 1 || (SPS == 2 && !EDGE), "two slabs per stage: whole tiles");
    constexpr int A_STAGE = SPS * OA::BYTES, B_STAGE = SPS * OB::BYTES;
    constexpr int B_BASE = NST * A_STAGE;
    constexpr int NREADS = TM * OA::READS + TN * OB::READS;
    constexpr int NREADS_PAIR = 2 * TM * OA::READS + TN;      // int8 B: LDS reads of a pair of k-blocks (B once per pair)
    // loads a wave may leave in flight at the end of a slab: everything but the next slab's
    // int8 B with four stages: the fragments of slab s + 1 are read while slab s is converted and multiplied, so the
    // loop's barrier must already cover slab s + 2 and one stage less is in flight
    constexpr bool PIPE = B_I8 && NST == 4;
    static_assert(!PIPE || SPS == 1, "fragments read a slab ahead: one slab per stage");
    // the wait counts below assume every wave that loads the int8 operand issues the same number of its instructions
    static_assert(!B_I8 || OB::NINSTR % NW == 0 || OB::NINSTR < NW, "int8 load instructions per wave");
    constexpr int VM_KEEP = (NST - (PIPE ? 3 : 2)) * SPS * (OA::IPW + OB::IPW);
    static_assert(NST >= 2 && NST <= 4 && VM_KEEP < 64, "stage count");
    static_assert(B_BASE + NST * B_STAGE <= 160 * 1024, "LDS budget");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = wave / (WAVES_M * WAVES_N), wmn = wave % (WAVES_M * WAVES_N);
    const int wm = wmn / WAVES_N, wn = wmn % WAVES_N;
    int tm, tn;
    int64_t batch = 0;
    if (gridDim.y == 1) tile_of_block(blockIdx.x, (int)((g.M + BM - 1) / BM), (int)((g.N + BN - 1) / BN), tm, tn);
    else tile_of_batched_block((int)((g.M + BM - 1) / BM), (int)((g.N + BN - 1) / BN), tm, tn, batch);
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const int mvalid = EDGE && g.M - m0 < BM ? (int)(g.M - m0) : BM, nvalid = EDGE && g.N - n0 < BN ? (int)(g.N - n0) : BN;
    const float *A = static_cast<const float *>(g.A) + batch * g.stride_a;
    const BSRC *B = static_cast<const BSRC *>(g.B) + batch * g.stride_b;
    float *C = g.C + batch * g.stride_c;
    // EDGE also takes a K that ends inside a slab (K a multiple of 4): the last slab's lanes whose four
    // k values lie past K load nothing and write zeros to their LDS place instead
    const int slabs = EDGE ? (int)((g.K + 31) / 32) : (int)(g.K / (32 * SPS));   // stages to walk
    const int ktail = EDGE ? (int)(g.K - (int64_t)(slabs - 1) * 32) : 32;     // k values in the last slab
    int left = slabs;                                                          // slabs not yet requested

    // ---- global -> LDS ----
    unsigned va[OA::IPW], vb[OB::IPW];
#pragma unroll
    for (int j = 0; j < OA::IPW; j++) va[j] = OA::lane_offset(j * NW + wave, lane, g.lda, mvalid);
#pragma unroll
    for (int j = 0; j < OB::IPW; j++) vb[j] = OB::lane_offset(j * NW + wave, lane, g.ldb, nvalid);
    const char *ga = reinterpret_cast<const char *>(A_KC ? A + m0 * g.lda : A + m0);
    const char *gb = reinterpret_cast<const char *>(B_KC ? B + n0 * g.ldb : B + n0);
    const int64_t step_a = A_KC ? 128 : 128 * g.lda, step_b = B_KC ? 32 * (int64_t)sizeof(BSRC) : 128 * g.ldb;   // bytes per slab
    const unsigned lds0 = (unsigned)(uintptr_t)lds_raw;
    const unsigned dma_a = lds0 + wave * OA::PITCH, dma_b = lds0 + wave * OB::PITCH;
    // does this lane's 16 bytes of load instruction j lie inside K in the last slab
    bool ta[OA::IPW], tb[OB::IPW];
#pragma unroll
    for (int j = 0; j < OA::IPW; j++) {
        const int q = j * NW + wave, row = q * 8 + (lane >> 3);
        ta[j] = A_KC ? (((lane & 7) ^ ((row >> 1) & 7)) * 4 < ktail) : (q * (256 / BM) + lane / (64 / (256 / BM)) < ktail);
    }
#pragma unroll
    for (int j = 0; j < OB::IPW; j++) {
        const int q = j * NW + wave, row = q * 8 + (lane >> 3);
        tb[j] = B_I8 ? true
                : B_KC ? (((lane & 7) ^ ((row >> 1) & 7)) * 4 < ktail) : (q * (256 / BN) + lane / (64 / (256 / BN)) < ktail);
    }

    // ---- LDS -> fragments ----
    const int frow = lane & 31, fhalf = lane >> 5;
    unsigned ra[NST][4], rb[NST][4];    // [stage][k-block]: the stage base does not fit a 16-bit immediate
#pragma unroll
    for (int st = 0; st < NST; st++)
#pragma unroll
        for (int kbi = 0; kbi < 4; kbi++) {
            // with a k split, entries 0 and 1 address this wave set's own two k-blocks
            const int kb = WAVES_K == 2 ? 2 * wk + (kbi & 1) : kbi;
            // with int8 B a lane holds 8 consecutive k of a pair of k-blocks (as its 8 weight bytes lie): the fragment of
            // k-block 2 P + j is the 16-byte chunk 4 P + 2 fhalf + j of the row
            ra[st][kbi] = lds0 + st * A_STAGE + (B_I8 ? OA::frag_base(wm * WTM, frow, kb & 1, (kb & ~1) + fhalf)
                                                      : OA::frag_base(wm * WTM, frow, fhalf, kb)) +
                          (WAVES_K == 2 && !A_KC ? wk * OA::k_imm(16) : 0);
            rb[st][kbi] = lds0 + B_BASE + st * B_STAGE + OB::frag_base(wn * WTN, frow, fhalf, kb) +
                          (WAVES_K == 2 && !B_KC ? wk * OB::k_imm(16) : 0);
        }

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    Frag<A_KC> fa[PIPE ? 8 : B_I8 ? 4 : 2][TM];
    typename std::conditional<B_I8, FragI8, Frag<B_KC>>::type fb[PIPE ? 8 : B_I8 ? 4 : 2][TN];

// loads of the next unread slab into stage ST
#define AXF_ISSUE(ST)                                                                            \
    do {                                                                                         \
        --left;                                                                                  \
        if (EDGE && left == 0 && ktail < 32) {                                                   \
            _Pragma("unroll") for (int j = 0; j < OA::IPW; j++) {                                \
                const unsigned at = wave * OA::PITCH + (ST) * A_STAGE + j * NW * OA::PITCH;      \
                if (ta[j]) AXF_LOAD_LDS(lds0 + at, va[j], ga);                                   \
                else *reinterpret_cast<v4f *>(lds_raw + at + lane * 16) = v4f{0.f, 0.f, 0.f, 0.f}; \
            }                                                                                    \
            _Pragma("unroll") for (int j = 0; j < OB::IPW; j++) {                                \
                const unsigned at = B_BASE + wave * OB::PITCH + (ST) * B_STAGE + j * NW * OB::PITCH; \
                if (!tb[j]) *reinterpret_cast<v4f *>(lds_raw + at + lane * 16) = v4f{0.f, 0.f, 0.f, 0.f}; \
                else if (STREAM_B) AXF_LOAD_LDS_NT(lds0 + at, vb[j], gb);                      \
                else AXF_LOAD_LDS(lds0 + at, vb[j], gb);                                         \
            }                                                                                    \
        } else {                                                                                 \
            _Pragma("unroll") for (int u = 0; u < SPS; u++) {                                    \
                _Pragma("unroll") for (int j = 0; j < OA::IPW; j++)                              \
                    AXF_LOAD_LDS(dma_a + (ST) * A_STAGE + u * OA::BYTES + j * NW * OA::PITCH, va[j], ga + u * step_a); \
                _Pragma("unroll") for (int j = 0; j < OB::IPW; j++)                              \
                    if (!B_I8 || j * NW + wave < OB::NINSTR) {                                   \
                        if (STREAM_B) AXF_LOAD_LDS_NT(dma_b + B_BASE + (ST) * B_STAGE + u * OB::BYTES + j * NW * OB::PITCH, vb[j], gb + u * step_b); \
                        else AXF_LOAD_LDS(dma_b + B_BASE + (ST) * B_STAGE + u * OB::BYTES + j * NW * OB::PITCH, vb[j], gb + u * step_b); \
                    }                                                                            \
            }                                                                                    \
        }                                                                                        \
        ga += SPS * step_a;                                                                      \
        gb += SPS * step_b;                                                                      \
    } while (0)

// fragments of k-block KBI of stage ST
#define AXF_FRAGS(BUF, ST, KBI, U)                                                               \
    do {                                                                                         \
        _Pragma("unroll") for (int t = 0; t < TM; t++) {                                         \
            if constexpr (A_KC) {                                                                \
                AXF_DS128(fa[BUF][t].q, ra[ST][KBI], t * 4096 + (U) * OA::BYTES);                \
            } else {                                                                             \
                AXF_DS32(fa[BUF][t].s0, ra[ST][0], OA::k_imm((KBI) * 8 + 0) + t * 128 + (U) * OA::BYTES); \
                AXF_DS32(fa[BUF][t].s1, ra[ST][0], OA::k_imm((KBI) * 8 + 1) + t * 128 + (U) * OA::BYTES); \
                AXF_DS32(fa[BUF][t].s2, ra[ST][0], OA::k_imm((KBI) * 8 + 2) + t * 128 + (U) * OA::BYTES); \
                AXF_DS32(fa[BUF][t].s3, ra[ST][0], OA::k_imm((KBI) * 8 + 3) + t * 128 + (U) * OA::BYTES); \
            }                                                                                    \
        }                                                                                        \
        _Pragma("unroll") for (int t = 0; t < TN; t++) {                                         \
            if constexpr (B_I8) {                                                                \
                if ((KBI) % 2 == 0) AXF_DS64(fb[BUF][t].raw, rb[ST][KBI], t * 1024 + (U) * OB::BYTES); \
            } else if constexpr (B_KC) {                                                         \
                AXF_DS128(fb[BUF][t].q, rb[ST][KBI], t * 4096 + (U) * OB::BYTES);                \
            } else {                                                                             \
                AXF_DS32(fb[BUF][t].s0, rb[ST][0], OB::k_imm((KBI) * 8 + 0) + t * 128 + (U) * OB::BYTES); \
                AXF_DS32(fb[BUF][t].s1, rb[ST][0], OB::k_imm((KBI) * 8 + 1) + t * 128 + (U) * OB::BYTES); \
                AXF_DS32(fb[BUF][t].s2, rb[ST][0], OB::k_imm((KBI) * 8 + 2) + t * 128 + (U) * OB::BYTES); \
                AXF_DS32(fb[BUF][t].s3, rb[ST][0], OB::k_imm((KBI) * 8 + 3) + t * 128 + (U) * OB::BYTES); \
            }                                                                                    \
        }                                                                                        \
    } while (0)

#define AXF_MFMAS(BUF)                                                                           \
    do {                                                                                         \
        __builtin_amdgcn_sched_barrier(0);                                                       \
        _Pragma("unroll") for (int e = 0; e < 4; e++)                                            \
            _Pragma("unroll") for (int i = 0; i < TM; i++)                                       \
                _Pragma("unroll") for (int j = 0; j < TN; j++)                                   \
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[BUF][j].get(e),          \
                                                                     fa[BUF][i].get(e), acc[i][j], 0, 0, 0); \
        __builtin_amdgcn_sched_barrier(0);                                                       \
    } while (0)

// int8 B: the k-blocks in fragment buffers B0 and B1 (16 k values) as three bf16 products per 32x32 tile.  All
// conversions come first, so that the products issue back to back (a conversion between two products that add
// into the same accumulator costs the pair its hand-over); the small terms are added first.
#define AXF_PAIR(B0, B1)                                                                         \
    do {                                                                                         \
        __builtin_amdgcn_sched_barrier(0);                                                       \
        Bf16x3 ax[TM];                                                                           \
        v4i bx[TN];                                                                              \
        _Pragma("unroll") for (int i = 0; i < TM; i++) ax[i] = bf16x3_of(fa[B0][i].q, fa[B1][i].q); \
        _Pragma("unroll") for (int j = 0; j < TN; j++) bx[j] = bf16_of_i8(fb[B0][j].raw.x, fb[B0][j].raw.y); \
        __builtin_amdgcn_sched_barrier(0);                                                       \
        _Pragma("unroll") for (int t = 0; t < 3; t++)                                            \
            _Pragma("unroll") for (int i = 0; i < TM; i++)                                       \
                _Pragma("unroll") for (int j = 0; j < TN; j++)                                   \
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(                         \
                        __builtin_bit_cast(v8bf, bx[j]),                                         \
                        __builtin_bit_cast(v8bf, t == 0 ? ax[i].lo : t == 1 ? ax[i].mid : ax[i].hi), acc[i][j], 0, 0, 0); \
        __builtin_amdgcn_sched_barrier(0);                                                       \
    } while (0)

// one slab out of stage ST; `more`: slab s+NST-1 exists and is fetched into the stage read last
#define AXF_SLAB(ST, more, next)                                                                 \
    do {                                                                                         \
        if (more) AXF_ISSUE(((ST) + NST - 1) % NST);                                             \
        if constexpr (PIPE) {                                                                    \
            /* this slab's fragments are in buffers 4 (ST & 1) ..., read a slab ago */            \
            constexpr int C0 = 4 * ((ST) & 1), N0 = 4 - C0, NS = ((ST) + 1) % NST;               \
            if (next) {                                                                          \
                AXF_FRAGS(N0, NS, 0, 0);                                                         \
                AXF_FRAGS(N0 + 1, NS, 1, 0);                                                     \
                if constexpr (WAVES_K == 1) {                                                    \
                    AXF_FRAGS(N0 + 2, NS, 2, 0);                                                 \
                    AXF_FRAGS(N0 + 3, NS, 3, 0);                                                 \
                }                                                                                \
                AXF_LGKM((WAVES_K == 1 ? 2 : 1) * NREADS_PAIR);                                  \
            } else AXF_LGKM(0);                                                                  \
            AXF_PAIR(C0, C0 + 1);                                                                \
            if constexpr (WAVES_K == 1) AXF_PAIR(C0 + 2, C0 + 3);                                \
        } else if constexpr (B_I8) {                                                             \
            _Pragma("unroll") for (int u = 0; u < SPS; u++) {                                    \
                AXF_FRAGS(0, ST, 0, u);                                                          \
                AXF_FRAGS(1, ST, 1, u);                                                          \
                if constexpr (WAVES_K == 1) {                                                    \
                    AXF_FRAGS(2, ST, 2, u);                                                      \
                    AXF_FRAGS(3, ST, 3, u);                                                      \
                    AXF_LGKM(NREADS_PAIR);                                                       \
                    AXF_PAIR(0, 1);                                                              \
                    AXF_LGKM(0);                                                                 \
                    AXF_PAIR(2, 3);                                                              \
                } else {                                                                         \
                    AXF_LGKM(0);                                                                 \
                    AXF_PAIR(0, 1);                                                              \
                }                                                                                \
            }                                                                                    \
        } else {                                                                                 \
            _Pragma("unroll") for (int u = 0; u < SPS; u++) {                                    \
                AXF_FRAGS(0, ST, 0, u);                                                          \
                AXF_FRAGS(1, ST, 1, u);                                                          \
                AXF_LGKM(NREADS);                                                                \
                AXF_MFMAS(0);                                                                    \
                if constexpr (WAVES_K == 1) {                                                    \
                    AXF_FRAGS(0, ST, 2, u);                                                      \
                    AXF_LGKM(NREADS);                                                            \
                    AXF_MFMAS(1);                                                                \
                    AXF_FRAGS(1, ST, 3, u);                                                      \
                    AXF_LGKM(NREADS);                                                            \
                    AXF_MFMAS(0);                                                                \
                }                                                                                \
                AXF_LGKM(0);                                                                     \
                AXF_MFMAS(1);                                                                    \
            }                                                                                    \
        }                                                                                        \
        if (VM_KEEP > 0 && (more)) {                                                             \
            /* a wave past the int8 operand's load instructions has only A's in flight */        \
            if (B_I8 && wave >= OB::NINSTR) AXF_VM((NST - (PIPE ? 3 : 2)) * SPS * OA::IPW); else AXF_VM(VM_KEEP); \
        } else AXF_VM(0);                                                                        \
        __builtin_amdgcn_s_barrier();                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                       \
    } while (0)

    // When K is exactly NST slabs the whole of it fits the stages: everything is fetched at once
    // (one load latency per tile instead of two) and the loop issues nothing.
    const bool ring = slabs != NST;
    AXF_ISSUE(0);
    if constexpr (NST > 2) { if (slabs > 1) AXF_ISSUE(1); }
    if constexpr (NST > 3) { if (slabs > 2) AXF_ISSUE(2); }
    if (!ring) AXF_ISSUE(NST - 1);
    AXF_VM(0);
    if constexpr (EDGE) AXF_LGKM(0);             // zeros written for a K tail that is already in the first slabs
    __builtin_amdgcn_s_barrier();
    if constexpr (PIPE) {
        AXF_FRAGS(0, 0, 0, 0);
        AXF_FRAGS(1, 0, 1, 0);
        if constexpr (WAVES_K == 1) {
            AXF_FRAGS(2, 0, 2, 0);
            AXF_FRAGS(3, 0, 3, 0);
        }
    }
    // whole rounds of the ring in a loop with one way out, then the slabs % NST that remain (nothing is
    // left to fetch by then): an exit between two slabs of the loop body makes the compiler copy the
    // accumulators from one register set to another every round
    int s = 0;
    for (; s + NST <= slabs; s += NST) {
        AXF_SLAB(0, ring && s + NST - 1 < slabs, s + 1 < slabs);
        AXF_SLAB(1, s + NST < slabs, s + 2 < slabs);
        if constexpr (NST > 2) AXF_SLAB(2, s + NST + 1 < slabs, s + 3 < slabs);
        if constexpr (NST > 3) AXF_SLAB(3, s + NST + 2 < slabs, s + 4 < slabs);
    }
    if (s < slabs) AXF_SLAB(0, false, s + 1 < slabs);
    if (s + 1 < slabs) AXF_SLAB(1, false, s + 2 < slabs);
    if constexpr (NST > 3) { if (s + 2 < slabs) AXF_SLAB(2, false, false); }
#undef AXF_ISSUE
#undef AXF_FRAGS
#undef AXF_MFMAS
#undef AXF_PAIR
#undef AXF_SLAB

    if constexpr (WAVES_K == 2) {
        // 4 KiB per 32x32 sub-tile, a wave's sub-tiles side by side (the stages are dead now)
        float *sum = reinterpret_cast<float *>(lds_raw + wmn * (TM * TN * 4096));
        if (wk == 1) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++)
                        *reinterpret_cast<v4f *>(sum + (i * TN + j) * 1024 + (q * 64 + lane) * 4) =
                            v4f{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
        }
        __syncthreads();
        if (wk == 1) return;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const v4f t = *reinterpret_cast<const v4f *>(sum + (i * TN + j) * 1024 + (q * 64 + lane) * 4);
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[i][j][4 * q + e] += t[e];
                }
    }

    // register v of lane l: m = i*32 + (l&31), n = j*32 + 8*(v>>2) + 4*(l>>5) + (v&3)
    const bool use_beta = g.beta != 0.0f;
    if constexpr (EPI == 0) {
        const int64_t row0 = m0 + wm * WTM + frow, col0 = n0 + wn * WTN + 4 * fhalf;
        float *dst = C + row0 * g.ldc + col0;
        const float *bp = g.bias ? g.bias + col0 : nullptr;
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int gq = 0; gq < 4; gq++) {
                v4f bv = {0.f, 0.f, 0.f, 0.f};
                if (bp) bv = *reinterpret_cast<const v4f *>(bp + j * 32 + 8 * gq);
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    float *cp = dst + (int64_t)i * 32 * g.ldc + j * 32 + 8 * gq;
                    v4f r;
#pragma unroll
                    for (int e = 0; e < 4; e++) r[e] = acc[i][j][4 * gq + e];
                    if (g.alpha != 1.0f) r *= g.alpha;
                    if (use_beta) r += g.beta * *reinterpret_cast<const v4f *>(cp);
                    if (bp) r += bv;
#pragma unroll
                    for (int e = 0; e < 4; e++) r[e] = apply_act(r[e], g.act);
                    *reinterpret_cast<v4f *>(cp) = r;
                }
            }
    } else {
        // Each wave turns its 32x32 sub-tiles through a private 4 KiB of LDS (the stages are
        // dead after the loop's last barrier) so that a store instruction writes 8 rows of 128
        // contiguous bytes instead of 32 rows of 32.  Rows of 128 bytes, 16-byte chunk c of row
        // r kept at chunk c ^ ((r>>1)&7): both the write (16 rows, one chunk column) and the
        // read (2 rows, all chunks) of a 16-lane group then touch every bank once.
        unsigned char *turn = lds_raw + wmn * (WAVES_K == 2 ? TM * TN * 4096 : 4096);   // inside the wave's own join area
        const int rrow = lane >> 3, rchunk = lane & 7;
        const int64_t col0 = n0 + wn * WTN + 4 * rchunk;
        float *dst = C + (m0 + wm * WTM + rrow) * g.ldc + col0;
        const float *bp = g.bias ? g.bias + col0 : nullptr;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const bool col_in = !EDGE || col0 + j * 32 < g.N;          // N % 4 == 0: the whole group or none of it
            v4f bv = {0.f, 0.f, 0.f, 0.f}, cs = {1.f, 1.f, 1.f, 1.f};
            if (bp && col_in) bv = *reinterpret_cast<const v4f *>(bp + j * 32);
            if (g.col_scale && col_in) cs = *reinterpret_cast<const v4f *>(g.col_scale + col0 + j * 32);
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int gq = 0; gq < 4; gq++) {
                    v4f r;
#pragma unroll
                    for (int e = 0; e < 4; e++) r[e] = acc[i][j][4 * gq + e];
                    *reinterpret_cast<v4f *>(turn + frow * 128 + (((2 * gq + fhalf) ^ ((frow >> 1) & 7)) << 4)) = r;
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                v4f r[4];
#pragma unroll
                for (int p = 0; p < 4; p++) {
                    const int row = p * 8 + rrow;
                    r[p] = *reinterpret_cast<const v4f *>(turn + row * 128 + ((rchunk ^ ((row >> 1) & 7)) << 4));
                }
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int p = 0; p < 4; p++) {
                    if (EDGE && (!col_in || m0 + wm * WTM + rrow + i * 32 + p * 8 >= g.M)) continue;
                    float *cp = dst + (int64_t)(i * 32 + p * 8) * g.ldc + j * 32;
                    v4f o = r[p];
                    if (g.alpha != 1.0f) o *= g.alpha;
                    if (g.col_scale) o *= cs;
                    if (use_beta) o += g.beta * *reinterpret_cast<const v4f *>(cp);
                    if (bp) o += bv;
#pragma unroll
                    for (int e = 0; e < 4; e++) o[e] = apply_act(o[e], g.act);
                    // streaming store: results are not re-read by this kernel and must not push the
                    // operand panels out of the XCD's L2 (Q K^T of 512 heads: 226 -> 201 us)
                    __builtin_nontemporal_store(o, reinterpret_cast<v4f *>(cp));
                }
            }
        }
    }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int NST, bool A_KC, bool B_KC, int EPI = 1, int WAVES_K = 1,
          bool EDGE = false, typename BSRC = float, int SPS = 1>
int launch_dma(const char *name, const SgemmArgs &g, int64_t batch) {
    static_assert(!EDGE || EPI == 1, "the edge form guards the turned write-back only");
    constexpr int NW = WAVES_M * WAVES_N * WAVES_K;
    using OB = typename std::conditional<sizeof(BSRC) == 1, DmaOperandI8<BN, NW>, DmaOperand<BN, B_KC, NW>>::type;
    constexpr int stage_bytes = NST * SPS * (DmaOperand<BM, A_KC, NW>::BYTES + OB::BYTES);
    // the write-back turns 4 KiB per output wave through the dead stages
    constexpr int after = WAVES_K == 2 ? BM * BN * 4 : WAVES_M * WAVES_N * 4096;   // the join of a k split needs the whole tile
    constexpr int smem = stage_bytes > after ? stage_bytes : after;
    // One row of tiles reads every byte of B once: large fp32 weights then arrive faster through non-temporal loads
    // (the K ranges of a split and the entries of a batch count together).  Weights in rotation, plain -> non-temporal:
    // 16 x 4096 x 4096 21.0 -> 19.3 us, 16 x 11008 x 4096 38.5 -> 36.3, 32 x 8192 x 8192 57.0 -> 53.2; the same matrix
    // multiplied back to back out of the caches loses 3-12 %, which only a benchmark loop does.  Not for int8 weights: a
    // slab takes 32 bytes of each of their 128-byte lines, and a line that is not kept is fetched four times
    // (8 x 11008 x 4096: 25.0 -> 31.0 us).  Built for the tiles of at most 64 rows, which are the ones few rows get.
    constexpr bool CAN_STREAM = sizeof(BSRC) == 4 && BM <= 64;
    const bool stream_b = CAN_STREAM && g.M <= BM && g.N * g.K * 4 * batch >= (int64_t(32) << 20);
    auto plain = k_sgemm_dma<BM, BN, WAVES_M, WAVES_N, NST, A_KC, B_KC, EPI, WAVES_K, EDGE, BSRC, SPS, false>;
    auto streams = k_sgemm_dma<BM, BN, WAVES_M, WAVES_N, NST, A_KC, B_KC, EPI, WAVES_K, EDGE, BSRC, SPS, CAN_STREAM>;
    auto kern = stream_b ? streams : plain;
    static bool attr_set[2] = {false, false};
    if (!attr_set[stream_b]) {
        AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, smem),
                      "hipFuncSetAttribute");
        attr_set[stream_b] = true;
    }
    const int64_t tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
    note_kernel(name);
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles, (unsigned)batch), dim3(NW * 64), smem, kStream, g);
    return check_launch(name);
}

// =====================================================================================
// C = alpha * A * B^T with a short K (32, 64, 96 or 128: the scores Q K^T of attention heads), both
// operands K-contiguous.  A product this shape writes eight times what it reads per workgroup and has
// only a few dozen MFMAs per output tile, so a workgroup per tile spends its life in its prologue, its
// load latency and its write-back.  Here a workgroup keeps a 128-row block of A in LDS for its whole
// life and walks the 64-column blocks of B^T through two buffers: the loads of block j+1 and the stores
// of tile j-1 are in flight while tile j is multiplied, and the address arithmetic is paid once per
// workgroup.  Within a wave, loads are issued before the stores they must not wait behind (loads and
// stores retire in issue order), so the wait for block j+1 never includes the stores of tile j-1.
// 4 waves as 2 (M) x 2 (N), wave tile 64 x 32.  LDS: A block KS x 16 KiB, two B blocks KS x 8 KiB each,
// 4 KiB per wave to turn the write-back into whole 128-byte rows; two workgroups share a CU up to K = 64.
template <int KS>
__global__ void __launch_bounds__(256) k_sgemm_nt_rows(SgemmArgs g) {
    constexpr int BM = 128, BN = 64, NW = 4, TM = 2;
    using OA = DmaOperand<BM, true, NW>;
    using OB = DmaOperand<BN, true, NW>;
    constexpr int A_BYTES = KS * OA::BYTES, B_BYTES = KS * OB::BYTES;     // the resident block, one B buffer
    constexpr int B_BASE = A_BYTES, TURN_BASE = A_BYTES + 2 * B_BYTES;
    constexpr int NSTORES = TM * 4;                                       // store instructions of a wave per tile
    static_assert(KS >= 1 && KS <= 4 && TURN_BASE + NW * 4096 <= 160 * 1024, "LDS budget");
    static_assert(3 * OA::BYTES + 4096 < 65536 && B_BYTES + 3 * OB::BYTES < 65536, "ds_read immediates are 16 bits");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    int tm = (int)blockIdx.x, tn = 0;
    int64_t batch = 0;
    if (gridDim.y > 1) tile_of_batched_block((int)(g.M / BM), 1, tm, tn, batch);
    const int64_t m0 = (int64_t)tm * BM;
    const float *A = static_cast<const float *>(g.A) + batch * g.stride_a + m0 * g.lda;
    const float *B = static_cast<const float *>(g.B) + batch * g.stride_b;
    float *C = g.C + batch * g.stride_c + m0 * g.ldc;
    const int nblk = (int)(g.N / BN);

    unsigned va[OA::IPW], vb[OB::IPW];
#pragma unroll
    for (int j = 0; j < OA::IPW; j++) va[j] = OA::lane_offset(j * NW + wave, lane, g.lda);
#pragma unroll
    for (int j = 0; j < OB::IPW; j++) vb[j] = OB::lane_offset(j * NW + wave, lane, g.ldb);
    const char *ga = reinterpret_cast<const char *>(A), *gb = reinterpret_cast<const char *>(B);
    const int64_t step_b = (int64_t)BN * g.ldb * 4;                       // bytes from one block of B to the next
    const unsigned lds0 = (unsigned)(uintptr_t)lds_raw;
    const unsigned dma_a = lds0 + wave * OA::PITCH, dma_b = lds0 + B_BASE + wave * OB::PITCH;

    const int frow = lane & 31, fhalf = lane >> 5;
    unsigned ra[4], rb[4];
#pragma unroll
    for (int kbi = 0; kbi < 4; kbi++) {
        ra[kbi] = lds0 + OA::frag_base(wm * 64, frow, fhalf, kbi);
        rb[kbi] = lds0 + B_BASE + OB::frag_base(wn * 32, frow, fhalf, kbi);
    }
    unsigned char *turn = lds_raw + TURN_BASE + wave * 4096;
    const int rrow = lane >> 3, rchunk = lane & 7;
    // where this lane's 16 bytes of a write-back row go, relative to the tile's first row and column block
    float *cdst = C + (int64_t)(wm * 64 + rrow) * g.ldc + wn * 32 + rchunk * 4;

    v16f acc[TM];
    Frag<true> fa[2][TM], fb[2];

// loads of the next block of B into buffer BUFK
#define AXN_ISSUE_B(BUFK)                                                                        \
    do {                                                                                         \
        _Pragma("unroll") for (int s = 0; s < KS; s++)                                           \
            _Pragma("unroll") for (int j = 0; j < OB::IPW; j++)                                  \
                AXF_LOAD_LDS(dma_b + (BUFK) * B_BYTES + s * OB::BYTES + j * NW * OB::PITCH, vb[j], gb + s * 128); \
        gb += step_b;                                                                            \
    } while (0)
// fragments of k-block KK (slab KK >> 2, block KK & 3) out of B buffer BUFK
#define AXN_FRAGS(BUF, BUFK, KK)                                                                 \
    do {                                                                                         \
        AXF_DS128(fa[BUF][0].q, ra[(KK) & 3], ((KK) >> 2) * OA::BYTES);                          \
        AXF_DS128(fa[BUF][1].q, ra[(KK) & 3], ((KK) >> 2) * OA::BYTES + 4096);                   \
        AXF_DS128(fb[BUF].q, rb[(KK) & 3], (BUFK) * B_BYTES + ((KK) >> 2) * OB::BYTES);          \
    } while (0)
// one tile out of B buffer BUFK: 4 * KS k-blocks, the fragments of the next one requested before the
// MFMAs of the current; the first MFMA of each accumulator starts from zero
#define AXN_TILE(BUFK)                                                                           \
    do {                                                                                         \
        AXN_FRAGS(0, BUFK, 0);                                                                   \
        _Pragma("unroll") for (int kk = 0; kk < 4 * KS; kk++) {                                  \
            if (kk + 1 < 4 * KS) {                                                               \
                AXN_FRAGS((kk + 1) & 1, BUFK, kk + 1);                                           \
                AXF_LGKM(3);                                                                     \
            } else {                                                                             \
                AXF_LGKM(0);                                                                     \
            }                                                                                    \
            __builtin_amdgcn_sched_barrier(0);                                                   \
            _Pragma("unroll") for (int e = 0; e < 4; e++)                                        \
                _Pragma("unroll") for (int i = 0; i < TM; i++)                                   \
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[kk & 1].get(e), fa[kk & 1][i].get(e), \
                                                                  (kk == 0 && e == 0) ? zero : acc[i], 0, 0, 0); \
            __builtin_amdgcn_sched_barrier(0);                                                   \
        }                                                                                        \
    } while (0)

    const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // Write-back of the tile in `acc` (columns n0 ..): each 32x32 sub-tile is turned through the wave's
    // 4 KiB of LDS (16-byte chunk c of row r at chunk c ^ ((r >> 1) & 7), conflict-free both ways) so
    // that a store instruction writes 8 rows of 128 contiguous bytes; streaming stores, the scores are
    // not read again by this kernel.
    auto write_back = [&](int64_t n0) {
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int gq = 0; gq < 4; gq++)
                *reinterpret_cast<v4f *>(turn + frow * 128 + (((2 * gq + fhalf) ^ ((frow >> 1) & 7)) << 4)) =
                    v4f{acc[i][4 * gq], acc[i][4 * gq + 1], acc[i][4 * gq + 2], acc[i][4 * gq + 3]};
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            v4f r[4];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const int row = p * 8 + rrow;
                r[p] = *reinterpret_cast<const v4f *>(turn + row * 128 + ((rchunk ^ ((row >> 1) & 7)) << 4));
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int p = 0; p < 4; p++) {
                v4f o = r[p];
                if (g.alpha != 1.0f) o *= g.alpha;
                __builtin_nontemporal_store(o, reinterpret_cast<v4f *>(cdst + (int64_t)(i * 32 + p * 8) * g.ldc + n0));
            }
        }
    };
    // One tile.  Order inside a wave: the loads of the block after this one, then the stores of the tile
    // before this one, then this tile's MFMAs; the wait that follows passes over the stores (NSTORES of
    // them are younger than the loads) and the barrier makes every wave's part of the next block visible
    // and frees this tile's buffer for the loads after next.
#define AXN_STEP(BUFK, j)                                                                        \
    do {                                                                                         \
        const bool more = (j) + 1 < nblk;                                                        \
        if (more) AXN_ISSUE_B(1 - (BUFK));                                                       \
        if ((j) > 0) write_back((int64_t)((j) - 1) * BN);                                        \
        AXN_TILE(BUFK);                                                                          \
        if (more) {                                                                              \
            if ((j) > 0) AXF_VM(NSTORES); else AXF_VM(0);                                        \
            __builtin_amdgcn_s_barrier();                                                        \
            __builtin_amdgcn_sched_barrier(0);                                                   \
        }                                                                                        \
    } while (0)

#pragma unroll
    for (int s = 0; s < KS; s++)
#pragma unroll
        for (int j = 0; j < OA::IPW; j++)
            AXF_LOAD_LDS(dma_a + s * OA::BYTES + j * NW * OA::PITCH, va[j], ga + s * 128);
    AXN_ISSUE_B(0);
    AXF_VM(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    for (int j = 0; j < nblk; j += 2) {
        AXN_STEP(0, j);
        if (j + 1 >= nblk) break;
        AXN_STEP(1, j + 1);
    }
    write_back((int64_t)(nblk - 1) * BN);
#undef AXN_ISSUE_B
#undef AXN_FRAGS
#undef AXN_TILE
#undef AXN_STEP
}

template <int KS>
int launch_nt_rows(const SgemmArgs &g, int64_t batch) {
    constexpr int smem = KS * (16 + 2 * 8) * 1024 + 4 * 4096;
    static bool attr_set = false;
    if (!attr_set) {
        AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(k_sgemm_nt_rows<KS>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, smem),
                      "hipFuncSetAttribute");
        attr_set = true;
    }
    note_kernel("sgemm_nt_rows128_dma");
    hipLaunchKernelGGL((k_sgemm_nt_rows<KS>), dim3((unsigned)(g.M / 128), (unsigned)batch), dim3(256), smem, kStream, g);
    return check_launch("sgemm_nt_rows128_dma");
}

// The short-K NT route: K a multiple of 32 up to 128, M on the 128 grid, N on the 64 grid with at least
// four column blocks, no beta / bias / activation, enough row blocks for the chip.  -1: not taken.
int try_nt_rows(const SgemmArgs &g, int64_t batch) {
    if (tuning().f32_tile != 0) return -1;
    if (g.K % 32 != 0 || g.K < 32 || g.K > 128 || g.M % 128 != 0 || g.N % 64 != 0 || g.N < 256) return -1;
    if (g.beta != 0.0f || g.bias || g.col_scale || g.act != AXHIP_ACT_NONE) return -1;
    if ((g.M / 128) * batch < 2 * cu_count() || batch > 65535 || g.M / 128 > 0x7fffffff) return -1;
    if ((((uintptr_t)g.A | (uintptr_t)g.B | (uintptr_t)g.C) & 15) != 0 || g.lda % 4 != 0 || g.ldb % 4 != 0 || g.ldc % 4 != 0 ||
        g.stride_a % 4 != 0 || g.stride_b % 4 != 0 || g.stride_c % 4 != 0 || g.lda >= (1 << 20) || g.ldb >= (1 << 20))
        return -1;
    switch (g.K / 32) {
        case 1: return launch_nt_rows<1>(g, batch);
        case 2: return launch_nt_rows<2>(g, batch);
        case 3: return launch_nt_rows<3>(g, batch);
        default: return launch_nt_rows<4>(g, batch);
    }
}

// =====================================================================================
// The same product walked the other way: a workgroup keeps 256 rows of B (= 256 columns of C) for its whole
// life — in registers: each of its four waves holds the fragments of its own 64 columns, 8 K / 32 vectors —
// and walks the rows of A in blocks of 32 through two LDS buffers.  Every step therefore finishes 32 rows of
// C over the workgroup's whole width: a wave's store instruction writes four pieces of 256 contiguous bytes,
// the four waves' pieces of a row are neighbours (1 KiB per row and step), and a row of C is complete after
// one step of the N / 256 workgroups that share it instead of being visited N / 64 times over the life of
// one.  The stream of stores that reaches memory is then made of long runs instead of 256-byte fragments
// spread over 128 rows.  Only the A fragments are read from LDS (one ds_read_b128 per 8 MFMAs); loads of the
// next block are issued before the stores of the previous tile, as above.  LDS: two A blocks of K / 32 x 4
// KiB, 8 KiB per wave to turn the write-back into rows of 256 bytes.
template <int KS>
__global__ void __launch_bounds__(256) k_sgemm_nt_cols(SgemmArgs g) {
    constexpr int BMS = 32, BN = 256, NW = 4, TN = 2;                    // rows per step, columns per workgroup
    using OA = DmaOperand<BMS, true, NW>;
    constexpr int A_BYTES = KS * OA::BYTES;                               // one A buffer
    constexpr int TURN_BASE = 2 * A_BYTES;
    constexpr int NSTORES = 8;                                            // store instructions of a wave per step
    static_assert(OA::IPW == 1, "one load instruction per wave and slab");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int tm = 0, tn = (int)blockIdx.x;
    int64_t batch = 0;
    if (gridDim.y > 1) tile_of_batched_block(1, (int)(g.N / BN), tm, tn, batch);
    const int64_t n0 = (int64_t)tn * BN + wave * 64;                      // this wave's first column
    const float *A = static_cast<const float *>(g.A) + batch * g.stride_a;
    const float *B = static_cast<const float *>(g.B) + batch * g.stride_b + n0 * g.ldb;
    float *C = g.C + batch * g.stride_c + n0;
    const int nblk = (int)(g.M / BMS);

    const unsigned va = OA::lane_offset(wave, lane, g.lda);
    const char *ga = reinterpret_cast<const char *>(A);
    const int64_t step_a = (int64_t)BMS * g.lda * 4;                      // bytes from one block of A to the next
    const unsigned lds0 = (unsigned)(uintptr_t)lds_raw;
    const unsigned dma_a = lds0 + wave * OA::PITCH;

    const int frow = lane & 31, fhalf = lane >> 5;
    unsigned ra[4];
#pragma unroll
    for (int kbi = 0; kbi < 4; kbi++) ra[kbi] = lds0 + OA::frag_base(0, frow, fhalf, kbi);

    // This wave's B fragments, kept for the workgroup's life: tile j, k-block kk -> row n0 + 32 j + frow of B,
    // k = 8 kk + 4 fhalf .. + 3 (the pairing of k values over the two lane halves is that of the A fragments).
    // Fetched as whole 128-byte lines (a load instruction takes one slab of 8 rows: lane l -> row l >> 3, 16-byte
    // chunk l & 7; all of them in flight at once) and brought into fragment order through the wave's own turn
    // area, one 32-row slab at a time, rows 144 bytes apart so that neither side meets a bank twice: loading the
    // fragments straight from memory touches every line with four instructions, 32 bytes at a time.
#define AXC_ISSUE_A(BUFK)                                                                        \
    do {                                                                                         \
        _Pragma("unroll") for (int s = 0; s < KS; s++)                                           \
            AXF_LOAD_LDS(dma_a + (BUFK) * A_BYTES + s * OA::BYTES, va, ga + s * 128);            \
        ga += step_a;                                                                            \
    } while (0)
    unsigned char *turn = lds_raw + TURN_BASE + wave * 8192;
    v4f fb[TN][4 * KS];
    {
        v4f raw[TN][KS][4];
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int sl = 0; sl < KS; sl++)
#pragma unroll
                for (int q = 0; q < 4; q++)
                    raw[j][sl][q] = *reinterpret_cast<const v4f *>(B + (int64_t)(j * 32 + q * 8 + (lane >> 3)) * g.ldb + sl * 32 + (lane & 7) * 4);
        AXC_ISSUE_A(0);                             // the first block of A, behind the loads of B
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int sl = 0; sl < KS; sl++) {
#pragma unroll
                for (int q = 0; q < 4; q++)
                    *reinterpret_cast<v4f *>(turn + (q * 8 + (lane >> 3)) * 144 + (lane & 7) * 16) = raw[j][sl][q];
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int kbi = 0; kbi < 4; kbi++)
                    fb[j][sl * 4 + kbi] = *reinterpret_cast<const v4f *>(turn + frow * 144 + (2 * kbi + fhalf) * 16);
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
    }
    const int rrow = lane >> 4, rchunk = lane & 15;
    float *cdst = C + (int64_t)rrow * g.ldc + rchunk * 4;                 // this lane's 16 bytes of a write-back row
    v16f acc[TN];
    Frag<true> fa[2];
    const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

#define AXC_FRAG(BUF, BUFK, KK) AXF_DS128(fa[BUF].q, ra[(KK) & 3], (BUFK) * A_BYTES + ((KK) >> 2) * OA::BYTES)
// one step out of A buffer BUFK: 4 * KS k-blocks of 8 MFMAs, the fragment of the next one requested first
#define AXC_TILE(BUFK)                                                                           \
    do {                                                                                         \
        AXC_FRAG(0, BUFK, 0);                                                                    \
        _Pragma("unroll") for (int kk = 0; kk < 4 * KS; kk++) {                                  \
            if (kk + 1 < 4 * KS) {                                                               \
                AXC_FRAG((kk + 1) & 1, BUFK, kk + 1);                                            \
                AXF_LGKM(1);                                                                     \
            } else {                                                                             \
                AXF_LGKM(0);                                                                     \
            }                                                                                    \
            __builtin_amdgcn_sched_barrier(0);                                                   \
            _Pragma("unroll") for (int e = 0; e < 4; e++)                                        \
                _Pragma("unroll") for (int j = 0; j < TN; j++)                                   \
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j][kk][e], fa[kk & 1].get(e), \
                                                                  (kk == 0 && e == 0) ? zero : acc[j], 0, 0, 0); \
            __builtin_amdgcn_sched_barrier(0);                                                   \
        }                                                                                        \
    } while (0)

    // Write-back of the 32 x 64 tile in `acc` (rows m0 ..): register v of lane l is row l & 31, column
    // 32 j + 8 (v >> 2) + 4 (l >> 5) + (v & 3).  The tile is turned through the wave's 8 KiB of LDS as rows of
    // 256 bytes (16-byte chunk c of row r kept at chunk c ^ (r & 15): 16 rows of one chunk column, or the 16
    // chunks of one row, touch every bank once), so that a store instruction writes 4 rows of 256 bytes.
    auto write_back = [&](int64_t m0) {
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int gq = 0; gq < 4; gq++)
                *reinterpret_cast<v4f *>(turn + frow * 256 + (((j * 8 + 2 * gq + fhalf) ^ (frow & 15)) << 4)) =
                    v4f{acc[j][4 * gq], acc[j][4 * gq + 1], acc[j][4 * gq + 2], acc[j][4 * gq + 3]};
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int half = 0; half < 2; half++) {
            v4f r[4];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const int row = (half * 4 + p) * 4 + rrow;
                r[p] = *reinterpret_cast<const v4f *>(turn + row * 256 + ((rchunk ^ (row & 15)) << 4));
            }
            if (half == 1) {
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
#pragma unroll
            for (int p = 0; p < 4; p++) {
                v4f o = r[p];
                if (g.alpha != 1.0f) o *= g.alpha;
                    __builtin_nontemporal_store(o, reinterpret_cast<v4f *>(cdst + (m0 + (half * 4 + p) * 4) * g.ldc));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
#define AXC_STEP(BUFK, i)                                                                        \
    do {                                                                                         \
        const bool more = (i) + 1 < nblk;                                                        \
        if (more) AXC_ISSUE_A(1 - (BUFK));                                                       \
        if ((i) > 0) write_back((int64_t)((i) - 1) * BMS);                                       \
        AXC_TILE(BUFK);                                                                          \
        if (more) {                                                                              \
            if ((i) > 0) AXF_VM(NSTORES); else AXF_VM(0);                                        \
            __builtin_amdgcn_s_barrier();                                                        \
            __builtin_amdgcn_sched_barrier(0);                                                   \
        }                                                                                        \
    } while (0)

    AXF_VM(0);                                    // the first block of A
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    for (int i = 0; i < nblk; i += 2) {
        AXC_STEP(0, i);
        if (i + 1 >= nblk) break;
        AXC_STEP(1, i + 1);
    }
    write_back((int64_t)(nblk - 1) * BMS);
#undef AXC_ISSUE_A
#undef AXC_FRAG
#undef AXC_TILE
#undef AXC_STEP
}

template <int KS>
int launch_nt_cols(const SgemmArgs &g, int64_t batch) {
    constexpr int smem = 2 * KS * 4096 + 4 * 8192;                        // 64 KiB at most
    note_kernel("sgemm_nt_cols256_dma");
    // One workgroup walks all the rows of A: cutting them into two or four runs (shorter workgroups, more of them) costs
    // more in loads of B fragments than it evens out at the end of the launch (512 heads of 512 x 512, K = 64, zeros:
    // 151.6 us whole, 154.0 in halves, 161.6 in quarters).
    hipLaunchKernelGGL((k_sgemm_nt_cols<KS>), dim3((unsigned)(g.N / 256), (unsigned)batch), dim3(256), smem, kStream, g);
    return check_launch("sgemm_nt_cols256_dma");
}

// Taken ahead of the row-block walk when the columns come in blocks of 256 and the rows in blocks of 32, from eight
// steps per workgroup on (same box, row-block walk -> this one; 512 heads of 512 x 512, K = 64: 171 -> 163 us on
// random operands, 155 -> 149 on zeros; K = 128: 305 -> 276; K = 32: 113 -> 108; 256 heads of 1024 x 1024: 337 ->
// 319; with M = 128, four steps, the row-block walk stays ahead, 92 against 94).  A forced AX_HIP_NT_WALK=2 takes
// it from four steps on.  -1: not taken.
int try_nt_cols(const SgemmArgs &g, int64_t batch) {
    if (tuning().f32_tile != 0 || tuning().nt_walk == 1) return -1;
    if (g.K % 32 != 0 || g.K < 32 || g.K > 128 || g.M % 32 != 0 || g.M < (tuning().nt_walk == 2 ? 128 : 256) || g.N % 256 != 0) return -1;
    if (g.beta != 0.0f || g.bias || g.col_scale || g.act != AXHIP_ACT_NONE) return -1;
    if ((g.N / 256) * batch < 2 * cu_count() || batch > 65535 || g.N / 256 > 0x7fffffff) return -1;
    if ((((uintptr_t)g.A | (uintptr_t)g.B | (uintptr_t)g.C) & 15) != 0 || g.lda % 4 != 0 || g.ldb % 4 != 0 || g.ldc % 4 != 0 ||
        g.stride_a % 4 != 0 || g.stride_b % 4 != 0 || g.stride_c % 4 != 0 || g.lda >= (1 << 20) || g.ldb >= (1 << 20))
        return -1;
    switch (g.K / 32) {
        case 1: return launch_nt_cols<1>(g, batch);
        case 2: return launch_nt_cols<2>(g, batch);
        case 3: return launch_nt_cols<3>(g, batch);
        default: return launch_nt_cols<4>(g, batch);
    }
}

// =====================================================================================
// C = alpha * A * B for batched products with many output tiles and a K of a few hundred (P V of
// attention heads: K = 512, N = 64).  With a workgroup per tile, a third of each workgroup's life is its
// first load latency and its write-back, and the workgroups that share a CU go through both together.
// Here a fixed set of workgroups (one or two per CU) each walk a list of 128 x 64 output tiles and treat
// the K slabs of all of them as one stream through a ring of three LDS stages: the first slabs of the
// next tile are in flight while the last ones of the current tile are multiplied, and the stores of a
// finished tile are issued after the loads of the slab that follows them, so that no wait for loads
// includes stores.  The ring position is a run-time offset (five additions per slab), the first slab of
// a tile is known at compile time: its first MFMAs start from zero and the accumulators never leave
// their registers.  4 waves as 2 x 2, wave tile 64 x 32; A K-contiguous, B N-contiguous; the MFMA takes
// the A fragment first here, so a lane owns one column n of eight rows and a store instruction writes
// two whole 128-byte rows.  Workgroup w serves batch entries w % 8, w % 8 + 8, ... (w % 8 is the XCD it
// runs on), tile after tile of one entry, so the tiles that share an entry's B run next to each other on
// one XCD's L2.
__global__ void __launch_bounds__(256) k_sgemm_nn_stream(SgemmArgs g, int batch, int slots) {
    constexpr int BM = 128, BN = 64, NW = 4, TM = 2, NST = 3;
    using OA = DmaOperand<BM, true, NW>;
    using OB = DmaOperand<BN, false, NW>;
    constexpr int B_BASE = NST * OA::BYTES;
    constexpr int LOADS = OA::IPW + OB::IPW;       // load instructions of a wave per slab
    constexpr int NSTORES = TM * 16;               // store instructions of a wave per tile
    static_assert(B_BASE + NST * OB::BYTES <= 80 * 1024, "two workgroups per CU");
    static_assert(LOADS + NSTORES < 64, "wait counts");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int xcd = (int)(blockIdx.x & 7), slot = (int)(blockIdx.x >> 3);
    const int cbs = (int)(g.N / BN), per_entry = (int)(g.M / BM) * cbs;
    const int items_here = xcd < batch ? ((batch - xcd + 7) / 8) * per_entry : 0;    // tiles of this XCD's entries
    if (slot >= items_here) return;
    const int n_items = (items_here - slot + slots - 1) / slots;                     // ... of which this workgroup's
    const int slabs = (int)(g.K / 32);
    const float *A = static_cast<const float *>(g.A), *B = static_cast<const float *>(g.B);

    // item q of this XCD: entry xcd + 8 * (q / per_entry), row block and column block from the remainder
    auto locate = [&](int q, const char *&pa, const char *&pb, float *&pc) {
        const int e = q / per_entry, r = q - e * per_entry, rb = r / cbs, cb = r - rb * cbs;
        const int64_t entry = xcd + 8 * (int64_t)e;
        pa = reinterpret_cast<const char *>(A + entry * g.stride_a + (int64_t)rb * BM * g.lda);
        pb = reinterpret_cast<const char *>(B + entry * g.stride_b + (int64_t)cb * BN);
        pc = g.C + entry * g.stride_c + (int64_t)rb * BM * g.ldc + (int64_t)cb * BN;
    };

    unsigned va[OA::IPW], vb[OB::IPW];
#pragma unroll
    for (int j = 0; j < OA::IPW; j++) va[j] = OA::lane_offset(j * NW + wave, lane, g.lda);
#pragma unroll
    for (int j = 0; j < OB::IPW; j++) vb[j] = OB::lane_offset(j * NW + wave, lane, g.ldb);
    const int64_t step_b = 128 * g.ldb;                                              // bytes per slab of B
    const unsigned lds0 = (unsigned)(uintptr_t)lds_raw;
    const unsigned dma_a = lds0 + wave * OA::PITCH, dma_b = lds0 + B_BASE + wave * OB::PITCH;

    const int frow = lane & 31, fhalf = lane >> 5;
    unsigned ra0[4];                               // fragment addresses in stage 0
#pragma unroll
    for (int kbi = 0; kbi < 4; kbi++) ra0[kbi] = lds0 + OA::frag_base(wm * 64, frow, fhalf, kbi);
    const unsigned rb0 = lds0 + B_BASE + OB::frag_base(wn * 32, frow, fhalf, 0);
    // register v of lane l: n = l & 31, m = i*32 + 8*(v>>2) + 4*(l>>5) + (v&3)
    const int64_t lane_c = (int64_t)(wm * 64 + 4 * fhalf) * g.ldc + wn * 32 + frow;

    // the load side of the stream runs ahead of the multiply side: each has its own item and ring position
    const char *ga, *gb;
    float *c_unused, *c_cur, *c_prev = nullptr;
    int lq = slot, lk = 0, to_load = n_items * slabs;
    unsigned load_a = 0, load_b = 0, mul_a = 0, mul_b = 0;        // byte offsets of the stage loaded / multiplied next
    locate(lq, ga, gb, c_unused);
    {
        const char *ua, *ub;
        locate(slot, ua, ub, c_cur);
    }

    v16f acc[TM];
    Frag<true> fa[2][TM];
    Frag<false> fb[2];
    const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < TM; i++) acc[i] = zero;
    unsigned ra[4], rb;

// loads of the stream's next slab into the ring
#define AXS_ISSUE()                                                                              \
    do {                                                                                         \
        _Pragma("unroll") for (int j = 0; j < OA::IPW; j++)                                      \
            /* A (the scores of P V, 537 MB at 512 heads) is read once: 157.5 -> 153.3 us */    \
            AXF_LOAD_LDS_NT(dma_a + load_a + j * NW * OA::PITCH, va[j], ga);                     \
        _Pragma("unroll") for (int j = 0; j < OB::IPW; j++)                                      \
            AXF_LOAD_LDS(dma_b + load_b + j * NW * OB::PITCH, vb[j], gb);                        \
        load_a = load_a == (NST - 1) * OA::BYTES ? 0 : load_a + OA::BYTES;                       \
        load_b = load_b == (NST - 1) * OB::BYTES ? 0 : load_b + OB::BYTES;                       \
        --to_load;                                                                               \
        if (++lk == slabs) {                                                                     \
            lk = 0;                                                                              \
            lq += slots;                                                                         \
            if (to_load > 0) locate(lq, ga, gb, c_unused);                                       \
        } else {                                                                                 \
            ga += 128;                                                                           \
            gb += step_b;                                                                        \
        }                                                                                        \
    } while (0)
// fragments of k-block KB of the stage being multiplied
#define AXS_FRAGS(BUF, KB)                                                                       \
    do {                                                                                         \
        AXF_DS128(fa[BUF][0].q, ra[KB], 0);                                                      \
        AXF_DS128(fa[BUF][1].q, ra[KB], 4096);                                                   \
        AXF_DS32(fb[BUF].s0, rb, OB::k_imm((KB) * 8 + 0));                                       \
        AXF_DS32(fb[BUF].s1, rb, OB::k_imm((KB) * 8 + 1));                                       \
        AXF_DS32(fb[BUF].s2, rb, OB::k_imm((KB) * 8 + 2));                                       \
        AXF_DS32(fb[BUF].s3, rb, OB::k_imm((KB) * 8 + 3));                                       \
    } while (0)
// the eight MFMAs of a k-block; ZERO: a tile's first, which start from a clean accumulator
#define AXS_MFMAS(BUF, ZERO)                                                                     \
    do {                                                                                         \
        __builtin_amdgcn_sched_barrier(0);                                                       \
        _Pragma("unroll") for (int e = 0; e < 4; e++)                                            \
            _Pragma("unroll") for (int i = 0; i < TM; i++)                                       \
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[BUF][i].get(e), fb[BUF].get(e), \
                                                              ((ZERO) && e == 0) ? zero : acc[i], 0, 0, 0); \
        __builtin_amdgcn_sched_barrier(0);                                                       \
    } while (0)

    // the finished tile: a store instruction writes one float per lane, two rows of 128 bytes
    auto write_back = [&]() {
        float *cp = c_prev + lane_c;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                float o = acc[i][v];
                if (g.alpha != 1.0f) o *= g.alpha;
                __builtin_nontemporal_store(o, cp + (int64_t)(i * 32 + 8 * (v >> 2) + (v & 3)) * g.ldc);
            }
    };

// One slab; FIRST: the first of a tile.  Order inside a wave: the loads of the slab two ahead, then
// (FIRST) the stores of the tile finished by the previous slab, then this slab's MFMAs; the wait that
// follows passes over whatever was issued after the next slab's loads, and the barrier makes every
// wave's part of that slab visible and frees this slab's stage for the loads issued next.
#define AXS_SLAB(FIRST)                                                                          \
    do {                                                                                         \
        const bool more = to_load > 0, wrote = (FIRST) && c_prev != nullptr;                     \
        if (more) AXS_ISSUE();                                                                   \
        if (wrote) write_back();                                                                 \
        _Pragma("unroll") for (int kbi = 0; kbi < 4; kbi++) ra[kbi] = ra0[kbi] + mul_a;          \
        rb = rb0 + mul_b;                                                                        \
        mul_a = mul_a == (NST - 1) * OA::BYTES ? 0 : mul_a + OA::BYTES;                          \
        mul_b = mul_b == (NST - 1) * OB::BYTES ? 0 : mul_b + OB::BYTES;                          \
        AXS_FRAGS(0, 0);                                                                         \
        AXS_FRAGS(1, 1);                                                                         \
        AXF_LGKM(6);                                                                             \
        AXS_MFMAS(0, FIRST);                                                                     \
        AXS_FRAGS(0, 2);                                                                         \
        AXF_LGKM(6);                                                                             \
        AXS_MFMAS(1, false);                                                                     \
        AXS_FRAGS(1, 3);                                                                         \
        AXF_LGKM(6);                                                                             \
        AXS_MFMAS(0, false);                                                                     \
        AXF_LGKM(0);                                                                             \
        AXS_MFMAS(1, false);                                                                     \
        if (more) {                                                                              \
            if (wrote) AXF_VM(LOADS + NSTORES); else AXF_VM(LOADS);                              \
        } else {                                                                                 \
            if (wrote) AXF_VM(NSTORES); else AXF_VM(0);                                          \
        }                                                                                        \
        __builtin_amdgcn_s_barrier();                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                       \
    } while (0)

    AXS_ISSUE();
    AXS_ISSUE();                                   // a tile has at least four slabs
    AXF_VM(LOADS);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    int cq = slot;
    for (int t = 0; t < n_items; t++) {
        AXS_SLAB(true);
        for (int s = 1; s < slabs; s++) AXS_SLAB(false);
        c_prev = c_cur;
        cq += slots;
        if (t + 1 < n_items) {
            const char *ua, *ub;
            locate(cq, ua, ub, c_cur);
        }
    }
    write_back();
#undef AXS_ISSUE
#undef AXS_FRAGS
#undef AXS_MFMAS
#undef AXS_SLAB
}

// The streamed NN route: a batch of at least 8 entries, K a multiple of 32 from 128 to 1024, M on the 128
// grid, N on the 64 grid, no beta / bias / activation, at least three tiles for every workgroup.  An
// XCD's share of the tiles is dealt to one or two workgroups per CU, whichever leaves the last round of
// tiles fuller.  -1: not taken.
int try_nn_stream(const SgemmArgs &g, int64_t batch) {
    if (tuning().f32_tile != 0) return -1;
    if (g.K < 128 || g.K > 1024 || g.K % 32 != 0 || g.M % 128 != 0 || g.N % 64 != 0 || batch < 8 || batch > 65535) return -1;
    if (g.beta != 0.0f || g.bias || g.col_scale || g.act != AXHIP_ACT_NONE) return -1;
    if ((((uintptr_t)g.A | (uintptr_t)g.B | (uintptr_t)g.C) & 15) != 0 || g.lda % 4 != 0 || g.ldb % 4 != 0 || g.ldc % 4 != 0 ||
        g.stride_a % 4 != 0 || g.stride_b % 4 != 0 || g.stride_c % 4 != 0 || g.lda >= (1 << 20) || g.ldb >= (1 << 20))
        return -1;
    const int64_t per_entry = (g.M / 128) * (g.N / 64), per_xcd = (batch + 7) / 8 * per_entry, cus = cu_count() / 8;
    if (per_entry > 4096 || cus < 1) return -1;
    int64_t slots = 0, best_num = 0, best_den = 1;
    for (int64_t w = 1; w <= 2; w++) {
        const int64_t rounds = (per_xcd + w * cus - 1) / (w * cus);
        // fill = per_xcd / (rounds * w * cus); two per CU wins a tie
        if (rounds >= 3 && per_xcd * best_den >= best_num * rounds * w * cus) {
            best_num = per_xcd;
            best_den = rounds * w * cus;
            slots = w * cus;
        }
    }
    if (slots == 0) return -1;
    constexpr int smem = 3 * (DmaOperand<128, true, 4>::BYTES + DmaOperand<64, false, 4>::BYTES);
    static bool attr_set = false;
    if (!attr_set) {
        AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(k_sgemm_nn_stream),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, smem),
                      "hipFuncSetAttribute");
        attr_set = true;
    }
    note_kernel("sgemm_nn_stream128x64_dma");
    hipLaunchKernelGGL(k_sgemm_nn_stream, dim3((unsigned)(8 * slots)), dim3(256), smem, kStream, g, (int)batch, (int)slots);
    return check_launch("sgemm_nn_stream128x64_dma");
}

// Up to 160 rows (K-contiguous) whose count of 32-row blocks is odd (1..32, 65..96, 129..160) run on 32x64 tiles
// instead of 64x64 tiles whose last row block is at least half padding (same box, 32 x 11008 x 4096: 71.9 ->
// 57.1 us and 32.4 with the K split that the smaller tiles then earn, with int8 weights 84.9 -> 32.9;
// 160 x 11008 x 4096: 181.6 -> 143.7).  A 32x64 tile costs about 0.55 of a 64x64 one, so from 224 rows on the
// padded row block is the cheaper choice again (224 x 11008 x 4096: 182.6 against 198.4).
inline bool half_row_tiles(int64_t M) { return M <= 160 && ((M + 31) / 32) % 2 == 1; }

// Chooses the largest tile that still leaves about eight waves per CU; returns -1 when the
// shape does not qualify for the fast path (the caller then uses the register-staged kernel).
// names: 128x128, 64x64, 64x64 with the k split.
template <bool A_KC, bool B_KC>
int try_dma(const char *const names[3], const SgemmArgs &g, int64_t batch) {
    const bool ok = g.K % 4 == 0 && g.K > 0 && ((uintptr_t)g.A % 16 == 0) && ((uintptr_t)g.B % 16 == 0) &&
                    ((uintptr_t)g.C % 16 == 0) && ((uintptr_t)g.bias % 16 == 0) && g.lda % 4 == 0 &&
                    g.ldb % 4 == 0 && g.ldc % 4 == 0 && g.stride_a % 4 == 0 && g.stride_b % 4 == 0 &&
                    g.stride_c % 4 == 0 && g.lda < (1 << 20) && g.ldb < (1 << 20) && batch <= 65535 &&
                    g.N % 4 == 0 && (A_KC || g.M % 4 == 0) && ((g.M + 63) / 64) * ((g.N + 63) / 64) <= 0x7fffffff;
    if (!ok) return -1;
    if constexpr (A_KC) {
        if (half_row_tiles(g.M) && g.K >= 64 && tuning().f32_tile == 0) {
            if (g.M % 32 == 0 && g.N % 64 == 0 && g.K % 32 == 0)
                return launch_dma<32, 64, 1, 2, 2, A_KC, B_KC, 1, 2>(B_KC ? "sgemm_nt_32x64k2_dma" : "sgemm_nn_32x64k2_dma", g, batch);
            return launch_dma<32, 64, 1, 2, 2, A_KC, B_KC, 1, 2, true>("sgemm_32x64k2_dma_edge", g, batch);
        }
    }
    if (g.M % 64 != 0 || g.N % 64 != 0 || g.K % 32 != 0) {  // off the tile grid: 64x64 tiles with guarded edges
        static const char *const edge_names[2] = {"sgemm_64x64_dma_edge", "sgemm_64x64k2_dma_edge"};
        if (g.K > 128) return launch_dma<64, 64, 2, 2, 2, A_KC, B_KC, 1, 2, true>(edge_names[1], g, batch);
        return launch_dma<64, 64, 2, 2, 2, A_KC, B_KC, 1, 1, true>(edge_names[0], g, batch);
    }
    auto count = [&](int64_t bm, int64_t bn) { return (g.M / bm) * (g.N / bn) * batch; };
    // Sustained timings over the benchmark shapes: 128x128 with eight waves (2 x 4, wave tile 64x32;
    // 64 KiB of LDS, so two workgroups share a CU and one's first loads and write-back run under the
    // other's MFMAs) wins once there is a tile for every CU: 8192^3 151 TFLOP/s against 145 on 128x256
    // tiles (one workgroup per CU) and 4096^3 148 against 143; the four-wave form of the same tile and
    // 128x64 are behind both.  Below that 64x64 tiles with the k split are best everywhere, and two
    // stages are as good as three or four.  With only a few slabs per tile (K <= 128) a workgroup's
    // life is mostly its loads and its write-back: plain 64x64 tiles, several workgroups per CU.
    const int force = tuning().f32_tile;         // 0 = by shape; 128, 64 or 642 (64x64 with the k split) where the shape permits
    if (force == 128 && g.M % 128 == 0 && g.N % 128 == 0 && g.K >= 64)
        return launch_dma<128, 128, 2, 4, 2, A_KC, B_KC, 1>(names[0], g, batch);
    if (force == 642 && g.K >= 64) return launch_dma<64, 64, 2, 2, 2, A_KC, B_KC, 1, 2>(names[2], g, batch);
    if (force == 64) return launch_dma<64, 64, 2, 2, 2, A_KC, B_KC, 1>(names[1], g, batch);
    if (g.K > 128) {
        // ... provided the tiles come out at nearly the same number for every CU: 384 tiles are one
        // each and a second one for half the CUs, which then take twice as long
        const int64_t big = count(128, 128), cus = cu_count(), rounds = (big + cus - 1) / cus;
        if (g.M % 128 == 0 && g.N % 128 == 0 && big >= cus && big * 10 >= rounds * cus * 9)
            return launch_dma<128, 128, 2, 4, 2, A_KC, B_KC, 1>(names[0], g, batch);
        // One round of tiles with operands too large to be met in the L2s: every workgroup's life is one stream
        // from memory with nothing else on its CU to cover the latency, and a third stage keeps more of it in
        // flight.  Operands in HBM (rotating sets): 256 x 4096 x 4096 84.0 -> 71.6 us, 512 x 2048 x 4096 86.0 -> 71.3,
        // 128 x 4096 x 1024 on 32x64 tiles 22.6 -> 14.3, 128 x 4096 x 768 18.1 -> 12.0, 256 x 4096 x 1024 24.1 -> 21.1;
        // the same operands in the Infinity Cache: 68.4 -> 70.5, 68.2 -> 70.1, 12.8 -> 13.3, 10.3 -> 10.8, 19.8 -> 20.5.
        // With two rounds or more the other workgroup of a CU covers the latency and two stages stay (within 1.5 %
        // either way).  The K ranges of a split count like tiles (128 x 4096 x 4096 in two ranges, from HBM:
        // 48.6 -> 41.6 us).  Operands of at most 8 MiB together, a quarter of the L2s, keep two stages.
        const bool streams = count(64, 64) <= cus && g.K >= 512 && (g.M + g.N) * g.K * 4 * batch > (int64_t(8) << 20);
        // 64x64 tiles whose count leaves the last round of one tile per CU mostly empty (300 tiles: a full
        // round and 44 CUs' worth) run as 32x64 tiles instead when that evens the rounds out: a half tile
        // costs about 0.55 of a whole one (1280 x 960 x 2048: 63.8 -> 53.1 us; 1152^3: 38.2 -> 31.8; 896 x
        // 1280 x 4096: 123 -> 102).  Rows of A must be K-contiguous for a 32-row tile (NN and NT).
        if constexpr (A_KC) {
            const int64_t whole = count(64, 64), rounds_whole = (whole + cus - 1) / cus, rounds_half = (2 * whole + cus - 1) / cus;
            if (rounds_half * 55 <= rounds_whole * 95) {
                if (streams)
                    return launch_dma<32, 64, 1, 2, 3, A_KC, B_KC, 1, 2>(B_KC ? "sgemm_nt_32x64k2_dma" : "sgemm_nn_32x64k2_dma", g, batch);
                return launch_dma<32, 64, 1, 2, 2, A_KC, B_KC, 1, 2>(B_KC ? "sgemm_nt_32x64k2_dma" : "sgemm_nn_32x64k2_dma", g, batch);
            }
        }
        // Two slabs per stage and barrier where K allows (a slab of a 64x64 tile is 8 MFMAs per wave, so the barrier is a
        // visible share of it), which also keeps as much in flight as the third stage did.  Cached / from HBM:
        // 256 x 4096 x 4096 70.1 / 72.0 -> 66.8 / 69.9 us, 512 x 2048 x 4096 70.1 / 71.1 -> 66.7 / 68.2, 256 x 4096 x 1024
        // 20.4 / 20.5 -> 19.6 / 19.9, 1024^3 19.7 / 20.1 -> 19.5 / 19.9, 256 x 11008 x 4096 182 / 194 -> 182 / 188; with three
        // stages of two slabs 68.3 / 70.1 on the first.
        if (g.K % 64 == 0) return launch_dma<64, 64, 2, 2, 2, A_KC, B_KC, 1, 2, false, float, 2>(names[2], g, batch);
        if (streams) return launch_dma<64, 64, 2, 2, 3, A_KC, B_KC, 1, 2>(names[2], g, batch);
        return launch_dma<64, 64, 2, 2, 2, A_KC, B_KC, 1, 2>(names[2], g, batch);
    }
    return launch_dma<64, 64, 2, 2, 2, A_KC, B_KC, 1>(names[1], g, batch);
}

// The same fast path with int8 weights as the B operand (W8A32: A fp32 [M,K], B int8 [N,K], the
// per-column scale applied in the write-back).  The products run on the bf16 matrix core: three exact
// bf16 terms per fp32 activation (Bf16x3), the int8 weight as one bf16, v_mfma_f32_32x32x16_bf16 with
// fp32 accumulation — 3/16 of the matrix-core time of the fp32 product at the same accuracy.  K must be a multiple of 32 (whole slabs, rows of B on
// 16-byte boundaries); M and N may be off the tile grid.  Returns -1 when the shape does not qualify.
const char *const kI8DmaNames[3] = {"qgemm_w8a32_mfma_128x128_dma", "qgemm_w8a32_mfma_64x64_dma", "qgemm_w8a32_mfma_64x64k2_dma"};
int try_dma_i8(const char *const names[3], const SgemmArgs &g, int64_t batch) {
    const bool ok = g.K % 32 == 0 && g.K > 0 && ((uintptr_t)g.A % 16 == 0) && ((uintptr_t)g.B % 16 == 0) &&
                    ((uintptr_t)g.C % 16 == 0) && ((uintptr_t)g.bias % 16 == 0) && ((uintptr_t)g.col_scale % 16 == 0) &&
                    g.lda % 4 == 0 && g.ldb % 16 == 0 && g.ldc % 4 == 0 && g.stride_a % 4 == 0 && g.stride_b % 16 == 0 &&
                    g.stride_c % 4 == 0 && g.lda < (1 << 20) && g.ldb < (1 << 22) && batch <= 65535 && g.N % 4 == 0 &&
                    ((g.M + 63) / 64) * ((g.N + 63) / 64) <= 0x7fffffff;
    if (!ok) return -1;
    if (half_row_tiles(g.M) && g.K >= 64 && tuning().f32_tile == 0 && (tuning().w8a32_tile == 0 || g.K <= 128)) {   // as for fp32 operands
        if (g.M % 32 == 0 && g.N % 64 == 0) {
            // two slabs per stage where K allows: level with cached weights, ahead with the weights in HBM
            // (32 x 4096 x 4096 12.7 / 15.8 -> 13.0 / 14.6 us, 96 x 4096 x 4096 23.6 / 24.8 -> 23.1 / 24.4)
            if (g.K % 64 == 0)
                return launch_dma<32, 64, 1, 2, 2, true, true, 1, 2, false, int8_t, 2>("qgemm_w8a32_mfma_32x64k2_dma", g, batch);
            return launch_dma<32, 64, 1, 2, 2, true, true, 1, 2, false, int8_t>("qgemm_w8a32_mfma_32x64k2_dma", g, batch);
        }
        return launch_dma<32, 64, 1, 2, 2, true, true, 1, 2, true, int8_t>("qgemm_w8a32_mfma_32x64k2_dma_edge", g, batch);
    }
    if (g.K > 128 && tuning().f32_tile == 0) {
        // Many output tiles.  The conversions to bf16 run on the vector pipe beside the products, and that pipe needs two
        // waves on a SIMD to stay busy.  A wave converts its own rows of A (6.5 instructions a value) and every column of
        // B it multiplies them with (1.5), so its tile is one 32-row block high and as wide as the tile allows, and the
        // tile is the largest that still gives the CUs enough workgroups (M, N, K, us before -> after: 4096^3 517 -> 353,
        // 2048 x 4096 x 4096 266 -> 203, 1024 x 4096 x 4096 153 -> 106, 512 x 11008 x 4096 214 -> 153, 512 x 4096 x 4096
        // 84 -> 65, 2048 x 1024 x 4096 85 -> 62, 256 x 4096 x 4096 54 -> 46, 1024^3 16.1 -> 14.4).  `eighths` = workgroups
        // per CU, in eighths, from which a tile shape pays (measured: the 128-row tiles have one wave per SIMD and need
        // two workgroups per CU, the k-split ones bring two waves themselves).  A shape off the tile grid takes the edge
        // form when the padding stays under an eighth of the output (1000 x 4096 x 4096 153 -> 111 us, 4000 x 4000 x 4096
        // 577 -> 355, 300 x 11008 x 4096 146 -> 102, 2000 x 2000 x 2048 79 -> 58).
        const int64_t cus = cu_count();
        const int forced = tuning().w8a32_tile;
        auto pays = [&](int64_t bm, int64_t bn, int64_t eighths, bool &whole) {
            const int64_t tm = (g.M + bm - 1) / bm, tn = (g.N + bn - 1) / bn, tiles = tm * tn * batch;
            whole = g.M % bm == 0 && g.N % bn == 0;
            if (forced) return forced == (bm == 128 ? (bn == 256 ? 1 : 2) : bm == 64 ? 3 : bn == 128 ? 4 : 5) && tiles <= 0x7fffffff;
            if (tiles * 8 < eighths * cus || tm * bm * tn * bn * 8 > g.M * g.N * 9) return false;
            // two of the 128-row workgroups share a CU: a last round of them that is mostly empty costs a whole round
            // (516 tiles of 128x128 at 768 x 11008 x 4096: 341 us against 310 on 64x64 tiles)
            if (bm == 128) {
                const int64_t rounds = (tiles + 2 * cus - 1) / (2 * cus);
                return tiles * 5 >= rounds * 2 * cus * 4;
            }
            return true;
        };
        bool whole;
        if (pays(128, 256, 15, whole))
            return whole ? launch_dma<128, 256, 4, 1, 2, true, true, 1, 1, false, int8_t>("qgemm_w8a32_mfma_128x256_dma", g, batch)
                         : launch_dma<128, 256, 4, 1, 2, true, true, 1, 1, true, int8_t>("qgemm_w8a32_mfma_128x256_dma_edge", g, batch);
        if (pays(128, 128, 15, whole))
            return whole ? launch_dma<128, 128, 4, 1, 3, true, true, 1, 1, false, int8_t>(names[0], g, batch)
                         : launch_dma<128, 128, 4, 1, 3, true, true, 1, 1, true, int8_t>("qgemm_w8a32_mfma_128x128_dma_edge", g, batch);
        if (pays(64, 128, 12, whole))
            return whole ? launch_dma<64, 128, 2, 1, 2, true, true, 1, 2, false, int8_t>("qgemm_w8a32_mfma_64x128k2_dma", g, batch)
                         : launch_dma<64, 128, 2, 1, 2, true, true, 1, 2, true, int8_t>("qgemm_w8a32_mfma_64x128k2_dma_edge", g, batch);
        if (pays(32, 128, 10, whole))
            return whole ? launch_dma<32, 128, 1, 2, 4, true, true, 1, 2, false, int8_t>("qgemm_w8a32_mfma_32x128k2_dma", g, batch)
                         : launch_dma<32, 128, 1, 2, 4, true, true, 1, 2, true, int8_t>("qgemm_w8a32_mfma_32x128k2_dma_edge", g, batch);
        if (pays(32, 64, 12, whole))
            return whole ? launch_dma<32, 64, 1, 2, 4, true, true, 1, 2, false, int8_t>("qgemm_w8a32_mfma_32x64k2_dma", g, batch)
                         : launch_dma<32, 64, 1, 2, 4, true, true, 1, 2, true, int8_t>("qgemm_w8a32_mfma_32x64k2_dma_edge", g, batch);
    }
    if (g.M % 64 != 0 || g.N % 64 != 0) {
        if (g.K > 128) return launch_dma<64, 64, 2, 2, 2, true, true, 1, 2, true, int8_t>(names[2], g, batch);
        return launch_dma<64, 64, 2, 2, 2, true, true, 1, 1, true, int8_t>(names[1], g, batch);
    }
    if (g.K > 128) {
        const int64_t big = (g.M / 128) * (g.N / 128) * batch, cus = cu_count(), rounds = (big + cus - 1) / cus;
        if (g.M % 128 == 0 && g.N % 128 == 0 && big >= cus && big * 10 >= rounds * cus * 9)
            return launch_dma<128, 128, 4, 1, 3, true, true, 1, 1, false, int8_t>(names[0], g, batch);
        // the last round of one 64x64 tile per CU mostly empty: 32x64 tiles, as for fp32 operands
        const int64_t whole = (g.M / 64) * (g.N / 64) * batch, rounds_whole = (whole + cus - 1) / cus,
                      rounds_half = (2 * whole + cus - 1) / cus;
        if (tuning().f32_tile == 0 && rounds_half * 55 <= rounds_whole * 95) {
            // (two slabs per stage, cached / from HBM: 128 x 4096 x 1024 12.9 / 14.5 -> 12.1 / 12.9 us, 128 x 3072 x 768 10.5 / 10.8 -> 9.9 / 10.1)
            if (g.K % 64 == 0)
                return launch_dma<32, 64, 1, 2, 2, true, true, 1, 2, false, int8_t, 2>("qgemm_w8a32_mfma_32x64k2_dma", g, batch);
            return launch_dma<32, 64, 1, 2, 2, true, true, 1, 2, false, int8_t>("qgemm_w8a32_mfma_32x64k2_dma", g, batch);
        }
        return launch_dma<64, 64, 2, 2, 2, true, true, 1, 2, false, int8_t>(names[2], g, batch);
    }
    return launch_dma<64, 64, 2, 2, 2, true, true, 1, 1, false, int8_t>(names[1], g, batch);
}

// ---- split-K for shapes with few output tiles -----------------------------------------
// A GEMM with a handful of 64x64 tiles and a long K (M of 9..128 against a wide weight) would
// occupy a handful of CUs.  It is run instead as a batched GEMM over `splits` equal K ranges —
// the ranges are sub-matrices reached by pointer offsets, so the batched kernels above serve
// unchanged — into a workspace of partial products, and one finishing pass adds the partials in
// split order and applies alpha, beta, the column scale's sibling terms, bias and activation.
// The order is fixed, so results do not vary from run to run.
// One workgroup covers 256 / LANES neighbouring items (four columns each when VEC); lane l adds
// the splits [l * per, (l + 1) * per) in order, with all its loads in flight together, and the
// lanes' sums are then joined in lane order by lane 0.
template <bool VEC, int LANES>
__global__ void __launch_bounds__(256)
k_splitk_finish(const float *__restrict__ part, int splits, int64_t M, int64_t N, float alpha, float beta,
                const float *__restrict__ bias, int act, float *__restrict__ C, int64_t ldc) {
    constexpr int ITEMS = 256 / LANES, W = VEC ? 4 : 1;
    typedef float vw __attribute__((ext_vector_type(W)));
    __shared__ vw sums[LANES][ITEMS];
    const int lane = threadIdx.x / ITEMS, it = threadIdx.x % ITEMS;
    const int64_t per_row = N / W, items = M * per_row;
    const int64_t t = (int64_t)blockIdx.x * ITEMS + it;
    const bool live = t < items;
    const int64_t m = live ? t / per_row : 0, n = live ? (t - m * per_row) * W : 0;
    const int per = (splits + LANES - 1) / LANES;
    const int k0 = lane * per, k1 = min(splits, k0 + per);
    vw s = 0.0f;
    if (live) {
        const float *p = part + m * N + n + (int64_t)k0 * M * N;
        int k = k0;
        for (; k + 4 <= k1; k += 4, p += 4 * M * N) {
            const vw x0 = *reinterpret_cast<const vw *>(p), x1 = *reinterpret_cast<const vw *>(p + M * N),
                     x2 = *reinterpret_cast<const vw *>(p + 2 * M * N), x3 = *reinterpret_cast<const vw *>(p + 3 * M * N);
            s = (((s + x0) + x1) + x2) + x3;
        }
        for (; k < k1; k++, p += M * N) s += *reinterpret_cast<const vw *>(p);
    }
    sums[lane][it] = s;
    __syncthreads();
    if (lane != 0 || !live) return;
#pragma unroll
    for (int l = 1; l < LANES; l++) s += sums[l][it];
    vw *dst = reinterpret_cast<vw *>(C + m * ldc + n);
    vw r = s * alpha;
    if (beta != 0.0f) r += *dst * beta;
    if (bias) r += *reinterpret_cast<const vw *>(bias + n);
#pragma unroll
    for (int e = 0; e < W; e++) r[e] = apply_act(r[e], act);
    *dst = r;
}

int dispatch_f32(const SgemmArgs &g, int transa, int transb, int64_t batch);

// how many K ranges to use (1: none).  Every range must be a whole number of 32-wide slabs.
int64_t split_count(int64_t M, int64_t N, int64_t K, bool a_rows_k_contiguous) {
    // whole 32x64 tiles count as 0.55 of a tile each
    const bool halves = a_rows_k_contiguous && tuning().f32_tile == 0 && half_row_tiles(M);
    const int64_t tiles = halves ? (((M + 31) / 32) * ((N + 63) / 64) * 11 + 19) / 20 : ((M + 63) / 64) * ((N + 63) / 64);
    const int64_t cus = cu_count();
    if (tuning().f32_splitk == 1 || K < 256 || K % 32 != 0) return 1;
    if (tiles * 2 > cus) {
        // More than half the CUs have a tile: a split pays only when a fifth of them would sit idle through a long
        // K (192 tiles, K = 4096: 68 -> 55..57 us with the operands in the Infinity Cache, 84..88 -> 58..61 from
        // HBM; with 256 tiles it loses 3 % cached and gains no more than a third stage does).
        if (tiles * 5 > cus * 4 || K < 4096 || halves || tuning().f32_splitk != 0) return 1;
        for (int64_t s = 4; s >= 2; s--)
            if (K % (s * 32) == 0) return s;
        return 1;
    }
    // One workgroup per CU measured best for tiles on the 64 grid (32x768x768: 10.5 us against 27
    // unsplit; 64x1024x4096: 12 against 70; 128x4096x1024: 16.5 against 20; more ranges only add
    // partial sums to move); strips off the grid, part of whose tiles is padding, gain from two
    // (4x4100x4096: 38 -> 30 us; 9x8000x8192: 78 -> 69).
    const bool ragged = halves || M % 64 != 0 || N % 64 != 0;     // small workgroups, too: two per CU (96 x 4096 x 4096: 33.9 us against 40.4)
    int64_t want = ((ragged ? 2 : 1) * cus + tiles - 1) / tiles;
    if (tuning().f32_splitk > 1) want = tuning().f32_splitk;
    const int64_t most = K / 64;                             // ranges of at least 64
    if (want > most) want = most;
    // K / 32 must divide into the ranges: the nearest count at or below the wish, or, when that is
    // under half of it (K = 4000 has only 5, 25 and 125), the nearest above up to twice the wish
    int64_t below = 1, above = 0;
    for (int64_t s = want; s >= 2; s--)
        if (K % (s * 32) == 0) { below = s; break; }
    for (int64_t s = want + 1; s <= 2 * want && s <= most; s++)
        if (K % (s * 32) == 0) { above = s; break; }
    return (below * 2 < want && above) ? above : below;
}

// With rows of A K-contiguous, a shape on the tile grid with few 64x64 tiles runs on 32x64 tiles with
// the k split (twice the workgroups, eight waves each), and that one launch costs 3.4 us plus 2.3 us
// per 256 of K up to K = 1536 whatever the tile count (K = 256: 5.7 us, 512: 8.0, 768: 10.3, 1024: 12.7,
// 1536: 17.5; from 2048 on the rows of A are 8 KiB apart and it takes 29).  The two launches of the split
// route take 7.8 to 10.5 us at K = 256, 9.3 to 12.2 at 512, 11.1 at 768, 11.8 to 12.3 at K = 1024 up to 64
// tiles and 15.9 with 128 (1024 x 512 x 1024), 20 at K = 1536 with 128 tiles; a dozen tiles split many
// ways take 8.1 at K = 768.  So the split is left out up to K = 512, up to K = 768 from 48 tiles on, and
// up to K = 1536 for more than 64 tiles.  The same holds with int8 weights as B (128 x 4096 x 1024:
// 18.3 -> 15.3 us).
bool one_launch_on_half_tiles(const SgemmArgs &g, int transa) {
    if (transa || tuning().f32_splitk != 0 || tuning().f32_tile != 0) return false;
    if (g.M % 64 != 0 || g.N % 64 != 0 || g.K % 32 != 0) return false;
    if ((((uintptr_t)g.A | (uintptr_t)g.B | (uintptr_t)g.C | (uintptr_t)g.bias | (uintptr_t)g.col_scale) & 15) != 0 ||
        g.lda % 4 != 0 || g.ldb % 16 != 0 || g.ldc % 4 != 0)
        return false;                                        // the fast kernels would not take it
    const int64_t tiles = (g.M / 64) * (g.N / 64);
    return g.K <= 512 || (g.K <= 768 && tiles >= 48) || (g.K <= 1536 && tiles > 64);
}

// returns -1 when the shape is left to the ordinary path
template <typename BSRC>
int try_split_k(const SgemmArgs &g, int transa, int transb, const char *name, const char *const i8_names[3]) {
    if (one_launch_on_half_tiles(g, transa)) return -1;
    const int64_t splits = split_count(g.M, g.N, g.K, !transa);
    if (splits < 2 || splits > 65535) return -1;
    const int64_t kr = g.K / splits;
    float *part = static_cast<float *>(workspace((size_t)splits * g.M * g.N * sizeof(float)));
    if (!part) return AXHIP_ERR_ALLOC;
    SgemmArgs p = g;
    p.K = kr;
    p.C = part;
    p.ldc = g.N;
    p.stride_a = transa ? kr * g.lda : kr;                 // op(A) = [M, K]: the K index runs along rows of A^T
    p.stride_b = transb ? kr : kr * g.ldb;
    p.stride_c = g.M * g.N;
    p.alpha = 1.0f;
    p.beta = 0.0f;
    p.bias = nullptr;
    p.act = AXHIP_ACT_NONE;
    int rc;
    if (std::is_same<BSRC, float>::value) rc = dispatch_f32(p, transa, transb, splits);
    else {
        rc = try_dma_i8(kI8DmaNames, p, splits);
        if (rc < 0) rc = pick_tile<true, true, int8_t>(i8_names, p, splits);
    }
    if (rc) return rc;
    const bool vec = g.N % 4 == 0 && g.ldc % 4 == 0 && (((uintptr_t)g.C | (uintptr_t)g.bias) & 15) == 0;
    const int64_t items = g.M * (vec ? g.N / 4 : g.N);
    // enough workgroups for the chip: 16 split lanes over 16 items when the result is small
    const bool wide = items >= 64 * 512 || splits < 8;
    const int64_t blocks = (items + (wide ? 63 : 15)) / (wide ? 64 : 16);
    if (blocks > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "sgemm split-k: result too large");
#define AX_FINISH(V, L)                                                                                     \
    hipLaunchKernelGGL((k_splitk_finish<V, L>), dim3((unsigned)blocks), dim3(256), 0, kStream, part, (int)splits, \
                       g.M, g.N, g.alpha, g.beta, g.bias, g.act, g.C, g.ldc)
    if (vec && wide) AX_FINISH(true, 4);
    else if (vec) AX_FINISH(true, 16);
    else if (wide) AX_FINISH(false, 4);
    else AX_FINISH(false, 16);
#undef AX_FINISH
    note_kernel(name);
    return check_launch("sgemm split-k finish");
}

int dispatch_f32(const SgemmArgs &g, int transa, int transb, int64_t batch) {
    static const char *const nn[3] = {"sgemm_nn_128x128", "sgemm_nn_64x64", "sgemm_nn_64x64_guarded"};
    static const char *const nt[3] = {"sgemm_nt_128x128", "sgemm_nt_64x64", "sgemm_nt_64x64_guarded"};
    static const char *const tn[3] = {"sgemm_tn_128x128", "sgemm_tn_64x64", "sgemm_tn_64x64_guarded"};
    static const char *const nn_d[3] = {"sgemm_nn_128x128_dma", "sgemm_nn_64x64_dma", "sgemm_nn_64x64k2_dma"};
    static const char *const nt_d[3] = {"sgemm_nt_128x128_dma", "sgemm_nt_64x64_dma", "sgemm_nt_64x64k2_dma"};
    static const char *const tn_d[3] = {"sgemm_tn_128x128_dma", "sgemm_tn_64x64_dma", "sgemm_tn_64x64k2_dma"};
    int rc = -1;
    if (!transa && transb) rc = try_nt_cols(g, batch);
    if (rc < 0 && !transa && transb) rc = try_nt_rows(g, batch);
    if (!transa && !transb) rc = try_nn_stream(g, batch);
    if (rc >= 0) return rc;
    if (!transa && !transb) rc = try_dma<true, false>(nn_d, g, batch);
    else if (!transa && transb) rc = try_dma<true, true>(nt_d, g, batch);
    else if (transa && !transb) rc = try_dma<false, false>(tn_d, g, batch);
    if (rc >= 0) return rc;
    if (!transa && !transb) return pick_tile<true, false, float>(nn, g, batch);
    if (!transa && transb) return pick_tile<true, true, float>(nt, g, batch);
    if (transa && !transb) return pick_tile<false, false, float>(tn, g, batch);
    return fail(AXHIP_ERR_NOT_IMPLEMENTED, "sgemm: A^T * B^T is not provided");
}

// A large fp32 shape off the tile grid runs on 64x64 tiles with guarded edges (4000^3: 125
// TFLOP/s against 141 for the large tiles on the grid).  When it is large enough for 128x128
// tiles, its interior on that grid goes to them and only the right and bottom fringes to the
// edge form; every block is a sub-matrix reached by pointer offsets.  Returns -1 when the shape
// is left alone.
int try_interior_and_fringes(const SgemmArgs &g, int transa, int transb) {
    if ((transa && transb) || g.K % 32 != 0 || g.K <= 0) return -1;
    if ((((uintptr_t)g.A | (uintptr_t)g.B | (uintptr_t)g.C | (uintptr_t)g.bias) & 15) != 0 || g.lda % 4 != 0 ||
        g.ldb % 4 != 0 || g.ldc % 4 != 0)
        return -1;                                           // the interior would not qualify for the fast kernels either
    if ((g.M / 128) * (g.N / 128) < 2 * (int64_t)cu_count()) return -1;
    const int64_t Mi = g.M / 128 * 128, Ni = g.N / 128 * 128;
    if (Mi == g.M && Ni == g.N) return -1;
    const float *A = static_cast<const float *>(g.A), *B = static_cast<const float *>(g.B);
    // a fringe is a strip of few tiles with the whole K: the split-K route when it qualifies
    auto fringe = [&](const SgemmArgs &f) {
        const int rc = try_split_k<float>(f, transa, transb, "sgemm_splitk", nullptr);
        return rc >= 0 ? rc : dispatch_f32(f, transa, transb, 1);
    };
    SgemmArgs p = g;
    p.M = Mi;
    p.N = Ni;
    int rc = dispatch_f32(p, transa, transb, 1);
    if (rc == AXHIP_OK && Ni < g.N) {                       // columns Ni.. of the interior's rows
        p = g;
        p.M = Mi;
        p.N = g.N - Ni;
        p.B = transb ? B + Ni * g.ldb : B + Ni;
        p.C = g.C + Ni;
        if (g.bias) p.bias = g.bias + Ni;
        rc = fringe(p);
    }
    if (rc == AXHIP_OK && Mi < g.M) {                       // rows Mi.., every column
        p = g;
        p.M = g.M - Mi;
        p.A = transa ? A + Mi : A + Mi * g.lda;
        p.C = g.C + Mi * g.ldc;
        rc = fringe(p);
    }
    note_kernel("sgemm_interior+fringes");
    return rc;
}

int run_f32(const SgemmArgs &g, int transa, int transb);

// K off the 32 grid keeps a large product off every fast kernel.  It is run as the product over the
// first K / 32 * 32 columns (alpha and beta as given, no bias or activation yet) followed by the
// few remaining columns accumulated on top (beta = 1) with the bias and activation of the whole.
// Returns -1 when the shape is left alone.
int try_k_tail(const SgemmArgs &g, int transa, int transb) {
    const int64_t Km = g.K / 32 * 32;
    if ((transa && transb) || Km == g.K || Km < 256) return -1;
    // K a multiple of 4 runs in one pass on the 64x64 tiles with guarded edges, which take a K tail
    // themselves; two passes are for the other K and for shapes whose main part earns 128x128 tiles
    if (g.K % 4 == 0 && (g.M / 128) * (g.N / 128) < 2 * (int64_t)cu_count()) return -1;
    const float *A = static_cast<const float *>(g.A), *B = static_cast<const float *>(g.B);
    SgemmArgs p = g;
    p.K = Km;
    p.bias = nullptr;
    p.act = AXHIP_ACT_NONE;
    int rc = run_f32(p, transa, transb);
    if (rc != AXHIP_OK) return rc;
    p = g;
    p.K = g.K - Km;
    p.A = transa ? A + Km * g.lda : A + Km;
    p.B = transb ? B + Km : B + Km * g.ldb;
    p.beta = 1.0f;
    rc = dispatch_f32(p, transa, transb, 1);
    note_kernel("sgemm_main+k_tail");
    return rc;
}

// a single product: the route for its shape
int run_f32(const SgemmArgs &g, int transa, int transb) {
    if (!(transa && transb)) {
        int rc = try_split_k<float>(g, transa, transb, "sgemm_splitk", nullptr);
        if (rc >= 0) return rc;
        rc = try_interior_and_fringes(g, transa, transb);
        if (rc >= 0) return rc;
        rc = try_k_tail(g, transa, transb);
        if (rc >= 0) return rc;
    }
    return dispatch_f32(g, transa, transb, 1);
}

}  // namespace

namespace axhip {
// W8A32 through the matrix cores: B is int8 [N,K].  The direct-to-LDS tiles multiply on the bf16 matrix core
// (try_dma_i8); shapes they do not take (K off the 32 grid, unaligned rows) convert B to fp32 while it is staged.
int sgemm_i8w(int64_t M, int64_t N, int64_t K, const float *a, const int8_t *w,
              const float *w_scales, float *out) {
    static const char *const names[3] = {"qgemm_w8a32_mfma_128x128", "qgemm_w8a32_mfma_64x64",
                                         "qgemm_w8a32_mfma_64x64_guarded"};
    SgemmArgs g{a, w, out, M, N, K, K, K, N, 0, 0, 0, 1.0f, 0.0f, w_scales, nullptr, AXHIP_ACT_NONE};
    auto run = [&](const SgemmArgs &p) {
        const int rc = try_split_k<int8_t>(p, 0, 1, "qgemm_w8a32_mfma_splitk", names);
        if (rc >= 0) return rc;
        const int rd = try_dma_i8(kI8DmaNames, p, 1);
        return rd >= 0 ? rd : pick_tile<true, true, int8_t>(names, p, 1);
    };
    // K off the 32 grid cannot be cut into ranges: the first K / 32 * 32 columns as above, then the
    // remaining few accumulated on top (the column scale applies to each part's sum alike)
    const int64_t Km = K / 32 * 32;
    if (Km != K && Km >= 512) {
        SgemmArgs p = g;
        p.K = Km;
        int rc = run(p);
        if (rc != AXHIP_OK) return rc;
        p = g;
        p.K = K - Km;
        p.A = a + Km;
        p.B = w + Km;
        p.beta = 1.0f;
        rc = pick_tile<true, true, int8_t>(names, p, 1);
        note_kernel("qgemm_w8a32_mfma_main+k_tail");
        return rc;
    }
    return run(g);
}
}  // namespace axhip

extern "C" int axhip_sgemm(int transa, int transb, int64_t M, int64_t N, int64_t K, float alpha,
                           const float *A, int64_t lda, const float *B, int64_t ldb, float beta,
                           float *C, int64_t ldc, const float *bias, int act) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (int rc = validate("sgemm", transa, transb, M, N, K, A, lda, B, ldb, C, ldc, act)) return rc;
    if (M == 0 || N == 0) return AXHIP_OK;
    // M = 9..16 on whole tiles: the 32x64 tiles with their K split are level with the streaming kernel at 4096 x 4096
    // and ahead on larger weights (M = 16, operands cached / from HBM: 11008 x 4096 41.1 / 48.4 -> 31.5 / 38.2 us,
    // 8192 x 8192 57.1 / 64.3 -> 48.9 / 55.7, 32000 x 4096 124 -> 101, 1024 x 1024 10.0 -> 8.0); off the tile grid the
    // streaming kernel stays ahead (4096 x 784: 10.8 against 10.9 cached, 12.6 against 18.8 from HBM)
    const bool tiles_for_rows = M >= 9 && K % 32 == 0 && N % 64 == 0;
    if (M <= 16 && !tiles_for_rows && !transa && !transb && alpha == 1.0f && beta == 0.0f)
        return axhip_sgemm_skinny(M, N, K, A, lda, B, ldb, C, ldc, bias, act);
    SgemmArgs g{A, B, C, M, N, K, lda, ldb, ldc, 0, 0, 0, alpha, beta, nullptr, bias, act};
    return run_f32(g, transa, transb);
}

extern "C" int axhip_sgemm_strided_batched(int transa, int transb, int64_t M, int64_t N, int64_t K,
                                           float alpha, const float *A, int64_t lda,
                                           int64_t stride_a, const float *B, int64_t ldb,
                                           int64_t stride_b, float beta, float *C, int64_t ldc,
                                           int64_t stride_c, int64_t batch) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (int rc = validate("sgemm_strided_batched", transa, transb, M, N, K, A, lda, B, ldb, C, ldc,
                          AXHIP_ACT_NONE))
        return rc;
    if (batch < 0 || stride_a < 0 || stride_b < 0 || stride_c < 0)
        return fail(AXHIP_ERR_SHAPE, "sgemm_strided_batched: negative batch or stride");
    if (M == 0 || N == 0 || batch == 0) return AXHIP_OK;
    // the batch index is the grid's second dimension (at most 65535): longer batches go in pieces
    constexpr int64_t kMostPerLaunch = 65535;
    for (int64_t b0 = 0; b0 < batch; b0 += kMostPerLaunch) {
        const int64_t nb = batch - b0 < kMostPerLaunch ? batch - b0 : kMostPerLaunch;
        SgemmArgs g{A + b0 * stride_a, B + b0 * stride_b, C + b0 * stride_c, M, N, K, lda, ldb, ldc, stride_a, stride_b,
                    stride_c, alpha, beta, nullptr, nullptr, AXHIP_ACT_NONE};
        if (int rc = dispatch_f32(g, transa, transb, nb)) return rc;
    }
    return AXHIP_OK;
}
