// int8 x int8 -> int32 GEMM (W8A8) with fused dequantize + bias + activation write-back.
//
//   acc[m,n] = sum_k x[m,k] * w[n,k]          x: [M,K] int8, w: [N,K] int8 (both K-contiguous)
//   out[m,n] = act((float)acc * (x_scale*w_scale[n]) + bias[n])
//
// One workgroup owns a BM x BN tile of the output and walks K in slabs of 128 bytes.
// Slabs are fetched with 16-byte global loads (8 consecutive lanes cover one 128-byte row
// segment), staged through registers into a double-buffered LDS tile, and consumed by
// v_mfma_i32_32x32x32_i8: lane l supplies row (l & 31), bytes [16*(l>>5), +16) of each
// 32-byte k-step.  Because A and B fragments use the same byte placement the integer dot
// product is exact whatever order the matrix core sums in.
//
// LDS rows are 128 bytes = 32 banks, so the 16-byte chunk index is XOR-swizzled with
// (row >> 1) & 7: the 16 lanes served together by a ds_read_b128 (16 consecutive rows, one
// chunk) and the 16 lanes of a ds_write_b128 (2 rows x 8 chunks) then touch 64 distinct banks.
#include "common.h"

namespace {
using namespace axhip;

constexpr int BK = 128;   // bytes of K per slab

__device__ __forceinline__ int swz(int row, int chunk) {
    return row * BK + ((chunk ^ ((row >> 1) & 7)) << 4);
}

template <bool GUARD>
__device__ __forceinline__ v4i load_chunk(const int8_t *base, int64_t row, int64_t rows,
                                          int64_t k, int64_t K, bool vec_ok) {
    if (!GUARD) return *reinterpret_cast<const v4i *>(base + row * K + k);
    v4i r = {0, 0, 0, 0};
    if (row >= rows || k >= K) return r;
    const int8_t *p = base + row * K + k;
    if (vec_ok && k + 16 <= K) return *reinterpret_cast<const v4i *>(p);
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
             int32_t *__restrict__ acc_out) {
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

    const bool vec_ok = !GUARD || ((((uintptr_t)X | (uintptr_t)W | (uintptr_t)K) & 15) == 0);
    const int64_t slabs = (K + BK - 1) / BK;

    v4i ra[CA], rb[CB];
    auto fetch = [&](int64_t slab) {
        const int64_t k0 = slab * BK;
#pragma unroll
        for (int i = 0; i < CA; i++) {
            int c = tid + i * T;
            ra[i] = load_chunk<GUARD>(X, m0 + (c >> 3), M, k0 + ((c & 7) << 4), K, vec_ok);
        }
#pragma unroll
        for (int i = 0; i < CB; i++) {
            int c = tid + i * T;
            rb[i] = load_chunk<GUARD>(W, n0 + (c >> 3), N, k0 + ((c & 7) << 4), K, vec_ok);
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
                if (acc_out) acc_out[row * N + col] = a;
                if (out) {
                    float f = (float)a;
                    float r = bias ? __builtin_fmaf(f, scale, bv) : f * scale;
                    out[row * N + col] = apply_act(r, act);
                }
            }
        }
    }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool GUARD>
int launch(const char *name, const int8_t *x, float x_scale, const int8_t *w,
           const float *w_scales, const float *bias, int act, float *out, int32_t *acc_out,
           int64_t M, int64_t N, int64_t K) {
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
                       w, M, N, K, x_scale, w_scales, bias, act, out, acc_out);
    return check_launch(name);
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
    const bool aligned = ((((uintptr_t)x | (uintptr_t)w) & 15) == 0) && (K % BK == 0) && K > 0;
    if (aligned && M % 256 == 0 && N % 256 == 0 && (M / 256) * (N / 256) >= 128)
        return launch<256, 256, 2, 4, false>("qgemm_w8a8_256x256", x, x_scale, w, w_scales, bias,
                                             act, out, acc_out, M, N, K);
    if (aligned && M % 128 == 0 && N % 128 == 0)
        return launch<128, 128, 2, 2, false>("qgemm_w8a8_128x128", x, x_scale, w, w_scales, bias,
                                             act, out, acc_out, M, N, K);
    return launch<64, 64, 2, 2, true>("qgemm_w8a8_64x64_guarded", x, x_scale, w, w_scales, bias,
                                      act, out, acc_out, M, N, K);
}
