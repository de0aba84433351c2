// W8A32: out[m,n] = w_scales[n] * sum_k a[m,k] * (float)w[n,k], fp32 accumulation.
//
// M <= 8 (the bandwidth-bound inference case): one wave owns 4 weight rows.  Lanes walk K in
// 16-element steps (a wave-wide load covers 1 KiB of one row), each lane keeps the activations of
// its k positions in registers across the 4 rows, and the 4*M partial sums are reduced over
// the wave together, in a fixed tree order, ending one per lane for the write-back.  Larger M goes through the fp32
// matrix-core GEMM with the int8 operand converted while it is staged in LDS.
#include "common.h"

namespace axhip {
int sgemm_i8w(int64_t M, int64_t N, int64_t K, const float *a, const int8_t *w,
              const float *w_scales, float *out);
}

namespace {
using namespace axhip;

constexpr int ROWS = 4;   // weight rows per wave

template <int MR>
__global__ void __launch_bounds__(64)
k_w8a32_gemv(const float *__restrict__ a, const int8_t *__restrict__ w,
             const float *__restrict__ w_scales, float *__restrict__ out, int64_t N, int64_t K) {
    const int lane = threadIdx.x;
    const int64_t n0 = (int64_t)blockIdx.x * ROWS;
    float acc[ROWS][MR];
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int m = 0; m < MR; m++) acc[r][m] = 0.0f;

    for (int64_t k = (int64_t)lane * 16; k < K; k += 64 * 16) {
        // A step wholly inside the row is fetched with 16-byte loads at whatever alignment K and
        // the base pointers leave (global memory takes unaligned vector loads); only the last,
        // partial step of a row goes element by element.
        const bool whole = k + 16 <= K;
        float xa[MR][16];
        if (whole) {
#pragma unroll
            for (int m = 0; m < MR; m++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    v4f t;
                    __builtin_memcpy(&t, a + m * K + k + 4 * q, 16);
                    xa[m][4 * q] = t.x; xa[m][4 * q + 1] = t.y; xa[m][4 * q + 2] = t.z; xa[m][4 * q + 3] = t.w;
                }
        } else {
#pragma unroll
            for (int m = 0; m < MR; m++)
#pragma unroll
                for (int e = 0; e < 16; e++) xa[m][e] = (k + e < K) ? a[m * K + k + e] : 0.0f;
        }
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const int64_t n = n0 + r;
            if (n >= N) break;
            float wf[16];
            if (whole) {
                v4i p;
                __builtin_memcpy(&p, w + n * K + k, 16);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int word = p[q];
                    wf[4 * q] = (float)(signed char)(word & 0xff);
                    wf[4 * q + 1] = (float)(signed char)((word >> 8) & 0xff);
                    wf[4 * q + 2] = (float)(signed char)((word >> 16) & 0xff);
                    wf[4 * q + 3] = (float)(signed char)((word >> 24) & 0xff);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 16; e++) wf[e] = (k + e < K) ? (float)w[n * K + k + e] : 0.0f;
            }
#pragma unroll
            for (int m = 0; m < MR; m++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[r][m] = __builtin_fmaf(xa[m][e], wf[e], acc[r][m]);
        }
    }
    constexpr int NV = ROWS * MR <= 4 ? 4 : ROWS * MR <= 8 ? 8 : ROWS * MR <= 16 ? 16 : 32;
    float v[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) v[i] = i < ROWS * MR ? acc[i / MR][i % MR] : 0.0f;
    wave_sum_spread(v, lane);
    const int idx = lane / (64 / NV), r = idx / MR, m = idx % MR;
    if (lane % (64 / NV) != 0 || idx >= ROWS * MR || n0 + r >= N) return;
    out[m * N + n0 + r] = v[0] * w_scales[n0 + r];
}

template <int MR>
int launch_gemv(const float *a, const int8_t *w, const float *s, float *out, int64_t N, int64_t K) {
    dim3 grid((unsigned)((N + ROWS - 1) / ROWS));
    hipLaunchKernelGGL(k_w8a32_gemv<MR>, grid, dim3(64), 0, kStream, a, w, s, out, N, K);
    return check_launch("qgemm_w8a32_gemv");
}
}  // namespace

extern "C" int axhip_qgemm_w8a32(const float *a, const int8_t *w, const float *w_scales, float *out,
                                 int64_t M, int64_t N, int64_t K) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!a || !w || !w_scales || !out) return fail(AXHIP_ERR_NULL_ARG, "qgemm_w8a32: NULL");
    if (M < 0 || N < 0 || K < 0) return fail(AXHIP_ERR_SHAPE, "qgemm_w8a32: negative dimension");
    if (M == 0 || N == 0) return AXHIP_OK;
    if (M > 8) return axhip::sgemm_i8w(M, N, K, a, w, w_scales, out);
    if ((N + ROWS - 1) / ROWS > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "qgemm_w8a32: N too large");
    note_kernel("qgemm_w8a32_gemv");
    switch (M) {
        case 1: return launch_gemv<1>(a, w, w_scales, out, N, K);
        case 2: return launch_gemv<2>(a, w, w_scales, out, N, K);
        case 3: return launch_gemv<3>(a, w, w_scales, out, N, K);
        case 4: return launch_gemv<4>(a, w, w_scales, out, N, K);
        case 5: return launch_gemv<5>(a, w, w_scales, out, N, K);
        case 6: return launch_gemv<6>(a, w, w_scales, out, N, K);
        case 7: return launch_gemv<7>(a, w, w_scales, out, N, K);
        default: return launch_gemv<8>(a, w, w_scales, out, N, K);
    }
}
