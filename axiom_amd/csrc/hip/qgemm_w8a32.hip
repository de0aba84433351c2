// W8A32: out[m,n] = w_scales[n] * sum_k a[m,k] * (float)w[n,k], fp32 accumulation.
//
// M = 2..6 (the bandwidth-bound inference case) streams the weights once.  A workgroup of four waves owns
// 4 * R consecutive weight rows, a wave R of them over all of K.  K is walked in windows of 1024: a
// wave-wide 16-byte load covers 1 KiB of one row, lane l the k values 16 l .. 16 l + 15 of the window.
// The activations of a slice of K sit in LDS, laid out so that the four 16-byte reads a lane makes per
// window and activation row are consecutive across lanes; a lane turns its 16 weight bytes of each of the
// R rows into floats and multiplies them into R * M running sums.  Weights of the next U windows
// (R * U = 8 loads of 16 bytes per lane) are requested before the current ones are used, and the first
// batch before the activations are staged, so 16 KiB per wave are in flight throughout.  The R * M sums
// are added over the wave together in a fixed tree order and end one per lane for the write-back.
// Rows at any byte alignment and any K: whole 16-byte steps are fetched with one load wherever the row
// starts (global memory takes unaligned vector loads), the last partial step byte by byte.
// M = 1, and up to four rows against fewer than 16384 weight rows, take a form without LDS (below).  Larger M goes through the fp32 matrix-core GEMM with the
// int8 operand converted while it is staged.
#include "common.h"

namespace axhip {
int sgemm_i8w(int64_t M, int64_t N, int64_t K, const float *a, const int8_t *w,
              const float *w_scales, float *out);
}

namespace {
using namespace axhip;

// windows requested together: 8 loads per lane in all, less where M activation rows leave no room for more in LDS
template <int MR, int R> constexpr int windows_per_step() {
    constexpr int most = MR <= 2 ? 8 : MR <= 4 ? 4 : 2;
    return 8 / R < most ? 8 / R : most;
}

// 16 weight bytes at any alignment.  STREAM marks the load non-temporal: every weight byte is read once per launch, and
// large weights that come from HBM arrive faster that way (M = 1, weights in rotation: 4096 x 11008 16.2 -> 14.7 us,
// 32000 x 4096 28.2 -> 26.4, 8192 x 8192 16.0 -> 15.3, 11008 x 4096 13.6 -> 13.3; M = 4, 32000 x 4096 50.9 -> 45.8), while
// one matrix multiplied again and again out of the Infinity Cache loses as much (8192 x 4096, 33.5 MB: 6.5 -> 9.0 us
// against 11.6 -> 11.5 from HBM).  The launchers set it from 40 MiB of weights on.
typedef int v4i_any __attribute__((ext_vector_type(4), aligned(1)));
template <bool STREAM>
__device__ __forceinline__ v4i load16(const int8_t *p) {
    if (STREAM) return __builtin_nontemporal_load(reinterpret_cast<const v4i_any *>(p));
    v4i v;
    __builtin_memcpy(&v, p, 16);
    return v;
}

template <int R, int U, bool STREAM>
__device__ __forceinline__ void w8a32_request(v4i (&dst)[R][U], const int8_t *w, int64_t first_row, int64_t N, int64_t k0, int lane,
                                              int64_t K, int used) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        if (u >= used) break;                                   // uniform: a short K fills fewer windows per step
        const int64_t k = k0 + (int64_t)u * 1024 + lane * 16;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int64_t n = first_row + r < N ? first_row + r : N - 1;     // rows past N repeat the last one, unstored
            const int8_t *row = w + n * K;
            v4i p = {0, 0, 0, 0};
            if (k + 16 <= K) {
                p = load16<STREAM>(row + k);
            } else if (k < K) {
#pragma unroll
                for (int e = 0; e < 16; e++)
                    if (k + e < K) p[e >> 2] |= (int)(unsigned char)row[k + e] << (8 * (e & 3));
            }
            dst[r][u] = p;
        }
    }
}

template <int MR, int R, int U>
__device__ __forceinline__ void w8a32_multiply(const v4i (&src)[R][U], float (&acc)[R][MR], const v4f *xs, int quads_per_row,
                                               int window0, int lane, int used) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        if (u >= used) break;
        v4f xa[MR][4];
#pragma unroll
        for (int m = 0; m < MR; m++)
#pragma unroll
            for (int q = 0; q < 4; q++) xa[m][q] = xs[m * quads_per_row + ((window0 + u) * 4 + q) * 64 + lane];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int word = src[r][u][q];
                const float f0 = (float)(signed char)(word & 0xff), f1 = (float)(signed char)((word >> 8) & 0xff),
                            f2 = (float)(signed char)((word >> 16) & 0xff), f3 = (float)(signed char)((word >> 24) & 0xff);
#pragma unroll
                for (int m = 0; m < MR; m++) {
                    float s = acc[r][m];
                    s = __builtin_fmaf(xa[m][q].x, f0, s);
                    s = __builtin_fmaf(xa[m][q].y, f1, s);
                    s = __builtin_fmaf(xa[m][q].z, f2, s);
                    s = __builtin_fmaf(xa[m][q].w, f3, s);
                    acc[r][m] = s;
                }
            }
    }
}

// slice: k values of the activations held in LDS at a time, a multiple of used * 1024.  groups: row groups of 4 * R
// rows a workgroup walks one after the other (more than one only when a single slice holds all of K, so the
// activations are staged once); the weight requests run ahead across group boundaries.
template <int MR, int R, bool STREAM>
__global__ void __launch_bounds__(256)
k_w8a32_rows(const float *__restrict__ a, const int8_t *__restrict__ w, const float *__restrict__ w_scales,
             float *__restrict__ out, int64_t N, int64_t K, int slice, int groups, int used) {
    constexpr int U = windows_per_step<MR, R>();
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    v4f *xs = reinterpret_cast<v4f *>(lds_raw);                 // [MR][slice / 4], permuted inside each window
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t base = (int64_t)blockIdx.x * groups * (4 * R) + wave * R;      // this wave's rows of group g: base + g * 4 R
    float acc[R][MR];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < MR; m++) acc[r][m] = 0.0f;

    const int span = used * 1024;                               // k values of a step: `used` <= U windows
    const int quads = slice / 4, steps_per_slice = slice / span;
    const int steps = (int)((K + span - 1) / span);
    // activations of slice s -> LDS: 16-byte piece q of lane l's 16 values of window v at quad (4 v + q) * 64 + l
    auto stage = [&](int64_t s) {
        for (int f = tid; f < MR * quads; f += 256) {
            const int m = f / quads, fr = f - m * quads;
            const int v = fr >> 8, q = (fr >> 6) & 3, l = fr & 63;
            const int64_t k = s * slice + v * 1024 + l * 16 + q * 4;
            v4f t = {0.f, 0.f, 0.f, 0.f};
            if (k + 4 <= K) {
                __builtin_memcpy(&t, a + m * K + k, 16);
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (k + e < K) t[e] = a[m * K + k + e];
            }
            xs[f] = t;
        }
    };
    // the sums of a finished group: added over the wave in a fixed tree, one result per lane, scaled and stored
    auto finish = [&](int64_t first_row) {
        constexpr int NV = R * MR <= 1 ? 1 : R * MR <= 2 ? 2 : R * MR <= 4 ? 4 : R * MR <= 8 ? 8 : R * MR <= 16 ? 16 : 32;
        float v[NV];
#pragma unroll
        for (int i = 0; i < NV; i++) v[i] = i < R * MR ? acc[i / MR][i % MR] : 0.0f;
        wave_sum_spread(v, lane);
        const int idx = lane / (64 / NV), r = idx / MR, m = idx % MR;
        if (lane % (64 / NV) == 0 && idx < R * MR && first_row + r < N) out[m * N + first_row + r] = v[0] * w_scales[first_row + r];
#pragma unroll
        for (int rr = 0; rr < R; rr++)
#pragma unroll
            for (int mm = 0; mm < MR; mm++) acc[rr][mm] = 0.0f;
    };
    v4i wa[R][U], wb[R][U];
    w8a32_request<R, U, STREAM>(wa, w, base, N, 0, lane, K, used);      // before the activations: the latency of both overlaps
    // One flat walk over (group, step): every quantity below is uniform over the workgroup.  Two steps per
    // round so that the two weight buffers keep their names.
    int g = 0, it = 0, in_slice = steps_per_slice;              // "slice full" forces the first staging
    int64_t s = 0;
    const int total = groups * steps;
    auto enter = [&]() {                                        // the slice of step `it` is in LDS
        if (in_slice == steps_per_slice && (groups == 1 || (g == 0 && it == 0))) {
            __syncthreads();
            stage(s++);
            __syncthreads();
            in_slice = 0;
        }
    };
    auto advance = [&]() {                                      // after a step: the group ends with its last one
        ++it;
        ++in_slice;
        if (it == steps) {
            finish(base + (int64_t)g * (4 * R));
            it = 0;
            ++g;
            if (groups > 1) in_slice = 0;                       // one slice holds all of K: start over in it
            else { in_slice = steps_per_slice; s = 0; }
        }
    };
    for (int t = 0; t < total;) {
        enter();
        if (t + 1 < total) {
            const bool wrap = it + 1 == steps;
            w8a32_request<R, U, STREAM>(wb, w, base + (int64_t)(g + wrap) * (4 * R), N, wrap ? 0 : (int64_t)(it + 1) * span, lane, K, used);
        }
        w8a32_multiply<MR, R, U>(wa, acc, xs, quads, in_slice * used, lane, used);
        advance();
        if (++t >= total) break;
        enter();
        if (t + 1 < total) {
            const bool wrap = it + 1 == steps;
            w8a32_request<R, U, STREAM>(wa, w, base + (int64_t)(g + wrap) * (4 * R), N, wrap ? 0 : (int64_t)(it + 1) * span, lane, K, used);
        }
        w8a32_multiply<MR, R, U>(wb, acc, xs, quads, in_slice * used, lane, used);
        advance();
        ++t;
    }
}

// ---- M = 1 (and up to four rows against fewer than 16384 weight rows) ------------------------------
// One activation row needs no LDS: a lane's 16 activations of a window are 64 bytes that every wave of the
// chip reads from cache, so they travel with the weight requests (two buffers of R * U weight loads and 4 U
// activation loads per lane) and no workgroup waits for a staging pass before its stream starts (same box, LDS form
// -> this one, cached / weights from HBM: 4096 x 4096 5.0 / 7.2 -> 4.6 / 5.9 us, 8192 x 8192 16.2 / 18.1 -> 13.2 / 15.9,
// 32000 x 4096 24.7 / 29.6 -> 22.7 / 28.0, 4096 x 11008 14.7 / 18.3 -> 11.9 / 15.2).  Otherwise the walk of the form above.
template <int MR, int R, int U>
struct W8a32DirectBuf {
    v4i w[R][U];
    v4f x[MR][U][4];
};

template <int MR, int R, int U, bool STREAM>
__device__ __forceinline__ void w8a32_direct_request(W8a32DirectBuf<MR, R, U> &b, const float *a, const int8_t *w, int64_t first_row,
                                                     int64_t N, int64_t k0, int lane, int64_t K, int used) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        if (u >= used) break;
        const int64_t k = k0 + (int64_t)u * 1024 + lane * 16;
#pragma unroll
        for (int m = 0; m < MR; m++) {
#pragma unroll
            for (int q = 0; q < 4; q++) b.x[m][u][q] = v4f{0.f, 0.f, 0.f, 0.f};
            if (k + 16 <= K) {
#pragma unroll
                for (int q = 0; q < 4; q++) __builtin_memcpy(&b.x[m][u][q], a + m * K + k + 4 * q, 16);
            } else if (k < K) {
#pragma unroll
                for (int q = 0; q < 4; q++)
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (k + 4 * q + e < K) b.x[m][u][q][e] = a[m * K + k + 4 * q + e];
            }
        }
    }
    w8a32_request<R, U, STREAM>(b.w, w, first_row, N, k0, lane, K, used);
}

template <int MR, int R, int U>
__device__ __forceinline__ void w8a32_direct_multiply(const W8a32DirectBuf<MR, R, U> &b, float (&acc)[R][MR], int used) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        if (u >= used) break;
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int word = b.w[r][u][q];
                const float f0 = (float)(signed char)(word & 0xff), f1 = (float)(signed char)((word >> 8) & 0xff),
                            f2 = (float)(signed char)((word >> 16) & 0xff), f3 = (float)(signed char)((word >> 24) & 0xff);
#pragma unroll
                for (int m = 0; m < MR; m++) {
                    float s = acc[r][m];
                    s = __builtin_fmaf(b.x[m][u][q].x, f0, s);
                    s = __builtin_fmaf(b.x[m][u][q].y, f1, s);
                    s = __builtin_fmaf(b.x[m][u][q].z, f2, s);
                    s = __builtin_fmaf(b.x[m][u][q].w, f3, s);
                    acc[r][m] = s;
                }
            }
    }
}

template <int MR, int R, int U, bool STREAM>
__global__ void __launch_bounds__(256)
k_w8a32_direct(const float *__restrict__ a, const int8_t *__restrict__ w, const float *__restrict__ w_scales,
               float *__restrict__ out, int64_t N, int64_t K, int groups, int used) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t base = (int64_t)blockIdx.x * groups * (4 * R) + wave * R;
    float acc[R][MR];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < MR; m++) acc[r][m] = 0.0f;
    const int span = used * 1024;
    const int steps = (int)((K + span - 1) / span), total = groups * steps;
    W8a32DirectBuf<MR, R, U> ba, bb;
    w8a32_direct_request<MR, R, U, STREAM>(ba, a, w, base, N, 0, lane, K, used);
    int g = 0, it = 0;
    auto finish = [&]() {                                       // the group's R * MR sums: over the wave, scaled, stored
        constexpr int NV = R * MR <= 1 ? 1 : R * MR <= 2 ? 2 : R * MR <= 4 ? 4 : R * MR <= 8 ? 8 : 16;
        static_assert(R * MR <= 16, "sums per wave");
        float v[NV];
#pragma unroll
        for (int i = 0; i < NV; i++) v[i] = i < R * MR ? acc[i / MR][i % MR] : 0.0f;
        wave_sum_spread(v, lane);
        const int idx = lane / (64 / NV), r = idx / MR, m = idx % MR;
        const int64_t n = base + (int64_t)g * (4 * R) + r;
        if (lane % (64 / NV) == 0 && idx < R * MR && n < N) out[m * N + n] = v[0] * w_scales[n];
#pragma unroll
        for (int rr = 0; rr < R; rr++)
#pragma unroll
            for (int mm = 0; mm < MR; mm++) acc[rr][mm] = 0.0f;
    };
    auto next_request = [&](W8a32DirectBuf<MR, R, U> &b) {      // operands of the step after (g, it)
        const bool wrap = it + 1 == steps;
        w8a32_direct_request<MR, R, U, STREAM>(b, a, w, base + (int64_t)(g + wrap) * (4 * R), N, wrap ? 0 : (int64_t)(it + 1) * span, lane, K,
                                       used);
    };
    auto advance = [&]() {
        if (++it == steps) {
            finish();
            it = 0;
            ++g;
        }
    };
    for (int t = 0; t < total;) {
        if (t + 1 < total) next_request(bb);
        w8a32_direct_multiply<MR, R, U>(ba, acc, used);
        advance();
        if (++t >= total) break;
        if (t + 1 < total) next_request(ba);
        w8a32_direct_multiply<MR, R, U>(bb, acc, used);
        advance();
        ++t;
    }
}

template <int MR, int R, int U>
int launch_direct(const float *a, const int8_t *w, const float *s, float *out, int64_t N, int64_t K) {
    const int64_t windows = (K + 1023) / 1024;
    int used = U;
    while (used > 1 && used / 2 >= windows) used /= 2;
    int64_t groups = N / (4 * R * 2 * (int64_t)cu_count());     // as many as still leave two workgroups for every CU
    if (groups < 1) groups = 1;
    if (groups > 64) groups = 64;
    const int64_t rows_per_block = 4 * R * groups, blocks = (N + rows_per_block - 1) / rows_per_block;
    if (N * K >= (int64_t(40) << 20))
        hipLaunchKernelGGL((k_w8a32_direct<MR, R, U, true>), dim3((unsigned)blocks), dim3(256), 0, kStream, a, w, s, out, N, K, (int)groups, used);
    else
        hipLaunchKernelGGL((k_w8a32_direct<MR, R, U, false>), dim3((unsigned)blocks), dim3(256), 0, kStream, a, w, s, out, N, K, (int)groups, used);
    return check_launch("qgemm_w8a32_gemv");
}

template <int MR, int R>
int launch_rows(const float *a, const int8_t *w, const float *s, float *out, int64_t N, int64_t K) {
    constexpr int U = windows_per_step<MR, R>();
    // windows of 1024 k a step takes: all U the registers allow, fewer when K does not fill them
    const int64_t windows = (K + 1023) / 1024;
    int used = U;
    while (used > 1 && used / 2 >= windows) used /= 2;
    const int64_t span = (int64_t)used * 1024;
    // up to 64 KiB of activations at a time (two workgroups share a CU), no more than K needs
    int64_t slice = (16384 / MR) / span * span;
    const int64_t need = (K + span - 1) / span * span;
    if (slice > need) slice = need;
    // With all of K in one slice a workgroup stages the activations once and walks several row groups, as
    // many as still leave two workgroups for every CU (M = 1: 32000 x 4096 30.1 -> 25.3 us, 16384 x 4096
    // 17.8 -> 15.2 against one group each; with short rows one group each stays ahead, 50000 x 2048: 18.5 against 20.9).
    int64_t groups = 1;
    if (slice == need) {
        groups = N / (4 * R * 2 * (int64_t)cu_count());
        if (groups < 1) groups = 1;
        if (groups > 64) groups = 64;
    }
    const size_t smem = (size_t)MR * slice * sizeof(float);
    const bool stream = N * K >= (int64_t(40) << 20);
    auto kern = stream ? k_w8a32_rows<MR, R, true> : k_w8a32_rows<MR, R, false>;
    static bool attr_set = false;
    if (!attr_set) {
        AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(k_w8a32_rows<MR, R, true>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 65536), "hipFuncSetAttribute");
        AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(k_w8a32_rows<MR, R, false>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 65536), "hipFuncSetAttribute");
        attr_set = true;
    }
    const int64_t rows_per_block = 4 * R * groups, blocks = (N + rows_per_block - 1) / rows_per_block;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), smem, kStream, a, w, s, out, N, K, (int)slice, (int)groups, used);
    return check_launch("qgemm_w8a32_gemv");
}

// Rows per wave: as many as still leave two workgroups for every CU (fewer, fuller workgroups measured slower at
// every M: 8 x 4096 x 4096 on four rows per wave and one workgroup per CU 20.6 us against 13.6).
template <int MR>
int launch_gemv(const float *a, const int8_t *w, const float *s, float *out, int64_t N, int64_t K) {
    const int64_t cus = cu_count();
    if constexpr (MR == 1) {
        // rows per wave x windows per request, by sweep (cached / weights from HBM, us): 32000 x 4096 on 4 x 1 22.7 / 28.0
        // (2 x 2: 30.0 / 39.6), 8192 x 8192 13.2 / 15.9, 4096 x 4096 on 2 x 4 4.6 / 5.9 (4 x 2: 4.8 / 8.0), 4096 x 11008 11.9 / 15.2
        if (N >= 32 * cus) return launch_direct<1, 4, 1>(a, w, s, out, N, K);
        if (N >= 16 * cus) return launch_direct<1, 2, 4>(a, w, s, out, N, K);
        if (N >= 8 * cus) return launch_direct<1, 2, 2>(a, w, s, out, N, K);
        return launch_direct<1, 1, 2>(a, w, s, out, N, K);
    }
    if constexpr (MR >= 2 && MR <= 4) {
        // up to four rows the same form without LDS is level or ahead below N = 16384 (cached / from HBM, M = 4:
        // 11008 x 4096 23.3 / 25.0 -> 19.2 / 20.8 us, 4096 x 11008 31.1 / 34.2 -> 23.5 / 25.4, 4096 x 4096 9.0 / 11.3 ->
        // 9.0 / 10.3); beyond, the staged form keeps the lead (32000 x 4096: 46.0 / 51.1 against 51.1 / 56.2)
        if (N < 64 * cus) {
            if (MR == 2 && N < 32 * cus) return launch_direct<MR, 2, 1>(a, w, s, out, N, K);
            return launch_direct<MR, 4, 1>(a, w, s, out, N, K);
        }
    }
    if (N >= 64 * cus) return launch_rows<MR, 4>(a, w, s, out, N, K);
    // eight rows of activations leave room for two workgroups per CU only: two weight rows per wave from 2560 on, so that one
    // round of workgroups covers N (M = 8, 3072 x 768: 9.7 -> 6.7 us; 2048 x 2048 stays on one, 7.2 against 8.0)
    if (N >= 16 * cus || (MR >= 8 && N >= 10 * cus)) return launch_rows<MR, 2>(a, w, s, out, N, K);
    return launch_rows<MR, 1>(a, w, s, out, N, K);
}

}  // namespace

extern "C" int axhip_qgemm_w8a32(const float *a, const int8_t *w, const float *w_scales, float *out,
                                 int64_t M, int64_t N, int64_t K) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!a || !w || !w_scales || !out) return fail(AXHIP_ERR_NULL_ARG, "qgemm_w8a32: NULL");
    if (M < 0 || N < 0 || K < 0) return fail(AXHIP_ERR_SHAPE, "qgemm_w8a32: negative dimension");
    if (M == 0 || N == 0) return AXHIP_OK;
    // The weight-streaming form pays M multiply-adds per weight byte on the vector ALU (4096 x 4096: 4.6 us at
    // M = 1, +1.4 us per further row); from M = 7 on the matrix-core tiles are level or ahead wherever K is long, and with a
    // long K already at M = 6, at M = 5 for large weights (us, streaming against tiles — M = 6: 4096 x 4096 11.7 / 11.5,
    // 1024 x 4096 10.0 / 8.2, 768 x 3072 10.0 / 8.5, 11008 x 4096 35.0 / 21.9; M = 5: 11008 x 4096 31.2 / 21.9 but
    // 4096 x 4096 10.5 / 11.5; with K = 768 or 1024 the streaming form stays ahead up to M = 6, 4.9-5.7 against 7.8-8.2).
    const bool tiles_for_rows = K >= 2048 && K % 32 == 0 && (M == 6 || (M == 5 && N * K > (int64_t(1) << 24)));
    // M = 7, 8 against a short K: the tiles' two launches (products, then the join of the K ranges) cost more than the
    // vector ALU's extra rows (us, weights cached / from HBM, streaming against tiles — 768 x 768: M = 7 5.3 / 5.3 against
    // 6.6 / 6.8, M = 8 5.5 / 5.6 against 6.6 / 7.4; 1024 x 1024, M = 8: 4.9 against 7.8; 4096 x 1024: 5.9 against 8.1 / 8.5;
    // 8192 x 1024: 7.5 / 8.7 against 10.1 / 11.2; 2048 x 2048: 7.2 / 7.7 against 8.0 / 8.5; but 16384 x 768: 12.5 / 16.0
    // against 11.5 / 13.7, 768 x 3072: 12.2 / 12.6 against 8.7 / 9.0, 4096 x 4096: 14.5 / 19.4 against 13.0 / 15.1).
    const bool small_rows = (M == 7 || M == 8) && tuning().w8a32_tile == 0 &&
                            ((K <= 1024 && N * K <= (int64_t(8) << 20)) || (K <= 2048 && N <= 2048));
    if ((M > 6 && !small_rows) || tiles_for_rows) return axhip::sgemm_i8w(M, N, K, a, w, w_scales, out);
    if ((N + 3) / 4 > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "qgemm_w8a32: N too large");
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
