// Row softmax (the .softmax_rowwise vtable slot; cpu_naive.c:235-270, cuda/ops_fused.cu:44-91)
// and layer normalisation forward (src/core/norm.c:1278-1399) over contiguous [rows, cols] fp32.
// HBM-bound.  A row of up to TPR*VPT columns is read once into registers (several rows per wave up
// to 128 columns, one wave per row up to 1024, one workgroup per row up to 6144), reduced, and
// written once; a row of up to 36864 columns is held in LDS by a workgroup of 1024 threads; longer
// rows are read twice.
#include <float.h>

#include "common.h"

namespace {
using namespace axhip;

// sum (or max) over the TPR threads that share a row
template <int TPR, bool MAX>
__device__ __forceinline__ float row_join(float v, float *lds, int wave) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_xor(v, off, 64);
        v = MAX ? fmaxf(v, o) : v + o;
    }
    if (TPR == 64) return v;
    __syncthreads();                             // the previous use of lds has been read
    if ((threadIdx.x & 63) == 0) lds[wave] = v;
    __syncthreads();
    const float a = lds[0], b = lds[1], c = lds[2], d = lds[3];
    return MAX ? fmaxf(fmaxf(a, b), fmaxf(c, d)) : (a + b) + (c + d);
}

// two sums at once (layer norm's sum and sum of squares): one LDS round instead of two
template <int TPR>
__device__ __forceinline__ void row_join2(float &a, float &b, float *lds, int wave) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        a += __shfl_xor(a, off, 64);
        b += __shfl_xor(b, off, 64);
    }
    if (TPR == 64) return;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) {
        lds[wave] = a;
        lds[4 + wave] = b;
    }
    __syncthreads();
    a = (lds[0] + lds[1]) + (lds[2] + lds[3]);
    b = (lds[4] + lds[5]) + (lds[6] + lds[7]);
}

struct LnArgs {
    const float *gamma, *beta;
    float *x_hat, *inv_std;
    float eps;
};

// KIND 0: softmax, 1: layer norm.  Thread t of a row holds columns t, t + TPR, ...
template <int TPR, int VPT, int KIND>
__global__ void __launch_bounds__(256)
k_rows_cached(const float *in, float *out, int64_t rows, int cols, LnArgs ln) {
    __shared__ float lds[8];
    constexpr int RPB = 256 / TPR;
    const int t = threadIdx.x % TPR, wave = threadIdx.x >> 6;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / TPR;
    if (TPR == 64 && row >= rows) return;        // whole waves leave; a workgroup row is never partial
    const float *x = in + row * cols;
    float v[VPT];
#pragma unroll
    for (int i = 0; i < VPT; i++) v[i] = (t + i * TPR < cols) ? x[t + i * TPR] : (KIND == 0 ? -FLT_MAX : 0.0f);
    if (KIND == 0) {
        float mx = -FLT_MAX;
#pragma unroll
        for (int i = 0; i < VPT; i++) mx = fmaxf(mx, v[i]);
        mx = row_join<TPR, true>(mx, lds, wave);
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            v[i] = (t + i * TPR < cols) ? expf(v[i] - mx) : 0.0f;
            sum += v[i];
        }
        sum = row_join<TPR, false>(sum, lds, wave);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int i = 0; i < VPT; i++)
            if (t + i * TPR < cols) out[row * cols + t + i * TPR] = v[i] * inv;
    } else {
        // scale and shift are requested now (L2 hits), so that they have arrived when the row's
        // sums are joined rather than being waited for after the barrier
        float gam[VPT], bet[VPT];
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int c = t + i * TPR;
            gam[i] = c < cols ? ln.gamma[c] : 0.0f;
            bet[i] = c < cols ? ln.beta[c] : 0.0f;
        }
        float s = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            s += v[i];
            s2 = __builtin_fmaf(v[i], v[i], s2);
        }
        row_join2<TPR>(s, s2, lds, wave);
        const float mean = s / (float)cols;
        float var = s2 / (float)cols - mean * mean;
        if (var < 0.0f) var = 0.0f;
        const float inv_std = 1.0f / sqrtf(var + ln.eps);
        if (ln.inv_std && t == 0) ln.inv_std[row] = inv_std;
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int c = t + i * TPR;
            if (c < cols) {
                const float xh = (v[i] - mean) * inv_std;
                out[row * cols + c] = __builtin_fmaf(gam[i], xh, bet[i]);
                if (ln.x_hat) ln.x_hat[row * cols + c] = xh;
            }
        }
    }
}

// ---- rows longer than the register cache ----------------------------------------------------
// Rows start wherever rows * cols puts them, so 16-byte accesses go through copies the compiler
// may emit at any alignment (global memory takes unaligned vector loads and stores).
__device__ __forceinline__ v4f load4(const float *p) {
    v4f v;
    __builtin_memcpy(&v, p, 16);
    return v;
}
__device__ __forceinline__ void store4(float *p, v4f v) { __builtin_memcpy(p, &v, 16); }

// sum (or max) over the NW waves of a workgroup, joined in wave order
template <int NW, bool MAX>
__device__ __forceinline__ float block_join(float v, float *lds, int wave) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_xor(v, off, 64);
        v = MAX ? fmaxf(v, o) : v + o;
    }
    __syncthreads();                             // the previous use of lds has been read
    if ((threadIdx.x & 63) == 0) lds[wave] = v;
    __syncthreads();
    float r = lds[0];
#pragma unroll
    for (int w = 1; w < NW; w++) r = MAX ? fmaxf(r, lds[w]) : r + lds[w];
    return r;
}

constexpr int kBig = 1024, kBigWaves = kBig / 64;   // threads of the long-row kernels

// Up to 36864 columns: one workgroup of 1024 threads per row, the row held in LDS (144 KiB), read
// from memory once and written once.  Thread t owns the 4-column groups t, t + 1024, ... and the
// columns of the ragged tail it picks up, in every pass, so it only ever re-reads its own LDS entries.
template <int KIND>
__global__ void __launch_bounds__(kBig)
k_rows_lds(const float *in, float *out, int64_t cols, LnArgs ln) {
    extern __shared__ __attribute__((aligned(16))) float rowbuf[];
    __shared__ float lds[2 * kBigWaves];
    const int t = threadIdx.x, wave = t >> 6;
    const int64_t row = blockIdx.x;
    const float *x = in + row * cols;
    float *y = out + row * cols;
    const int n = (int)cols, groups = n / 4, tail0 = groups * 4;
    for (int i = t; i < groups; i += kBig) *reinterpret_cast<v4f *>(rowbuf + 4 * i) = load4(x + 4 * i);
    for (int c = tail0 + t; c < n; c += kBig) rowbuf[c] = x[c];
    if (KIND == 0) {
        float mx = -FLT_MAX;
        for (int i = t; i < groups; i += kBig) {
            const v4f v = *reinterpret_cast<const v4f *>(rowbuf + 4 * i);
            mx = fmaxf(fmaxf(mx, fmaxf(v.x, v.y)), fmaxf(v.z, v.w));
        }
        for (int c = tail0 + t; c < n; c += kBig) mx = fmaxf(mx, rowbuf[c]);
        mx = block_join<kBigWaves, true>(mx, lds, wave);
        float sum = 0.0f;
        for (int i = t; i < groups; i += kBig) {
            v4f v = *reinterpret_cast<const v4f *>(rowbuf + 4 * i);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                v[e] = expf(v[e] - mx);
                sum += v[e];
            }
            *reinterpret_cast<v4f *>(rowbuf + 4 * i) = v;
        }
        for (int c = tail0 + t; c < n; c += kBig) {
            const float e = expf(rowbuf[c] - mx);
            rowbuf[c] = e;
            sum += e;
        }
        sum = block_join<kBigWaves, false>(sum, lds, wave);
        const float inv = 1.0f / sum;
        for (int i = t; i < groups; i += kBig) store4(y + 4 * i, *reinterpret_cast<const v4f *>(rowbuf + 4 * i) * inv);
        for (int c = tail0 + t; c < n; c += kBig) y[c] = rowbuf[c] * inv;
    } else {
        float s = 0.0f, s2 = 0.0f;
        for (int i = t; i < groups; i += kBig) {
            const v4f v = *reinterpret_cast<const v4f *>(rowbuf + 4 * i);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                s += v[e];
                s2 = __builtin_fmaf(v[e], v[e], s2);
            }
        }
        for (int c = tail0 + t; c < n; c += kBig) {
            const float v = rowbuf[c];
            s += v;
            s2 = __builtin_fmaf(v, v, s2);
        }
        s = block_join<kBigWaves, false>(s, lds, wave);
        s2 = block_join<kBigWaves, false>(s2, lds + kBigWaves, wave);
        const float mean = s / (float)cols;
        float var = s2 / (float)cols - mean * mean;
        if (var < 0.0f) var = 0.0f;
        const float inv_std = 1.0f / sqrtf(var + ln.eps);
        if (ln.inv_std && t == 0) ln.inv_std[row] = inv_std;
        float *xh_row = ln.x_hat ? ln.x_hat + row * cols : nullptr;
        for (int i = t; i < groups; i += kBig) {
            const v4f xh = (*reinterpret_cast<const v4f *>(rowbuf + 4 * i) - mean) * inv_std;
            const v4f g = load4(ln.gamma + 4 * i), b = load4(ln.beta + 4 * i);
            v4f o;
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = __builtin_fmaf(g[e], xh[e], b[e]);
            store4(y + 4 * i, o);
            if (xh_row) store4(xh_row + 4 * i, xh);
        }
        for (int c = tail0 + t; c < n; c += kBig) {
            const float xh = (rowbuf[c] - mean) * inv_std;
            y[c] = __builtin_fmaf(ln.gamma[c], xh, ln.beta[c]);
            if (xh_row) xh_row[c] = xh;
        }
    }
}

// Longer still: one workgroup per row, the row read twice (the second time mostly out of the
// caches: a workgroup re-reads what it has just streamed) and written once.  Softmax keeps a
// running maximum m and the sum of exp(x - m) per thread in the first pass, rescaling the sum when
// the maximum moves (four columns at a time: five exponentials per four columns), so no pass is
// spent on the maximum alone; the threads' pairs are joined as sum_i s_i * exp(m_i - M).
template <int KIND>
__global__ void __launch_bounds__(kBig)
k_rows_streamed(const float *in, float *out, int64_t cols, LnArgs ln) {
    __shared__ float lds[2 * kBigWaves];
    const int t = threadIdx.x, wave = t >> 6;
    const int64_t row = blockIdx.x;
    const float *x = in + row * cols;
    float *y = out + row * cols;
    const int64_t groups = cols / 4, tail0 = groups * 4;
    if (KIND == 0) {
        float m = -FLT_MAX, s = 0.0f;
        for (int64_t i = t; i < groups; i += kBig) {
            const v4f v = load4(x + 4 * i);
            const float m4 = fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w));
            if (m4 > m) {
                s *= expf(m - m4);
                m = m4;
            }
            s += (expf(v.x - m) + expf(v.y - m)) + (expf(v.z - m) + expf(v.w - m));
        }
        for (int64_t c = tail0 + t; c < cols; c += kBig) {
            const float v = x[c];
            if (v > m) {
                s *= expf(m - v);
                m = v;
            }
            s += expf(v - m);
        }
        const float mx = block_join<kBigWaves, true>(m, lds, wave);
        const float sum = block_join<kBigWaves, false>(s * expf(m - mx), lds + kBigWaves, wave);
        const float inv = 1.0f / sum;
        for (int64_t i = t; i < groups; i += kBig) {
            v4f v = load4(x + 4 * i);
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = expf(v[e] - mx) * inv;
            store4(y + 4 * i, v);
        }
        for (int64_t c = tail0 + t; c < cols; c += kBig) y[c] = expf(x[c] - mx) * inv;
    } else {
        float s = 0.0f, s2 = 0.0f;
        for (int64_t i = t; i < groups; i += kBig) {
            const v4f v = load4(x + 4 * i);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                s += v[e];
                s2 = __builtin_fmaf(v[e], v[e], s2);
            }
        }
        for (int64_t c = tail0 + t; c < cols; c += kBig) {
            const float v = x[c];
            s += v;
            s2 = __builtin_fmaf(v, v, s2);
        }
        s = block_join<kBigWaves, false>(s, lds, wave);
        s2 = block_join<kBigWaves, false>(s2, lds + kBigWaves, wave);
        const float mean = s / (float)cols;
        float var = s2 / (float)cols - mean * mean;
        if (var < 0.0f) var = 0.0f;
        const float inv_std = 1.0f / sqrtf(var + ln.eps);
        if (ln.inv_std && t == 0) ln.inv_std[row] = inv_std;
        float *xh_row = ln.x_hat ? ln.x_hat + row * cols : nullptr;
        for (int64_t i = t; i < groups; i += kBig) {
            const v4f xh = (load4(x + 4 * i) - mean) * inv_std;
            const v4f g = load4(ln.gamma + 4 * i), b = load4(ln.beta + 4 * i);
            v4f o;
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = __builtin_fmaf(g[e], xh[e], b[e]);
            store4(y + 4 * i, o);
            if (xh_row) store4(xh_row + 4 * i, xh);
        }
        for (int64_t c = tail0 + t; c < cols; c += kBig) {
            const float xh = (x[c] - mean) * inv_std;
            y[c] = __builtin_fmaf(ln.gamma[c], xh, ln.beta[c]);
            if (xh_row) xh_row[c] = xh;
        }
    }
}

// Short rows (up to 64 * VPT <= 128 columns): a wave per row has too few bytes in flight to cover
// HBM latency, so a wave takes RPW consecutive rows and requests all of them before it reduces any.
template <int VPT, int RPW, int KIND>
__global__ void __launch_bounds__(256)
k_rows_short(const float *in, float *out, int64_t rows, int cols, LnArgs ln) {
    const int t = threadIdx.x & 63;
    const int64_t row0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * RPW;
    if (row0 >= rows) return;
    float v[RPW][VPT];
#pragma unroll
    for (int r = 0; r < RPW; r++)
#pragma unroll
        for (int i = 0; i < VPT; i++)
            v[r][i] = (row0 + r < rows && t + i * 64 < cols) ? in[(row0 + r) * cols + t + i * 64]
                                                             : (KIND == 0 ? -FLT_MAX : 0.0f);
    float gam[VPT], bet[VPT];
    if (KIND == 1) {
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int c = t + i * 64;
            gam[i] = c < cols ? ln.gamma[c] : 0.0f;
            bet[i] = c < cols ? ln.beta[c] : 0.0f;
        }
    }
#pragma unroll
    for (int r = 0; r < RPW; r++) {
        const int64_t row = row0 + r;
        if (row >= rows) break;
        if (KIND == 0) {
            float mx = -FLT_MAX;
#pragma unroll
            for (int i = 0; i < VPT; i++) mx = fmaxf(mx, v[r][i]);
            mx = row_join<64, true>(mx, nullptr, 0);
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < VPT; i++) {
                v[r][i] = (t + i * 64 < cols) ? expf(v[r][i] - mx) : 0.0f;
                sum += v[r][i];
            }
            sum = row_join<64, false>(sum, nullptr, 0);
            const float inv = 1.0f / sum;
#pragma unroll
            for (int i = 0; i < VPT; i++)
                if (t + i * 64 < cols) out[row * cols + t + i * 64] = v[r][i] * inv;
        } else {
            float s = 0.0f, s2 = 0.0f;
#pragma unroll
            for (int i = 0; i < VPT; i++) {
                s += v[r][i];
                s2 = __builtin_fmaf(v[r][i], v[r][i], s2);
            }
            row_join2<64>(s, s2, nullptr, 0);
            const float mean = s / (float)cols;
            float var = s2 / (float)cols - mean * mean;
            if (var < 0.0f) var = 0.0f;
            const float inv_std = 1.0f / sqrtf(var + ln.eps);
            if (ln.inv_std && t == 0) ln.inv_std[row] = inv_std;
#pragma unroll
            for (int i = 0; i < VPT; i++) {
                const int c = t + i * 64;
                if (c < cols) {
                    const float xh = (v[r][i] - mean) * inv_std;
                    out[row * cols + c] = __builtin_fmaf(gam[i], xh, bet[i]);
                    if (ln.x_hat) ln.x_hat[row * cols + c] = xh;
                }
            }
        }
    }
}

template <int KIND>
int launch_rows(const float *in, float *out, int64_t rows, int64_t cols, const LnArgs &ln, const char *what) {
    if (cols <= 1024) {
        const int64_t blocks = (rows + 3) / 4;
        if (blocks > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "%s: too many rows", what);
        if (cols <= 64)
            hipLaunchKernelGGL((k_rows_short<1, 8, KIND>), dim3((unsigned)((rows + 31) / 32)), dim3(256), 0, kStream, in, out, rows, (int)cols, ln);
        else if (cols <= 128)
            hipLaunchKernelGGL((k_rows_short<2, 4, KIND>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, kStream, in, out, rows, (int)cols, ln);
        else if (cols <= 256)
            hipLaunchKernelGGL((k_rows_cached<64, 4, KIND>), dim3((unsigned)blocks), dim3(256), 0, kStream, in, out, rows, (int)cols, ln);
        else if (cols <= 512)
            hipLaunchKernelGGL((k_rows_cached<64, 8, KIND>), dim3((unsigned)blocks), dim3(256), 0, kStream, in, out, rows, (int)cols, ln);
        else
            hipLaunchKernelGGL((k_rows_cached<64, 16, KIND>), dim3((unsigned)blocks), dim3(256), 0, kStream, in, out, rows, (int)cols, ln);
    } else {
        if (rows > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "%s: too many rows", what);
        if (cols <= 4096) {
            hipLaunchKernelGGL((k_rows_cached<256, 16, KIND>), dim3((unsigned)rows), dim3(256), 0, kStream, in, out, rows, (int)cols, ln);
        } else if (cols <= 6144) {
            // still in registers (24 values a thread): faster than the LDS form up to here, slower from about 8192
            hipLaunchKernelGGL((k_rows_cached<256, 24, KIND>), dim3((unsigned)rows), dim3(256), 0, kStream, in, out, rows, (int)cols, ln);
        } else if (cols <= 36864) {
            static bool attr_set = false;
            if (!attr_set) {
                AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(k_rows_lds<KIND>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, 36864 * 4),
                              "hipFuncSetAttribute");
                attr_set = true;
            }
            const size_t smem = (size_t)((cols + 3) / 4 * 4) * sizeof(float);
            hipLaunchKernelGGL((k_rows_lds<KIND>), dim3((unsigned)rows), dim3(kBig), smem, kStream, in, out, cols, ln);
        } else {
            hipLaunchKernelGGL((k_rows_streamed<KIND>), dim3((unsigned)rows), dim3(kBig), 0, kStream, in, out, cols, ln);
        }
    }
    return check_launch(what);
}
}  // namespace

extern "C" int axhip_softmax_rows(const float *in, float *out, int64_t rows, int64_t cols) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!in || !out) return fail(AXHIP_ERR_NULL_ARG, "softmax_rows: NULL");
    if (rows < 0 || cols < 0) return fail(AXHIP_ERR_SHAPE, "softmax_rows: negative extent");
    if (rows == 0 || cols == 0) return AXHIP_OK;
    return launch_rows<0>(in, out, rows, cols, LnArgs{}, "softmax_rows");
}

extern "C" int axhip_layernorm_fwd(const float *x, const float *gamma, const float *beta, float *out, float *x_hat,
                                   float *inv_std, int64_t rows, int64_t cols, float eps) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!x || !gamma || !beta || !out) return fail(AXHIP_ERR_NULL_ARG, "layernorm_fwd: NULL");
    if (rows < 0 || cols <= 0) return fail(AXHIP_ERR_SHAPE, "layernorm_fwd: bad extent");
    if (rows == 0) return AXHIP_OK;
    return launch_rows<1>(x, out, rows, cols, LnArgs{gamma, beta, x_hat, inv_std, eps}, "layernorm_fwd");
}
