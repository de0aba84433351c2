// Row softmax (the .softmax_rowwise vtable slot; cpu_naive.c:235-270, cuda/ops_fused.cu:44-91)
// and layer normalisation forward (src/core/norm.c:1278-1399) over contiguous [rows, cols] fp32.
// HBM-bound.  A row of up to TPR*VPT columns is read once into registers (one wave per row up to
// 1024 columns, one workgroup per row up to 4096), reduced, and written once; longer rows are
// re-read from memory by one workgroup per row.
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
k_rows_cached(const float *__restrict__ in, float *__restrict__ out, int64_t rows, int cols, LnArgs ln) {
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
                out[row * cols + c] = __builtin_fmaf(ln.gamma[c], xh, ln.beta[c]);
                if (ln.x_hat) ln.x_hat[row * cols + c] = xh;
            }
        }
    }
}

// rows longer than the register cache: one workgroup per row, the row re-read from memory
template <int KIND>
__global__ void __launch_bounds__(256)
k_rows_streamed(const float *__restrict__ in, float *__restrict__ out, int64_t cols, LnArgs ln) {
    __shared__ float lds[8];
    const int t = threadIdx.x, wave = t >> 6;
    const int64_t row = blockIdx.x;
    const float *x = in + row * cols;
    float *y = out + row * cols;
    if (KIND == 0) {
        float mx = -FLT_MAX;
        for (int64_t c = t; c < cols; c += 256) mx = fmaxf(mx, x[c]);
        mx = row_join<256, true>(mx, lds, wave);
        float sum = 0.0f;
        for (int64_t c = t; c < cols; c += 256) {
            const float e = expf(x[c] - mx);
            y[c] = e;
            sum += e;
        }
        sum = row_join<256, false>(sum, lds, wave);
        const float inv = 1.0f / sum;
        for (int64_t c = t; c < cols; c += 256) y[c] *= inv;      // each thread re-reads its own writes
    } else {
        float s = 0.0f, s2 = 0.0f;
        for (int64_t c = t; c < cols; c += 256) {
            const float v = x[c];
            s += v;
            s2 = __builtin_fmaf(v, v, s2);
        }
        row_join2<256>(s, s2, lds, wave);
        const float mean = s / (float)cols;
        float var = s2 / (float)cols - mean * mean;
        if (var < 0.0f) var = 0.0f;
        const float inv_std = 1.0f / sqrtf(var + ln.eps);
        if (ln.inv_std && t == 0) ln.inv_std[row] = inv_std;
        for (int64_t c = t; c < cols; c += 256) {
            const float xh = (x[c] - mean) * inv_std;
            y[c] = __builtin_fmaf(ln.gamma[c], xh, ln.beta[c]);
            if (ln.x_hat) ln.x_hat[row * cols + c] = xh;
        }
    }
}

template <int KIND>
int launch_rows(const float *in, float *out, int64_t rows, int64_t cols, const LnArgs &ln, const char *what) {
    if (cols <= 1024) {
        const int64_t blocks = (rows + 3) / 4;
        if (blocks > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "%s: too many rows", what);
        if (cols <= 128)
            hipLaunchKernelGGL((k_rows_cached<64, 2, KIND>), dim3((unsigned)blocks), dim3(256), 0, kStream, in, out, rows, (int)cols, ln);
        else if (cols <= 512)
            hipLaunchKernelGGL((k_rows_cached<64, 8, KIND>), dim3((unsigned)blocks), dim3(256), 0, kStream, in, out, rows, (int)cols, ln);
        else
            hipLaunchKernelGGL((k_rows_cached<64, 16, KIND>), dim3((unsigned)blocks), dim3(256), 0, kStream, in, out, rows, (int)cols, ln);
    } else {
        if (rows > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "%s: too many rows", what);
        if (cols <= 4096)
            hipLaunchKernelGGL((k_rows_cached<256, 16, KIND>), dim3((unsigned)rows), dim3(256), 0, kStream, in, out, rows, (int)cols, ln);
        else
            hipLaunchKernelGGL((k_rows_streamed<KIND>), dim3((unsigned)rows), dim3(256), 0, kStream, in, out, cols, ln);
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
