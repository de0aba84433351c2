// Elementwise vtable slots (bias_add, relu, gelu, fill) and the per-row int8 quantizer.
// All are one pass over memory: 16-byte accesses where alignment allows, grid-stride loops.
#include "common.h"

namespace {
using namespace axhip;

template <int OP>   // 0 relu, 1 gelu
__global__ void __launch_bounds__(256) k_unary(const float *in, float *out,
                                               int64_t n, int vec) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        const int64_t n4 = n >> 2;
        for (int64_t j = i; j < n4; j += stride) {
            v4f v = reinterpret_cast<const v4f *>(in)[j];
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = OP == 0 ? (v[e] > 0.0f ? v[e] : 0.0f) : gelu_tanh(v[e]);
            reinterpret_cast<v4f *>(out)[j] = v;
        }
        for (int64_t j = (n4 << 2) + i; j < n; j += stride)
            out[j] = OP == 0 ? (in[j] > 0.0f ? in[j] : 0.0f) : gelu_tanh(in[j]);
    } else {
        for (; i < n; i += stride) out[i] = OP == 0 ? (in[i] > 0.0f ? in[i] : 0.0f) : gelu_tanh(in[i]);
    }
}

__global__ void __launch_bounds__(256) k_fill(float *__restrict__ dst, float value, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = value;
}

__global__ void __launch_bounds__(256)
k_bias_add(const float *in, const float *__restrict__ bias, int64_t axis_len,
           int64_t inner, int64_t total, float *out) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride)
        out[i] = in[i] + bias[(i / inner) % axis_len];
}

// one workgroup per weight row: absmax over the row, then round-to-nearest-even and clamp.
__global__ void __launch_bounds__(256)
k_quantize_rows(const float *__restrict__ w, int64_t K, int8_t *__restrict__ q,
                float *__restrict__ scales) {
    __shared__ float red[256];
    const int64_t n = blockIdx.x;
    const float *row = w + n * K;
    float top = 0.0f;
    for (int64_t k = threadIdx.x; k < K; k += 256) top = fmaxf(top, fabsf(row[k]));
    red[threadIdx.x] = top;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + s]);
        __syncthreads();
    }
    top = red[0];
    const float scale = top > 0.0f ? __fdiv_rn(top, 127.0f) : 1.0f;
    const float inv = __fdiv_rn(1.0f, scale);
    if (threadIdx.x == 0) scales[n] = scale;
    for (int64_t k = threadIdx.x; k < K; k += 256) {
        float v = rintf(__fmul_rn(row[k], inv));
        v = fminf(fmaxf(v, -127.0f), 127.0f);
        q[n * K + k] = (int8_t)(int)v;
    }
}

unsigned grid_for(int64_t work_items) {
    int64_t b = (work_items + 255) / 256;
    if (b < 1) b = 1;
    if (b > 256 * 32) b = 256 * 32;
    return (unsigned)b;
}
}  // namespace

extern "C" {

int axhip_relu(const float *in, float *out, int64_t n) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!in || !out) return fail(AXHIP_ERR_NULL_ARG, "relu: NULL");
    if (n <= 0) return n < 0 ? fail(AXHIP_ERR_SHAPE, "relu: negative size") : AXHIP_OK;
    int vec = (((uintptr_t)in | (uintptr_t)out) & 15) == 0;
    hipLaunchKernelGGL(k_unary<0>, dim3(grid_for(vec ? n / 4 + 1 : n)), dim3(256), 0, kStream, in, out, n, vec);
    return check_launch("relu");
}

int axhip_gelu(const float *in, float *out, int64_t n) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!in || !out) return fail(AXHIP_ERR_NULL_ARG, "gelu: NULL");
    if (n <= 0) return n < 0 ? fail(AXHIP_ERR_SHAPE, "gelu: negative size") : AXHIP_OK;
    int vec = (((uintptr_t)in | (uintptr_t)out) & 15) == 0;
    hipLaunchKernelGGL(k_unary<1>, dim3(grid_for(vec ? n / 4 + 1 : n)), dim3(256), 0, kStream, in, out, n, vec);
    return check_launch("gelu");
}

int axhip_fill_f32(float *dst, float value, int64_t n) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!dst) return fail(AXHIP_ERR_NULL_ARG, "fill: NULL");
    if (n <= 0) return n < 0 ? fail(AXHIP_ERR_SHAPE, "fill: negative size") : AXHIP_OK;
    hipLaunchKernelGGL(k_fill, dim3(grid_for(n)), dim3(256), 0, kStream, dst, value, n);
    return check_launch("fill");
}

int axhip_bias_add(const float *in, const float *bias, int64_t outer, int64_t axis_len,
                   int64_t inner, float *out) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!in || !bias || !out) return fail(AXHIP_ERR_NULL_ARG, "bias_add: NULL");
    if (outer < 0 || axis_len < 0 || inner < 0) return fail(AXHIP_ERR_SHAPE, "bias_add: negative extent");
    const int64_t total = outer * axis_len * inner;
    if (total == 0) return AXHIP_OK;
    hipLaunchKernelGGL(k_bias_add, dim3(grid_for(total)), dim3(256), 0, kStream, in, bias, axis_len,
                       inner, total, out);
    return check_launch("bias_add");
}

int axhip_quantize_rows(const float *w, int64_t N, int64_t K, int8_t *q, float *scales) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!w || !q || !scales) return fail(AXHIP_ERR_NULL_ARG, "quantize_rows: NULL");
    if (N <= 0 || K <= 0) return fail(AXHIP_ERR_SHAPE, "quantize_rows: N and K must be positive");
    if (N > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "quantize_rows: N too large");
    hipLaunchKernelGGL(k_quantize_rows, dim3((unsigned)N), dim3(256), 0, kStream, w, K, q, scales);
    return check_launch("quantize_rows");
}

}  // extern "C"
