// Sum reductions behind the .sum vtable slot: out[o, i] = sum_a in[o, a, i] for a contiguous
// fp32 tensor viewed as [outer, axis_len, inner] (the reference's reduction_dims,
// cuda/ops_reduce.cu:246-251).  HBM-bound: one pass over the input.
//
//   inner > 1  (column sums; axis 0 of [rows, cols] is the dense layer's bias gradient):
//              the skinny-M GEMM with a row of ones as the activations, out = 1^T * in.  A
//              fused multiply-add by 1.0 is an exact addition, so this is a plain sum in the
//              kernel's fixed order, streamed at the skinny route's rate.
//   inner == 1 (row sums): one wave per row, lanes stride over the row, then a fixed-order
//              cross-lane tree.
//   axis == -1 (everything): row sums over equal chunks, then one row sum over the partials.
// All orders are fixed, so results are bit-identical run to run.
#include "common.h"

namespace {
using namespace axhip;

// Row r covers in[r*stride, r*stride + min(len, total - r*stride)).
template <bool VEC>
__global__ void __launch_bounds__(256)
k_rowsum(const float *__restrict__ in, int64_t rows, int64_t stride, int64_t len, int64_t total,
         float *__restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const int64_t begin = r * stride;
    int64_t n = total - begin;
    if (n > len) n = len;
    const float *p = in + begin;
    float s = 0.0f;
    if (VEC) {
        int64_t c = (int64_t)lane * 4;
        for (; c + 4 <= n; c += 256) {
            const v4f v = *reinterpret_cast<const v4f *>(p + c);
            s += (v.x + v.y) + (v.z + v.w);
        }
        for (; c < n; c++) s += p[c];          // at most one lane holds the ragged tail
    } else {
        for (int64_t c = lane; c < n; c += 64) s += p[c];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off, 64);
    if (lane == 0) out[r] = s;
}

int launch_rowsum(const float *in, int64_t rows, int64_t stride, int64_t len, int64_t total, float *out) {
    const int64_t blocks = (rows + 3) / 4;
    if (blocks > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "sum: too many rows");
    const bool vec = ((uintptr_t)in % 16 == 0) && (stride % 4 == 0);
    if (vec)
        hipLaunchKernelGGL(k_rowsum<true>, dim3((unsigned)blocks), dim3(256), 0, kStream, in, rows, stride, len, total, out);
    else
        hipLaunchKernelGGL(k_rowsum<false>, dim3((unsigned)blocks), dim3(256), 0, kStream, in, rows, stride, len, total, out);
    return check_launch("sum_rows");
}

__global__ void __launch_bounds__(256)
k_axpy(const float *__restrict__ x, float alpha, float *__restrict__ y, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        y[i] = __builtin_fmaf(alpha, x[i], y[i]);
}

}  // namespace

extern "C" int axhip_sum_axis(const float *in, int64_t outer, int64_t axis_len, int64_t inner, float *out) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!in || !out) return fail(AXHIP_ERR_NULL_ARG, "sum: NULL");
    if (outer < 0 || axis_len < 0 || inner < 0) return fail(AXHIP_ERR_SHAPE, "sum: negative extent");
    if (outer == 0 || inner == 0) return AXHIP_OK;
    if (axis_len == 0) return axhip_fill_f32(out, 0.0f, outer * inner);
    if (inner == 1) return launch_rowsum(in, outer, axis_len, axis_len, outer * axis_len, out);
    float *ones = axhip::ones_vector((size_t)axis_len);
    if (!ones) return AXHIP_ERR_ALLOC;
    for (int64_t o = 0; o < outer; o++) {
        const int rc = axhip_sgemm_skinny(1, inner, axis_len, ones, axis_len, in + o * axis_len * inner, inner,
                                          out + o * inner, inner, nullptr, AXHIP_ACT_NONE);
        if (rc) return rc;
    }
    axhip::note_kernel("sum_columns_skinny");
    return AXHIP_OK;
}

extern "C" int axhip_sum_all(const float *in, int64_t n, float *out) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!in || !out) return fail(AXHIP_ERR_NULL_ARG, "sum: NULL");
    if (n < 0) return fail(AXHIP_ERR_SHAPE, "sum: negative extent");
    if (n == 0) return axhip_fill_f32(out, 0.0f, 1);
    if (n <= 4096) return launch_rowsum(in, 1, n, n, n, out);
    int64_t parts = (n + 4095) / 4096;
    if (parts > 1024) parts = 1024;
    int64_t len = (n + parts - 1) / parts;
    len = (len + 3) / 4 * 4;
    parts = (n + len - 1) / len;
    float *partial = static_cast<float *>(axhip::workspace((size_t)parts * sizeof(float)));
    if (!partial) return AXHIP_ERR_ALLOC;
    if (int rc = launch_rowsum(in, parts, len, len, n, partial)) return rc;
    return launch_rowsum(partial, 1, parts, parts, parts, out);
}

extern "C" int axhip_axpy(const float *x, float alpha, float *y, int64_t n) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!x || !y) return fail(AXHIP_ERR_NULL_ARG, "axpy: NULL");
    if (n < 0) return fail(AXHIP_ERR_SHAPE, "axpy: negative extent");
    if (n == 0) return AXHIP_OK;
    int64_t blocks = (n + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(k_axpy, dim3((unsigned)blocks), dim3(256), 0, kStream, x, alpha, y, n);
    return check_launch("axpy");
}
