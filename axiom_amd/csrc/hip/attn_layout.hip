// Layout transforms around attention: the split of a fused [B*S, 3D] projection into per-head
// Q, K, V of shape [B*H, S, dk] (optionally adding the [3D] bias), the merge of per-head outputs
// back to [B, S, H*dk], its inverse, and the assembly of the fused [D, 3D] weight panel and [3D]
// bias from the three projections.  They take the place of the layout members of the reference's
// GPU extension table (include/axiom/internal/cuda_extension.h:45-84; CPU forms in
// src/core/attention/layout.c:121-152, 215-262 and src/core/attention/cache.c:49-57, 79-81).
// Pure copies, HBM-bound: 16-byte accesses when dk (or D) is a multiple of 4 and the pointers
// are aligned, one element per thread otherwise.
#include "common.h"

namespace {
using namespace axhip;

// one item = VW consecutive floats of one (b, s, h) row of dk floats
template <int VW, bool BIAS>
__global__ void __launch_bounds__(256)
k_split_qkv(const float *__restrict__ src, const float *__restrict__ bqkv, float *__restrict__ q,
            float *__restrict__ k, float *__restrict__ v, int64_t S, int64_t H, int64_t dk, int64_t D, int64_t items) {
    const int64_t stride = (int64_t)gridDim.x * 256, per_row = dk / VW;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < items; t += stride) {
        // items are numbered in destination order: ((b*H + h)*S + s)*per_row + c
        const int64_t c = t % per_row, r = t / per_row;
        const int64_t s = r % S, bh = r / S, h = bh % H, b = bh / H;
        const int64_t col = h * dk + c * VW;
        const float *in = src + (b * S + s) * 3 * D + col;
        const int64_t out = r * dk + c * VW;
        if (VW == 4) {
            v4f vq = *reinterpret_cast<const v4f *>(in), vk = *reinterpret_cast<const v4f *>(in + D),
                vv = *reinterpret_cast<const v4f *>(in + 2 * D);
            if (BIAS) {
                vq += *reinterpret_cast<const v4f *>(bqkv + col);
                vk += *reinterpret_cast<const v4f *>(bqkv + D + col);
                vv += *reinterpret_cast<const v4f *>(bqkv + 2 * D + col);
            }
            *reinterpret_cast<v4f *>(q + out) = vq;
            *reinterpret_cast<v4f *>(k + out) = vk;
            *reinterpret_cast<v4f *>(v + out) = vv;
        } else {
            q[out] = in[0] + (BIAS ? bqkv[col] : 0.0f);
            k[out] = in[D] + (BIAS ? bqkv[D + col] : 0.0f);
            v[out] = in[2 * D] + (BIAS ? bqkv[2 * D + col] : 0.0f);
        }
    }
}

// TO_HEADS: [B, S, H, dk] -> [B*H, S, dk]; otherwise the reverse.  Items in destination order.
template <int VW, bool TO_HEADS>
__global__ void __launch_bounds__(256)
k_head_permute(const float *__restrict__ src, float *__restrict__ dst, int64_t S, int64_t H, int64_t dk, int64_t items) {
    const int64_t stride = (int64_t)gridDim.x * 256, per_row = dk / VW;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < items; t += stride) {
        const int64_t c = t % per_row, r = t / per_row;
        int64_t from;
        if (TO_HEADS) {                              // r = (b*H + h)*S + s
            const int64_t s = r % S, bh = r / S, h = bh % H, b = bh / H;
            from = ((b * S + s) * H + h) * dk;
        } else {                                     // r = (b*S + s)*H + h
            const int64_t h = r % H, bs = r / H, s = bs % S, b = bs / S;
            from = ((b * H + h) * S + s) * dk;
        }
        if (VW == 4) *reinterpret_cast<v4f *>(dst + r * dk + c * 4) = *reinterpret_cast<const v4f *>(src + from + c * 4);
        else dst[r * dk + c] = src[from + c];
    }
}

// dst[i, j] for j in [0, 3*cols): a[i, j], b[i, j - cols] or c[i, j - 2*cols]; rows = 1 gives the bias form
template <int VW>
__global__ void __launch_bounds__(256)
k_concat3(float *__restrict__ dst, const float *__restrict__ a, const float *__restrict__ b,
          const float *__restrict__ c, int64_t cols, int64_t items) {
    const int64_t stride = (int64_t)gridDim.x * 256, per_row = 3 * cols / VW;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < items; t += stride) {
        const int64_t i = t / per_row, j = (t - i * per_row) * VW;
        const int part = (int)(j / cols);
        const float *from = (part == 0 ? a : part == 1 ? b : c) + i * cols + (j - part * cols);
        if (VW == 4) *reinterpret_cast<v4f *>(dst + i * 3 * cols + j) = *reinterpret_cast<const v4f *>(from);
        else dst[i * 3 * cols + j] = *from;
    }
}

unsigned blocks_for(int64_t items) {
    int64_t b = (items + 255) / 256;
    if (b < 1) b = 1;
    if (b > 256 * 32) b = 256 * 32;
    return (unsigned)b;
}

bool aligned16(std::initializer_list<const void *> ptrs) {
    for (const void *p : ptrs)
        if ((uintptr_t)p & 15) return false;
    return true;
}
}  // namespace

extern "C" {

int axhip_head_split_qkv(const float *qkv, const float *bqkv, float *q, float *k, float *v, int64_t B, int64_t S,
                         int64_t H, int64_t dk, int64_t D) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!qkv || !q || !k || !v) return fail(AXHIP_ERR_NULL_ARG, "head_split_qkv: NULL");
    if (B < 0 || S < 0 || H <= 0 || dk <= 0 || D != H * dk) return fail(AXHIP_ERR_SHAPE, "head_split_qkv: D must equal H * dk");
    if (B == 0 || S == 0) return AXHIP_OK;
    const bool vec = dk % 4 == 0 && aligned16({qkv, bqkv, q, k, v});
    const int64_t items = B * H * S * (vec ? dk / 4 : dk);
    const dim3 grid(blocks_for(items)), block(256);
    if (vec && bqkv) hipLaunchKernelGGL((k_split_qkv<4, true>), grid, block, 0, kStream, qkv, bqkv, q, k, v, S, H, dk, D, items);
    else if (vec) hipLaunchKernelGGL((k_split_qkv<4, false>), grid, block, 0, kStream, qkv, bqkv, q, k, v, S, H, dk, D, items);
    else if (bqkv) hipLaunchKernelGGL((k_split_qkv<1, true>), grid, block, 0, kStream, qkv, bqkv, q, k, v, S, H, dk, D, items);
    else hipLaunchKernelGGL((k_split_qkv<1, false>), grid, block, 0, kStream, qkv, bqkv, q, k, v, S, H, dk, D, items);
    return check_launch("head_split_qkv");
}

static int head_permute(const float *src, float *dst, int64_t B, int64_t S, int64_t H, int64_t dk, bool to_heads) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!src || !dst) return fail(AXHIP_ERR_NULL_ARG, "head layout: NULL");
    if (B < 0 || S < 0 || H <= 0 || dk <= 0) return fail(AXHIP_ERR_SHAPE, "head layout: bad extent");
    if (B == 0 || S == 0) return AXHIP_OK;
    const bool vec = dk % 4 == 0 && aligned16({src, dst});
    const int64_t items = B * H * S * (vec ? dk / 4 : dk);
    const dim3 grid(blocks_for(items)), block(256);
    if (vec && to_heads) hipLaunchKernelGGL((k_head_permute<4, true>), grid, block, 0, kStream, src, dst, S, H, dk, items);
    else if (vec) hipLaunchKernelGGL((k_head_permute<4, false>), grid, block, 0, kStream, src, dst, S, H, dk, items);
    else if (to_heads) hipLaunchKernelGGL((k_head_permute<1, true>), grid, block, 0, kStream, src, dst, S, H, dk, items);
    else hipLaunchKernelGGL((k_head_permute<1, false>), grid, block, 0, kStream, src, dst, S, H, dk, items);
    return check_launch("head layout");
}

int axhip_head_interleave(const float *src, float *dst, int64_t B, int64_t S, int64_t H, int64_t dk) {
    return head_permute(src, dst, B, S, H, dk, true);
}

int axhip_head_deinterleave(const float *src, float *dst, int64_t B, int64_t S, int64_t H, int64_t dk) {
    return head_permute(src, dst, B, S, H, dk, false);
}

int axhip_concat3_rows(float *dst, const float *a, const float *b, const float *c, int64_t rows, int64_t cols) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!dst || !a || !b || !c) return fail(AXHIP_ERR_NULL_ARG, "concat3_rows: NULL");
    if (rows < 0 || cols < 0) return fail(AXHIP_ERR_SHAPE, "concat3_rows: negative extent");
    if (rows == 0 || cols == 0) return AXHIP_OK;
    const bool vec = cols % 4 == 0 && aligned16({dst, a, b, c});
    const int64_t items = rows * 3 * cols / (vec ? 4 : 1);
    if (vec) hipLaunchKernelGGL((k_concat3<4>), dim3(blocks_for(items)), dim3(256), 0, kStream, dst, a, b, c, cols, items);
    else hipLaunchKernelGGL((k_concat3<1>), dim3(blocks_for(items)), dim3(256), 0, kStream, dst, a, b, c, cols, items);
    return check_launch("concat3_rows");
}

}  // extern "C"
