// Reductions behind the .sum/.mean/.max_op/.min_op vtable slots, row softmax and layer
// normalisation.  out[o, i] = reduce_a in[o, a, i] for a contiguous fp32 tensor viewed as
// [outer, axis_len, inner] (the reference's reduction_dims, cuda/ops_reduce.cu:246-251).
// HBM-bound: one pass over the input.  Sums:
//
//   inner > 1  (column sums; axis 0 of [rows, cols] is the dense layer's bias gradient), wide
//              (2048 columns and up; narrower ones take the column kernel below, which is the
//              faster of the two there):
//              the skinny-M GEMM with a row of ones as the activations, out = 1^T * in.  A
//              fused multiply-add by 1.0 is an exact addition, so this is a plain sum in the
//              kernel's fixed order, streamed at the skinny route's rate.
//   inner == 1 (row sums): one wave per row, lanes stride over the row, then a fixed-order
//              cross-lane tree.
//   axis == -1 (everything): row sums over equal chunks, then one row sum over the partials.
// All orders are fixed, so results are bit-identical run to run.  Maxima and minima start from
// -FLT_MAX / +FLT_MAX and take a value only when it compares strictly beyond the running one
// (cpu_naive.c:395-433, 441-479), so NaNs are passed over and the result does not depend on order.
#include <float.h>

#include "common.h"

namespace {
using namespace axhip;

template <int OP> __device__ __forceinline__ float red_init() {
    return OP == AXHIP_RED_MAX ? -FLT_MAX : OP == AXHIP_RED_MIN ? FLT_MAX : 0.0f;
}
template <int OP> __device__ __forceinline__ float red_join(float acc, float v) {
    if (OP == AXHIP_RED_MAX) return v > acc ? v : acc;
    if (OP == AXHIP_RED_MIN) return v < acc ? v : acc;
    return acc + v;
}

// LPR lanes per segment: a wave (64), or 16 / 4 lanes for segments of up to 128 / 32 elements,
// where a wave per segment would leave most lanes without a load (2M rows of 32: 315 -> 79 us
// with 16 lanes).  Segment R = (row r, part p) with
// r = R / parts covers in[r*row_stride + p*part_len, ... + min(part_len, row_len - p*part_len)).
template <int OP, int LPR>
__global__ void __launch_bounds__(256)
k_reduce_rows(const float *__restrict__ in, int64_t segments, int64_t parts, int64_t row_stride,
              int64_t part_len, int64_t row_len, float *__restrict__ out) {
    const int lane = threadIdx.x & (LPR - 1);
    const int64_t seg = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
    if (seg >= segments) return;
    const int64_t r = seg / parts, part = seg - r * parts;
    int64_t n = row_len - part * part_len;
    if (n > part_len) n = part_len;
    const float *p = in + r * row_stride + part * part_len;
    float s = red_init<OP>();
    // 16-byte loads at whatever alignment the row has (global memory takes unaligned vector loads;
    // a row of odd length starts off the 16-byte grid: 4096 x 16385 summed in 85 us by elements)
    int64_t c = (int64_t)lane * 4;
    for (; c + 4 <= n; c += LPR * 4) {
        v4f v;
        __builtin_memcpy(&v, p + c, 16);
        if (OP == AXHIP_RED_SUM) {
            s += (v.x + v.y) + (v.z + v.w);
        } else {                                  // the running value must stay on the left: it is never NaN
#pragma unroll
            for (int e = 0; e < 4; e++) s = red_join<OP>(s, v[e]);
        }
    }
    for (; c < n; c++) s = red_join<OP>(s, p[c]);              // at most one lane holds the ragged tail
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) s = red_join<OP>(s, __shfl_down(s, off, 64));   // lane 0 of a segment only ever takes in its own lanes
    if (lane == 0) out[seg] = s;
}

template <int OP>
int launch_rows(const float *in, int64_t rows, int64_t parts, int64_t row_stride, int64_t part_len,
                int64_t row_len, float *out) {
    // lanes per segment by its length: 4 up to 32 elements, 16 up to 128, else a wave
    const int64_t len = part_len < row_len ? part_len : row_len;
    const int lpr = len <= 32 ? 4 : len <= 128 ? 16 : 64;
    const int64_t segments = rows * parts, per_block = 256 / lpr, blocks = (segments + per_block - 1) / per_block;
    if (blocks > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "reduce: too many rows");
#define AX_ROWS(L)                                                                                             \
    hipLaunchKernelGGL((k_reduce_rows<OP, L>), dim3((unsigned)blocks), dim3(256), 0, kStream, in, segments, parts, \
                       row_stride, part_len, row_len, out)
    if (lpr == 4) AX_ROWS(4);
    else if (lpr == 16) AX_ROWS(16);
    else AX_ROWS(64);
#undef AX_ROWS
    return check_launch("reduce_rows");
}

// Row reductions of [rows, len]: few long rows are cut into parts first so that the whole chip
// streams, then the parts of each row are reduced.
template <int OP>
int reduce_rows(const float *in, int64_t rows, int64_t len, float *out) {
    int64_t parts = 1;
    if (rows < 2048 && len > 8192) {
        parts = 4096 / rows;
        const int64_t most = (len + 4095) / 4096;
        if (parts > most) parts = most;
        if (parts < 1) parts = 1;
    }
    if (parts == 1) return launch_rows<OP>(in, rows, 1, len, len, len, out);
    int64_t part_len = (len + parts - 1) / parts;
    part_len = (part_len + 3) / 4 * 4;
    parts = (len + part_len - 1) / part_len;
    float *partial = static_cast<float *>(workspace((size_t)(rows * parts) * sizeof(float)));
    if (!partial) return AXHIP_ERR_ALLOC;
    if (int rc = launch_rows<OP>(in, rows, parts, len, part_len, len, partial)) return rc;
    return launch_rows<OP>(partial, rows, 1, parts, parts, parts, out);
}

// Column reductions of [outer, axis_len, inner], inner > 1.  A workgroup is TY axis positions
// by TX column groups of VW columns; it walks a slice of the axis TY positions at a time and
// joins its TY partial rows through LDS.  Slice s of `splits` writes out[(o*splits + s), :].
template <int OP, int VW>
__global__ void __launch_bounds__(256)
k_reduce_cols(const float *__restrict__ in, int64_t axis_len, int64_t inner, int tx_log2, int64_t col_blocks,
              int64_t splits, int64_t slice, float *__restrict__ out) {
    __shared__ float join[256 * VW];
    const int tx = threadIdx.x & ((1 << tx_log2) - 1), ty = threadIdx.x >> tx_log2, TY = 256 >> tx_log2;
    int64_t b = blockIdx.x;
    const int64_t cb = b % col_blocks;
    b /= col_blocks;
    const int64_t s = b % splits, o = b / splits;
    const int64_t col = (cb << tx_log2) * VW + (int64_t)tx * VW;
    float acc[VW];
#pragma unroll
    for (int e = 0; e < VW; e++) acc[e] = red_init<OP>();
    int64_t a1 = (s + 1) * slice;
    if (a1 > axis_len) a1 = axis_len;
    if (col < inner) {
        const float *base = in + o * axis_len * inner + col;
        int64_t a = s * slice + ty;
        // eight rows in flight per thread, then joined in ascending order
        for (; a + 7 * TY < a1; a += 8 * TY) {
            float v[8][VW];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                if (VW == 4) {
                    const v4f t = *reinterpret_cast<const v4f *>(base + (a + u * TY) * inner);
#pragma unroll
                    for (int e = 0; e < VW; e++) v[u][e] = t[e];
                } else {
                    v[u][0] = base[(a + u * TY) * inner];
                }
            }
#pragma unroll
            for (int u = 0; u < 8; u++)
#pragma unroll
                for (int e = 0; e < VW; e++) acc[e] = red_join<OP>(acc[e], v[u][e]);
        }
        for (; a < a1; a += TY) {
            if (VW == 4) {
                const v4f v = *reinterpret_cast<const v4f *>(base + a * inner);
#pragma unroll
                for (int e = 0; e < VW; e++) acc[e] = red_join<OP>(acc[e], v[e]);
            } else {
                acc[0] = red_join<OP>(acc[0], base[a * inner]);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < VW; e++) join[e * 256 + threadIdx.x] = acc[e];
    __syncthreads();
    if (ty == 0 && col < inner) {
        for (int y = 1; y < TY; y++)
#pragma unroll
            for (int e = 0; e < VW; e++) acc[e] = red_join<OP>(acc[e], join[e * 256 + (y << tx_log2) + tx]);
        float *dst = out + (o * splits + s) * inner + col;
#pragma unroll
        for (int e = 0; e < VW; e++) dst[e] = acc[e];
    }
}

template <int OP>
int launch_cols(const float *in, int64_t outer, int64_t axis_len, int64_t inner, int64_t splits, float *out) {
    const bool vec = ((uintptr_t)in % 16 == 0) && inner % 4 == 0;
    const int64_t groups = vec ? inner / 4 : inner;
    int tx_log2 = 0;
    while (tx_log2 < 8 && (int64_t(1) << tx_log2) < groups) tx_log2++;
    const int64_t slice = (axis_len + splits - 1) / splits;
    // Few workgroups over a long axis (the join of a split reduction is the usual case): narrower
    // column blocks, so that more threads share the axis and the serial walk of each is short.
    while (tx_log2 > 2 && ((groups + (int64_t(1) << tx_log2) - 1) >> tx_log2) * splits * outer < 256 &&
           slice >= 4 * (256 >> (tx_log2 - 1)))
        tx_log2--;
    const int64_t col_blocks = (groups + (int64_t(1) << tx_log2) - 1) >> tx_log2;
    const int64_t blocks = col_blocks * splits * outer;
    if (blocks > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "reduce: too many column blocks");
    if (vec)
        hipLaunchKernelGGL((k_reduce_cols<OP, 4>), dim3((unsigned)blocks), dim3(256), 0, kStream, in, axis_len, inner,
                           tx_log2, col_blocks, splits, slice, out);
    else
        hipLaunchKernelGGL((k_reduce_cols<OP, 1>), dim3((unsigned)blocks), dim3(256), 0, kStream, in, axis_len, inner,
                           tx_log2, col_blocks, splits, slice, out);
    return check_launch("reduce_cols");
}

template <int OP>
int reduce_cols(const float *in, int64_t outer, int64_t axis_len, int64_t inner, float *out) {
    // enough workgroups to stream from every CU: cut the axis when outer x column blocks is small
    const int64_t groups = (inner + 3) / 4, col_blocks = (groups + 255) / 256;
    int64_t splits = 1;
    if (outer * col_blocks < 2048) {
        splits = 2048 / (outer * col_blocks);
        const int64_t most = axis_len / (axis_len >= 8192 ? 32 : 64);       // rows per slice, at least
        if (splits > most) splits = most;
        if (splits < 1) splits = 1;
    }
    if (splits == 1) return launch_cols<OP>(in, outer, axis_len, inner, 1, out);
    float *partial = static_cast<float *>(workspace((size_t)(outer * splits * inner) * sizeof(float)));
    if (!partial) return AXHIP_ERR_ALLOC;
    if (int rc = launch_cols<OP>(in, outer, axis_len, inner, splits, partial)) return rc;
    return launch_cols<OP>(partial, outer, splits, inner, 1, out);
}

template <int OP>
int reduce_axis(const float *in, int64_t outer, int64_t axis_len, int64_t inner, float *out) {
    if (inner == 1) return reduce_rows<OP>(in, outer, axis_len, out);
    return reduce_cols<OP>(in, outer, axis_len, inner, out);
}

__global__ void __launch_bounds__(256)
k_axpy(const float *__restrict__ x, float alpha, float *__restrict__ y, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        y[i] = __builtin_fmaf(alpha, x[i], y[i]);
}

// first index of the largest value along the axis (cpu_opt.c:7236-7247)
__global__ void __launch_bounds__(256)
k_argmax(const float *__restrict__ in, int64_t outer, int64_t axis_len, int64_t inner, int64_t *__restrict__ out) {
    const int64_t stride = (int64_t)gridDim.x * 256, total = outer * inner;
    for (int64_t oi = (int64_t)blockIdx.x * 256 + threadIdx.x; oi < total; oi += stride) {
        const int64_t o = oi / inner, i = oi - o * inner;
        const float *base = in + o * axis_len * inner + i;
        int64_t best = 0;
        float bestv = base[0];
        for (int64_t a = 1; a < axis_len; a++) {
            const float v = base[a * inner];
            if (v > bestv) {
                bestv = v;
                best = a;
            }
        }
        out[oi] = best;
    }
}

// Argmax down columns (inner > 1) of a long axis, in two steps like the column reductions: a
// workgroup of TX columns by TY axis positions walks one slice of the axis and leaves, per column,
// the first index of the slice's maximum among its non-NaN values (-1: none); the finishing pass
// takes the slices in ascending order.  The rule reproduced is the scan that starts from element 0
// and replaces on strictly greater: NaNs are passed over, except that a NaN in element 0 is never
// replaced and the answer is then 0.
__global__ void __launch_bounds__(256)
k_argmax_cols_part(const float *__restrict__ in, int64_t axis_len, int64_t inner, int tx_log2, int64_t col_blocks,
                   int64_t splits, int64_t slice, float *__restrict__ part_v, int64_t *__restrict__ part_i) {
    __shared__ float jv[256];
    __shared__ int64_t ji[256];
    const int tx = threadIdx.x & ((1 << tx_log2) - 1), ty = threadIdx.x >> tx_log2, TY = 256 >> tx_log2;
    int64_t b = blockIdx.x;
    const int64_t cb = b % col_blocks;
    b /= col_blocks;
    const int64_t s = b % splits, o = b / splits;
    const int64_t col = (cb << tx_log2) + tx;
    int64_t a1 = (s + 1) * slice;
    if (a1 > axis_len) a1 = axis_len;
    float bestv = 0.0f;
    int64_t best = -1;
    if (col < inner) {
        const float *base = in + o * axis_len * inner + col;
#pragma unroll 8
        for (int64_t a = s * slice + ty; a < a1; a += TY) {
            const float v = base[a * inner];
            if (best < 0 ? v == v : v > bestv) {
                bestv = v;
                best = a;
            }
        }
    }
    jv[threadIdx.x] = bestv;
    ji[threadIdx.x] = best;
    __syncthreads();
    if (ty == 0 && col < inner) {
        for (int y = 1; y < TY; y++) {
            const float ov = jv[(y << tx_log2) + tx];
            const int64_t oi = ji[(y << tx_log2) + tx];
            if (oi >= 0 && (best < 0 || ov > bestv || (ov == bestv && oi < best))) {
                bestv = ov;
                best = oi;
            }
        }
        const int64_t at = (o * splits + s) * inner + col;
        part_v[at] = bestv;
        part_i[at] = best;
    }
}

__global__ void __launch_bounds__(256)
k_argmax_cols_finish(const float *__restrict__ in, const float *__restrict__ part_v, const int64_t *__restrict__ part_i,
                     int64_t outer, int64_t axis_len, int64_t inner, int64_t splits, int64_t *__restrict__ out) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= outer * inner) return;
    const int64_t o = t / inner, i = t - o * inner;
    const float first = in[o * axis_len * inner + i];
    float bestv = 0.0f;
    int64_t best = -1;
#pragma unroll 4
    for (int64_t s = 0; s < splits; s++) {
        const int64_t at = (o * splits + s) * inner + i, oi = part_i[at];
        const float ov = part_v[at];
        if (oi >= 0 && (best < 0 || ov > bestv)) {
            bestv = ov;
            best = oi;
        }
    }
    out[t] = (first != first || best < 0) ? 0 : best;
}

// LPR lanes per row (a wave; 16 or 4 lanes for short rows, as in the row reductions), for rows
// along the contiguous axis
template <int LPR>
__global__ void __launch_bounds__(256)
k_argmax_rows(const float *__restrict__ in, int64_t rows, int64_t len, int64_t *__restrict__ out) {
    const int lane = threadIdx.x & (LPR - 1);
    const int64_t r = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
    if (r >= rows) return;
    const float *p = in + r * len;
    // lanes scan interleaved positions in ascending order, so each keeps its first maximum;
    // a lane without elements, or with NaNs only ahead of row element 0's rule, defers below
    float bestv = p[0];
    int64_t best = 0;
    for (int64_t c = lane; c < len; c += LPR) {
        const float v = p[c];
        if (v > bestv || (v == bestv && c < best)) {
            bestv = v;
            best = c;
        }
    }
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) {          // lane 0 of a row only ever takes in its own lanes
        const float ov = __shfl_down(bestv, off, 64);
        const int64_t oi = __shfl_down(best, off, 64);
        if (ov > bestv || (ov == bestv && oi < best)) {
            bestv = ov;
            best = oi;
        }
    }
    if (lane == 0) out[r] = best;
}

}  // namespace

extern "C" int axhip_reduce_axis(int op, const float *in, int64_t outer, int64_t axis_len, int64_t inner,
                                 float *out) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!in || !out) return fail(AXHIP_ERR_NULL_ARG, "reduce: NULL");
    if (outer < 0 || axis_len < 0 || inner < 0) return fail(AXHIP_ERR_SHAPE, "reduce: negative extent");
    if (outer == 0 || inner == 0) return AXHIP_OK;
    switch (op) {
        case AXHIP_RED_SUM: return axhip_sum_axis(in, outer, axis_len, inner, out);
        case AXHIP_RED_MEAN: {
            if (axis_len == 0) return fail(AXHIP_ERR_SHAPE, "mean: empty axis");
            if (int rc = axhip_sum_axis(in, outer, axis_len, inner, out)) return rc;
            return axhip_unary(AXHIP_UN_MUL_SCALAR, out, out, outer * inner, 1.0f / (float)axis_len);
        }
        case AXHIP_RED_MAX:
            if (axis_len == 0) return axhip_fill_f32(out, -FLT_MAX, outer * inner);
            return reduce_axis<AXHIP_RED_MAX>(in, outer, axis_len, inner, out);
        case AXHIP_RED_MIN:
            if (axis_len == 0) return axhip_fill_f32(out, FLT_MAX, outer * inner);
            return reduce_axis<AXHIP_RED_MIN>(in, outer, axis_len, inner, out);
        default: return fail(AXHIP_ERR_SHAPE, "reduce: unknown op %d", op);
    }
}

extern "C" int axhip_reduce_all(int op, const float *in, int64_t n, float *out) {
    if (op == AXHIP_RED_SUM) return axhip_sum_all(in, n, out);
    if (op == AXHIP_RED_MEAN) {
        if (n <= 0) return fail(AXHIP_ERR_SHAPE, "mean: empty tensor");
        if (int rc = axhip_sum_all(in, n, out)) return rc;
        return axhip_unary(AXHIP_UN_MUL_SCALAR, out, out, 1, 1.0f / (float)n);
    }
    return axhip_reduce_axis(op, in, 1, n, 1, out);
}

extern "C" int axhip_argmax_axis(const float *in, int64_t outer, int64_t axis_len, int64_t inner, int64_t *out) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!in || !out) return fail(AXHIP_ERR_NULL_ARG, "argmax: NULL");
    if (outer < 0 || axis_len <= 0 || inner < 0) return fail(AXHIP_ERR_SHAPE, "argmax: bad extent");
    if (outer == 0 || inner == 0) return AXHIP_OK;
    if (inner == 1 && axis_len >= 8) {      // shorter rows: a thread per row, below
        const int lpr = axis_len > 128 ? 64 : axis_len > 32 ? 16 : 4;      // 2 Mi rows of 32: 1062 us a thread per row, 90 us so
        const int64_t per_block = 256 / lpr, blocks = (outer + per_block - 1) / per_block;
        if (blocks > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "argmax: too many rows");
        if (lpr == 64)
            hipLaunchKernelGGL(k_argmax_rows<64>, dim3((unsigned)blocks), dim3(256), 0, kStream, in, outer, axis_len, out);
        else if (lpr == 16)
            hipLaunchKernelGGL(k_argmax_rows<16>, dim3((unsigned)blocks), dim3(256), 0, kStream, in, outer, axis_len, out);
        else
            hipLaunchKernelGGL(k_argmax_rows<4>, dim3((unsigned)blocks), dim3(256), 0, kStream, in, outer, axis_len, out);
        return check_launch("argmax_rows");
    }
    if (inner > 1 && axis_len >= 64) {      // a long axis: slices of it in parallel, then a join
        int tx_log2 = 2;
        while (tx_log2 < 6 && (int64_t(1) << tx_log2) < inner) tx_log2++;      // at least 4 axis positions a workgroup: fewer slices to join
        const int64_t col_blocks = (inner + (int64_t(1) << tx_log2) - 1) >> tx_log2;
        int64_t splits = 2048 / (outer * col_blocks);
        if (splits > axis_len / 64) splits = axis_len / 64;
        if (splits < 1) splits = 1;
        const int64_t slice = (axis_len + splits - 1) / splits, cells = outer * splits * inner;
        const int64_t part_blocks = col_blocks * splits * outer, out_blocks = (outer * inner + 255) / 256;
        if (part_blocks > 0x7fffffff || out_blocks > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "argmax: too many columns");
        char *ws = static_cast<char *>(axhip::workspace((size_t)cells * 12));
        if (!ws) return AXHIP_ERR_ALLOC;
        int64_t *part_i = reinterpret_cast<int64_t *>(ws);
        float *part_v = reinterpret_cast<float *>(ws + (size_t)cells * 8);
        hipLaunchKernelGGL(k_argmax_cols_part, dim3((unsigned)part_blocks), dim3(256), 0, kStream, in, axis_len, inner,
                           tx_log2, col_blocks, splits, slice, part_v, part_i);
        hipLaunchKernelGGL(k_argmax_cols_finish, dim3((unsigned)out_blocks), dim3(256), 0, kStream, in, part_v, part_i,
                           outer, axis_len, inner, splits, out);
        return check_launch("argmax_cols");
    }
    int64_t blocks = (outer * inner + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(k_argmax, dim3((unsigned)blocks), dim3(256), 0, kStream, in, outer, axis_len, inner, out);
    return check_launch("argmax");
}

extern "C" int axhip_sum_axis(const float *in, int64_t outer, int64_t axis_len, int64_t inner, float *out) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!in || !out) return fail(AXHIP_ERR_NULL_ARG, "sum: NULL");
    if (outer < 0 || axis_len < 0 || inner < 0) return fail(AXHIP_ERR_SHAPE, "sum: negative extent");
    if (outer == 0 || inner == 0) return AXHIP_OK;
    if (axis_len == 0) return axhip_fill_f32(out, 0.0f, outer * inner);
    if (inner == 1) return reduce_rows<AXHIP_RED_SUM>(in, outer, axis_len, out);
    if (outer > 4 || inner < 2048) return reduce_cols<AXHIP_RED_SUM>(in, outer, axis_len, inner, out);
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
    return reduce_rows<AXHIP_RED_SUM>(in, 1, n, out);
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
