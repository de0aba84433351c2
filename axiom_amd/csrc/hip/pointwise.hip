// Broadcasting binary ops, unary/scalar ops and the fused optimizer updates behind the
// elementwise vtable slots (the reference's GPU definitions: cuda/ops_elementwise.cu:44-66,
// 135-203, cuda/ops_activations.cu:23-52, cuda/ops_fused.cu:13-33, cuda/ops_optim.cu:17-62).
// All are one pass over memory, HBM-bound: 16-byte accesses wherever alignment and the
// broadcast pattern allow, otherwise one element per thread.
#include <float.h>

#include "common.h"

namespace {
using namespace axhip;

template <int OP>
__device__ __forceinline__ float binop(float a, float b) {
    if (OP == AXHIP_BIN_ADD) return a + b;
    if (OP == AXHIP_BIN_SUB) return a - b;
    if (OP == AXHIP_BIN_MUL) return a * b;
    if (OP == AXHIP_BIN_DIV) return a / b;
    if (OP == AXHIP_BIN_EQUAL) return a == b ? 1.0f : 0.0f;
    if (OP == AXHIP_BIN_GREATER) return a > b ? 1.0f : 0.0f;
    const float v = a + b;                       // AXHIP_BIN_ADD_RELU
    return v > 0.0f ? v : 0.0f;
}

template <int OP>
__device__ __forceinline__ float unop(float v, float p) {
    if (OP == AXHIP_UN_NEG) return -v;
    if (OP == AXHIP_UN_ABS) return fabsf(v);
    if (OP == AXHIP_UN_EXP) return expf(v);
    if (OP == AXHIP_UN_LOG) return v > 0.0f ? logf(v) : -FLT_MAX;
    if (OP == AXHIP_UN_SQRT) return v >= 0.0f ? sqrtf(v) : 0.0f;
    if (OP == AXHIP_UN_SQUARE) return v * v;
    if (OP == AXHIP_UN_SIGMOID) return 1.0f / (1.0f + expf(-v));
    if (OP == AXHIP_UN_TANH) return tanhf(v);
    if (OP == AXHIP_UN_LEAKY_RELU) return v > 0.0f ? v : p * v;
    if (OP == AXHIP_UN_ELU) return v > 0.0f ? v : p * (expf(v) - 1.0f);
    if (OP == AXHIP_UN_SWISH) return v / (1.0f + expf(-v));
    if (OP == AXHIP_UN_ADD_SCALAR) return v + p;
    return v * p;                                // AXHIP_UN_MUL_SCALAR
}

// The output seen as [rows..., inner]: `nouter` collapsed outer dimensions (sizes and the two
// operands' element strides, 0 where an operand is broadcast), innermost extent `inner` with
// operand strides ia, ib.
struct Bcast {
    int nouter;
    int64_t size[7], sa[7], sb[7];
    int64_t inner, ia, ib;
};

template <typename IDX>
__device__ __forceinline__ void row_offsets(const Bcast &g, IDX row, int64_t &oa, int64_t &ob) {
    oa = ob = 0;
    for (int d = g.nouter - 1; d >= 0; d--) {
        const IDX sz = (IDX)g.size[d];
        const IDX q = row / sz, idx = row - q * sz;
        row = q;
        oa += (int64_t)idx * g.sa[d];
        ob += (int64_t)idx * g.sb[d];
    }
}

// VEC: every thread owns 4 consecutive elements of the inner dimension (inner strides 0 or 1),
// moved as 16 bytes at whatever alignment the row has (global memory takes unaligned vector
// accesses); the last group of a row whose length is not a multiple of 4 goes by element.
// Otherwise one element per thread.
template <int OP, bool VEC, typename IDX>
__global__ void __launch_bounds__(256)
k_binary(const float *a, const float *b, float *out, Bcast g,
         int64_t items) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    const IDX per_row = (IDX)(VEC ? (g.inner + 3) / 4 : g.inner);
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < items; t += stride) {
        const IDX row = (IDX)t / per_row, col = (IDX)t - row * per_row;
        int64_t oa, ob;
        row_offsets<IDX>(g, row, oa, ob);
        if (VEC) {
            const int64_t c = (int64_t)col * 4;
            float *dst = out + (int64_t)row * g.inner + c;
            if (c + 4 <= g.inner) {
                v4f va, vb, r;
                if (g.ia) __builtin_memcpy(&va, a + oa + c, 16);
                else va = v4f{a[oa], a[oa], a[oa], a[oa]};
                if (g.ib) __builtin_memcpy(&vb, b + ob + c, 16);
                else vb = v4f{b[ob], b[ob], b[ob], b[ob]};
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = binop<OP>(va[e], vb[e]);
                __builtin_memcpy(dst, &r, 16);
            } else {
                for (int64_t e = 0; c + e < g.inner; e++)
                    dst[e] = binop<OP>(a[oa + (c + e) * g.ia], b[ob + (c + e) * g.ib]);
            }
        } else {
            out[t] = binop<OP>(a[oa + (int64_t)col * g.ia], b[ob + (int64_t)col * g.ib]);
        }
    }
}

template <int OP>
__global__ void __launch_bounds__(256)
k_unary_p(const float *in, float *out, int64_t n, float p, int vec) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        const int64_t n4 = n >> 2;
        for (int64_t j = i; j < n4; j += stride) {
            v4f v;
            __builtin_memcpy(&v, in + 4 * j, 16);         // any alignment
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = unop<OP>(v[e], p);
            __builtin_memcpy(out + 4 * j, &v, 16);
        }
        for (int64_t j = (n4 << 2) + i; j < n; j += stride) out[j] = unop<OP>(in[j], p);
    } else {
        for (int64_t j = i; j < n; j += stride) out[j] = unop<OP>(in[j], p);
    }
}

// w, m, v updated in place; one thread per element (cuda/ops_optim.cu:17-35)
__global__ void __launch_bounds__(256)
k_adam(float *__restrict__ w, const float *__restrict__ g, float *__restrict__ m, float *__restrict__ v,
       int64_t n, float lr, float beta1, float beta2, float eps, float decay_scale, float wd_grad,
       float bc1, float bc2) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const float wi = w[i] * decay_scale;
        const float gi = g[i] + wd_grad * wi;
        const float mi = beta1 * m[i] + (1.0f - beta1) * gi;
        const float vi = beta2 * v[i] + (1.0f - beta2) * gi * gi;
        const float mh = mi / bc1, vh = vi / bc2;
        w[i] = wi - lr * mh / (sqrtf(vh) + eps);
        m[i] = mi;
        v[i] = vi;
    }
}

// cuda/ops_optim.cu:40-62
__global__ void __launch_bounds__(256)
k_sgd(float *__restrict__ w, const float *__restrict__ g, float *__restrict__ mom, int64_t n, float lr,
      float momentum, float weight_decay, int nesterov) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        float gi = g[i];
        if (weight_decay > 0.0f) gi += weight_decay * w[i];
        if (mom && momentum > 0.0f) {
            const float vi = momentum * mom[i] + gi;
            mom[i] = vi;
            w[i] -= nesterov ? lr * (gi + momentum * vi) : lr * vi;
        } else {
            w[i] -= lr * gi;
        }
    }
}

unsigned blocks_for(int64_t items) {
    int64_t b = (items + 255) / 256;
    if (b < 1) b = 1;
    if (b > 256 * 32) b = 256 * 32;
    return (unsigned)b;
}

template <int OP>
int launch_binary(const float *a, const float *b, float *out, const Bcast &g, int64_t rows) {
    const bool vec = g.inner >= 4 && (g.ia == 0 || g.ia == 1) && (g.ib == 0 || g.ib == 1);
    const int64_t items = rows * (vec ? (g.inner + 3) / 4 : g.inner);
    const bool narrow = items < 0x7fffffff && rows < 0x7fffffff && g.inner < 0x7fffffff;
    const dim3 grid(blocks_for(items)), block(256);
    if (vec && narrow) hipLaunchKernelGGL((k_binary<OP, true, unsigned>), grid, block, 0, kStream, a, b, out, g, items);
    else if (vec) hipLaunchKernelGGL((k_binary<OP, true, int64_t>), grid, block, 0, kStream, a, b, out, g, items);
    else if (narrow) hipLaunchKernelGGL((k_binary<OP, false, unsigned>), grid, block, 0, kStream, a, b, out, g, items);
    else hipLaunchKernelGGL((k_binary<OP, false, int64_t>), grid, block, 0, kStream, a, b, out, g, items);
    return check_launch("binary");
}

template <int OP>
int launch_unary(const float *in, float *out, int64_t n, float p) {
    const int vec = 1;
    hipLaunchKernelGGL(k_unary_p<OP>, dim3(blocks_for(vec ? n / 4 + 1 : n)), dim3(256), 0, kStream, in, out, n, p, vec);
    return check_launch("unary");
}
}  // namespace

extern "C" {

int axhip_binary(int op, const float *a, const float *b, float *out, int ndim, const int64_t *out_shape,
                 const int64_t *a_strides, const int64_t *b_strides) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!a || !b || !out) return fail(AXHIP_ERR_NULL_ARG, "binary: NULL tensor");
    if (ndim < 0 || ndim > 8 || (ndim > 0 && (!out_shape || !a_strides || !b_strides)))
        return fail(AXHIP_ERR_SHAPE, "binary: 0..8 dimensions with shape and strides");
    if (op < AXHIP_BIN_ADD || op > AXHIP_BIN_ADD_RELU) return fail(AXHIP_ERR_SHAPE, "binary: unknown op %d", op);
    // drop extent-1 dimensions, then merge neighbours that both operands walk as one run
    int64_t size[8], sa[8], sb[8];
    int nd = 0;
    int64_t total = 1;
    for (int d = 0; d < ndim; d++) {
        if (out_shape[d] < 0) return fail(AXHIP_ERR_SHAPE, "binary: negative extent");
        total *= out_shape[d];
        if (out_shape[d] == 1) continue;
        if (a_strides[d] < 0 || b_strides[d] < 0) return fail(AXHIP_ERR_SHAPE, "binary: negative stride");
        if (nd > 0 && sa[nd - 1] == a_strides[d] * out_shape[d] && sb[nd - 1] == b_strides[d] * out_shape[d]) {
            size[nd - 1] *= out_shape[d];
            sa[nd - 1] = a_strides[d];
            sb[nd - 1] = b_strides[d];
        } else {
            size[nd] = out_shape[d];
            sa[nd] = a_strides[d];
            sb[nd] = b_strides[d];
            nd++;
        }
    }
    if (total == 0) return AXHIP_OK;
    Bcast g{};
    if (nd == 0) {
        g.inner = 1;
    } else {
        g.inner = size[nd - 1];
        g.ia = sa[nd - 1];
        g.ib = sb[nd - 1];
        g.nouter = nd - 1;
        for (int d = 0; d < nd - 1; d++) {
            g.size[d] = size[d];
            g.sa[d] = sa[d];
            g.sb[d] = sb[d];
        }
    }
    const int64_t rows = total / g.inner;
    switch (op) {
        case AXHIP_BIN_ADD: return launch_binary<AXHIP_BIN_ADD>(a, b, out, g, rows);
        case AXHIP_BIN_SUB: return launch_binary<AXHIP_BIN_SUB>(a, b, out, g, rows);
        case AXHIP_BIN_MUL: return launch_binary<AXHIP_BIN_MUL>(a, b, out, g, rows);
        case AXHIP_BIN_DIV: return launch_binary<AXHIP_BIN_DIV>(a, b, out, g, rows);
        case AXHIP_BIN_EQUAL: return launch_binary<AXHIP_BIN_EQUAL>(a, b, out, g, rows);
        case AXHIP_BIN_GREATER: return launch_binary<AXHIP_BIN_GREATER>(a, b, out, g, rows);
        default: return launch_binary<AXHIP_BIN_ADD_RELU>(a, b, out, g, rows);
    }
}

int axhip_unary(int op, const float *in, float *out, int64_t n, float param) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!in || !out) return fail(AXHIP_ERR_NULL_ARG, "unary: NULL tensor");
    if (n <= 0) return n < 0 ? fail(AXHIP_ERR_SHAPE, "unary: negative size") : AXHIP_OK;
    switch (op) {
        case AXHIP_UN_NEG: return launch_unary<AXHIP_UN_NEG>(in, out, n, param);
        case AXHIP_UN_ABS: return launch_unary<AXHIP_UN_ABS>(in, out, n, param);
        case AXHIP_UN_EXP: return launch_unary<AXHIP_UN_EXP>(in, out, n, param);
        case AXHIP_UN_LOG: return launch_unary<AXHIP_UN_LOG>(in, out, n, param);
        case AXHIP_UN_SQRT: return launch_unary<AXHIP_UN_SQRT>(in, out, n, param);
        case AXHIP_UN_SQUARE: return launch_unary<AXHIP_UN_SQUARE>(in, out, n, param);
        case AXHIP_UN_SIGMOID: return launch_unary<AXHIP_UN_SIGMOID>(in, out, n, param);
        case AXHIP_UN_TANH: return launch_unary<AXHIP_UN_TANH>(in, out, n, param);
        case AXHIP_UN_LEAKY_RELU: return launch_unary<AXHIP_UN_LEAKY_RELU>(in, out, n, param);
        case AXHIP_UN_ELU: return launch_unary<AXHIP_UN_ELU>(in, out, n, param);
        case AXHIP_UN_SWISH: return launch_unary<AXHIP_UN_SWISH>(in, out, n, param);
        case AXHIP_UN_ADD_SCALAR: return launch_unary<AXHIP_UN_ADD_SCALAR>(in, out, n, param);
        case AXHIP_UN_MUL_SCALAR: return launch_unary<AXHIP_UN_MUL_SCALAR>(in, out, n, param);
        default: return fail(AXHIP_ERR_SHAPE, "unary: unknown op %d", op);
    }
}

int axhip_adam_update(float *w, const float *g, float *m, float *v, int64_t n, float lr, float beta1,
                      float beta2, float eps, float weight_decay, float bc1, float bc2, int decoupled) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!w || !g || !m || !v) return fail(AXHIP_ERR_NULL_ARG, "adam_update: NULL tensor");
    if (n <= 0) return n < 0 ? fail(AXHIP_ERR_SHAPE, "adam_update: negative size") : AXHIP_OK;
    // cuda/ops_optim.cu:75-77
    float decay_scale = decoupled ? (1.0f - lr * weight_decay) : 1.0f;
    if (decay_scale < 0.0f) decay_scale = 0.0f;
    const float wd_grad = (!decoupled && weight_decay > 0.0f) ? weight_decay : 0.0f;
    hipLaunchKernelGGL(k_adam, dim3(blocks_for(n)), dim3(256), 0, kStream, w, g, m, v, n, lr, beta1, beta2, eps,
                       decay_scale, wd_grad, bc1, bc2);
    return check_launch("adam_update");
}

int axhip_sgd_update(float *w, const float *g, float *momentum_buf, int64_t n, float lr, float momentum,
                     float weight_decay, int nesterov) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!w || !g) return fail(AXHIP_ERR_NULL_ARG, "sgd_update: NULL tensor");
    if (n <= 0) return n < 0 ? fail(AXHIP_ERR_SHAPE, "sgd_update: negative size") : AXHIP_OK;
    hipLaunchKernelGGL(k_sgd, dim3(blocks_for(n)), dim3(256), 0, kStream, w, g, momentum_buf, n, lr, momentum,
                       weight_decay, nesterov ? 1 : 0);
    return check_launch("sgd_update");
}

}  // extern "C"
