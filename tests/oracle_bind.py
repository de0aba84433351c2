"""ctypes bindings for the two checkers used by the tests.

* ``Oracle``  — oracle/libax_oracle.so, this repository's CPU restatement of the path.
* ``RefLib``  — oracle/_ref/libaxref.so, the unmodified reference library compiled by
  oracle/Makefile.  Optional: absent unless it was built where the reference tree exists.

Checker code only: nothing under axiom_amd/ imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_SO = os.path.join(ROOT, "oracle", "libax_oracle.so")
REF_SO = os.path.join(ROOT, "oracle", "_ref", "libaxref.so")

f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
i8p = np.ctypeslib.ndpointer(np.int8, flags="C_CONTIGUOUS")
i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
i64 = C.c_int64


def build_oracle():
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "oracle"])


class Oracle:
    def __init__(self):
        if not os.path.exists(ORACLE_SO):
            build_oracle()
        L = self.L = C.CDLL(ORACLE_SO)
        L.axo_rng_seed.argtypes = [C.c_uint64]
        L.axo_rng_uint64.restype = C.c_uint64
        L.axo_rng_float.restype = C.c_float
        L.axo_rng_uniform.restype = C.c_float
        L.axo_rng_uniform.argtypes = [C.c_float, C.c_float]
        L.axo_rng_normal.restype = C.c_float
        L.axo_rng_bounded.restype = C.c_uint64
        L.axo_rng_bounded.argtypes = [C.c_uint64]
        L.axo_fill_uniform.argtypes = [f32p, i64, C.c_float, C.c_float]
        L.axo_fill_normal.argtypes = [f32p, i64, C.c_float, C.c_float]
        L.axo_fill_kaiming_uniform.argtypes = [f32p, i64, i64]
        L.axo_fill_int8.argtypes = [i8p, i64]
        L.axo_gemm_f64.argtypes = [f32p, f32p, f64p, i64, i64, i64, C.c_int]
        L.axo_gemm_abs_f64.argtypes = [f32p, f32p, f64p, i64, i64, i64, C.c_int]
        L.axo_gemm_naive.argtypes = [f32p, f32p, f32p, i64, i64, i64]
        L.axo_gemm_takes_small_route.argtypes = [i64, i64, i64]
        L.axo_gemm_opt.argtypes = [f32p, f32p, f32p, i64, i64, i64]
        L.axo_gemm_opt_nt.argtypes = [f32p, f32p, f32p, i64, i64, i64]
        L.axo_bias_add_cols.argtypes = [f32p, f32p, i64, i64]
        L.axo_bias_relu.argtypes = [f32p, C.c_void_p, i64, i64]
        L.axo_sum_axis0.argtypes = [f32p, i64, i64, f32p]
        L.axo_sum_axis_f64.argtypes = [f32p, i64, i64, i64, f64p, C.c_void_p]
        L.axo_axpy.argtypes = [f32p, C.c_float, f32p, i64]
        L.axo_sdpa_fwd.argtypes = [f32p, f32p, f32p, f32p, f32p, i64, i64, i64, C.c_float, C.c_int]
        L.axo_sdpa_fwd_f64.argtypes = [f32p, f32p, f32p, f64p, f64p, i64, i64, i64, C.c_float, C.c_int]
        L.axo_gelu_tanh.restype = C.c_float
        L.axo_gelu_tanh.argtypes = [C.c_float]
        L.axo_gelu_f64.restype = C.c_double
        L.axo_gelu_f64.argtypes = [C.c_double]
        L.axo_gelu.argtypes = [f32p, i64]
        L.axo_quantize_rows.argtypes = [f32p, i64, i64, i8p, f32p]
        L.axo_dequantize_rows.argtypes = [i8p, f32p, i64, i64, f32p]
        L.axo_qgemm_w8a32.argtypes = [f32p, i8p, f32p, f32p, i64, i64, i64]
        L.axo_qgemm_w8a8_acc.argtypes = [i8p, i8p, i32p, i64, i64, i64]
        L.axo_w8a8_epilogue.argtypes = [i32p, C.c_float, f32p, C.c_void_p, C.c_int, f32p, i64, i64]
        i64p = np.ctypeslib.ndpointer(np.int64, flags="C_CONTIGUOUS")
        L.axo_binary.argtypes = [C.c_int, f32p, i64p, C.c_int, f32p, i64p, C.c_int, f32p, i64p, C.c_int]
        L.axo_unary.argtypes = [C.c_int, f32p, f32p, i64, C.c_float]
        L.axo_reduce_axis.argtypes = [C.c_int, f32p, i64, i64, i64, f32p]
        L.axo_argmax_axis.argtypes = [f32p, i64, i64, i64, i64p]
        L.axo_softmax_rows.argtypes = [f32p, f32p, i64, i64]
        L.axo_layernorm_fwd.argtypes = [f32p, f32p, f32p, f32p, C.c_void_p, C.c_void_p, i64, i64, C.c_float]
        L.axo_adam_update.argtypes = [f32p, f32p, f32p, f32p, i64] + [C.c_float] * 7 + [C.c_int]
        L.axo_sgd_update.argtypes = [f32p, f32p, C.c_void_p, i64, C.c_float, C.c_float, C.c_float, C.c_int]

    # ---- RNG -------------------------------------------------------------
    def seed(self, s, drop_spare=True):
        self.L.axo_rng_seed(s)
        if drop_spare:
            self.L.axo_rng_drop_spare()

    def uniform(self, shape, lo, hi):
        out = np.empty(shape, np.float32)
        self.L.axo_fill_uniform(out.reshape(-1), out.size, lo, hi)
        return out

    def normal(self, shape, mean=0.0, std=1.0):
        out = np.empty(shape, np.float32)
        self.L.axo_fill_normal(out.reshape(-1), out.size, mean, std)
        return out

    def kaiming(self, shape, fan_in):
        out = np.empty(shape, np.float32)
        self.L.axo_fill_kaiming_uniform(out.reshape(-1), out.size, fan_in)
        return out

    def int8(self, shape):
        out = np.empty(shape, np.int8)
        self.L.axo_fill_int8(out.reshape(-1), out.size)
        return out

    # ---- GEMM ------------------------------------------------------------
    def gemm_f64(self, a, b, transb=False):
        M, K = a.shape
        N = b.shape[0] if transb else b.shape[1]
        c = np.empty((M, N), np.float64)
        self.L.axo_gemm_f64(a, b, c, M, N, K, int(transb))
        return c

    def gemm_abs_f64(self, a, b, transb=False):
        M, K = a.shape
        N = b.shape[0] if transb else b.shape[1]
        c = np.empty((M, N), np.float64)
        self.L.axo_gemm_abs_f64(a, b, c, M, N, K, int(transb))
        return c

    def gemm_naive(self, a, b):
        M, K = a.shape
        N = b.shape[1]
        c = np.empty((M, N), np.float32)
        self.L.axo_gemm_naive(a, b, c, M, N, K)
        return c

    def gemm_opt(self, a, b):
        M, K = a.shape
        N = b.shape[1]
        c = np.empty((M, N), np.float32)
        self.L.axo_gemm_opt(a, b, c, M, N, K)
        return c

    def gemm_opt_nt(self, a, b):
        M, K = a.shape
        N = b.shape[0]
        c = np.empty((M, N), np.float32)
        self.L.axo_gemm_opt_nt(a, b, c, M, N, K)
        return c

    def small_route(self, m, n, k):
        return bool(self.L.axo_gemm_takes_small_route(m, n, k))

    def bias_add(self, c, bias):
        c = np.ascontiguousarray(c, np.float32).copy()
        self.L.axo_bias_add_cols(c, bias, c.shape[0], c.shape[1])
        return c

    def bias_relu(self, c, bias):
        c = np.ascontiguousarray(c, np.float32).copy()
        bp = bias.ctypes.data_as(C.c_void_p) if bias is not None else None
        self.L.axo_bias_relu(c, bp, c.shape[0], c.shape[1])
        return c

    def sum_axis0(self, x):
        x = np.ascontiguousarray(x, np.float32)
        rows, cols = x.shape[0], int(np.prod(x.shape[1:]))
        out = np.empty(cols, np.float32)
        self.L.axo_sum_axis0(x.reshape(-1), rows, cols, out)
        return out.reshape(x.shape[1:])

    def sum_axis_f64(self, x, axis):
        """(fp64 sums over `axis`, fp64 sums of |x| over `axis`)"""
        x = np.ascontiguousarray(x, np.float32)
        outer, inner = int(np.prod(x.shape[:axis])), int(np.prod(x.shape[axis + 1:]))
        out, out_abs = np.empty(outer * inner, np.float64), np.empty(outer * inner, np.float64)
        self.L.axo_sum_axis_f64(x.reshape(-1), outer, x.shape[axis], inner, out, out_abs.ctypes.data_as(C.c_void_p))
        shape = x.shape[:axis] + x.shape[axis + 1:]
        return out.reshape(shape), out_abs.reshape(shape)

    def axpy(self, x, alpha, y):
        y = np.ascontiguousarray(y, np.float32).copy()
        self.L.axo_axpy(np.ascontiguousarray(x, np.float32).reshape(-1), alpha, y.reshape(-1), y.size)
        return y

    def sdpa(self, q, k, v, scale, causal=False, f64=False):
        """(O, L) for q, k, v of shape [BH, S, dk]; fp32 textbook evaluation, or the fp64 ground truth."""
        BH, S, dk = q.shape
        q, k, v = (np.ascontiguousarray(t, np.float32).reshape(-1) for t in (q, k, v))
        dt = np.float64 if f64 else np.float32
        o, l = np.empty(BH * S * dk, dt), np.empty(BH * S, dt)
        (self.L.axo_sdpa_fwd_f64 if f64 else self.L.axo_sdpa_fwd)(q, k, v, o, l, BH, S, dk, scale, int(causal))
        return o.reshape(BH, S, dk), l.reshape(BH, S)

    BINARY = {"add": 0, "sub": 1, "mul": 2, "div": 3, "equal": 4, "greater": 5, "add_relu": 6}
    UNARY = {"neg": 0, "abs": 1, "exp": 2, "log": 3, "sqrt": 4, "square": 5, "sigmoid": 6, "tanh": 7,
             "leaky_relu": 8, "elu": 9, "swish": 10, "add_scalar": 11, "mul_scalar": 12}
    REDUCE = {"sum": 0, "mean": 1, "max": 2, "min": 3}

    def binary(self, name, a, b):
        a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
        shape = np.broadcast_shapes(a.shape, b.shape)
        out = np.empty(shape, np.float32)
        sh = lambda t: np.array(t.shape if t.ndim else (1,), np.int64)
        self.L.axo_binary(self.BINARY[name], a.reshape(-1), sh(a), max(a.ndim, 1), b.reshape(-1), sh(b),
                          max(b.ndim, 1), out.reshape(-1), np.array(shape, np.int64), len(shape))
        return out

    def unary(self, name, x, param=0.0):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty_like(x)
        self.L.axo_unary(self.UNARY[name], x.reshape(-1), out.reshape(-1), x.size, param)
        return out

    def reduce(self, name, x, axis):
        """axis -1 reduces everything (to shape (1,))."""
        x = np.ascontiguousarray(x, np.float32)
        if axis == -1:
            out = np.empty(1, np.float32)
            self.L.axo_reduce_axis(self.REDUCE[name], x.reshape(-1), 1, x.size, 1, out)
            return out
        outer, inner = int(np.prod(x.shape[:axis])), int(np.prod(x.shape[axis + 1:]))
        out = np.empty(outer * inner, np.float32)
        self.L.axo_reduce_axis(self.REDUCE[name], x.reshape(-1), outer, x.shape[axis], inner, out)
        return out.reshape(x.shape[:axis] + x.shape[axis + 1:])

    def argmax(self, x, axis):
        x = np.ascontiguousarray(x, np.float32)
        if axis == -1:
            out = np.empty(1, np.int64)
            self.L.axo_argmax_axis(x.reshape(-1), 1, x.size, 1, out)
            return out
        outer, inner = int(np.prod(x.shape[:axis])), int(np.prod(x.shape[axis + 1:]))
        out = np.empty(outer * inner, np.int64)
        self.L.axo_argmax_axis(x.reshape(-1), outer, x.shape[axis], inner, out)
        return out.reshape(x.shape[:axis] + x.shape[axis + 1:])

    def softmax_rows(self, x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty_like(x)
        self.L.axo_softmax_rows(x.reshape(-1), out.reshape(-1), x.shape[0], x.shape[1])
        return out

    def layernorm(self, x, gamma, beta, eps):
        """(out, x_hat, inv_std) over the last axis."""
        x = np.ascontiguousarray(x, np.float32)
        rows, cols = int(np.prod(x.shape[:-1])), x.shape[-1]
        out, xh, inv = np.empty_like(x), np.empty_like(x), np.empty(rows, np.float32)
        self.L.axo_layernorm_fwd(x.reshape(-1), np.ascontiguousarray(gamma, np.float32),
                                 np.ascontiguousarray(beta, np.float32), out.reshape(-1), xh.ctypes.data,
                                 inv.ctypes.data, rows, cols, eps)
        return out, xh, inv

    def adam_update(self, w, g, m, v, lr, beta1, beta2, eps, wd, bc1, bc2, decoupled):
        """Updates w, m, v (float32 arrays) in place."""
        self.L.axo_adam_update(w.reshape(-1), np.ascontiguousarray(g, np.float32).reshape(-1), m.reshape(-1),
                               v.reshape(-1), w.size, lr, beta1, beta2, eps, wd, bc1, bc2, int(decoupled))

    def sgd_update(self, w, g, mom, lr, momentum, wd, nesterov):
        self.L.axo_sgd_update(w.reshape(-1), np.ascontiguousarray(g, np.float32).reshape(-1),
                              mom.ctypes.data if mom is not None else None, w.size, lr, momentum, wd, int(nesterov))

    def gelu(self, x):
        x = np.ascontiguousarray(x, np.float32).copy()
        self.L.axo_gelu(x.reshape(-1), x.size)
        return x

    def dense(self, x, w, bias=None, act=0):
        """act(x @ w + bias[n]) through the cpu_opt restatement; act 0 none, 1 relu, 2 gelu."""
        c = self.gemm_opt(x, w)
        if act == 1:
            return self.bias_relu(c, bias)
        if bias is not None:
            c = self.bias_add(c, bias)
        if act == 2:
            c = self.gelu(c)
        return c

    # ---- int8 ------------------------------------------------------------
    def quantize_rows(self, w):
        N, K = w.shape
        q = np.empty((N, K), np.int8)
        s = np.empty(N, np.float32)
        self.L.axo_quantize_rows(w, N, K, q, s)
        return q, s

    def dequantize_rows(self, q, s):
        out = np.empty(q.shape, np.float32)
        self.L.axo_dequantize_rows(q, s, q.shape[0], q.shape[1], out)
        return out

    def qgemm_w8a32(self, a, q, s):
        M, K = a.shape
        N = q.shape[0]
        out = np.empty((M, N), np.float32)
        self.L.axo_qgemm_w8a32(a, q, s, out, M, N, K)
        return out

    def qgemm_w8a8_acc(self, x, w):
        M, K = x.shape
        N = w.shape[0]
        acc = np.empty((M, N), np.int32)
        self.L.axo_qgemm_w8a8_acc(x, w, acc, M, N, K)
        return acc

    def w8a8_epilogue(self, acc, x_scale, w_scales, bias=None, act=0):
        M, N = acc.shape
        out = np.empty((M, N), np.float32)
        bp = bias.ctypes.data_as(C.c_void_p) if bias is not None else None
        self.L.axo_w8a8_epilogue(acc, x_scale, w_scales, bp, act, out, M, N)
        return out


# ---------------------------------------------------------------------------
# the compiled reference
# ---------------------------------------------------------------------------
AX_MAX_DIMS = 8


class RefStorage(C.Structure):            # include/axiom/tensor.h:29-43
    _fields_ = [("data", C.c_void_p), ("size_bytes", C.c_size_t), ("refcount", C.c_int),
                ("device", C.c_int), ("is_arena_temp", C.c_bool), ("generation", C.c_uint64)]


class RefTensor(C.Structure):             # include/axiom/tensor.h:53-70
    pass


RefTensor._fields_ = [("storage", C.POINTER(RefStorage)), ("shape", i64 * AX_MAX_DIMS),
                      ("strides", i64 * AX_MAX_DIMS), ("ndim", C.c_int), ("dtype", C.c_int),
                      ("offset", i64), ("requires_grad", C.c_bool),
                      ("grad", C.POINTER(RefTensor)), ("grad_fn", C.c_void_p),
                      ("layout", C.c_int)]


class RefQWeight(C.Structure):            # include/axiom/quantize.h:50-55
    _fields_ = [("data", C.POINTER(C.c_int8)), ("scales", C.POINTER(C.c_float)),
                ("N", i64), ("K", i64)]


def ref_available():
    return os.path.exists(REF_SO)


class RefLib:
    """The reference library itself (CPU backends), driven through its public C API."""
    CPU_NAIVE, CPU_SIMD = 0, 1

    def __init__(self):
        # keep the reference from calibrating / writing a cache under $HOME
        os.environ.setdefault("AX_NO_CALIB_CACHE", "1")
        os.environ.setdefault("AX_GEMM_CALIBRATE", "0")
        os.environ.setdefault("AX_NO_AUTOTUNE", "1")
        L = self.L = C.CDLL(REF_SO, mode=C.RTLD_GLOBAL)
        TP = C.POINTER(RefTensor)
        L.ax_rng_seed.argtypes = [C.c_uint64]
        L.ax_rng_uint64.restype = C.c_uint64
        L.ax_rng_float.restype = C.c_float
        L.ax_rng_uniform.restype = C.c_float
        L.ax_rng_uniform.argtypes = [C.c_float, C.c_float]
        L.ax_rng_normal.restype = C.c_float
        L.ax_rng_bounded.restype = C.c_uint64
        L.ax_rng_bounded.argtypes = [C.c_uint64]
        L.ax_set_seed.argtypes = [C.c_uint]
        L.ax_tensor_create.restype = TP
        L.ax_tensor_create.argtypes = [C.POINTER(i64), C.c_int, C.c_int]
        L.ax_tensor_zeros.restype = TP
        L.ax_tensor_zeros.argtypes = [C.POINTER(i64), C.c_int, C.c_int]
        L.ax_tensor_rand.restype = TP
        L.ax_tensor_rand.argtypes = [C.POINTER(i64), C.c_int, C.c_float, C.c_float]
        L.ax_tensor_destroy.argtypes = [TP]
        L.ax_compute_init.restype = C.c_int
        L.ax_compute_set_backend.argtypes = [C.c_int]
        L.ax_compute_set_backend.restype = C.c_int
        for name in ("ax_compute_gemm", "ax_compute_gemm_nt"):
            getattr(L, name).argtypes = [TP, TP, TP]
            getattr(L, name).restype = C.c_int
        L.ax_compute_gemm_relu.argtypes = [TP, TP, TP, TP]
        L.ax_compute_gemm_relu.restype = C.c_int
        L.ax_compute_bias_add.argtypes = [TP, TP, C.c_int, TP]
        for name in ("ax_fused_attention_fwd", "ax_fused_attention_fwd_causal"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [f32p, f32p, f32p, f32p, f32p, i64, i64, i64, C.c_float]
        L.ax_compute_sum.argtypes = [TP, C.c_int, TP]
        L.ax_compute_axpy.argtypes = [TP, C.c_float, TP]
        L.ax_compute_bias_add.restype = C.c_int
        L.ax_gelu.restype = TP
        L.ax_gelu.argtypes = [TP]
        L.ax_no_grad.restype = None
        L.ax_qweight_create_from_fp32.restype = C.POINTER(RefQWeight)
        L.ax_qweight_create_from_fp32.argtypes = [f32p, i64, i64]
        L.ax_qweight_destroy.argtypes = [C.POINTER(RefQWeight)]
        L.ax_qgemm_w8a32.restype = C.c_int
        L.ax_qgemm_w8a32.argtypes = [f32p, C.POINTER(RefQWeight), f32p, i64]
        L.ax_init_kaiming_uniform.argtypes = [TP, i64]
        L.ax_dense_create.restype = C.c_void_p
        L.ax_dense_create.argtypes = [i64, i64, C.c_bool]
        L.ax_relu_layer_create.restype = C.c_void_p
        L.ax_sequential_create.restype = C.c_void_p
        L.ax_sequential_add.restype = C.c_void_p
        L.ax_sequential_add.argtypes = [C.c_void_p, C.c_void_p]
        L.ax_layer_forward.restype = TP
        L.ax_layer_forward.argtypes = [C.c_void_p, TP]
        L.ax_layer_destroy.argtypes = [C.c_void_p]
        L.ax_layer_get_params.restype = C.c_int
        L.ax_layer_get_params.argtypes = [C.c_void_p, C.POINTER(TP), C.c_int]
        for name in ("add", "sub", "mul", "div", "equal", "greater", "add_relu"):
            getattr(L, "ax_compute_" + name).argtypes = [TP, TP, TP]
            getattr(L, "ax_compute_" + name).restype = C.c_int
        for name in ("neg", "abs", "exp", "log", "sqrt", "square", "sigmoid", "tanh", "relu", "softmax_rowwise"):
            getattr(L, "ax_compute_" + name).argtypes = [TP, TP]
            getattr(L, "ax_compute_" + name).restype = C.c_int
        for name in ("add_scalar", "mul_scalar"):
            getattr(L, "ax_compute_" + name).argtypes = [TP, C.c_double, TP]
            getattr(L, "ax_compute_" + name).restype = C.c_int
        for name in ("sum", "mean", "max", "min", "argmax"):
            getattr(L, "ax_compute_" + name).argtypes = [TP, C.c_int, TP]
            getattr(L, "ax_compute_" + name).restype = C.c_int
        for name in ("ax_leaky_relu", "ax_elu"):
            getattr(L, name).argtypes = [TP, C.c_float]
            getattr(L, name).restype = TP
        L.ax_swish.argtypes = [TP]
        L.ax_swish.restype = TP
        L.ax_layernorm_create.restype = C.c_void_p
        L.ax_layernorm_create.argtypes = [i64, C.c_float]
        PP = C.POINTER(TP)
        L.ax_adam_create.restype = C.c_void_p
        L.ax_adam_create.argtypes = [PP, C.c_int] + [C.c_float] * 5
        L.ax_adamw_create.restype = C.c_void_p
        L.ax_adamw_create.argtypes = [PP, C.c_int] + [C.c_float] * 5
        L.ax_sgd_create.restype = C.c_void_p
        L.ax_sgd_create.argtypes = [PP, C.c_int, C.c_float, C.c_float, C.c_float, C.c_bool]
        L.ax_optimizer_step.argtypes = [C.c_void_p]
        L.ax_optimizer_destroy.argtypes = [C.c_void_p]
        L.ax_compute_init()
        L.ax_no_grad()

    # ---- tensors ----------------------------------------------------------
    def tensor(self, arr):
        arr = np.ascontiguousarray(arr, np.float32)
        shape = (i64 * arr.ndim)(*arr.shape)
        t = self.L.ax_tensor_create(shape, arr.ndim, 0)
        C.memmove(t.contents.storage.contents.data, arr.ctypes.data, arr.nbytes)
        return t

    def empty(self, *shape):
        sh = (i64 * len(shape))(*shape)
        return self.L.ax_tensor_zeros(sh, len(shape), 0)

    @staticmethod
    def numpy(t):
        tt = t.contents
        shape = [tt.shape[i] for i in range(tt.ndim)]
        n = int(np.prod(shape))
        buf = (C.c_float * n).from_address(tt.storage.contents.data + 4 * tt.offset)
        return np.frombuffer(buf, np.float32).reshape(shape).copy()

    def free(self, *ts):
        for t in ts:
            self.L.ax_tensor_destroy(t)

    def backend(self, which):
        assert self.L.ax_compute_set_backend(which) == 0

    # ---- ops --------------------------------------------------------------
    def gemm(self, a, b, backend=1, nt=False):
        self.backend(backend)
        ta, tb = self.tensor(a), self.tensor(b)
        N = b.shape[0] if nt else b.shape[1]
        to = self.empty(a.shape[0], N)
        fn = self.L.ax_compute_gemm_nt if nt else self.L.ax_compute_gemm
        st = fn(ta, tb, to)
        assert st == 0, st
        out = self.numpy(to)
        self.free(ta, tb, to)
        return out

    def gemm_tn(self, a_km, b, backend=1):
        """a_km is [K,M]; returns a_km^T x b, [M,N]."""
        self.backend(backend)
        ta, tb = self.tensor(a_km), self.tensor(b)
        to = self.empty(a_km.shape[1], b.shape[1])
        st = self.L.ax_compute_gemm_tn(ta, tb, to)
        assert st == 0, st
        out = self.numpy(to)
        self.free(ta, tb, to)
        return out

    def sum(self, x, axis, backend=1):
        self.backend(backend)
        x = np.ascontiguousarray(x, np.float32)
        shape = (1,) if axis == -1 else x.shape[:axis] + x.shape[axis + 1:]
        t, to = self.tensor(x), self.empty(*shape)
        st = self.L.ax_compute_sum(t, axis, to)
        assert st == 0, st
        out = self.numpy(to)
        self.free(t, to)
        return out

    def axpy(self, x, alpha, y, backend=1):
        self.backend(backend)
        tx, ty = self.tensor(x), self.tensor(y)
        st = self.L.ax_compute_axpy(tx, alpha, ty)
        assert st == 0, st
        out = self.numpy(ty)
        self.free(tx, ty)
        return out

    def sdpa(self, q, k, v, scale, causal=False):
        """The reference's fused CPU attention (src/core/fused_attention.c:559-573): (O, L)."""
        BH, S, dk = q.shape
        q, k, v = (np.ascontiguousarray(t, np.float32).reshape(-1) for t in (q, k, v))
        o, l = np.zeros(BH * S * dk, np.float32), np.zeros(BH * S, np.float32)
        fn = self.L.ax_fused_attention_fwd_causal if causal else self.L.ax_fused_attention_fwd
        fn(q, k, v, o, l, BH, S, dk, scale)
        return o.reshape(BH, S, dk), l.reshape(BH, S)

    def gemm_relu(self, a, b, bias):
        self.backend(self.CPU_SIMD)
        ta, tb = self.tensor(a), self.tensor(b)
        tbias = self.tensor(bias) if bias is not None else None
        to = self.empty(a.shape[0], b.shape[1])
        st = self.L.ax_compute_gemm_relu(ta, tb, tbias, to)
        assert st == 0, st
        out = self.numpy(to)
        self.free(ta, tb, to)
        if tbias:
            self.free(tbias)
        return out

    def gelu(self, x):
        t = self.tensor(x)
        o = self.L.ax_gelu(t)
        out = self.numpy(o)
        self.free(t, o)
        return out

    def quantize_rows(self, w):
        N, K = w.shape
        qw = self.L.ax_qweight_create_from_fp32(np.ascontiguousarray(w), N, K)
        q = np.ctypeslib.as_array(qw.contents.data, (N, K)).copy()
        s = np.ctypeslib.as_array(qw.contents.scales, (N,)).copy()
        self.L.ax_qweight_destroy(qw)
        return q, s

    def qgemm_w8a32(self, a, q, s):
        """The reference routine on a hand-filled ax_qweight_t (a public struct)."""
        q = np.ascontiguousarray(q, np.int8)
        s = np.ascontiguousarray(s, np.float32)
        qw = RefQWeight(q.ctypes.data_as(C.POINTER(C.c_int8)),
                        s.ctypes.data_as(C.POINTER(C.c_float)), q.shape[0], q.shape[1])
        out = np.empty((a.shape[0], q.shape[0]), np.float32)
        st = self.L.ax_qgemm_w8a32(np.ascontiguousarray(a, np.float32), C.byref(qw), out,
                                   a.shape[0])
        assert st == 0
        return out

    # ---- the remaining elementwise / reduction / optimizer slots ----------------------------
    def empty_dtype(self, shape, dtype):
        sh = (i64 * len(shape))(*shape)
        return self.L.ax_tensor_zeros(sh, len(shape), dtype)

    def binary(self, name, a, b, backend=1):
        self.backend(backend)
        a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
        ta, tb = self.tensor(a), self.tensor(b)
        to = self.empty(*np.broadcast_shapes(a.shape, b.shape))
        st = getattr(self.L, "ax_compute_" + name)(ta, tb, to)
        assert st == 0, (name, st)
        out = self.numpy(to)
        self.free(ta, tb, to)
        return out

    def unary(self, name, x, backend=1, scalar=None):
        self.backend(backend)
        t, to = self.tensor(x), self.empty(*np.shape(x))
        fn = getattr(self.L, "ax_compute_" + name)
        st = fn(t, to) if scalar is None else fn(t, scalar, to)
        assert st == 0, (name, st)
        out = self.numpy(to)
        self.free(t, to)
        return out

    def reduce(self, name, x, axis, backend=1):
        self.backend(backend)
        x = np.ascontiguousarray(x, np.float32)
        shape = (1,) if axis == -1 else x.shape[:axis] + x.shape[axis + 1:]
        t = self.tensor(x)
        to = self.empty_dtype(shape, 3) if name == "argmax" else self.empty(*shape)
        st = getattr(self.L, "ax_compute_" + name)(t, axis, to)
        assert st == 0, (name, st)
        if name == "argmax":
            n = int(np.prod(shape))
            buf = (C.c_int64 * n).from_address(to.contents.storage.contents.data)
            out = np.frombuffer(buf, np.int64).reshape(shape).copy()
        else:
            out = self.numpy(to)
        self.free(t, to)
        return out

    def activation(self, name, x, alpha=None):
        """ax_leaky_relu / ax_elu / ax_swish (src/core/activations.c) on host tensors."""
        t = self.tensor(x)
        fn = getattr(self.L, "ax_" + name)
        o = fn(t) if alpha is None else fn(t, alpha)
        out = self.numpy(o)
        self.free(t, o)
        return out

    def layernorm(self, x, gamma, beta, eps):
        ln = self.L.ax_layernorm_create(x.shape[-1], eps)
        params = (C.POINTER(RefTensor) * 4)()
        assert self.L.ax_layer_get_params(ln, params, 4) == 2
        for prm, val in zip(params, (gamma, beta)):
            val = np.ascontiguousarray(val, np.float32)
            C.memmove(prm.contents.storage.contents.data, val.ctypes.data, val.nbytes)
        t = self.tensor(x)
        o = self.L.ax_layer_forward(ln, t)
        out = self.numpy(o)
        self.free(t, o)
        self.L.ax_layer_destroy(ln)
        return out

    def optimizer_steps(self, kind, w0, grads, fetch=None, **kw):
        """Runs one reference optimizer step per gradient in `grads` on a single parameter
        tensor; returns the weights after each step.  kind: adam, adamw, sgd.  Tensors are made
        with ax_tensor_from_array on the reference's default device; `fetch` reads one back when
        that device is not the CPU."""
        def from_host(arr):
            arr = np.ascontiguousarray(arr, np.float32)
            return self.L.ax_tensor_from_array(arr.ctypes.data, (i64 * arr.ndim)(*arr.shape), arr.ndim, 0)
        self.L.ax_tensor_from_array.restype = C.POINTER(RefTensor)
        self.L.ax_tensor_from_array.argtypes = [C.c_void_p, C.POINTER(i64), C.c_int, C.c_int]
        tw = from_host(w0)
        params = (C.POINTER(RefTensor) * 1)(tw)
        if kind == "sgd":
            opt = self.L.ax_sgd_create(params, 1, kw["lr"], kw["momentum"], kw["wd"], kw["nesterov"])
        else:
            make = self.L.ax_adam_create if kind == "adam" else self.L.ax_adamw_create
            opt = make(params, 1, kw["lr"], kw["beta1"], kw["beta2"], kw["eps"], kw["wd"])
        outs = []
        for g in grads:
            tg = from_host(g)
            tw.contents.grad = tg
            self.L.ax_optimizer_step(opt)
            tw.contents.grad = None
            self.free(tg)
            outs.append(fetch(tw) if fetch else self.numpy(tw))
        self.L.ax_optimizer_destroy(opt)
        self.free(tw)
        return outs
