"""ctypes binding of libaxhip.so (include/axhip.h).  Loading fails loudly when the library
has not been built; compute calls fail with AxHipError when no gfx950 GPU is present."""
import ctypes as C
import os

import numpy as np

LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
LIB_PATH = os.path.join(LIB_DIR, "libaxhip.so")

ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2
i64 = C.c_int64
vp = C.c_void_p

# every symbol include/axhip.h declares: (restype, argtypes)
SIGNATURES = {
    "axhip_init": (C.c_int, []),
    "axhip_shutdown": (None, []),
    "axhip_synchronize": (C.c_int, []),
    "axhip_device_count": (C.c_int, []),
    "axhip_last_error": (C.c_char_p, []),
    "axhip_device_name": (C.c_char_p, []),
    "axhip_tuning_reload": (C.c_int, []),
    "axhip_tuning_get": (C.c_int, [C.c_char_p]),
    "axhip_workspace_reserve": (C.c_int, [C.c_size_t, C.POINTER(C.c_size_t)]),
    "axhip_malloc": (vp, [C.c_size_t]),
    "axhip_malloc_uninit": (vp, [C.c_size_t]),
    "axhip_free": (None, [vp]),
    "axhip_alloc_stats": (None, [C.POINTER(C.c_int64)] * 6),
    "axhip_reset_alloc_stats": (None, []),
    "axhip_device_free_bytes": (C.c_int64, []),
    "axhip_memset": (C.c_int, [vp, C.c_int, C.c_size_t]),
    "axhip_memcpy_h2d": (C.c_int, [vp, vp, C.c_size_t]),
    "axhip_memcpy_d2h": (C.c_int, [vp, vp, C.c_size_t]),
    "axhip_memcpy_d2d": (C.c_int, [vp, vp, C.c_size_t]),
    "axhip_sgemm": (C.c_int, [C.c_int, C.c_int, i64, i64, i64, C.c_float, vp, i64, vp, i64,
                              C.c_float, vp, i64, vp, C.c_int]),
    "axhip_sgemm_strided_batched": (C.c_int, [C.c_int, C.c_int, i64, i64, i64, C.c_float, vp, i64,
                                              i64, vp, i64, i64, C.c_float, vp, i64, i64, i64]),
    "axhip_sgemm_skinny": (C.c_int, [i64, i64, i64, vp, i64, vp, i64, vp, i64, vp, C.c_int]),
    "axhip_sgemm_skinny_head": (C.c_int, [i64, i64, i64, vp, i64, vp, i64, vp, i64, vp, C.c_int, i64, vp, vp, C.c_int, vp]),
    "axhip_sgemm_skinny_static": (C.c_int, [i64, i64, i64, vp, i64, vp, i64, vp, i64, vp, C.c_int]),
    "axhip_sgemm_skinny_reset": (C.c_int, []),
    "axhip_probe_int8_matrix_core": (C.c_int, [C.c_int, C.c_int, vp, vp]),
    "axhip_probe_fp32_matrix_core": (C.c_int, [C.c_int, C.c_int, vp, vp]),
    "axhip_qgemm_w8a8": (C.c_int, [vp, C.c_float, vp, vp, vp, C.c_int, vp, vp, i64, i64, i64]),
    "axhip_qgemm_w8a32": (C.c_int, [vp, vp, vp, vp, i64, i64, i64]),
    "axhip_quantize_rows": (C.c_int, [vp, i64, i64, vp, vp]),
    "axhip_bias_add": (C.c_int, [vp, vp, i64, i64, i64, vp]),
    "axhip_sdpa_fwd": (C.c_int, [vp, vp, vp, vp, vp, i64, i64, i64, C.c_float, C.c_int]),
    "axhip_sdpa_fwd_rows": (C.c_int, [vp, vp, vp, i64, vp, i64, vp, i64, i64, i64, i64, C.c_float, C.c_int]),
    "axhip_sum_axis": (C.c_int, [vp, i64, i64, i64, vp]),
    "axhip_sum_all": (C.c_int, [vp, i64, vp]),
    "axhip_axpy": (C.c_int, [vp, C.c_float, vp, i64]),
    "axhip_binary": (C.c_int, [C.c_int, vp, vp, vp, C.c_int, C.POINTER(i64), C.POINTER(i64), C.POINTER(i64)]),
    "axhip_unary": (C.c_int, [C.c_int, vp, vp, i64, C.c_float]),
    "axhip_reduce_axis": (C.c_int, [C.c_int, vp, i64, i64, i64, vp]),
    "axhip_reduce_all": (C.c_int, [C.c_int, vp, i64, vp]),
    "axhip_argmax_axis": (C.c_int, [vp, i64, i64, i64, vp]),
    "axhip_softmax_rows": (C.c_int, [vp, vp, i64, i64]),
    "axhip_layernorm_fwd": (C.c_int, [vp, vp, vp, vp, vp, vp, i64, i64, C.c_float]),
    "axhip_adam_update": (C.c_int, [vp, vp, vp, vp, i64] + [C.c_float] * 7 + [C.c_int]),
    "axhip_sgd_update": (C.c_int, [vp, vp, vp, i64, C.c_float, C.c_float, C.c_float, C.c_int]),
    "axhip_head_split_qkv": (C.c_int, [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64]),
    "axhip_head_interleave": (C.c_int, [vp, vp, i64, i64, i64, i64]),
    "axhip_head_deinterleave": (C.c_int, [vp, vp, i64, i64, i64, i64]),
    "axhip_concat3_rows": (C.c_int, [vp, vp, vp, vp, i64, i64]),
    "axhip_relu": (C.c_int, [vp, vp, i64]),
    "axhip_gelu": (C.c_int, [vp, vp, i64]),
    "axhip_fill_f32": (C.c_int, [vp, C.c_float, i64]),
    "axhip_event_create": (vp, []),
    "axhip_event_destroy": (None, [vp]),
    "axhip_event_record": (C.c_int, [vp]),
    "axhip_event_elapsed_ms": (C.c_int, [vp, vp, C.POINTER(C.c_float)]),
    "axhip_last_kernel": (C.c_char_p, []),
}


class AxHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"axhip error {code}: {message}")
        self.code = code


class DeviceArray:
    """A typed, shaped view of device memory owned through axhip_malloc."""

    def __init__(self, hip, shape, dtype):
        self.hip = hip
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        self.ptr = hip.L.axhip_malloc(max(self.nbytes, 1))
        if not self.ptr:
            raise AxHipError(2, hip.last_error())

    def upload(self, host):
        host = np.ascontiguousarray(host, self.dtype)
        assert host.shape == self.shape, (host.shape, self.shape)
        if self.nbytes:
            self.hip.check(self.hip.L.axhip_memcpy_h2d(self.ptr, host.ctypes.data, self.nbytes))
        return self

    def numpy(self):
        out = np.empty(self.shape, self.dtype)
        if self.nbytes:
            self.hip.check(self.hip.L.axhip_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes))
        return out

    def free(self):
        if self.ptr:
            self.hip.L.axhip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class AxHip:
    def __init__(self, path=LIB_PATH):
        if not os.path.exists(path):
            raise ImportError(f"{path} is missing: build it with `make -C axiom_amd/csrc` "
                              "(there is no CPU fallback)")
        self.L = C.CDLL(path, mode=C.RTLD_GLOBAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(self.L, name)
            fn.restype, fn.argtypes = res, args

    # ---- helpers ---------------------------------------------------------
    def last_error(self):
        return (self.L.axhip_last_error() or b"").decode()

    def check(self, rc):
        if rc != 0:
            raise AxHipError(rc, self.last_error())

    def init(self):
        self.check(self.L.axhip_init())

    def sync(self):
        self.check(self.L.axhip_synchronize())

    def last_kernel(self):
        return (self.L.axhip_last_kernel() or b"").decode()

    def array(self, host):
        host = np.ascontiguousarray(host)
        return DeviceArray(self, host.shape, host.dtype).upload(host)

    def empty(self, shape, dtype=np.float32):
        return DeviceArray(self, shape, dtype)

    @staticmethod
    def _p(x):
        return x.ptr if x is not None else None

    # ---- GEMMs (host-array convenience forms; device-resident forms take DeviceArray) ----
    def sgemm(self, a, b, transa=False, transb=False, alpha=1.0, beta=0.0, c=None, bias=None, act=0):
        """a, b (and c, bias) are DeviceArray; returns the output DeviceArray."""
        M = a.shape[1] if transa else a.shape[0]
        K = a.shape[0] if transa else a.shape[1]
        N = b.shape[0] if transb else b.shape[1]
        if c is None:
            c = self.empty((M, N))
        self.check(self.L.axhip_sgemm(int(transa), int(transb), M, N, K, alpha, a.ptr, a.shape[1],
                                      b.ptr, b.shape[1], beta, c.ptr, N, self._p(bias), act))
        return c

    def sgemm_batched(self, a, b, transb=False, alpha=1.0):
        """a [B,M,K]; b [B,K,N] or [B,N,K] when transb; returns [B,M,N]."""
        Bn, M, K = a.shape
        N = b.shape[1] if transb else b.shape[2]
        c = self.empty((Bn, M, N))
        self.check(self.L.axhip_sgemm_strided_batched(
            0, int(transb), M, N, K, alpha, a.ptr, K, M * K, b.ptr, b.shape[2],
            b.shape[1] * b.shape[2], 0.0, c.ptr, N, M * N, Bn))
        return c

    def sgemm_skinny(self, a, b, bias=None, act=0, c=None):
        M, K = a.shape
        N = b.shape[1]
        if c is None:
            c = self.empty((M, N))
        self.check(self.L.axhip_sgemm_skinny(M, N, K, a.ptr, K, b.ptr, N, c.ptr, N, self._p(bias), act))
        return c

    def qgemm_w8a8(self, x, x_scale, w, w_scales, bias=None, act=0, want_out=True, want_acc=True):
        M, K = x.shape
        N = w.shape[0]
        out = self.empty((M, N), np.float32) if want_out else None
        acc = self.empty((M, N), np.int32) if want_acc else None
        self.check(self.L.axhip_qgemm_w8a8(x.ptr, x_scale, w.ptr, self._p(w_scales), self._p(bias),
                                           act, self._p(out), self._p(acc), M, N, K))
        return out, acc

    def qgemm_w8a32(self, a, w, w_scales):
        M, K = a.shape
        N = w.shape[0]
        out = self.empty((M, N))
        self.check(self.L.axhip_qgemm_w8a32(a.ptr, w.ptr, w_scales.ptr, out.ptr, M, N, K))
        return out

    def quantize_rows(self, w):
        N, K = w.shape
        q = self.empty((N, K), np.int8)
        s = self.empty((N,), np.float32)
        self.check(self.L.axhip_quantize_rows(w.ptr, N, K, q.ptr, s.ptr))
        return q, s

    # ---- timing ----------------------------------------------------------
    def time_ms(self, fn, iters=1):
        """Average milliseconds per call of fn() over `iters` back-to-back calls, by HIP events
        recorded on the stream the kernels run on."""
        e0, e1 = self.L.axhip_event_create(), self.L.axhip_event_create()
        self.check(self.L.axhip_event_record(e0))
        for _ in range(iters):
            fn()
        self.check(self.L.axhip_event_record(e1))
        ms = C.c_float()
        self.check(self.L.axhip_event_elapsed_ms(e0, e1, C.byref(ms)))
        self.L.axhip_event_destroy(e0)
        self.L.axhip_event_destroy(e1)
        return ms.value / iters
