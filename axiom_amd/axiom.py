"""ctypes binding of libaxiom_hip.so — the C host core (include/axiom/*.h) with the ax_hip_ops
backend.  Mirrors the reference's public C API for the GEMM path: same names, arguments and
error behaviour.  Used by the tests and examples; the library itself is plain C."""
import ctypes as C
import os

import numpy as np

from .hip import LIB_DIR

LIB_PATH = os.path.join(LIB_DIR, "libaxiom_hip.so")
i64 = C.c_int64
AX_MAX_DIMS = 8
DEVICE_CPU, DEVICE_CUDA, DEVICE_HIP = 0, 1, 2
BACKEND_HIP = 4
FLOAT32, INT32, UINT8 = 0, 2, 4
ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2


class Storage(C.Structure):
    _fields_ = [("data", C.c_void_p), ("size_bytes", C.c_size_t), ("refcount", C.c_int),
                ("device", C.c_int), ("is_arena_temp", C.c_bool), ("generation", C.c_uint64)]


class Tensor(C.Structure):
    pass


Tensor._fields_ = [("storage", C.POINTER(Storage)), ("shape", i64 * AX_MAX_DIMS),
                   ("strides", i64 * AX_MAX_DIMS), ("ndim", C.c_int), ("dtype", C.c_int),
                   ("offset", i64), ("requires_grad", C.c_bool), ("grad", C.POINTER(Tensor)),
                   ("grad_fn", C.c_void_p), ("layout", C.c_int)]
TP = C.POINTER(Tensor)


class QWeight(C.Structure):
    _fields_ = [("data", C.c_void_p), ("scales", C.c_void_p), ("N", i64), ("K", i64)]


QP = C.POINTER(QWeight)
f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")

SIGNATURES = {
    "ax_init": (C.c_int, []), "ax_shutdown": (None, []),
    "ax_compute_init": (C.c_int, []), "ax_compute_shutdown": (None, []),
    "ax_compute_set_backend": (C.c_int, [C.c_int]), "ax_compute_get_backend": (C.c_int, []),
    "ax_compute_backend_name": (C.c_char_p, []),
    "ax_compute_register_backend": (C.c_int, [C.c_int, C.c_void_p]),
    "ax_compute_get_ops": (C.c_void_p, []), "ax_backend_for_device": (C.c_void_p, [C.c_int]),
    "ax_compute_gemm": (C.c_int, [TP, TP, TP]), "ax_compute_gemm_nt": (C.c_int, [TP, TP, TP]),
    "ax_compute_gemm_tn": (C.c_int, [TP, TP, TP]),
    "ax_compute_gemm_relu": (C.c_int, [TP, TP, TP, TP]),
    "ax_compute_gemm_ex": (C.c_int, [TP, TP, C.c_float, C.c_float, TP]),
    "ax_compute_bias_add": (C.c_int, [TP, TP, C.c_int, TP]),
    "ax_compute_relu": (C.c_int, [TP, TP]), "ax_compute_gelu": (C.c_int, [TP, TP]),
    "ax_compute_fill": (C.c_int, [TP, C.c_double]), "ax_compute_copy": (C.c_int, [TP, TP]),
    "ax_hip_sdpa_fwd": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, i64, i64, i64,
                                 C.c_float, C.c_bool, C.c_void_p]),
    "ax_compute_sum": (C.c_int, [TP, C.c_int, TP]), "ax_compute_axpy": (C.c_int, [TP, C.c_float, TP]),
    **{"ax_compute_" + n: (C.c_int, [TP, TP, TP]) for n in ("add", "sub", "mul", "div", "equal", "greater", "add_relu")},
    **{"ax_compute_" + n: (C.c_int, [TP, TP]) for n in ("neg", "abs", "exp", "log", "sqrt", "square", "sigmoid", "tanh",
                                                        "swish", "softmax_rowwise")},
    **{"ax_compute_" + n: (C.c_int, [TP, C.c_double, TP]) for n in ("add_scalar", "mul_scalar")},
    **{"ax_compute_" + n: (C.c_int, [TP, C.c_float, TP]) for n in ("leaky_relu", "elu")},
    **{"ax_compute_" + n: (C.c_int, [TP, C.c_int, TP]) for n in ("mean", "max", "min", "argmax")},
    "ax_compute_adam_update": (C.c_int, [TP, TP, TP, TP] + [C.c_float] * 7 + [C.c_bool]),
    "ax_compute_sgd_update": (C.c_int, [TP, TP, TP, C.c_float, C.c_float, C.c_float, C.c_bool]),
    "ax_compute_has_adam_update": (C.c_int, []), "ax_compute_has_sgd_update": (C.c_int, []),
    "ax_compute_layernorm": (C.c_int, [TP, TP, TP, C.c_float, TP, TP, TP]),
    "ax_layernorm_create": (C.c_void_p, [C.c_int64, C.c_float]),
    "ax_mha_create": (C.c_void_p, [C.c_int64, C.c_int, C.c_bool, C.c_bool]),
    "ax_init_xavier_uniform": (None, [TP, C.c_int64, C.c_int64]),
    "ax_compute_register_cuda_extension": (C.c_int, [C.c_void_p]),
    "ax_compute_get_cuda_extension": (C.c_void_p, []),
    "ax_sigmoid_layer_create": (C.c_void_p, []), "ax_tanh_layer_create": (C.c_void_p, []),
    "ax_swish_layer_create": (C.c_void_p, []), "ax_leaky_relu_layer_create": (C.c_void_p, [C.c_float]),
    "ax_elu_layer_create": (C.c_void_p, [C.c_float]), "ax_softmax_layer_create": (C.c_void_p, [C.c_int]),
    "ax_sigmoid": (TP, [TP]), "ax_tanh_op": (TP, [TP]), "ax_swish": (TP, [TP]),
    "ax_leaky_relu": (TP, [TP, C.c_float]), "ax_elu": (TP, [TP, C.c_float]), "ax_softmax": (TP, [TP, C.c_int]),
    "ax_tensor_write": (C.c_int, [TP, C.c_void_p, C.c_size_t]),
    "ax_model_create": (C.c_void_p, [C.c_void_p]), "ax_model_predict": (TP, [C.c_void_p, TP]),
    "ax_model_destroy": (None, [C.c_void_p]),
    "ax_model_save": (C.c_int, [C.c_void_p, C.c_char_p]), "ax_model_load": (C.c_void_p, [C.c_char_p]),
    "ax_tensor_save": (C.c_int, [TP, C.c_char_p]), "ax_tensor_load": (TP, [C.c_char_p]),
    "ax_qweight_save": (C.c_int, [QP, C.c_char_p]), "ax_qweight_load": (QP, [C.c_char_p]),
    "ax_compute_gemm_bias_act": (C.c_int, [TP, TP, TP, C.c_int, TP]),
    "ax_compute_has_gemm_relu": (C.c_int, []), "ax_compute_has_gemm_nt": (C.c_int, []),
    "ax_compute_has_gemm_tn": (C.c_int, []), "ax_compute_has_gemm_ex": (C.c_int, []),
    "ax_compute_has_bias_add": (C.c_int, []), "ax_compute_has_gemm_bias_act": (C.c_int, []),
    "ax_compute_has_gemm_act_head": (C.c_int, []),
    "ax_compute_gemm_act_head": (C.c_int, [TP, TP, TP, C.c_int, TP, TP, C.c_int, TP]),
    "ax_matmul_bias_act_head": (TP, [TP, TP, TP, C.c_int, TP, TP, C.c_int]),
    "ax_device_count": (C.c_int, [C.c_int]), "ax_device_synchronize": (None, [C.c_int]),
    "ax_device_is_available": (C.c_int, [C.c_int]),
    "ax_err_clear": (None, []), "ax_err_last_status": (C.c_int, []),
    "ax_err_last_message": (C.c_char_p, []), "ax_status_name": (C.c_char_p, [C.c_int]),
    "ax_storage_create": (C.POINTER(Storage), [C.c_size_t, C.c_int]),
    "ax_storage_retain": (None, [C.POINTER(Storage)]), "ax_storage_release": (None, [C.POINTER(Storage)]),
    "ax_tensor_create": (TP, [C.POINTER(i64), C.c_int, C.c_int]),
    "ax_tensor_zeros": (TP, [C.POINTER(i64), C.c_int, C.c_int]),
    "ax_tensor_from_array": (TP, [C.c_void_p, C.POINTER(i64), C.c_int, C.c_int]),
    "ax_tensor_rand": (TP, [C.POINTER(i64), C.c_int, C.c_float, C.c_float]),
    "ax_tensor_destroy": (None, [TP]), "ax_set_seed": (None, [C.c_uint]),
    "ax_tensor_numel": (i64, [TP]), "ax_tensor_is_contiguous": (C.c_bool, [TP]),
    "ax_tensor_reshape": (TP, [TP, C.POINTER(i64), C.c_int]),
    "ax_set_default_device": (None, [C.c_int]), "ax_get_default_device": (C.c_int, []),
    "ax_tensor_to_device": (TP, [TP, C.c_int]), "ax_tensor_to_cpu": (TP, [TP]),
    "ax_tensor_read": (C.c_int, [TP, C.c_void_p, C.c_size_t]),
    "ax_rng_seed": (None, [C.c_uint64]), "ax_rng_is_seeded": (C.c_bool, []),
    "ax_rng_uint64": (C.c_uint64, []), "ax_rng_float": (C.c_float, []),
    "ax_rng_uniform": (C.c_float, [C.c_float, C.c_float]), "ax_rng_normal": (C.c_float, []),
    "ax_rng_normal_params": (C.c_float, [C.c_float, C.c_float]),
    "ax_rng_bounded": (C.c_uint64, [C.c_uint64]),
    "ax_init_kaiming_uniform": (None, [TP, i64]), "ax_init_normal": (None, [TP, C.c_float, C.c_float]),
    "ax_init_uniform": (None, [TP, C.c_float, C.c_float]),
    "ax_matmul": (TP, [TP, TP]), "ax_matmul_bias": (TP, [TP, TP, TP]),
    "ax_matmul_bias_relu": (TP, [TP, TP, TP]), "ax_matmul_bias_gelu": (TP, [TP, TP, TP]),
    "ax_relu": (TP, [TP]), "ax_gelu": (TP, [TP]),
    "ax_dense_create": (C.c_void_p, [i64, i64, C.c_bool]), "ax_relu_layer_create": (C.c_void_p, []),
    "ax_gelu_layer_create": (C.c_void_p, []), "ax_sequential_create": (C.c_void_p, []),
    "ax_sequential_add": (C.c_void_p, [C.c_void_p, C.c_void_p]),
    "ax_layer_forward": (TP, [C.c_void_p, TP]),
    "ax_layer_get_params": (C.c_int, [C.c_void_p, C.POINTER(TP), C.c_int]),
    "ax_layer_destroy": (None, [C.c_void_p]),
    "ax_qweight_create_from_fp32": (QP, [f32p, i64, i64]), "ax_qweight_destroy": (None, [QP]),
    "ax_qweight_dequantize": (None, [QP, f32p]),
    "ax_qweight_to_device": (QP, [QP, C.c_int]), "ax_qweight_device_destroy": (None, [QP, C.c_int]),
    "ax_qgemm_w8a32": (C.c_int, [f32p, QP, f32p, i64]),
    "ax_qgemm_w8a32_dev": (C.c_int, [C.c_void_p, QP, C.c_void_p, i64]),
    "ax_qgemm_w8a8_dev": (C.c_int, [C.c_void_p, C.c_float, QP, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, i64]),
    "ax_hip_ops_for_device": (C.c_void_p, [C.c_int]),
}
DATA_SYMBOLS = ["ax_hip_ops", "ax_hip_extension"]


class Axiom:
    def __init__(self, path=LIB_PATH):
        if not os.path.exists(path):
            raise ImportError(f"{path} is missing: build it with `make -C axiom_amd/csrc`")
        self.L = C.CDLL(path, mode=C.RTLD_GLOBAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(self.L, name)
            fn.restype, fn.argtypes = res, args

    def err(self):
        return self.L.ax_err_last_status(), (self.L.ax_err_last_message() or b"").decode()

    @staticmethod
    def shape_arg(shape):
        return (i64 * len(shape))(*shape), len(shape)

    def from_numpy(self, arr, device=DEVICE_HIP):
        arr = np.ascontiguousarray(arr, np.float32)
        sh, nd = self.shape_arg(arr.shape)
        prev = self.L.ax_get_default_device()
        self.L.ax_set_default_device(device)
        t = self.L.ax_tensor_from_array(arr.ctypes.data, sh, nd, FLOAT32)
        self.L.ax_set_default_device(prev)
        if not t:
            raise RuntimeError("ax_tensor_from_array: %s" % (self.err(),))
        return t

    def empty(self, shape, device=DEVICE_HIP):
        sh, nd = self.shape_arg(shape)
        prev = self.L.ax_get_default_device()
        self.L.ax_set_default_device(device)
        t = self.L.ax_tensor_create(sh, nd, FLOAT32)
        self.L.ax_set_default_device(prev)
        if not t:
            raise RuntimeError("ax_tensor_create: %s" % (self.err(),))
        return t

    def to_numpy(self, t):
        tt = t.contents
        shape = tuple(tt.shape[i] for i in range(tt.ndim))
        out = np.empty(shape, np.float32)
        st = self.L.ax_tensor_read(t, out.ctypes.data, out.nbytes)
        if st != 0:
            raise RuntimeError("ax_tensor_read: %s" % (self.err(),))
        return out

    def free(self, *ts):
        for t in ts:
            if t:
                self.L.ax_tensor_destroy(t)
