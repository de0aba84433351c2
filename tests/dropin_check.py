"""Run by tests/test_gpu_host.py in a fresh process.  Loads the UNMODIFIED reference library
(oracle/_ref/libaxref.so, built from the reference's own sources), registers this repository's
backend object in the reference's GPU slot through the reference's public registration call, and
drives the reference's own tensors / ops / layers on the MI355X, comparing with the reference's
CPU backend in the same process."""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
sys.path.insert(0, HERE)
from oracle_bind import RefLib, RefTensor, i64  # noqa: E402

REF_DEVICE_GPU = 1       # AX_DEVICE_CUDA in the reference's include/axiom/types.h:106-110
REF_BACKEND_GPU = 3      # AX_BACKEND_CUDA in the reference's include/axiom/compute.h:46-52
REF_BACKEND_CPU = 1      # AX_BACKEND_CPU_SIMD

ref = RefLib()           # RTLD_GLOBAL: the reference's ax_err_set / ax_tensor_* serve the plugin
L = ref.L
plugin = C.CDLL(os.path.join(ROOT, "axiom_amd", "lib", "libax_hip_plugin.so"), mode=C.RTLD_GLOBAL)
plugin.ax_hip_ops_for_device.restype = C.c_void_p
plugin.ax_hip_ops_for_device.argtypes = [C.c_int]
TP = C.POINTER(RefTensor)
L.ax_compute_register_backend.argtypes = [C.c_int, C.c_void_p]
L.ax_compute_register_backend.restype = C.c_int
L.ax_device_count.argtypes = [C.c_int]
L.ax_set_default_device.argtypes = [C.c_int]
L.ax_tensor_from_array.restype = TP
L.ax_tensor_from_array.argtypes = [C.c_void_p, C.POINTER(i64), C.c_int, C.c_int]
L.ax_tensor_to_cpu.restype = TP
L.ax_tensor_to_cpu.argtypes = [TP]
L.ax_matmul_bias_relu.restype = TP
L.ax_matmul_bias_relu.argtypes = [TP, TP, TP]
L.ax_compute_backend_name.restype = C.c_char_p
L.ax_err_last_message.restype = C.c_char_p

ops = plugin.ax_hip_ops_for_device(REF_DEVICE_GPU)
assert L.ax_compute_register_backend(REF_BACKEND_GPU, ops) == 0, L.ax_err_last_message()
assert L.ax_device_count(REF_DEVICE_GPU) >= 1
print("registered:", L.ax_device_count(REF_DEVICE_GPU), "device(s)", flush=True)


def on_gpu():
    L.ax_set_default_device(REF_DEVICE_GPU)
    assert L.ax_compute_set_backend(REF_BACKEND_GPU) == 0
    assert L.ax_compute_backend_name() == b"hip"


def on_cpu():
    L.ax_set_default_device(0)
    assert L.ax_compute_set_backend(REF_BACKEND_CPU) == 0


def dev_tensor(arr):
    arr = np.ascontiguousarray(arr, np.float32)
    sh = (i64 * arr.ndim)(*arr.shape)
    t = L.ax_tensor_from_array(arr.ctypes.data, sh, arr.ndim, 0)
    assert t and t.contents.storage.contents.device == REF_DEVICE_GPU
    return t


def fetch(t):
    c = L.ax_tensor_to_cpu(t)
    out = ref.numpy(c)
    ref.free(c)
    return out


rng = np.random.default_rng(0)
# 1. the reference's ax_compute_gemm / gemm_nt / gemm_relu on device tensors
for (M, K, N) in [(64, 128, 32), (256, 512, 384), (1, 784, 4096), (37, 73, 19)]:
    a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    b = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    bias = rng.normal(0, 0.5, N).astype(np.float32)
    on_cpu()
    want, want_relu = ref.gemm(a, b), ref.gemm_relu(a, b, bias)
    on_gpu()
    ta, tb, tbias = dev_tensor(a), dev_tensor(b), dev_tensor(bias)
    out = L.ax_tensor_zeros((i64 * 2)(M, N), 2, 0)
    assert out.contents.storage.contents.device == REF_DEVICE_GPU
    assert L.ax_compute_gemm(ta, tb, out) == 0, L.ax_err_last_message()
    got = fetch(out)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max(), (M, K, N)
    tbt = dev_tensor(np.ascontiguousarray(b.T))
    assert L.ax_compute_gemm_nt(ta, tbt, out) == 0
    assert np.abs(fetch(out) - want).max() <= 1e-4 * np.abs(want).max()
    y = L.ax_matmul_bias_relu(ta, tb, tbias)               # the reference's op layer -> our gemm_relu slot
    assert y, L.ax_err_last_message()
    assert np.abs(fetch(y) - want_relu).max() <= 1e-4 * np.abs(want).max()
    ref.free(ta, tb, tbias, out, tbt, y)
    print("gemm", M, K, N, "ok", flush=True)

# 2. the reference's own Sequential MLP, built twice from the same seed: once on the CPU backend,
#    once with its parameters allocated on the MI355X through our storage hooks
def build_and_run(x):
    L.ax_set_seed(99)
    seq = L.ax_sequential_create()
    for (i, o, relu) in ((784, 4096, True), (4096, 4096, True), (4096, 10, False)):
        L.ax_sequential_add(seq, L.ax_dense_create(i, o, True))
        if relu:
            L.ax_sequential_add(seq, L.ax_relu_layer_create())
    sh = (i64 * 2)(*x.shape)
    tx = L.ax_tensor_from_array(x.ctypes.data, sh, 2, 0)
    y = L.ax_layer_forward(seq, tx)
    assert y, L.ax_err_last_message()
    out = fetch(y) if y.contents.storage.contents.device != 0 else ref.numpy(y)
    ref.free(tx, y)
    L.ax_layer_destroy(seq)
    return out


for M in (1, 8, 128):
    x = rng.uniform(0, 1, (M, 784)).astype(np.float32)
    on_cpu()
    want = build_and_run(x)
    on_gpu()
    got = build_and_run(x)
    assert got.shape == (M, 10)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max(), M
    print("sequential M=%d ok" % M, flush=True)

# 3. the reference's own autograd node for the dense layer (matmul_bias_backward,
#    src/core/autograd_ops.c:603-757) run on the MI355X: gemm_nt, gemm_tn, sum and copy slots.
#    The node's backward function is the first member of ax_grad_fn_t (include/axiom/autograd.h:48-50).
L.ax_matmul_bias.restype = TP
L.ax_matmul_bias.argtypes = [TP, TP, TP]
BACKWARD = C.CFUNCTYPE(None, C.c_void_p, TP)


def dense_backward(x, w, b, dy):
    sh = lambda a: (i64 * a.ndim)(*a.shape)
    ts = [L.ax_tensor_from_array(np.ascontiguousarray(a, np.float32).ctypes.data, sh(a), a.ndim, 0)
          for a in (x, w, b, dy)]
    tx, tw, tb, tdy = ts
    for t in (tx, tw, tb):
        t.contents.requires_grad = True
    L.ax_enable_grad()
    y = L.ax_matmul_bias(tx, tw, tb)
    assert y and y.contents.grad_fn, L.ax_err_last_message()
    fn = BACKWARD(C.cast(y.contents.grad_fn, C.POINTER(C.c_void_p))[0])
    fn(y.contents.grad_fn, tdy)
    L.ax_no_grad()
    grads = []
    for t in (tx, tw, tb):
        g = t.contents.grad
        assert g, "gradient was not produced"
        grads.append(fetch(g) if g.contents.storage.contents.device != 0 else ref.numpy(g))
    return grads


for (M, K, N) in [(48, 40, 24), (256, 512, 384)]:
    x = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    w = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    b = rng.uniform(-1, 1, N).astype(np.float32)
    dy = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    on_cpu()
    want = dense_backward(x, w, b, dy)
    on_gpu()
    got = dense_backward(x, w, b, dy)
    for name, g, r_ in zip(("dX", "dW", "dBias"), got, want):
        assert g.shape == r_.shape, name
        assert np.abs(g - r_).max() <= 1e-4 * np.abs(r_).max(), (name, M, K, N)
    print("dense backward", M, K, N, "ok", flush=True)

# 4. the reference's tensor-level ops (src/core/ops.c:107-283, 444-537) on device tensors: each
#    allocates its result through our storage hooks and dispatches to our elementwise / reduction slots
for name in ("ax_add", "ax_sub", "ax_mul", "ax_div"):
    getattr(L, name).restype = TP
    getattr(L, name).argtypes = [TP, TP]
for name in ("ax_neg", "ax_exp", "ax_square", "ax_sigmoid", "ax_tanh_op", "ax_relu"):
    getattr(L, name).restype = TP
    getattr(L, name).argtypes = [TP]
for name in ("ax_sum", "ax_mean", "ax_max", "ax_min"):
    getattr(L, name).restype = TP
    getattr(L, name).argtypes = [TP, C.c_int]


def run_ops(a, b):
    ta, tb = (L.ax_tensor_from_array(v.ctypes.data, (i64 * v.ndim)(*v.shape), v.ndim, 0) for v in (a, b))
    outs = {}
    for name in ("ax_add", "ax_sub", "ax_mul", "ax_div"):
        outs[name] = getattr(L, name)(ta, tb)
    for name in ("ax_neg", "ax_exp", "ax_square", "ax_sigmoid", "ax_tanh_op", "ax_relu"):
        outs[name] = getattr(L, name)(ta)
    for name in ("ax_sum", "ax_mean", "ax_max", "ax_min"):
        for axis in (-1, 0, 1, 2):
            outs[f"{name}{axis}"] = getattr(L, name)(ta, axis)
    res = {}
    for k, t in outs.items():
        assert t, (k, L.ax_err_last_message())
        res[k] = fetch(t) if t.contents.storage.contents.device != 0 else ref.numpy(t)
        ref.free(t)
    ref.free(ta, tb)
    return res


a = rng.uniform(-2, 2, (6, 5, 32)).astype(np.float32)
b = rng.uniform(0.5, 2, (5, 1)).astype(np.float32)
L.ax_no_grad()
on_cpu()
want = run_ops(a, b)
on_gpu()
got = run_ops(a, b)
for k in want:
    assert got[k].shape == want[k].shape, k
    assert np.abs(got[k] - want[k]).max() <= 2e-5 * max(1.0, np.abs(want[k]).max()), k
print("tensor ops ok:", len(want), flush=True)

# 5. the reference's optimizers (src/core/optim.c): with a parameter on the device, sgd_step and
#    adam_step hand each update to the backend's sgd_update / adam_update slot (optim.c:78-110, 243-266)
on_cpu()
w0 = rng.uniform(-1, 1, 500).astype(np.float32)
grads = [rng.uniform(-1, 1, 500).astype(np.float32) for _ in range(3)]
for kind, kw in (("adam", dict(lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01)),
                 ("adamw", dict(lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01)),
                 ("sgd", dict(lr=5e-2, momentum=0.9, wd=0.01, nesterov=True)),
                 ("sgd", dict(lr=5e-2, momentum=0.0, wd=0.0, nesterov=False))):
    on_cpu()
    want = ref.optimizer_steps(kind, w0, grads, **kw)
    on_gpu()
    got = ref.optimizer_steps(kind, w0, grads, fetch=fetch, **kw)
    for step, (g_, w_) in enumerate(zip(got, want)):
        assert np.abs(g_ - w_).max() <= 2e-6, (kind, step)
    print("optimizer", kind, "ok", flush=True)

# 6. the extension table through the reference's own registry (src/compute/dispatch.c:286-300).  The
#    reference's attention layer rebuilds its fused projection cache through the table
#    (ax_attn_refresh_fused_qkv, src/core/attention/cache.c:24-85); its forward pass itself cannot be
#    driven on any GPU device: it wraps the input in a stack view labelled AX_DEVICE_CPU
#    (src/core/attention.c:71-89,176-179) and then decides `on_cuda` from that label (:211), so it
#    walks device pointers with host memcpy.  What runs here: registration, the cache rebuild by the
#    reference's code, and every forward member of the table on the reference's device tensors.
class RefLayer(C.Structure):                 # include/axiom/layer.h:72-85
    _fields_ = [("forward", C.c_void_p), ("destroy", C.c_void_p), ("type", C.c_int), ("training", C.c_bool),
                ("params", TP * 8), ("n_params", C.c_int), ("buffers", TP * 4), ("n_buffers", C.c_int),
                ("input_features", i64), ("output_features", i64)]


class RefMHA(C.Structure):                   # include/axiom/attention.h:59-89
    _fields_ = [("base", RefLayer), ("d_model", i64), ("n_heads", C.c_int), ("d_k", i64), ("use_bias", C.c_bool),
                ("causal", C.c_bool), ("Wq", TP), ("Wk", TP), ("Wv", TP), ("Wo", TP), ("bq", TP), ("bk", TP), ("bv", TP),
                ("bo", TP), ("Wqkv_cache", TP), ("bqkv_cache", TP)]


EXT_FIELDS = [("split", C.CFUNCTYPE(None, *([C.c_void_p] * 4 + [i64] * 5))),
              ("split_bias", C.CFUNCTYPE(None, *([C.c_void_p] * 5 + [i64] * 5))),
              ("interleave", C.CFUNCTYPE(None, C.c_void_p, C.c_void_p, i64, i64, i64, i64)),
              ("deinterleave", C.CFUNCTYPE(None, C.c_void_p, C.c_void_p, i64, i64, i64, i64)),
              ("merge", C.c_void_p), ("qkv_cache_build", C.c_void_p), ("bias_cache_build", C.c_void_p),
              ("sdpa_fwd", C.CFUNCTYPE(C.c_int, *([C.c_void_p] * 5 + [i64] * 3 + [C.c_float, C.c_bool, C.c_void_p])))]


class RefExtension(C.Structure):             # include/axiom/internal/cuda_extension.h:41-140, leading members
    _fields_ = EXT_FIELDS


ext_addr = C.addressof(C.c_char.in_dll(plugin, "ax_hip_extension"))
L.ax_compute_register_cuda_extension.argtypes = [C.c_void_p]
L.ax_compute_register_cuda_extension.restype = C.c_int
L.ax_compute_get_cuda_extension.restype = C.c_void_p
assert L.ax_compute_register_cuda_extension(ext_addr) == 0
assert L.ax_compute_get_cuda_extension() == ext_addr
L.ax_mha_create.restype = C.c_void_p
L.ax_mha_create.argtypes = [C.c_int64, C.c_int, C.c_bool, C.c_bool]
L.ax_attn_refresh_fused_qkv.argtypes = [C.c_void_p]
on_gpu()
L.ax_set_seed(4242)
D, H = 96, 6
layer = L.ax_mha_create(D, H, True, False)
assert layer, L.ax_err_last_message()
mha = C.cast(layer, C.POINTER(RefMHA)).contents
assert mha.d_model == D and mha.n_heads == H and mha.Wq.contents.storage.contents.device == REF_DEVICE_GPU
L.ax_attn_refresh_fused_qkv(layer)
assert mha.Wqkv_cache and mha.Wqkv_cache.contents.storage.contents.device == REF_DEVICE_GPU
wq, wk, wv = fetch(mha.Wq), fetch(mha.Wk), fetch(mha.Wv)
assert np.array_equal(fetch(mha.Wqkv_cache), np.concatenate([wq, wk, wv], axis=1))
assert np.array_equal(fetch(mha.bqkv_cache), np.concatenate([fetch(mha.bq), fetch(mha.bk), fetch(mha.bv)]))
# the forward members, called through the registered table on the reference's device tensors
ext = C.cast(L.ax_compute_get_cuda_extension(), C.POINTER(RefExtension)).contents
B, S, dk = 2, 40, D // H
x = rng.uniform(-1, 1, (B * S, D)).astype(np.float32)
tx = dev_tensor(x)
qkv = L.ax_tensor_zeros((i64 * 2)(B * S, 3 * D), 2, 0)
assert L.ax_compute_gemm(tx, mha.Wqkv_cache, qkv) == 0, L.ax_err_last_message()
heads = [L.ax_tensor_zeros((i64 * 3)(B * H, S, dk), 3, 0) for _ in range(4)]
attn = L.ax_tensor_zeros((i64 * 2)(B * S, D), 2, 0)
ptr = lambda t: t.contents.storage.contents.data
ext.split_bias(ptr(qkv), ptr(mha.bqkv_cache), ptr(heads[0]), ptr(heads[1]), ptr(heads[2]), B, S, H, dk, D)
assert ext.sdpa_fwd(ptr(heads[0]), ptr(heads[1]), ptr(heads[2]), ptr(heads[3]), None, B * H, S, dk,
                    1.0 / np.sqrt(dk), False, None) == 0, L.ax_err_last_message()
ext.deinterleave(ptr(heads[3]), ptr(attn), B, S, H, dk)
got = fetch(attn)
on_cpu()
full = ref.gemm(x, np.concatenate([wq, wk, wv], axis=1)) + fetch(mha.bqkv_cache)
hq, hk, hv = (np.ascontiguousarray(full[:, i * D:(i + 1) * D].reshape(B, S, H, dk).transpose(0, 2, 1, 3)).reshape(B * H, S, dk)
              for i in range(3))
o, _ = ref.sdpa(hq, hk, hv, float(1.0 / np.sqrt(dk)))
want = o.reshape(B, H, S, dk).transpose(0, 2, 1, 3).reshape(B * S, D)
assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max()), np.abs(got - want).max()
on_gpu()
ref.free(tx, qkv, attn, *heads)
L.ax_layer_destroy(layer)
L.ax_compute_register_cuda_extension(None)
print("extension table ok", flush=True)

on_cpu()
print("DROPIN OK", flush=True)
