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

on_cpu()
print("DROPIN OK", flush=True)
