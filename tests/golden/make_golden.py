"""Writes tests/golden/golden.npz from the compiled reference (oracle/_ref/libaxref.so).

Run where the reference was built:  python tests/golden/make_golden.py
Every array is an input/output vector of the reference's public C API; the file holds
data only.  Inputs that tests can regenerate (seeded fills) are stored as checksums.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from fills import property_case, xorshift32_unit  # noqa: E402
from oracle_bind import RefLib  # noqa: E402

r = RefLib()
L = r.L
G = {}

# ---- RNG known answers (src/core/rng.c) -----------------------------------
for seed in (0, 42):
    L.ax_rng_seed(seed)
    G[f"rng_u64_seed{seed}"] = np.array([L.ax_rng_uint64() for _ in range(8)], np.uint64)
    L.ax_rng_seed(seed)
    G[f"rng_uniform_seed{seed}"] = np.array([L.ax_rng_uniform(-1.0, 1.0) for _ in range(8)], np.float32)
    L.ax_rng_seed(seed)
    G[f"rng_normal_seed{seed}"] = np.array([L.ax_rng_normal() for _ in range(8)], np.float32)
    L.ax_rng_seed(seed)
    G[f"rng_bounded255_seed{seed}"] = np.array([L.ax_rng_bounded(255) for _ in range(32)], np.uint64)


def ref_uniform(n, lo, hi):
    return np.array([L.ax_rng_uniform(lo, hi) for _ in range(n)], np.float32)


# ---- quantizer (src/core/quantize.c:21-57) --------------------------------
hand = np.array([[0.5, -1.0, 0.25, 0.1], [0.0, 0.0, 0.0, 0.0]], np.float32)
G["quant_hand_w"] = hand
G["quant_hand_q"], G["quant_hand_s"] = r.quantize_rows(hand)
s = np.float32(1.0) / np.float32(127.0)
ties = np.array([[127 * s, 0.5 * s, 1.5 * s, 2.5 * s, -0.5 * s, -1.5 * s, -2.5 * s, 3.5 * s]], np.float32)
G["quant_ties_w"] = ties
G["quant_ties_q"], G["quant_ties_s"] = r.quantize_rows(ties)
for (N, K) in ((8, 8), (128, 128), (64, 1024)):          # tests/test_quantize.c:60-69 shapes
    w = xorshift32_unit(N * K, 42).reshape(N, K)
    q, sc = r.quantize_rows(w)
    G[f"quant_{N}x{K}_q"], G[f"quant_{N}x{K}_s"] = q, sc

# ---- W8A32 (src/core/quantize.c:100-177) at tests/test_quantize.c:133-137 shapes
for (M, N, K) in ((1, 8, 8), (4, 16, 32), (8, 64, 128), (32, 128, 512), (16, 256, 1024), (3, 17, 45)):
    a = xorshift32_unit(M * K, 7).reshape(M, K)
    w = xorshift32_unit(N * K, 13).reshape(N, K)
    q, sc = r.quantize_rows(w)
    G[f"w8a32_{M}x{N}x{K}_out"] = r.qgemm_w8a32(a, q, sc)

# ---- int8 accumulators through the reference's W8A32 routine with unit scales
for K in (8, 32, 128, 512, 1024):
    L.ax_rng_seed(1000 + K)
    x = np.array([int(L.ax_rng_bounded(255)) - 127 for _ in range(4 * K)], np.int8).reshape(4, K)
    w = np.array([int(L.ax_rng_bounded(255)) - 127 for _ in range(64 * K)], np.int8).reshape(64, K)
    G[f"acc_K{K}_x_sum"] = np.array([x.astype(np.int64).sum()])
    G[f"acc_K{K}_w_sum"] = np.array([w.astype(np.int64).sum()])
    G[f"acc_K{K}"] = r.qgemm_w8a32(x.astype(np.float32), w, np.ones(64, np.float32))
xs = np.full((2, 1024), 127, np.int8)
ws = np.full((3, 1024), -127, np.int8)
G["acc_extreme"] = r.qgemm_w8a32(xs.astype(np.float32), ws, np.ones(3, np.float32))

# ---- fp32 GEMM ---------------------------------------------------------------
# known answers held by the reference's tests (test_compute.c:162-199, test_cuda.c:44-58)
a = np.arange(1, 7, dtype=np.float32).reshape(2, 3)
b = np.arange(7, 13, dtype=np.float32).reshape(3, 2)
G["gemm_2x3x2"] = r.gemm(a, b)
G["gemm_2x2x2"] = r.gemm(np.array([[1, 2], [3, 4]], np.float32), np.array([[5, 6], [7, 8]], np.float32))
for (M, K, N) in ((37, 73, 19), (64, 128, 32), (32, 2048, 16), (1, 784, 64), (7, 300, 130)):
    L.ax_rng_seed(M * 1000 + N)
    a = ref_uniform(M * K, -1.0, 1.0).reshape(M, K)
    b = ref_uniform(K * N, -1.0, 1.0).reshape(K, N)
    G[f"gemm_{M}x{K}x{N}_opt"] = r.gemm(a, b, backend=1)
    G[f"gemm_{M}x{K}x{N}_naive"] = r.gemm(a, b, backend=0)
    G[f"gemm_nt_{M}x{K}x{N}_opt"] = r.gemm(a, np.ascontiguousarray(b.T), backend=1, nt=True)
# 1024^3 from ax_set_seed(0): checksums only
L.ax_set_seed(0)
A = ref_uniform(1024 * 1024, -1.0, 1.0).reshape(1024, 1024)
B = ref_uniform(1024 * 1024, -1.0, 1.0).reshape(1024, 1024)
Cm = r.gemm(A, B)
G["gemm_1024_probe"] = np.array([A[0, 0], B[0, 0], Cm[0, 0], Cm[-1, -1]], np.float32)
G["gemm_1024_sums"] = np.array([Cm.astype(np.float64).sum(), np.abs(Cm).astype(np.float64).sum()])
G["gemm_1024_row0"] = Cm[0].copy()
G["gemm_1024_diag"] = np.diagonal(Cm).copy()
# the 60 property cases (tests/test_property.c:176-208)
shapes, sums = [], []
for i in range(60):
    M, N, K, a, b = property_case(i)
    cn = r.gemm(a, b, backend=0)
    co = r.gemm(a, b, backend=1)
    shapes.append((M, N, K))
    sums.append((cn.astype(np.float64).sum(), co.astype(np.float64).sum(),
                 np.abs(co).astype(np.float64).sum(), float(co[0, 0]), float(co[-1, -1])))
G["prop_shapes"] = np.array(shapes, np.int64)
G["prop_sums"] = np.array(sums, np.float64)

# ---- fused bias + relu (cpu_opt.c:7401-7440) and GELU (activations.c:267-316)
L.ax_rng_seed(77)
a = ref_uniform(33 * 100, -1.0, 1.0).reshape(33, 100)
b = ref_uniform(100 * 40, -1.0, 1.0).reshape(100, 40)
bias = ref_uniform(40, -0.5, 0.5)
G["gemm_relu_33x100x40"] = r.gemm_relu(a, b, bias)
G["gemm_relu_33x100x40_nobias"] = r.gemm_relu(a, b, None)
xg = np.linspace(-6, 6, 1201, dtype=np.float32)
G["gelu_x"] = xg
G["gelu_y"] = r.gelu(xg.reshape(1, -1)).reshape(-1)

# ---- dense backward building blocks (src/core/autograd_ops.c:603-757): dA = dY W^T (gemm_nt),
# dW = X^T dY (gemm_tn), dBias = sum(dY, 0), accumulation by axpy
L.ax_rng_seed(4242)
Mb, Kb, Nb = 48, 40, 24                                   # tokens, in features, out features
xb = ref_uniform(Mb * Kb, -1.0, 1.0).reshape(Mb, Kb)
wb = ref_uniform(Kb * Nb, -1.0, 1.0).reshape(Kb, Nb)      # Dense weight is [in, out]
dyb = ref_uniform(Mb * Nb, -1.0, 1.0).reshape(Mb, Nb)
G["dense_bwd_dA"] = r.gemm(dyb, wb, backend=1, nt=True)   # [M,N] x [K,N]^T
G["dense_bwd_dW"] = r.gemm_tn(xb, dyb, backend=1)         # [M,K]^T x [M,N]
G["dense_bwd_db"] = r.sum(dyb, 0, backend=1)
G["dense_bwd_db_naive"] = r.sum(dyb, 0, backend=0)
L.ax_rng_seed(4343)
s2 = ref_uniform(37 * 19, -1.0, 1.0).reshape(37, 19)
s3 = ref_uniform(4 * 9 * 10, -1.0, 1.0).reshape(4, 9, 10)
for name, arr in (("sum2d", s2), ("sum3d", s3)):
    for axis in [-1] + list(range(arr.ndim)):
        G[f"{name}_axis{axis}"] = r.sum(arr, axis, backend=1)
        G[f"{name}_axis{axis}_naive"] = r.sum(arr, axis, backend=0)
xa, ya = ref_uniform(1003, -1.0, 1.0), ref_uniform(1003, -1.0, 1.0)
G["axpy_1003"] = r.axpy(xa, 0.37, ya, backend=1)
G["axpy_1003_naive"] = r.axpy(xa, 0.37, ya, backend=0)

# ---- scaled dot-product attention forward (src/core/fused_attention.c:559-573) at the shapes
# of tests/test_attention.c:54-60,101-104 and one with dk = 64
for (BH, S, dk, causal) in ((6, 24, 16, 0), (2, 16, 8, 1), (3, 128, 64, 0), (3, 128, 64, 1), (2, 40, 32, 1)):
    L.ax_rng_seed(5000 + BH * 100 + S + dk + causal)
    q = ref_uniform(BH * S * dk, -0.5, 0.5).reshape(BH, S, dk)
    k = ref_uniform(BH * S * dk, -0.5, 0.5).reshape(BH, S, dk)
    v = ref_uniform(BH * S * dk, -0.5, 0.5).reshape(BH, S, dk)
    o, l = r.sdpa(q, k, v, float(np.float32(1.0) / np.sqrt(np.float32(dk))), bool(causal))
    G[f"sdpa_{BH}x{S}x{dk}_c{causal}_O"], G[f"sdpa_{BH}x{S}x{dk}_c{causal}_L"] = o, l

# ---- remaining elementwise / reduction / optimizer slots --------------------------------
# inputs come from ax_rng_seed + ax_rng_uniform so that the tests can regenerate them; the
# shapes follow tests/test_compute.c (broadcast [2,3]+[3], [2,1]+[1,3]) and tests/test_cuda.c
BCAST = (((5, 7), (5, 7)), ((2, 3), (3,)), ((2, 1), (1, 3)), ((4, 1, 6), (3, 1)), ((2, 3, 4), (1,)),
         ((3, 8, 16), (8, 1)))
for case, (sa, sb) in enumerate(BCAST):
    L.ax_rng_seed(7000 + case)
    # values on a coarse grid so that equal / greater see ties
    a = np.round(ref_uniform(int(np.prod(sa)), -2.0, 2.0) * 4) / 4
    b = np.round(ref_uniform(int(np.prod(sb)), -2.0, 2.0) * 4) / 4
    a, b = a.reshape(sa).astype(np.float32), b.reshape(sb).astype(np.float32)
    for name in ("add", "sub", "mul", "div", "equal", "greater"):
        G[f"bin_{name}_{case}"] = r.binary(name, a, b, backend=0)
        assert np.array_equal(G[f"bin_{name}_{case}"], r.binary(name, a, b, backend=1), equal_nan=True)
    if sa == sb:
        G[f"bin_add_relu_{case}"] = r.binary("add_relu", a, b, backend=0)
L.ax_rng_seed(7100)
ux = np.concatenate([ref_uniform(200, -4.0, 4.0), np.array([0.0, -0.0, 1.0, -1.0, 30.0, -30.0, 1e-20], np.float32)])
for name in ("neg", "abs", "exp", "log", "sqrt", "square", "sigmoid", "tanh"):
    G[f"un_{name}"] = r.unary(name, ux, backend=0)
G["un_add_scalar"] = r.unary("add_scalar", ux, backend=0, scalar=0.37)
G["un_mul_scalar"] = r.unary("mul_scalar", ux, backend=0, scalar=-1.7)
G["un_leaky_relu"] = r.activation("leaky_relu", ux, 0.1)
G["un_elu"] = r.activation("elu", ux, 0.7)
G["un_swish"] = r.activation("swish", ux)
L.ax_rng_seed(7200)
for name_shape in (((6, 10),), ((4, 5, 6),), ((3, 200),)):
    shp = name_shape[0]
    arr = ref_uniform(int(np.prod(shp)), -1.0, 1.0).reshape(shp)
    tag = "x".join(map(str, shp))
    for axis in range(-1, len(shp)):
        for name in ("mean", "max", "min"):
            G[f"red_{name}_{tag}_axis{axis}"] = r.reduce(name, arr, axis, backend=1)
            G[f"red_{name}_{tag}_axis{axis}_naive"] = r.reduce(name, arr, axis, backend=0)
        G[f"red_argmax_{tag}_axis{axis}"] = r.reduce("argmax", arr, axis, backend=1)
L.ax_rng_seed(7300)
for (rows, cols) in ((5, 7), (3, 300), (2, 1000), (4, 64)):
    arr = ref_uniform(rows * cols, -6.0, 6.0).reshape(rows, cols)
    G[f"softmax_{rows}x{cols}"] = r.unary("softmax_rowwise", arr, backend=1)
    G[f"softmax_{rows}x{cols}_naive"] = r.unary("softmax_rowwise", arr, backend=0)
L.ax_rng_seed(7400)
for shp in ((6, 16), (2, 5, 100), (3, 768)):
    arr = ref_uniform(int(np.prod(shp)), -3.0, 5.0).reshape(shp)
    gamma, beta = ref_uniform(shp[-1], 0.5, 1.5), ref_uniform(shp[-1], -1.0, 1.0)
    G["layernorm_" + "x".join(map(str, shp))] = r.layernorm(arr, gamma, beta, 1e-5)
L.ax_rng_seed(7500)
w0 = ref_uniform(300, -1.0, 1.0)
grads = [ref_uniform(300, -1.0, 1.0) for _ in range(3)]
G["opt_adam"] = np.stack(r.optimizer_steps("adam", w0, grads, lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01))
G["opt_adamw"] = np.stack(r.optimizer_steps("adamw", w0, grads, lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01))
G["opt_sgd_plain"] = np.stack(r.optimizer_steps("sgd", w0, grads, lr=5e-2, momentum=0.0, wd=0.0, nesterov=False))
G["opt_sgd_momentum"] = np.stack(r.optimizer_steps("sgd", w0, grads, lr=5e-2, momentum=0.9, wd=0.01, nesterov=False))
G["opt_sgd_nesterov"] = np.stack(r.optimizer_steps("sgd", w0, grads, lr=5e-2, momentum=0.9, wd=0.01, nesterov=True))

# ---- model files written by the reference (src/core/serialize.c) ------------------------------
import ctypes as C  # noqa: E402

for name in ("ax_relu_layer_create", "ax_sigmoid_layer_create", "ax_tanh_layer_create", "ax_gelu_layer_create",
             "ax_swish_layer_create", "ax_flatten_create"):
    getattr(L, name).restype = C.c_void_p
    getattr(L, name).argtypes = []
for name in ("ax_leaky_relu_layer_create", "ax_elu_layer_create"):
    getattr(L, name).restype = C.c_void_p
    getattr(L, name).argtypes = [C.c_float]
L.ax_softmax_layer_create.restype = C.c_void_p
L.ax_softmax_layer_create.argtypes = [C.c_int]
L.ax_model_create.restype = C.c_void_p
L.ax_model_create.argtypes = [C.c_void_p]
L.ax_model_save.argtypes = [C.c_void_p, C.c_char_p]
L.ax_model_destroy.argtypes = [C.c_void_p]
L.ax_tensor_save.argtypes = [C.POINTER(type(r.empty(1).contents)), C.c_char_p]


def ref_model(tag, layers, in_shape, seed):
    """Builds a Sequential in the reference, perturbs every parameter, saves it and records the
    reference's CPU forward of a seeded input."""
    L.ax_set_seed(seed)
    seq = L.ax_sequential_create()
    for make in layers:
        assert L.ax_sequential_add(seq, make())
    params = (C.POINTER(type(r.empty(1).contents)) * 64)()
    n = L.ax_layer_get_params(seq, params, 64)
    L.ax_rng_seed(seed + 1)
    for i in range(n):                                   # biases / gamma / beta away from 0 and 1
        t = params[i].contents
        cnt = int(np.prod([t.shape[d] for d in range(t.ndim)]))
        buf = (C.c_float * cnt).from_address(t.storage.contents.data)
        if t.ndim == 1:
            buf[:] = list(np.frombuffer(buf, np.float32) + ref_uniform(cnt, -0.5, 0.5))
    x = ref_uniform(int(np.prod(in_shape)), -1.0, 1.0).reshape(in_shape)
    r.backend(1)
    tx = r.tensor(x)
    y = L.ax_layer_forward(seq, tx)
    G[f"axm_{tag}_out"] = r.numpy(y)
    r.free(tx, y)
    model = L.ax_model_create(seq)
    assert L.ax_model_save(model, os.path.join(HERE, f"ref_{tag}.axm").encode()) == 0
    L.ax_model_destroy(model)


ref_model("mlp", [lambda: L.ax_dense_create(12, 20, True), L.ax_relu_layer_create,
                  lambda: L.ax_layernorm_create(20, 1e-5), lambda: L.ax_dense_create(20, 6, False),
                  lambda: L.ax_leaky_relu_layer_create(0.1), lambda: L.ax_softmax_layer_create(1)], (5, 12), 8100)
# a Dense that is not followed by ReLU carries no bias here: the reference's unfused path hands its
# bias to bias_add with axis 0 (src/core/ops.c:357), which rejects it or adds it down the rows, so
# its outputs for such layers are not the layer's definition
ref_model("ffn", [lambda: L.ax_layernorm_create(64, 1e-5), lambda: L.ax_dense_create(64, 256, False),
                  L.ax_gelu_layer_create, lambda: L.ax_dense_create(256, 64, False)], (2, 7, 64), 8200)
ref_model("acts", [lambda: L.ax_dense_create(9, 9, False), L.ax_sigmoid_layer_create, L.ax_tanh_layer_create,
                   lambda: L.ax_elu_layer_create(0.7), L.ax_swish_layer_create], (4, 9), 8300)
L.ax_mha_create.restype = C.c_void_p
L.ax_mha_create.argtypes = [C.c_int64, C.c_int, C.c_bool, C.c_bool]
# the encoder block of benchmarks/bench_transformer.c:33-44 (LN, MHA, LN, Dense, GELU, Dense) and a
# causal attention layer whose head size takes the fused kernel
ref_model("encoder", [lambda: L.ax_layernorm_create(64, 1e-5), lambda: L.ax_mha_create(64, 4, True, False),
                      lambda: L.ax_layernorm_create(64, 1e-5), lambda: L.ax_dense_create(64, 128, False),
                      L.ax_gelu_layer_create, lambda: L.ax_dense_create(128, 64, False)], (2, 24, 64), 8600)
ref_model("mha_causal", [lambda: L.ax_mha_create(128, 2, True, True)], (2, 128, 128), 8700)
# a file whose first layer has no forward pass in the port: it must be refused, not misread
L.ax_set_seed(8400)
seq = L.ax_sequential_create()
L.ax_sequential_add(seq, L.ax_flatten_create())
L.ax_sequential_add(seq, L.ax_dense_create(4, 3, True))
model = L.ax_model_create(seq)
assert L.ax_model_save(model, os.path.join(HERE, "ref_flatten.axm").encode()) == 0
L.ax_model_destroy(model)
L.ax_rng_seed(8500)
tt = r.tensor(ref_uniform(3 * 4 * 5, -1.0, 1.0).reshape(3, 4, 5))
assert L.ax_tensor_save(tt, os.path.join(HERE, "ref_tensor.axt").encode()) == 0
r.free(tt)

np.savez_compressed(os.path.join(HERE, "golden.npz"), **G)
print("wrote", len(G), "arrays,", os.path.getsize(os.path.join(HERE, "golden.npz")), "bytes")

# ---- struct layout of the reference's boundary types -----------------------------------
import subprocess  # noqa: E402
import tempfile  # noqa: E402

with tempfile.TemporaryDirectory() as tmp:
    exe = os.path.join(tmp, "abi_probe")
    subprocess.check_call(["gcc", "-std=gnu11", "-I/root/reference/include",
                           os.path.join(HERE, "abi_probe.c"), "-o", exe])
    layout = subprocess.check_output([exe]).decode()
open(os.path.join(HERE, "abi_layout.json"), "w").write(layout)
print("wrote abi_layout.json")
