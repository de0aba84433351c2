"""GPU tests of the host side: the Axiom C API of libaxiom_hip.so driving ax_hip_ops, and the
backend object dropped into the unmodified reference library through its own
ax_compute_register_backend()."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REL = 1e-4     # fp32: max |gpu - cpu| / max |cpu|
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def ax():
    from axiom_amd.axiom import Axiom
    a = Axiom()
    assert a.L.ax_init() == 0, a.err()
    assert a.L.ax_compute_backend_name() == b"hip"
    a.L.ax_set_default_device(2)
    yield a
    a.L.ax_set_default_device(0)


def close(got, ref, rel=REL):
    return np.abs(got - ref).max() <= rel * max(np.abs(ref).max(), 1e-30)


def test_dispatch_wrappers(ax, oracle):
    L = ax.L
    assert L.ax_device_count(2) >= 1 and L.ax_device_is_available(2) == 1
    assert all(f() == 1 for f in (L.ax_compute_has_gemm_relu, L.ax_compute_has_gemm_nt, L.ax_compute_has_gemm_tn,
                                  L.ax_compute_has_gemm_ex, L.ax_compute_has_bias_add, L.ax_compute_has_gemm_bias_act))
    oracle.seed(5)
    M, K, N = 70, 130, 90
    a, b = oracle.uniform((M, K), -1, 1), oracle.uniform((K, N), -1, 1)
    bias = oracle.normal((N,), 0, 0.5)
    ref = oracle.gemm_opt(a, b)
    ta, tb, tbias = ax.from_numpy(a), ax.from_numpy(b), ax.from_numpy(bias)
    out = ax.empty((M, N))
    gen0 = out.contents.storage.contents.generation
    assert L.ax_compute_gemm(ta, tb, out) == 0
    assert out.contents.storage.contents.generation == gen0 + 1          # dispatch.c:347-350
    assert close(ax.to_numpy(out), ref)
    tbt = ax.from_numpy(np.ascontiguousarray(b.T))
    assert L.ax_compute_gemm_nt(ta, tbt, out) == 0 and close(ax.to_numpy(out), ref)
    tat = ax.from_numpy(np.ascontiguousarray(a.T))
    assert L.ax_compute_gemm_tn(tat, tb, out) == 0 and close(ax.to_numpy(out), ref)
    assert L.ax_compute_gemm_relu(ta, tb, tbias, out) == 0
    assert close(ax.to_numpy(out), oracle.dense(a, b, bias, 1))
    assert L.ax_compute_gemm_relu(ta, tb, None, out) == 0
    assert close(ax.to_numpy(out), oracle.dense(a, b, None, 1))
    assert L.ax_compute_gemm_bias_act(ta, tb, tbias, 2, out) == 0
    assert np.abs(ax.to_numpy(out) - oracle.dense(a, b, bias, 2)).max() <= 1e-5 + REL * np.abs(ref).max()
    # gemm_ex: alpha/beta, beta = 1 accumulates (cpu_opt.c:7442-7497)
    c0 = oracle.uniform((M, N), -1, 1)
    tc = ax.from_numpy(c0)
    assert L.ax_compute_gemm_ex(ta, tb, 1.0, 1.0, tc) == 0 and close(ax.to_numpy(tc), ref + c0)
    assert L.ax_compute_gemm_ex(ta, tb, 0.5, 0.0, tc) == 0 and close(ax.to_numpy(tc), 0.5 * ref)
    # bias_add along either axis of [M,N] (cpu_opt.c:7148-7194)
    lin = ax.from_numpy(ref)
    assert L.ax_compute_bias_add(lin, tbias, 1, out) == 0
    assert np.array_equal(ax.to_numpy(out), ref + bias[None, :])
    rb = oracle.normal((M,), 0, 1)
    trb = ax.from_numpy(rb)
    assert L.ax_compute_bias_add(lin, trb, 0, out) == 0
    assert np.array_equal(ax.to_numpy(out), ref + rb[:, None])
    assert L.ax_compute_bias_add(lin, tbias, 0, out) == 3          # [N] bias against axis 0 of [M,N]
    assert L.ax_compute_bias_add(lin, tbias, 2, out) == 5          # AX_ERR_INVALID_AXIS
    assert L.ax_compute_relu(lin, out) == 0 and np.array_equal(ax.to_numpy(out), np.maximum(ref, 0))
    assert L.ax_compute_gelu(lin, out) == 0 and np.abs(ax.to_numpy(out) - oracle.gelu(ref)).max() <= 2e-6 * max(1, np.abs(ref).max())
    assert L.ax_compute_fill(out, 1.5) == 0 and (ax.to_numpy(out) == 1.5).all()
    assert L.ax_compute_copy(lin, out) == 0 and np.array_equal(ax.to_numpy(out), ref)
    # errors follow the reference backend's convention (cuda/ops_gemm.cu:16-23)
    bad = ax.empty((M, N + 1))
    assert L.ax_compute_gemm(ta, tb, bad) == 3
    t3 = ax.empty((2, 3, 4))
    assert L.ax_compute_gemm(t3, tb, out) == 3
    host = ax.from_numpy(a, device=0)
    assert L.ax_compute_gemm(host, tb, out) == 9 and b"hip device" in L.ax_err_last_message()
    ax.free(ta, tb, tbias, out, tbt, tat, tc, lin, trb, bad, t3, host)


def test_dense_backward_through_dispatch(ax, oracle):
    """The call sequence of the reference's matmul_bias_backward (src/core/autograd_ops.c:603-757)
    on device tensors: gemm_nt, gemm_tn, sum(axis 0) + copy for fresh gradients, temp + axpy for
    gradients that already hold a value."""
    L = ax.L
    oracle.seed(31)
    M, K, N = 96, 160, 72
    x, w, dy = oracle.uniform((M, K), -1, 1), oracle.uniform((K, N), -1, 1), oracle.uniform((M, N), -1, 1)
    tx, tw, tdy = ax.from_numpy(x), ax.from_numpy(w), ax.from_numpy(dy)
    dA, dW, db, tmp = ax.empty((M, K)), ax.empty((K, N)), ax.empty((N,)), ax.empty((N,))
    assert L.ax_compute_has_gemm_tn() == 1
    assert L.ax_compute_gemm_nt(tdy, tw, dA) == 0 and close(ax.to_numpy(dA), oracle.gemm_opt_nt(dy, w))
    xt = np.ascontiguousarray(x.T)
    assert L.ax_compute_gemm_tn(tx, tdy, dW) == 0 and close(ax.to_numpy(dW), oracle.gemm_opt(xt, dy))
    assert L.ax_compute_sum(tdy, 0, tmp) == 0 and L.ax_compute_copy(tmp, db) == 0
    want_db = oracle.sum_axis0(dy)
    assert np.abs(ax.to_numpy(db) - want_db).max() <= 1e-5 * np.abs(dy).sum(axis=0).max()
    # second backward pass into the same gradients: += semantics
    assert L.ax_compute_axpy(tmp, 1.0, db) == 0
    assert np.array_equal(ax.to_numpy(db), ax.to_numpy(tmp) * 2)
    g = ax.empty((K, N))
    assert L.ax_compute_gemm_tn(tx, tdy, g) == 0 and L.ax_compute_axpy(g, 1.0, dW) == 0
    assert close(ax.to_numpy(dW), 2 * oracle.gemm_opt(xt, dy))
    # other axes, the full reduction, and the error codes of cuda_sum (cuda/ops_reduce.cu:262-295)
    rows = ax.empty((M,))
    assert L.ax_compute_sum(tdy, 1, rows) == 0
    assert np.abs(ax.to_numpy(rows) - dy.astype(np.float64).sum(axis=1)).max() <= 1e-5 * np.abs(dy).sum(axis=1).max()
    one = ax.empty((1,))
    assert L.ax_compute_sum(tdy, -1, one) == 0
    assert abs(float(ax.to_numpy(one)[0]) - dy.astype(np.float64).sum()) <= 1e-5 * np.abs(dy).sum()
    assert L.ax_compute_sum(tdy, 2, rows) == 5                     # AX_ERR_INVALID_AXIS
    assert L.ax_compute_sum(tdy, 0, rows) == 3                     # wrong output size
    assert L.ax_compute_axpy(tmp, 1.0, rows) == 3                  # numel mismatch
    ax.free(tx, tw, tdy, dA, dW, db, tmp, g, rows, one)


def test_attention_forward_extension_entry(ax, oracle):
    """ax_hip_sdpa_fwd: the sdpa_fwd member of the reference's GPU extension table
    (include/axiom/internal/cuda_extension.h:86-92) on device tensors of the host core."""
    L = ax.L
    oracle.seed(64)
    BH, S, dk = 4, 256, 64
    q, k, v = (oracle.uniform((BH, S, dk), -0.5, 0.5) for _ in range(3))
    tq, tk, tv = ax.from_numpy(q), ax.from_numpy(k), ax.from_numpy(v)
    to, tl = ax.empty((BH, S, dk)), ax.empty((BH, S))
    ptr = lambda t: t.contents.storage.contents.data
    for causal in (False, True):
        assert L.ax_hip_sdpa_fwd(ptr(tq), ptr(tk), ptr(tv), ptr(to), ptr(tl), BH, S, dk, 0.125, causal, None) == 0
        o64, l64 = oracle.sdpa(q, k, v, 0.125, causal, f64=True)
        assert np.abs(ax.to_numpy(to) - o64).max() <= 1e-5
        assert np.abs(ax.to_numpy(tl) - l64).max() <= 1e-5 * max(1.0, np.abs(l64).max())
    assert L.ax_hip_sdpa_fwd(ptr(tq), ptr(tk), ptr(tv), ptr(to), None, BH, S, dk, 0.125, False, ptr(tl)) == 10
    assert b"P_save" in L.ax_err_last_message()
    ax.free(tq, tk, tv, to, tl)


def test_reference_gpu_vs_cpu_template(ax, oracle):
    """tests/test_cuda.c:213-244: 64x128 . 128x32, rand(-0.1,0.1), every element within 1e-3."""
    L = ax.L
    L.ax_set_seed(7)
    sa, _ = ax.shape_arg((64, 128))
    sb, _ = ax.shape_arg((128, 32))
    a, b = L.ax_tensor_rand(sa, 2, -0.1, 0.1), L.ax_tensor_rand(sb, 2, -0.1, 0.1)
    assert a.contents.storage.contents.device == 2
    c = L.ax_matmul(a, b)
    got = ax.to_numpy(c)
    oracle.seed(7)
    an, bn = oracle.uniform((64, 128), -0.1, 0.1), oracle.uniform((128, 32), -0.1, 0.1)
    assert np.array_equal(ax.to_numpy(a), an) and np.array_equal(ax.to_numpy(b), bn)
    assert np.abs(got - oracle.gemm_opt(an, bn)).max() <= 1e-3
    assert close(got, oracle.gemm_opt(an, bn))
    cpu = L.ax_tensor_to_cpu(c)
    assert cpu.contents.storage.contents.device == 0 and np.array_equal(ax.to_numpy(cpu), got)
    ax.free(a, b, c, cpu)


def test_matmul_bias_adds_to_columns(ax, oracle):
    L = ax.L
    oracle.seed(9)
    x, w, bias = oracle.normal((6, 5, 48)), oracle.normal((48, 40), 0, 0.1), oracle.normal((40,), 0, 1)
    tx, tw, tb = ax.from_numpy(x), ax.from_numpy(w), ax.from_numpy(bias)
    y = L.ax_matmul_bias(tx, tw, tb)                       # [B,S,K] input is flattened and viewed back
    assert [y.contents.shape[i] for i in range(y.contents.ndim)] == [6, 5, 40]
    ref = oracle.dense(x.reshape(30, 48), w, bias, 0).reshape(6, 5, 40)
    assert close(ax.to_numpy(y), ref)
    tx2 = ax.from_numpy(x.reshape(30, 48))
    y2 = L.ax_matmul_bias_relu(tx2, tw, tb)
    assert close(ax.to_numpy(y2), np.maximum(ref.reshape(30, 40), 0))
    assert not L.ax_matmul_bias_relu(tx, tw, tb)           # 3-D input: rejected like the reference (ops.c:405)
    g = L.ax_gelu(y2)
    assert np.abs(ax.to_numpy(g) - oracle.gelu(ax.to_numpy(y2))).max() <= 2e-6
    ax.free(tx, tw, tb, y, tx2, y2, g)


@pytest.mark.parametrize("M", [1, 8, 64])
def test_config1_sequential_mlp(ax, oracle, M):
    """Sequential(Dense 784-4096, ReLU, Dense 4096-4096, ReLU, Dense 4096-10) built after
    ax_set_seed: the weights equal the oracle's draw, the output equals the oracle's MLP."""
    L = ax.L
    L.ax_set_seed(1234)
    seq = L.ax_sequential_create()
    for (i, o, relu) in ((784, 4096, True), (4096, 4096, True), (4096, 10, False)):
        assert L.ax_sequential_add(seq, L.ax_dense_create(i, o, True))
        if relu:
            assert L.ax_sequential_add(seq, L.ax_relu_layer_create())
    oracle.seed(1234)
    w1, w2, w3 = oracle.kaiming((784, 4096), 784), oracle.kaiming((4096, 4096), 4096), oracle.kaiming((4096, 10), 4096)
    from axiom_amd.axiom import TP
    params = (TP * 8)()
    assert L.ax_layer_get_params(seq, params, 8) == 6
    assert np.array_equal(ax.to_numpy(params[2]), w2) and params[2].contents.storage.contents.device == 2
    x = oracle.uniform((M, 784), 0, 1)
    tx = ax.from_numpy(x)
    y = L.ax_layer_forward(seq, tx)
    assert y, ax.err()
    ref = oracle.dense(oracle.dense(oracle.dense(x, w1, None, 1), w2, None, 1), w3, None, 0)
    assert close(ax.to_numpy(y), ref)
    ax.free(tx, y)
    L.ax_layer_destroy(seq)


def test_sequential_dense_with_narrow_head(ax, oracle):
    """Sequential fuses Dense [+ act] -> Dense(<= 16) [+ act] on a few rows into one backend call and runs the
    same layers one by one otherwise; both give the oracle's result."""
    L = ax.L
    from axiom_amd.axiom import TP
    assert L.ax_compute_has_gemm_act_head()
    for (M, hidden, head, act1, act2) in ((3, 512, 7, "gelu", "relu"), (16, 300, 16, None, None), (17, 512, 7, "relu", None),
                                          (4, 512, 17, "relu", None)):
        L.ax_set_seed(99)
        seq = L.ax_sequential_create()
        L.ax_sequential_add(seq, L.ax_dense_create(200, hidden, True))
        if act1:
            L.ax_sequential_add(seq, L.ax_gelu_layer_create() if act1 == "gelu" else L.ax_relu_layer_create())
        L.ax_sequential_add(seq, L.ax_dense_create(hidden, head, True))
        if act2:
            L.ax_sequential_add(seq, L.ax_relu_layer_create())
        params = (TP * 4)()
        assert L.ax_layer_get_params(seq, params, 4) == 4
        oracle.seed(M + hidden + head)
        b1, b2 = oracle.normal((hidden,), 0, 0.3), oracle.normal((head,), 0, 0.3)
        assert L.ax_tensor_write(params[1], b1.ctypes.data, b1.nbytes) == 0
        assert L.ax_tensor_write(params[3], b2.ctypes.data, b2.nbytes) == 0
        w1, w2 = ax.to_numpy(params[0]), ax.to_numpy(params[2])
        x = oracle.uniform((M, 200), -1, 1)
        tx = ax.from_numpy(x)
        L.ax_err_clear()
        y = L.ax_layer_forward(seq, tx)
        assert y, ax.err()
        code = {None: 0, "relu": 1, "gelu": 2}
        ref = oracle.dense(oracle.dense(x, w1, b1, code[act1]), w2, b2, code[act2])
        assert close(ax.to_numpy(y), ref), (M, hidden, head)
        assert ax.err()[0] == 0                                # a fall-back to the layer-by-layer path is not an error
        ax.free(tx, y)
        L.ax_layer_destroy(seq)
    # the operation itself: refused shapes report AX_ERR_NOT_IMPLEMENTED, bad shapes a shape error
    oracle.seed(5)
    a, w1, w2 = oracle.uniform((2, 64), -1, 1), oracle.uniform((64, 128), -1, 1), oracle.uniform((128, 5), -1, 1)
    ta, tw1, tw2 = ax.from_numpy(a), ax.from_numpy(w1), ax.from_numpy(w2)
    y = L.ax_matmul_bias_act_head(ta, tw1, None, 1, tw2, None, 0)
    assert y and close(ax.to_numpy(y), oracle.dense(oracle.dense(a, w1, None, 1), w2, None, 0))
    big = ax.from_numpy(oracle.uniform((40, 64), -1, 1))
    assert not L.ax_matmul_bias_act_head(big, tw1, None, 1, tw2, None, 0) and ax.err()[0] == 10
    assert not L.ax_matmul_bias_act_head(ta, tw2, None, 1, tw1, None, 0) and ax.err()[0] == 3
    ax.free(ta, tw1, tw2, y, big)


def test_config3_ffn_through_layers(ax, oracle):
    L = ax.L
    L.ax_set_seed(3)
    seq = L.ax_sequential_create()
    d1, d2 = L.ax_dense_create(1024, 4096, True), L.ax_dense_create(4096, 1024, True)
    for layer in (d1, L.ax_gelu_layer_create(), d2):
        L.ax_sequential_add(seq, layer)
    from axiom_amd.axiom import TP
    params = (TP * 4)()
    L.ax_layer_get_params(seq, params, 4)
    oracle.seed(33)
    w1, b1 = oracle.normal((1024, 4096), 0, 0.02), oracle.normal((4096,), 0, 0.02)
    w2, b2 = oracle.normal((4096, 1024), 0, 0.02), oracle.normal((1024,), 0, 0.02)
    hooks = L.ax_backend_for_device(2)
    assert hooks
    for t, v in zip(params, (w1, b1, w2, b2)):            # overwrite the parameters in place
        src = ax.from_numpy(v)
        assert L.ax_compute_copy(src, t) == 0
        ax.free(src)
    x = oracle.normal((4, 512, 1024))
    tx = ax.from_numpy(x)
    y = L.ax_layer_forward(seq, tx)
    assert [y.contents.shape[i] for i in range(3)] == [4, 512, 1024]
    h = oracle.dense(x.reshape(2048, 1024), w1, b1, 2)
    ref = oracle.dense(h, w2, b2, 0).reshape(4, 512, 1024)
    assert close(ax.to_numpy(y), ref)
    ax.free(tx, y)
    L.ax_layer_destroy(seq)


def test_quantized_entry_points(ax, oracle):
    L = ax.L
    oracle.seed(13)
    M, N, K = 8, 768, 768
    w, a = oracle.uniform((N, K), -1, 1), oracle.uniform((M, K), -1, 1)
    qw = L.ax_qweight_create_from_fp32(w, N, K)
    q, s = oracle.quantize_rows(w)
    ref = oracle.qgemm_w8a32(a, q, s)
    out = np.zeros((M, N), np.float32)
    assert L.ax_qgemm_w8a32(a, qw, out, M) == 0           # reference signature: host pointers
    assert close(out, ref)
    dq = L.ax_qweight_to_device(qw, 2)
    ta, tout = ax.from_numpy(a), ax.empty((M, N))
    assert L.ax_qgemm_w8a32_dev(ta.contents.storage.contents.data, dq, tout.contents.storage.contents.data, M) == 0
    assert close(ax.to_numpy(tout), ref)
    # W8A8 on device-resident operands
    from axiom_amd import AxHip
    hip = AxHip()
    x8 = oracle.int8((M, K))
    bias = oracle.normal((N,), 0, 0.02)
    dx, db = hip.array(x8), hip.array(bias)
    dout, dacc = hip.empty((M, N)), hip.empty((M, N), np.int32)
    assert L.ax_qgemm_w8a8_dev(dx.ptr, 0.02, dq, db.ptr, 1, dout.ptr, dacc.ptr, M) == 0
    acc = oracle.qgemm_w8a8_acc(x8, q)
    assert np.array_equal(dacc.numpy(), acc)
    assert np.array_equal(dout.numpy(), oracle.w8a8_epilogue(acc, np.float32(0.02), s, bias, 1))
    assert L.ax_qgemm_w8a8_dev(None, 0.02, dq, None, 0, dout.ptr, None, M) == 1
    L.ax_qweight_device_destroy(dq, 2)
    L.ax_qweight_destroy(qw)
    ax.free(ta, tout)


def test_backend_dropped_into_the_unmodified_reference(oracle):
    """Load the reference library itself, register ax_hip_ops through the reference's own
    ax_compute_register_backend (src/compute/dispatch.c:302-315) in its GPU slot, and run the
    reference's tensors, ops and Sequential on the MI355X."""
    import subprocess
    import sys
    ref_so = os.path.join(ROOT, "oracle", "_ref", "libaxref.so")
    if not os.path.exists(ref_so):
        pytest.skip("oracle/_ref/libaxref.so was not built (needs the reference tree)")
    # a fresh process: the reference's ax_* symbols must be the first ones in scope
    r = subprocess.run([sys.executable, "-u", os.path.join(ROOT, "tests", "dropin_check.py")],
                       capture_output=True, text=True, timeout=170)
    say(r.stdout[-3000:], r.stderr[-3000:])
    assert r.returncode == 0
    assert "DROPIN OK" in r.stdout


def test_elementwise_reduction_optimizer_slots(ax, oracle, golden):
    """The remaining vtable slots through the ax_compute_* wrappers on device tensors, against the
    reference vectors (inputs regenerated from their seeds) and the CPU restatement."""
    import slot_cases as sc
    L = ax.L
    # broadcasting binaries: bit-exact
    for case in range(len(sc.BCAST)):
        a, b = sc.binary_inputs(oracle, case)
        ta, tb = ax.from_numpy(a), ax.from_numpy(b)
        out = ax.empty(np.broadcast_shapes(a.shape, b.shape))
        for name in sc.BINARY:
            assert getattr(L, "ax_compute_" + name)(ta, tb, out) == 0, ax.err()
            assert np.array_equal(ax.to_numpy(out), golden[f"bin_{name}_{case}"], equal_nan=True), (name, case)
        if a.shape == b.shape:
            assert L.ax_compute_add_relu(ta, tb, out) == 0
            assert np.array_equal(ax.to_numpy(out), golden[f"bin_add_relu_{case}"])
        ax.free(ta, tb, out)
    # a strided operand: the transpose view [K, M] of an [M, K] tensor, added to a contiguous [K, M]
    oracle.seed(77)
    m = oracle.uniform((6, 10), -1, 1)
    tm, tn = ax.from_numpy(m), ax.from_numpy(np.ascontiguousarray(m.T) * 2)
    view = ax.from_numpy(m)
    v = view.contents
    v.shape[0], v.shape[1], v.strides[0], v.strides[1] = 10, 6, 1, 10
    out = ax.empty((10, 6))
    assert L.ax_compute_add(view, tn, out) == 0 and np.array_equal(ax.to_numpy(out), m.T + 2 * m.T)
    bad = ax.empty((7, 6))
    assert L.ax_compute_add(tm, tn, bad) == 3                      # [6,10] does not broadcast to [7,6]
    v.shape[0], v.shape[1], v.strides[0], v.strides[1] = 6, 10, 10, 1
    # a GEMM operand whose rows overlap (row stride below the row length, e.g. an expanded row) is refused,
    # not read as a dense matrix
    ga, gb, gout = ax.from_numpy(m), ax.from_numpy(oracle.uniform((10, 4), -1, 1)), ax.empty((6, 4))
    assert L.ax_compute_gemm(ga, gb, gout) == 0
    ga.contents.strides[0] = 0
    assert L.ax_compute_gemm(ga, gb, gout) == 3 and "overlap" in ax.err()[1]
    ga.contents.strides[0] = 5
    assert L.ax_compute_gemm(ga, gb, gout) == 3
    ga.contents.strides[0] = 10
    ax.free(tm, tn, view, out, bad, ga, gb, gout)
    # unary / scalar / activation slots
    x = sc.unary_input(oracle)
    tx, out = ax.from_numpy(x), ax.empty(x.shape)
    calls = {"neg": (L.ax_compute_neg,), "abs": (L.ax_compute_abs,), "exp": (L.ax_compute_exp,),
             "log": (L.ax_compute_log,), "sqrt": (L.ax_compute_sqrt,), "square": (L.ax_compute_square,),
             "sigmoid": (L.ax_compute_sigmoid,), "tanh": (L.ax_compute_tanh,), "swish": (L.ax_compute_swish,),
             "leaky_relu": (L.ax_compute_leaky_relu, 0.1), "elu": (L.ax_compute_elu, 0.7),
             "add_scalar": (L.ax_compute_add_scalar, 0.37), "mul_scalar": (L.ax_compute_mul_scalar, -1.7)}
    for name, call in calls.items():
        st = call[0](tx, out) if len(call) == 1 else call[0](tx, call[1], out)
        assert st == 0, (name, ax.err())
        ref = golden[f"un_{name}"]
        assert (np.abs(ax.to_numpy(out) - ref) <= 1e-6 * np.maximum(np.abs(ref), 1)).all(), name
    assert ax.to_numpy(out).shape == x.shape
    ax.free(tx, out)
    # reductions (int64 argmax through a tensor of that dtype)
    for shp, arr in zip(sc.REDUCE_SHAPES, sc.reduce_inputs(oracle)):
        tag = "x".join(map(str, shp))
        t = ax.from_numpy(arr)
        for axis in range(-1, len(shp)):
            oshape = (1,) if axis == -1 else shp[:axis] + shp[axis + 1:]
            out = ax.empty(oshape)
            for name in ("mean", "max", "min"):
                assert getattr(L, "ax_compute_" + name)(t, axis, out) == 0, ax.err()
                assert np.abs(ax.to_numpy(out) - golden[f"red_{name}_{tag}_axis{axis}_naive"]).max() < 2e-6
            sh, nd = ax.shape_arg(oshape)
            L.ax_set_default_device(2)
            idx = L.ax_tensor_create(sh, nd, 3)                    # AX_INT64
            assert L.ax_compute_argmax(t, axis, idx) == 0, ax.err()
            got = np.empty(oshape, np.int64)
            assert L.ax_tensor_read(idx, got.ctypes.data, got.nbytes) == 0
            assert np.array_equal(got, golden[f"red_argmax_{tag}_axis{axis}"])
            assert L.ax_compute_argmax(t, axis, out) == 4          # AX_ERR_DTYPE_MISMATCH: float output
            ax.free(out, idx)
        assert L.ax_compute_max(t, len(shp), t) == 5               # AX_ERR_INVALID_AXIS
        ax.free(t)
    # softmax_rowwise and its shape rule
    for (rows, cols), arr in zip(sc.SOFTMAX_SHAPES, sc.softmax_inputs(oracle)):
        t, out = ax.from_numpy(arr), ax.empty((rows, cols))
        assert L.ax_compute_softmax_rowwise(t, out) == 0
        assert np.abs(ax.to_numpy(out) - golden[f"softmax_{rows}x{cols}_naive"]).max() < 1e-6
        ax.free(t, out)
    t3, o3 = ax.from_numpy(np.zeros((2, 3, 4), np.float32)), ax.empty((2, 3, 4))
    assert L.ax_compute_softmax_rowwise(t3, o3) == 3
    ax.free(t3, o3)
    # the LayerNorm layer: gamma ones / beta zeros at creation, then the reference's vectors
    for shp, (xv, gamma, beta) in zip(sc.LAYERNORM_SHAPES, sc.layernorm_inputs(oracle)):
        ln = L.ax_layernorm_create(shp[-1], 1e-5)
        from axiom_amd.axiom import TP
        params = (TP * 4)()
        assert L.ax_layer_get_params(ln, params, 4) == 2
        assert np.array_equal(ax.to_numpy(params[0]), np.ones(shp[-1], np.float32))
        assert np.array_equal(ax.to_numpy(params[1]), np.zeros(shp[-1], np.float32))
        for prm, val in zip(params, (gamma, beta)):
            tv_ = ax.from_numpy(val)
            assert L.ax_compute_copy(tv_, prm) == 0
            ax.free(tv_)
        t = ax.from_numpy(xv)
        y = L.ax_layer_forward(ln, t)
        assert y, ax.err()
        assert np.abs(ax.to_numpy(y) - golden["layernorm_" + "x".join(map(str, shp))]).max() < 5e-6
        ax.free(t, y)
        L.ax_layer_destroy(ln)
    # optimizer slots over three steps
    assert L.ax_compute_has_adam_update() == 1 and L.ax_compute_has_sgd_update() == 1
    w0, grads = sc.optimizer_inputs(oracle)
    for key, (kind, kw) in sc.OPTIMIZERS.items():
        tw, tm_, tv = ax.from_numpy(w0), ax.from_numpy(np.zeros_like(w0)), ax.from_numpy(np.zeros_like(w0))
        for step, g in enumerate(grads, 1):
            tg = ax.from_numpy(g)
            if kind == "sgd":
                st = L.ax_compute_sgd_update(tw, tg, tm_ if kw["momentum"] > 0 else None, kw["lr"], kw["momentum"],
                                             kw["wd"], kw["nesterov"])
            else:
                bc1, bc2 = sc.bias_corrections(kw["beta1"], kw["beta2"], step)
                st = L.ax_compute_adam_update(tw, tg, tm_, tv, kw["lr"], kw["beta1"], kw["beta2"], kw["eps"], kw["wd"],
                                              bc1, bc2, kind == "adamw")
            assert st == 0, ax.err()
            assert np.abs(ax.to_numpy(tw) - golden[key][step - 1]).max() < 2e-6, (key, step)
            ax.free(tg)
        ax.free(tw, tm_, tv)


@pytest.mark.parametrize("tag,in_shape,seed", [("mlp", (5, 12), 8100), ("ffn", (2, 7, 64), 8200), ("acts", (4, 9), 8300),
                                               ("encoder", (2, 24, 64), 8600), ("mha_causal", (2, 128, 128), 8700)])
def test_reference_model_file_runs_on_device(ax, oracle, golden, tag, in_shape, seed, tmp_path):
    """A model the reference built, initialised and saved (tests/golden/ref_*.axm) is loaded onto
    the GPU, reproduces the reference's CPU forward of the same input, and is written back from
    device memory byte for byte."""
    L = ax.L
    path = os.path.join(ROOT, "tests", "golden", f"ref_{tag}.axm")
    L.ax_set_default_device(2)
    model = L.ax_model_load(path.encode())
    assert model, ax.err()
    from axiom_amd.axiom import TP
    params = (TP * 64)()
    net = C.cast(model, C.POINTER(C.c_void_p))[0]
    n = L.ax_layer_get_params(net, params, 64)
    assert n > 0 and all(params[i].contents.storage.contents.device == 2 for i in range(n))
    # the input the generator drew: parameters' perturbations first, then x, from seed + 1
    oracle.seed(seed + 1)
    for i in range(n):
        t = params[i].contents
        if t.ndim == 1:
            oracle.uniform((t.shape[0],), -0.5, 0.5)
    x = oracle.uniform(in_shape, -1.0, 1.0)
    tx = ax.from_numpy(x)
    y = L.ax_model_predict(model, tx)
    assert y, ax.err()
    want = golden[f"axm_{tag}_out"]
    got = ax.to_numpy(y)
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max()), np.abs(got - want).max()
    out = tmp_path / "from_device.axm"
    assert L.ax_model_save(model, str(out).encode()) == 0, ax.err()
    assert out.read_bytes() == open(path, "rb").read()
    ax.free(tx, y)
    L.ax_model_destroy(model)


@pytest.mark.parametrize("B,S,D,H,bias,causal", [(2, 128, 128, 2, True, True), (1, 256, 256, 4, False, False),
                                                 (3, 40, 96, 6, True, False), (2, 77, 64, 2, True, True),
                                                 (2, 50, 90, 6, True, False), (2, 130, 288, 3, False, True)])
def test_attention_layer_forward(ax, oracle, B, S, D, H, bias, causal):
    """ax_mha_create + forward on the device against the layer restated from the oracle's pieces
    (pinned to the reference's own layer output in test_oracle.py)."""
    import attn_cases as ac
    from axiom_amd.axiom import TP
    L = ax.L
    L.ax_set_default_device(2)
    L.ax_set_seed(1234)
    layer = L.ax_mha_create(D, H, bias, causal)
    assert layer, ax.err()
    params = (TP * 8)()
    n = L.ax_layer_get_params(layer, params, 8)
    assert n == (8 if bias else 4)
    oracle.seed(B + S + D)
    w = [ax.to_numpy(params[i]) for i in range(4)]
    limit = np.sqrt(np.float32(6.0) / np.float32(2 * D))
    assert all(np.abs(m).max() <= limit and m.std() > 0.4 * limit for m in w)       # Xavier-uniform
    if bias:
        for i in range(4, 8):
            b = oracle.uniform((D,), -0.5, 0.5)
            tb = ax.from_numpy(b)
            assert L.ax_compute_copy(tb, params[i]) == 0
            ax.free(tb)
            w.append(b)
    x = oracle.uniform((B, S, D), -1, 1)
    tx = ax.from_numpy(x)
    y = L.ax_layer_forward(layer, tx)
    assert y, ax.err()
    want = ac.mha_forward(oracle, x, w, H, causal)
    got = ax.to_numpy(y)
    assert got.shape == (B, S, D)
    assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max()), np.abs(got - want).max()
    # a second call reuses the fused projection cache; a changed weight invalidates it
    y2 = L.ax_layer_forward(layer, tx)
    assert np.array_equal(ax.to_numpy(y2), got)
    w[0] = w[0] * 0.5
    tw = ax.from_numpy(w[0])
    assert L.ax_compute_copy(tw, params[0]) == 0
    y3 = L.ax_layer_forward(layer, tx)
    want3 = ac.mha_forward(oracle, x, w, H, causal)
    assert np.abs(ax.to_numpy(y3) - want3).max() <= 2e-5 * max(1.0, np.abs(want3).max())
    bad = ax.from_numpy(np.zeros((2, D), np.float32))
    assert not L.ax_layer_forward(layer, bad)
    ax.free(tx, y, y2, y3, tw, bad)
    L.ax_layer_destroy(layer)


@pytest.mark.gpu
def test_no_device_memory_is_left_behind(ax):
    """Build, run and destroy an encoder-shaped model (layer norm, attention with bias on both of its
    forward routes, dense + GELU) and a quantized weight: every device block the host core asked for comes
    back, counted by the allocator itself."""
    import ctypes as C
    from axiom_amd import AxHip
    hip = AxHip()
    L = ax.L
    L.ax_set_default_device(2)
    st = [C.c_int64() for _ in range(6)]

    def stats():
        hip.L.axhip_alloc_stats(*[C.byref(v) for v in st])
        return [v.value for v in st]

    hip.L.axhip_reset_alloc_stats()
    for (D, H) in ((128, 2), (90, 6)):                           # dk 64: direct route; dk 15: split route
        seq = L.ax_sequential_create()
        for layer in (L.ax_layernorm_create(D, 1e-5), L.ax_mha_create(D, H, True, True), L.ax_layernorm_create(D, 1e-5),
                      L.ax_dense_create(D, 4 * D, True), L.ax_gelu_layer_create(), L.ax_dense_create(4 * D, D, True),
                      L.ax_softmax_layer_create(-1)):
            assert L.ax_sequential_add(seq, layer)
        model = L.ax_model_create(seq)
        x = ax.from_numpy(np.random.default_rng(D).uniform(-1, 1, (3, 70, D)).astype(np.float32))
        for _ in range(3):
            y = L.ax_model_predict(model, x)
            assert y, ax.err()
            assert np.isfinite(ax.to_numpy(y)).all()
            ax.free(y)
        bad = ax.from_numpy(np.zeros((3, 70, D + 4), np.float32))   # a refused input must not strand temporaries
        assert not L.ax_model_predict(model, bad)
        ax.free(x, bad)
        L.ax_model_destroy(model)
    allocs, frees, b_alloc, b_free, _, _ = stats()
    assert allocs > 50 and allocs == frees and b_alloc == b_free, (allocs, frees, b_alloc, b_free)

