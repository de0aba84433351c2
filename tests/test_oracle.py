"""Pins the CPU oracle: golden vectors from the reference, the compiled reference itself
(when built), and what the mathematics fixes.  No GPU."""
import numpy as np
import pytest

from fills import property_case, xorshift32_unit


# ---------------------------------------------------------------- RNG
@pytest.mark.parametrize("seed", [0, 42])
def test_rng_matches_reference_vectors(oracle, golden, seed):
    L = oracle.L
    oracle.seed(seed)
    assert [L.axo_rng_uint64() for _ in range(8)] == list(golden[f"rng_u64_seed{seed}"])
    oracle.seed(seed)
    got = np.array([L.axo_rng_uniform(-1.0, 1.0) for _ in range(8)], np.float32)
    assert np.array_equal(got, golden[f"rng_uniform_seed{seed}"])
    oracle.seed(seed)
    got = np.array([L.axo_rng_normal() for _ in range(8)], np.float32)
    assert np.array_equal(got, golden[f"rng_normal_seed{seed}"])
    oracle.seed(seed)
    assert [L.axo_rng_bounded(255) for _ in range(32)] == list(golden[f"rng_bounded255_seed{seed}"])


def test_rng_published_known_answers(oracle):
    # xoshiro256** seeded by splitmix64(0): first outputs are a published test vector
    oracle.seed(0)
    assert oracle.L.axo_rng_uint64() == 0x99EC5F36CB75F2B4
    assert oracle.L.axo_rng_uint64() == 0xBF6E1F784956452A


def test_rng_statistics(oracle):
    oracle.seed(123)
    u = oracle.uniform((200000,), -1.0, 1.0)
    assert u.min() >= -1.0 and u.max() < 1.0 and abs(u.mean()) < 0.01
    n = oracle.normal((200000,), 0.0, 0.02)
    assert abs(n.mean()) < 2e-4 and abs(n.std() - 0.02) < 2e-4
    q = oracle.int8((100000,))
    assert q.min() == -127 and q.max() == 127


# ---------------------------------------------------------------- quantizer
def test_quantizer_hand_vectors(oracle, golden):
    q, s = oracle.quantize_rows(golden["quant_hand_w"])
    assert np.array_equal(q, golden["quant_hand_q"]) and np.array_equal(s, golden["quant_hand_s"])
    assert q[0].tolist() == [64, -127, 32, 13] and s[1] == 1.0 and not q[1].any()
    q, s = oracle.quantize_rows(golden["quant_ties_w"])
    assert np.array_equal(q, golden["quant_ties_q"]) and np.array_equal(s, golden["quant_ties_s"])
    assert q[0, :4].tolist() == [127, 0, 2, 2]          # round-half-to-even


@pytest.mark.parametrize("N,K", [(8, 8), (128, 128), (64, 1024)])
def test_quantizer_reference_shapes(oracle, golden, N, K):
    w = xorshift32_unit(N * K, 42).reshape(N, K)
    q, s = oracle.quantize_rows(w)
    assert np.array_equal(q, golden[f"quant_{N}x{K}_q"])
    assert np.array_equal(s, golden[f"quant_{N}x{K}_s"])
    # the reference's own invariant (tests/test_quantize.c:47-57)
    assert (np.abs(w - oracle.dequantize_rows(q, s)) <= 1.5 * s[:, None]).all()


# ---------------------------------------------------------------- W8A32
@pytest.mark.parametrize("M,N,K", [(1, 8, 8), (4, 16, 32), (8, 64, 128), (32, 128, 512),
                                   (16, 256, 1024), (3, 17, 45)])
def test_w8a32_matches_reference_output(oracle, golden, M, N, K):
    a = xorshift32_unit(M * K, 7).reshape(M, K)
    w = xorshift32_unit(N * K, 13).reshape(N, K)
    q, s = oracle.quantize_rows(w)
    out = oracle.qgemm_w8a32(a, q, s)
    assert np.array_equal(out, golden[f"w8a32_{M}x{N}x{K}_out"])
    # and the closed form the reference's test uses (tests/test_quantize.c:94-111)
    want = a.astype(np.float64) @ oracle.dequantize_rows(q, s).astype(np.float64).T
    diff = np.abs(out - want)
    assert not ((diff > 1e-2) & (diff / np.maximum(np.abs(want), 1e-30) > 1e-3)).any()


# ---------------------------------------------------------------- int8 accumulators
@pytest.mark.parametrize("K", [8, 32, 128, 512, 1024])
def test_int8_acc_equals_reference_w8a32_with_unit_scales(oracle, golden, K):
    oracle.seed(1000 + K)
    x = oracle.int8((4, K))
    w = oracle.int8((64, K))
    assert x.astype(np.int64).sum() == golden[f"acc_K{K}_x_sum"][0]
    assert w.astype(np.int64).sum() == golden[f"acc_K{K}_w_sum"][0]
    acc = oracle.qgemm_w8a8_acc(x, w)
    assert np.array_equal(acc.astype(np.float64), golden[f"acc_K{K}"].astype(np.float64))


def test_int8_acc_brute_force_and_extremes(oracle, golden):
    oracle.seed(5)
    x, w = oracle.int8((5, 37)), oracle.int8((7, 37))
    brute = [[sum(int(x[m, k]) * int(w[n, k]) for k in range(37)) for n in range(7)] for m in range(5)]
    assert oracle.qgemm_w8a8_acc(x, w).tolist() == brute
    xs, ws = np.full((2, 1024), 127, np.int8), np.full((3, 1024), -127, np.int8)
    acc = oracle.qgemm_w8a8_acc(xs, ws)
    assert (acc == -127 * 127 * 1024).all()
    assert np.array_equal(acc.astype(np.float64), golden["acc_extreme"].astype(np.float64))
    big = oracle.qgemm_w8a8_acc(np.full((1, 8192), -127, np.int8), np.full((1, 8192), -127, np.int8))
    assert big[0, 0] == 127 * 127 * 8192                 # largest magnitude at K = 8192


def test_w8a8_epilogue_against_fp64(oracle):
    oracle.seed(9)
    x, w = oracle.int8((6, 300)), oracle.int8((10, 300))
    ws = oracle.uniform((10,), 1e-3, 1e-2)
    bias = oracle.normal((10,), 0.0, 0.02)
    acc = oracle.qgemm_w8a8_acc(x, w)
    xs = np.float32(0.0123)
    for act in (0, 1, 2):
        got = oracle.w8a8_epilogue(acc, xs, ws, bias, act)
        v = acc.astype(np.float64) * (np.float64(xs) * ws.astype(np.float64)) + bias
        if act == 1:
            v = np.maximum(v, 0)
        if act == 2:
            v = 0.5 * v * (1 + np.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3)))
        assert np.abs(got - v).max() <= 1e-6 * max(1.0, np.abs(v).max())
    nob = oracle.w8a8_epilogue(acc, xs, ws, None, 0)
    assert np.array_equal(nob, acc.astype(np.float32) * (xs * ws)[None, :])


# ---------------------------------------------------------------- fp32 GEMM
def test_gemm_known_answers(oracle, golden):
    a = np.arange(1, 7, dtype=np.float32).reshape(2, 3)
    b = np.arange(7, 13, dtype=np.float32).reshape(3, 2)
    for fn in (oracle.gemm_opt, oracle.gemm_naive, oracle.gemm_f64):
        assert fn(a, b).reshape(-1).tolist() == [58, 64, 139, 154]
    assert golden["gemm_2x3x2"].reshape(-1).tolist() == [58, 64, 139, 154]
    c = oracle.gemm_opt(np.array([[1, 2], [3, 4]], np.float32), np.array([[5, 6], [7, 8]], np.float32))
    assert c.reshape(-1).tolist() == [19, 22, 43, 50] == golden["gemm_2x2x2"].reshape(-1).tolist()
    oracle.seed(3)
    a = oracle.uniform((40, 40), -1, 1)
    assert np.array_equal(oracle.gemm_opt(a, np.eye(40, dtype=np.float32)), a)
    assert not oracle.gemm_opt(np.zeros((9, 300), np.float32), oracle.uniform((300, 500), -1, 1)).any()
    # K = 1 outer product
    u, v = oracle.uniform((33, 1), -1, 1), oracle.uniform((1, 65), -1, 1)
    assert np.array_equal(oracle.gemm_opt(u, v), u * v)


@pytest.mark.parametrize("M,K,N", [(37, 73, 19), (64, 128, 32), (32, 2048, 16), (1, 784, 64), (7, 300, 130)])
def test_gemm_matches_reference_outputs(oracle, golden, M, K, N):
    oracle.seed(M * 1000 + N)
    a = oracle.uniform((M, K), -1, 1)
    b = oracle.uniform((K, N), -1, 1)
    assert np.array_equal(oracle.gemm_naive(a, b), golden[f"gemm_{M}x{K}x{N}_naive"])
    ref = golden[f"gemm_{M}x{K}x{N}_opt"]
    got = oracle.gemm_opt(a, b)
    assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max()
    if oracle.small_route(M, N, K):
        assert np.array_equal(got, ref)                  # order fully specified on this route
    nt = oracle.gemm_opt_nt(a, np.ascontiguousarray(b.T))
    assert np.abs(nt - golden[f"gemm_nt_{M}x{K}x{N}_opt"]).max() <= 1e-4 * np.abs(ref).max()
    c64, cabs = oracle.gemm_f64(a, b), oracle.gemm_abs_f64(a, b)
    assert (np.abs(got - c64) <= 1e-5 * cabs + 1e-30).all()
    assert np.allclose(c64, a.astype(np.float64) @ b.astype(np.float64), rtol=1e-12, atol=1e-12)


def test_gemm_1024_cube_against_reference_checksums(oracle, golden):
    oracle.seed(0)
    a = oracle.uniform((1024, 1024), -1, 1)
    b = oracle.uniform((1024, 1024), -1, 1)
    c = oracle.gemm_opt(a, b)
    probe = golden["gemm_1024_probe"]
    assert a[0, 0] == probe[0] and b[0, 0] == probe[1]
    assert np.abs(c[0] - golden["gemm_1024_row0"]).max() <= 1e-4 * 60
    assert np.abs(np.diagonal(c) - golden["gemm_1024_diag"]).max() <= 1e-4 * 60
    s, sabs = golden["gemm_1024_sums"]
    assert abs(c.astype(np.float64).sum() - s) <= 1e-6 * sabs
    assert abs(np.abs(c).astype(np.float64).sum() - sabs) <= 1e-6 * sabs


def test_gemm_property_cases(oracle, golden):
    shapes, sums = golden["prop_shapes"], golden["prop_sums"]
    for i in range(60):
        M, N, K, a, b = property_case(i)
        assert (M, N, K) == tuple(shapes[i])
        cn, co = oracle.gemm_naive(a, b), oracle.gemm_opt(a, b)
        # the reference's own gate (tests/test_property.c:198): atol 1e-3 + rtol 1e-4
        assert (np.abs(cn - co) <= 1e-3 + 1e-4 * np.abs(cn)).all()
        assert abs(cn.astype(np.float64).sum() - sums[i, 0]) <= 1e-9 * max(1.0, sums[i, 2])
        assert abs(co.astype(np.float64).sum() - sums[i, 1]) <= 1e-5 * max(1.0, sums[i, 2])


def test_route_predicate(oracle):
    # src/compute/backends/cpu_opt.c:3509 with MR = 6
    assert oracle.small_route(1, 4096, 784)              # 3.2 M, m < 6
    assert not oracle.small_route(1, 4096, 4096)         # 16.8 M
    assert oracle.small_route(1, 10, 4096)
    assert oracle.small_route(46, 46, 47) and not oracle.small_route(47, 47, 47)
    assert not oracle.small_route(6, 100, 1000) and oracle.small_route(5, 100, 1000)


def test_bias_relu_and_gelu(oracle, golden):
    oracle.seed(77)
    a, b = oracle.uniform((33, 100), -1, 1), oracle.uniform((100, 40), -1, 1)
    bias = oracle.uniform((40,), -0.5, 0.5)
    assert np.array_equal(oracle.dense(a, b, bias, 1), golden["gemm_relu_33x100x40"])
    assert np.array_equal(oracle.dense(a, b, None, 1), golden["gemm_relu_33x100x40_nobias"])
    lin = oracle.dense(a, b, bias, 0)
    assert np.array_equal(lin, oracle.gemm_opt(a, b) + bias[None, :])
    x = golden["gelu_x"]
    y = oracle.gelu(x)
    assert np.abs(y - golden["gelu_y"]).max() <= 2e-6
    y64 = np.array([oracle.L.axo_gelu_f64(float(v)) for v in x])
    assert np.abs(y - y64).max() <= 1e-6
    assert oracle.L.axo_gelu_tanh(0.0) == 0.0 and abs(oracle.L.axo_gelu_tanh(10.0) - 10.0) < 1e-6


# ---------------------------------------------------------------- dense backward blocks
def test_dense_backward_blocks_match_reference_vectors(oracle, golden):
    """dA = dY W^T, dW = X^T dY, dBias = sum(dY, 0), axpy: the restatement against what the
    reference produced for the same seeded inputs (both of its CPU backends where they exist)."""
    oracle.seed(4242)
    M, K, N = 48, 40, 24
    x, w, dy = oracle.uniform((M, K), -1, 1), oracle.uniform((K, N), -1, 1), oracle.uniform((M, N), -1, 1)
    dA = oracle.gemm_opt_nt(dy, w)
    assert np.abs(dA - golden["dense_bwd_dA"]).max() <= 1e-5 * np.abs(golden["dense_bwd_dA"]).max()
    dW = oracle.gemm_opt(np.ascontiguousarray(x.T), dy)
    assert np.abs(dW - golden["dense_bwd_dW"]).max() <= 1e-5 * np.abs(golden["dense_bwd_dW"]).max()
    db = oracle.sum_axis0(dy)
    assert np.array_equal(db, golden["dense_bwd_db"]) and np.array_equal(db, golden["dense_bwd_db_naive"])
    oracle.seed(4343)
    s2, s3 = oracle.uniform((37, 19), -1, 1), oracle.uniform((4, 9, 10), -1, 1)
    for name, arr in (("sum2d", s2), ("sum3d", s3)):
        assert np.array_equal(oracle.sum_axis0(arr), golden[f"{name}_axis0"])        # bit-exact order
        for axis in range(arr.ndim):
            s64, sabs = oracle.sum_axis_f64(arr, axis)
            for tag in ("", "_naive"):
                ref = golden[f"{name}_axis{axis}{tag}"]
                assert (np.abs(ref - s64) <= 1e-6 * sabs + 1e-30).all()
        full = np.float64(arr.astype(np.float64).sum())
        assert abs(golden[f"{name}_axis-1"][0] - full) <= 1e-6 * np.abs(arr).sum()
    xa, ya = oracle.uniform((1003,), -1, 1), oracle.uniform((1003,), -1, 1)
    got = oracle.axpy(xa, 0.37, ya)
    # vector body is a fused multiply-add (bit-exact); the scalar tail of the SIMD backend and
    # the naive backend may round the product first: allow one rounding of the product
    for tag in ("", "_naive"):
        ref = golden[f"axpy_1003{tag}"]
        assert np.abs(got - ref).max() <= 2e-7
    assert np.array_equal(got[:1000], golden["axpy_1003"][:1000])
    # closed forms
    assert np.array_equal(oracle.sum_axis0(np.ones((1000, 7), np.float32)), np.full(7, 1000, np.float32))
    assert np.array_equal(oracle.axpy(np.ones(5, np.float32), 2.0, np.arange(5, dtype=np.float32)),
                          np.arange(5, dtype=np.float32) + 2)


# ---------------------------------------------------------------- attention forward
SDPA_GOLDEN = [(6, 24, 16, 0), (2, 16, 8, 1), (3, 128, 64, 0), (3, 128, 64, 1), (2, 40, 32, 1)]


def sdpa_inputs(oracle, BH, S, dk, causal):
    oracle.seed(5000 + BH * 100 + S + dk + causal)
    return tuple(oracle.uniform((BH, S, dk), -0.5, 0.5) for _ in range(3))


@pytest.mark.parametrize("BH,S,dk,causal", SDPA_GOLDEN)
def test_sdpa_restatement_against_reference_vectors(oracle, golden, BH, S, dk, causal):
    """The textbook evaluation (the yardstick of tests/test_attention.c) against what the
    reference's fused CPU kernel produced, at the reference test's gate of 1e-4, and against
    the fp64 ground truth; plus what the mathematics fixes."""
    q, k, v = sdpa_inputs(oracle, BH, S, dk, causal)
    scale = float(np.float32(1.0) / np.sqrt(np.float32(dk)))
    o, l = oracle.sdpa(q, k, v, scale, causal)
    o64, l64 = oracle.sdpa(q, k, v, scale, causal, f64=True)
    ref_o, ref_l = golden[f"sdpa_{BH}x{S}x{dk}_c{causal}_O"], golden[f"sdpa_{BH}x{S}x{dk}_c{causal}_L"]
    assert np.abs(o - ref_o).max() < 1e-4 and np.abs(l - ref_l).max() < 1e-4
    assert np.abs(o - o64).max() < 2e-6 and np.abs(ref_o - o64).max() < 1e-5
    assert np.abs(l - l64).max() < 1e-5 and np.abs(ref_l - l64).max() < 1e-4
    # numpy evaluation of the definition
    s = np.einsum("hid,hjd->hij", q.astype(np.float64), k.astype(np.float64)) * scale
    if causal:
        s = np.where(np.tril(np.ones((S, S), bool))[None], s, -np.inf)
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    want = np.einsum("hij,hjd->hid", p / p.sum(axis=-1, keepdims=True), v.astype(np.float64))
    assert np.abs(o64 - want).max() < 1e-12
    assert np.abs(l64 - (s.max(axis=-1) + np.log(p.sum(axis=-1)))).max() < 1e-12


def test_sdpa_closed_forms(oracle):
    # identical keys: uniform attention, O = mean of V, L = score + log S
    BH, S, dk = 2, 33, 8
    oracle.seed(9)
    q, v = oracle.uniform((BH, S, dk), -1, 1), oracle.uniform((BH, S, dk), -1, 1)
    k = np.repeat(oracle.uniform((BH, 1, dk), -1, 1), S, axis=1)
    o, l = oracle.sdpa(q, k, v, 0.5)
    assert np.abs(o - v.mean(axis=1, keepdims=True)).max() < 1e-6
    score = 0.5 * np.einsum("hid,hd->hi", q, k[:, 0])
    assert np.abs(l - (score + np.log(S))).max() < 1e-5
    # causal: the first query sees only key 0; a one-hot dominant key selects its value row
    o, l = oracle.sdpa(q, k, v, 0.5, causal=True)
    assert np.abs(o[:, 0] - v[:, 0]).max() < 1e-7
    q1 = np.zeros((1, 4, 4), np.float32); q1[0, :, 0] = 1
    k1 = np.zeros((1, 4, 4), np.float32); k1[0, 2, 0] = 100
    v1 = np.arange(16, dtype=np.float32).reshape(1, 4, 4)
    o, _ = oracle.sdpa(q1, k1, v1, 1.0)
    assert np.abs(o[0] - v1[0, 2]).max() < 1e-6


# ---------------------------------------------------------------- live cross-check
def test_oracle_equals_compiled_reference(oracle, reflib):
    oracle.seed(11)
    for (M, K, N) in [(5, 333, 77), (130, 700, 260), (1, 4096, 512), (256, 512, 384)]:
        a, b = oracle.uniform((M, K), -1, 1), oracle.uniform((K, N), -1, 1)
        ref = reflib.gemm(a, b)
        assert np.abs(oracle.gemm_opt(a, b) - ref).max() <= 1e-4 * np.abs(ref).max()
        assert np.array_equal(oracle.gemm_naive(a, b), reflib.gemm(a, b, backend=0)) or M * N * K > 2e7
    w = oracle.normal((96, 333), 0, 0.02)
    q, s = oracle.quantize_rows(w)
    q2, s2 = reflib.quantize_rows(w)
    assert np.array_equal(q, q2) and np.array_equal(s, s2)
    a = oracle.normal((9, 333))
    assert np.array_equal(oracle.qgemm_w8a32(a, q, s), reflib.qgemm_w8a32(a, q, s))
    x, wq = oracle.int8((3, 4096)), oracle.int8((32, 4096))
    via_ref = reflib.qgemm_w8a32(x.astype(np.float32), wq, np.ones(32, np.float32))
    assert np.array_equal(oracle.qgemm_w8a8_acc(x, wq).astype(np.float64), via_ref.astype(np.float64))


# ---------------------------------------------------------------- elementwise / reduction / optimizer slots
import slot_cases as sc  # noqa: E402


@pytest.mark.parametrize("case", range(len(sc.BCAST)))
def test_binary_broadcast_against_reference_vectors(oracle, golden, case):
    """Bit-exact against both reference CPU backends (they agree, checked when the vectors were
    written), and against numpy's broadcasting, which fixes the index mapping independently."""
    a, b = sc.binary_inputs(oracle, case)
    with np.errstate(divide="ignore", invalid="ignore"):
        want = {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b,
                "equal": (a == b).astype(np.float32), "greater": (a > b).astype(np.float32)}
    for name in sc.BINARY:
        got = oracle.binary(name, a, b)
        assert np.array_equal(got, golden[f"bin_{name}_{case}"], equal_nan=True), name
        assert np.array_equal(got, want[name], equal_nan=True), name
    assert np.array_equal(oracle.binary("equal", a, a), np.ones_like(a)) and not oracle.binary("greater", a, a).any()
    if a.shape == b.shape:
        got = oracle.binary("add_relu", a, b)
        assert np.array_equal(got, golden[f"bin_add_relu_{case}"]) and np.array_equal(got, np.maximum(a + b, 0))


def test_unary_against_reference_vectors(oracle, golden):
    """Bit-exact with the reference's naive backend and activation functions (same libm here);
    numpy float64 closed forms bound the values themselves."""
    x = sc.unary_input(oracle)
    x64 = x.astype(np.float64)
    with np.errstate(all="ignore"):
        closed = {"neg": -x64, "abs": np.abs(x64), "exp": np.exp(x64),
                  "log": np.where(x64 > 0, np.log(np.where(x64 > 0, x64, 1)), -np.finfo(np.float32).max),
                  "sqrt": np.where(x64 >= 0, np.sqrt(np.abs(x64)), 0.0), "square": x64 * x64,
                  "sigmoid": 1 / (1 + np.exp(-x64)), "tanh": np.tanh(x64),
                  "leaky_relu": np.where(x64 > 0, x64, np.float32(0.1) * x64),
                  "elu": np.where(x64 > 0, x64, np.float32(0.7) * np.expm1(x64)),
                  "swish": x64 / (1 + np.exp(-x64)),
                  "add_scalar": x64 + np.float32(0.37), "mul_scalar": x64 * np.float32(-1.7)}
    params = {"leaky_relu": 0.1, "elu": 0.7, "add_scalar": 0.37, "mul_scalar": -1.7}
    for name, want in closed.items():
        got = oracle.unary(name, x, params.get(name, 0.0))
        assert np.array_equal(got, golden[f"un_{name}"], equal_nan=True), name
        assert np.allclose(got, want, rtol=2e-6, atol=1e-6), name


def test_reductions_against_reference_vectors(oracle, golden):
    for shp, arr in zip(sc.REDUCE_SHAPES, sc.reduce_inputs(oracle)):
        tag = "x".join(map(str, shp))
        for axis in range(-1, len(shp)):
            np_axis = None if axis == -1 else axis
            for name, fn in (("mean", np.mean), ("max", np.max), ("min", np.min)):
                got = oracle.reduce(name, arr, axis)
                # the naive backend adds in the same order; the optimised one in lanes
                assert np.array_equal(got, golden[f"red_{name}_{tag}_axis{axis}_naive"]), (name, tag, axis)
                assert np.allclose(got, golden[f"red_{name}_{tag}_axis{axis}"], rtol=0, atol=2e-6)
                assert np.allclose(got.reshape(-1), np.asarray(fn(arr.astype(np.float64), axis=np_axis)).reshape(-1),
                                   rtol=0, atol=2e-6)
            got = oracle.argmax(arr, axis)
            assert np.array_equal(got, golden[f"red_argmax_{tag}_axis{axis}"])
            assert np.array_equal(got.reshape(-1), np.asarray(np.argmax(arr, axis=np_axis)).reshape(-1))
    # ties take the first index; values that fail every comparison leave the starting value
    assert oracle.argmax(np.array([[1, 3, 3, 2]], np.float32), 1)[0] == 1
    assert oracle.reduce("max", np.array([[np.nan, -np.inf]], np.float32), 1)[0] == -np.finfo(np.float32).max


def test_softmax_rows_against_reference_vectors(oracle, golden):
    for (rows, cols), arr in zip(sc.SOFTMAX_SHAPES, sc.softmax_inputs(oracle)):
        got = oracle.softmax_rows(arr)
        assert np.array_equal(got, golden[f"softmax_{rows}x{cols}_naive"])
        assert np.abs(got - golden[f"softmax_{rows}x{cols}"]).max() < 2e-6      # polynomial exp there
        e = np.exp(arr.astype(np.float64) - arr.max(axis=1, keepdims=True))
        assert np.abs(got - e / e.sum(axis=1, keepdims=True)).max() < 1e-6
        assert np.abs(got.sum(axis=1) - 1).max() < 1e-5
    # shift invariance and the uniform row
    x = sc.softmax_inputs(oracle)[0]
    assert np.abs(oracle.softmax_rows(x + 3.0) - oracle.softmax_rows(x)).max() < 1e-6
    assert np.allclose(oracle.softmax_rows(np.full((2, 8), 5.0, np.float32)), 0.125)


def test_layernorm_against_reference_vectors(oracle, golden):
    for shp, (x, gamma, beta) in zip(sc.LAYERNORM_SHAPES, sc.layernorm_inputs(oracle)):
        out, xh, inv = oracle.layernorm(x, gamma, beta, 1e-5)
        ref = golden["layernorm_" + "x".join(map(str, shp))]
        assert np.abs(out - ref).max() < 5e-6
        x64 = x.astype(np.float64)
        mu, var = x64.mean(axis=-1, keepdims=True), x64.var(axis=-1, keepdims=True)
        want_xh = (x64 - mu) / np.sqrt(var + 1e-5)
        assert np.abs(xh - want_xh).max() < 5e-6 and np.abs(ref - (gamma * want_xh + beta)).max() < 5e-6
        assert np.abs(out - (gamma * want_xh + beta)).max() < 5e-6
        assert np.allclose(inv, 1 / np.sqrt(var.reshape(-1) + 1e-5), rtol=2e-6)
    # a constant row has zero variance: x_hat = 0 and the output is beta
    out, xh, inv = oracle.layernorm(np.full((1, 12), 3.0, np.float32), np.ones(12, np.float32),
                                    np.arange(12, dtype=np.float32), 1e-5)
    assert np.array_equal(xh, np.zeros((1, 12), np.float32)) and np.array_equal(out[0], np.arange(12, dtype=np.float32))


@pytest.mark.parametrize("key", list(sc.OPTIMIZERS))
def test_optimizer_updates_against_reference_vectors(oracle, golden, key):
    """The per-element update formulas against what the reference's CPU optimizers produced
    over three steps (its Adam folds the bias corrections into the step size, hence a tolerance),
    and against a float64 evaluation of the textbook recurrences."""
    kind, kw = sc.OPTIMIZERS[key]
    w0, grads = sc.optimizer_inputs(oracle)
    w, m, v = w0.copy(), np.zeros_like(w0), np.zeros_like(w0)
    w64, m64, v64 = w0.astype(np.float64), np.zeros(300), np.zeros(300)
    for step, g in enumerate(grads, 1):
        g64 = g.astype(np.float64)
        if kind == "sgd":
            oracle.sgd_update(w, g, m if kw["momentum"] > 0 else None, kw["lr"], kw["momentum"], kw["wd"], kw["nesterov"])
            gi = g64 + kw["wd"] * w64
            if kw["momentum"] > 0:
                m64 = kw["momentum"] * m64 + gi
                w64 = w64 - kw["lr"] * ((gi + kw["momentum"] * m64) if kw["nesterov"] else m64)
            else:
                w64 = w64 - kw["lr"] * gi
        else:
            bc1, bc2 = sc.bias_corrections(kw["beta1"], kw["beta2"], step)
            oracle.adam_update(w, g, m, v, kw["lr"], kw["beta1"], kw["beta2"], kw["eps"], kw["wd"], bc1, bc2,
                               kind == "adamw")
            if kind == "adamw":
                w64 = w64 * (1 - kw["lr"] * kw["wd"])
                gi = g64
            else:
                gi = g64 + kw["wd"] * w64
            m64 = kw["beta1"] * m64 + (1 - kw["beta1"]) * gi
            v64 = kw["beta2"] * v64 + (1 - kw["beta2"]) * gi * gi
            w64 = w64 - kw["lr"] * (m64 / (1 - kw["beta1"] ** step)) / (np.sqrt(v64 / (1 - kw["beta2"] ** step)) + kw["eps"])
        assert np.abs(w - golden[key][step - 1]).max() < 2e-6, step
        assert np.abs(w - w64).max() < 2e-6, step


# ---------------------------------------------------------------- attention layer
def test_mha_layer_restatement_against_reference_vectors(oracle, golden):
    """GEMM + head split + attention + head merge + GEMM, assembled from the oracle's pieces,
    against what the reference's own layer produced (its CPU path fuses these differently)."""
    import attn_cases as ac
    _, w = ac.fixture_model("mha_causal")
    x = ac.fixture_input(oracle, w, (2, 128, 128), 8700)
    got = ac.mha_forward(oracle, x, w, 2, True)
    want = golden["axm_mha_causal_out"]
    assert np.abs(got - want).max() <= 1e-5 * max(1.0, np.abs(want).max())
    # numpy float64 evaluation of the definition
    B, S, D, H, dk = 2, 128, 128, 2, 64
    x64 = x.astype(np.float64).reshape(B * S, D)
    q, k, v = ((x64 @ w[i] + w[4 + i]).reshape(B, S, H, dk).transpose(0, 2, 1, 3) for i in range(3))
    s = q @ k.transpose(0, 1, 3, 2) / np.sqrt(dk)
    s = np.where(np.tril(np.ones((S, S), bool)), s, -np.inf)
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    o = (p / p.sum(axis=-1, keepdims=True)) @ v
    ref = o.transpose(0, 2, 1, 3).reshape(B * S, D) @ w[3] + w[7]
    assert np.abs(want.reshape(B * S, D) - ref).max() <= 1e-5 * max(1.0, np.abs(ref).max())
    # the two layout maps are inverses of numpy's own transposes
    t = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(6, 20)
    assert np.array_equal(ac.merge_heads(ac.split_heads(t, 2, 3, 4, 5), 2, 3, 4, 5), t)
