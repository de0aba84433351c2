"""GPU parity: the HIP path, called through the C ABI of libaxhip.so, against the CPU oracle
on identical seeded inputs.  int32 accumulators and int8 outputs: bit-exact.  fp32: the gates
stated next to each assert."""
import os

import numpy as np
import pytest

from fills import property_case, xorshift32_unit

pytestmark = pytest.mark.gpu

REL_FP32 = 1e-4      # max |gpu - cpu| / max |cpu|                      (fp32 GEMM vs the CPU path)
BOUND_FP32 = 1e-5    # |gpu - c64| <= BOUND * sum_k |a_ik||b_kj|        (vs fp64 ground truth)


def say(*a):
    print(*a, flush=True)


def check_fp32(oracle, got, a, b, transb=False, ref=None):
    c64 = oracle.gemm_f64(a, b, transb)
    cabs = oracle.gemm_abs_f64(a, b, transb)
    assert (np.abs(got - c64) <= BOUND_FP32 * cabs + 1e-30).all(), \
        f"fp64 bound violated: {(np.abs(got - c64) / (cabs + 1e-30)).max()}"
    if ref is not None:
        assert np.abs(got - ref).max() <= REL_FP32 * max(np.abs(ref).max(), 1e-30)


# ------------------------------------------------------------------ int8 W8A8
INT8_SHAPES = [(1, 1, 1), (3, 17, 45), (5, 7, 16), (64, 64, 128), (100, 200, 300), (33, 64, 1000),
               (128, 128, 256), (128, 256, 128), (256, 512, 384), (384, 128, 4096),
               (2048, 4096, 512), (256, 4096, 4096),
               # M <= 4 with whole 16-byte steps of K: the wave-per-rows dot-product route (and M = 5..8, on the tiles since)
               (1, 768, 3072), (1, 4096, 4096), (8, 768, 768), (3, 5, 16), (7, 1001, 1040), (2, 3, 4112),
               (4, 33, 64), (5, 9, 48), (6, 130, 256), (4, 11008, 512), (3, 4100, 2064),
               # staggered walks over K: a start slab that is odd with two slabs per stage, and with the K split
               (256, 4096, 1536), (128, 2048, 2560),
               # off the 256 grid with a large interior: persistent kernel inside, smaller tiles on the fringes
               (2112, 4128, 256), (4100, 2304, 128), (2048, 4100, 128),
               # rows that start at odd byte offsets (K % 16 != 0)
               (70, 90, 1037), (130, 257, 4099),
               # large with K off the 128 grid: zero-padded copies of both operands, then the fast kernels
               (2048, 4096, 520), (2112, 4128, 600),
               # M or N off the 64 grid with K on the 128 grid: the direct-to-LDS kernel with clamped edge tiles
               (100, 4096, 512), (130, 260, 256), (2000, 2000, 128), (63, 60, 128), (9, 4, 128), (500, 1000, 1024),
               (65, 64, 256), (64, 68, 384), (2900, 3000, 128),
               (500, 4096, 512), (900, 1004, 384), (260, 6148, 256),   # 128x64 tiles with clamped edges, and M = 260 that stays on 64x64
               # K a multiple of 16 off the 128 grid: the last slab's tail is zero-filled in LDS
               (100, 4096, 784), (64, 64, 16), (130, 260, 144), (256, 4096, 784), (2900, 3000, 400), (9, 4, 48),
               (64, 128, 1040), (128, 128, 112),
               # few tiles against a long K: workgroups split K and the last one of a tile adds the int32 partials
               (64, 1024, 4096), (64, 64, 8192), (256, 2048, 8192), (512, 1024, 4096), (100, 4096, 4096), (70, 200, 2064),
               (128, 128, 2048),
               # more than one 64x64 tile per CU, fewer than one 128x128 tile per CU: 128x64 tiles on eight waves
               (512, 4096, 512), (384, 2752, 256), (256, 6144, 1152), (2048, 2048, 2048)]


@pytest.mark.parametrize("M,N,K", INT8_SHAPES)
def test_w8a8_accumulators_bit_exact(hip, oracle, M, N, K):
    say("w8a8", M, N, K)
    oracle.seed(M * 7 + N * 3 + K)
    x, w = oracle.int8((M, K)), oracle.int8((N, K))
    ws = oracle.uniform((N,), 1e-3, 1e-2)
    bias = oracle.normal((N,), 0.0, 0.02)
    xs = float(np.float32(0.0173))
    dx, dw, dws, db = hip.array(x), hip.array(w), hip.array(ws), hip.array(bias)
    want_acc = oracle.qgemm_w8a8_acc(x, w)
    for act in (0, 1, 2):
        out, acc = hip.qgemm_w8a8(dx, xs, dw, dws, db, act)
        say("  kernel", hip.last_kernel(), "act", act)
        assert np.array_equal(acc.numpy(), want_acc)
        want = oracle.w8a8_epilogue(want_acc, xs, ws, bias, act)
        got = out.numpy()
        if act != 2:
            assert np.array_equal(got, want)              # same op order: bit-identical
        else:                                             # tanhf differs between libms
            assert np.abs(got - want).max() <= 1e-6 * max(1.0, np.abs(want).max())
    out, _ = hip.qgemm_w8a8(dx, xs, dw, dws, None, 0, want_acc=False)
    assert np.array_equal(out.numpy(), oracle.w8a8_epilogue(want_acc, xs, ws, None, 0))
    _, acc = hip.qgemm_w8a8(dx, xs, dw, None, None, 0, want_out=False)
    assert np.array_equal(acc.numpy(), want_acc)


@pytest.mark.parametrize("M,N,K", [(8, 11008, 4096), (64, 8192, 5120), (16, 4100, 11008)])
def test_w8a8_streaming_weights_bit_exact(hip, M, N, K):
    """One row of tiles against 40 MiB of weights and more: the weights are fetched with non-temporal loads.  The int32
    accumulators stay exact (checked against an fp64 product, which is exact at these magnitudes)."""
    say("w8a8 streaming", M, N, K)
    rng = np.random.default_rng(M + N + K)
    x = rng.integers(-127, 128, (M, K), dtype=np.int8)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    _, acc = hip.qgemm_w8a8(hip.array(x), 0.01, hip.array(w), None, None, 0, want_out=False)
    say("  kernel", hip.last_kernel())
    assert hip.last_kernel().startswith("qgemm_w8a8_64x64")
    want = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.int64)
    assert np.array_equal(acc.numpy().astype(np.int64), want)


def test_w8a8_extreme_values_and_golden(hip, oracle, golden):
    x = np.full((128, 8192), -127, np.int8)
    w = np.full((128, 8192), -127, np.int8)
    _, acc = hip.qgemm_w8a8(hip.array(x), 1.0, hip.array(w), None, want_out=False)
    assert (acc.numpy() == 127 * 127 * 8192).all()
    xg = hip.array(x[:4].copy())                          # same through the M <= 4 route
    wg = hip.array(np.full((128, 8192), -128, np.int8))
    _, acc = hip.qgemm_w8a8(xg, 1.0, wg, None, want_out=False)
    assert hip.last_kernel() == "qgemm_w8a8_gemv" and (acc.numpy() == 127 * 128 * 8192).all()
    for K in (8, 32, 128, 512, 1024):                     # the reference's W8A32 with unit scales
        oracle.seed(1000 + K)
        x, w = oracle.int8((4, K)), oracle.int8((64, K))
        _, acc = hip.qgemm_w8a8(hip.array(x), 1.0, hip.array(w), None, want_out=False)
        assert np.array_equal(acc.numpy().astype(np.float64), golden[f"acc_K{K}"].astype(np.float64))


@pytest.mark.parametrize("M,N,K", [(8192, 8192, 8192), (4096, 8192, 384), (4096, 8192, 512), (2048, 4096, 128),
                                   (2048, 4096, 2048), (2048, 11008 // 256 * 256, 2048)])
def test_w8a8_persistent_tiles_properties(hip, oracle, M, N, K):
    """Shapes served by the persistent 256x256 kernel, several tiles per workgroup, with an even
    slab count (next tile's first slab fetched under the write-back), an odd one, and one slab;
    the first is the full size of the headline config.  The last two have whole tiles for half the
    CUs / a short last round and a long K: they run on 256x128 tiles.  Exact row/column checksums and 4096
    sampled entries of the accumulators; the fp32 output of the out-only call (the form the
    benchmark times) against the epilogue applied to those accumulators."""
    oracle.seed(M + N + K)
    x, w = oracle.int8((M, K)), oracle.int8((N, K))
    ws = oracle.uniform((N,), 1e-3, 1e-2)
    bias = oracle.normal((N,), 0.0, 0.02)
    xs = float(np.float32(0.011))
    dx, dw, dws, db = hip.array(x), hip.array(w), hip.array(ws), hip.array(bias)
    say("w8a8 persistent", M, N, K)
    out, acc = hip.qgemm_w8a8(dx, xs, dw, dws, db, 0)
    say("  kernel", hip.last_kernel())
    assert hip.last_kernel() == ("qgemm_w8a8_256x128_dma" if K == 2048 else "qgemm_w8a8_256x256_dma")
    a = acc.numpy()
    xi, wi = x.astype(np.int64), w.astype(np.int64)
    assert np.array_equal(a.astype(np.int64).sum(axis=0), wi @ xi.sum(axis=0))   # column sums
    assert np.array_equal(a.astype(np.int64).sum(axis=1), xi @ wi.sum(axis=0))   # row sums
    rng = np.random.default_rng(1)
    ms, ns = rng.integers(0, M, 4096), rng.integers(0, N, 4096)
    exact = np.einsum("ik,ik->i", xi[ms], wi[ns])
    assert np.array_equal(a[ms, ns].astype(np.int64), exact)
    want = oracle.w8a8_epilogue(a, xs, ws, bias, 0)
    assert np.array_equal(out.numpy(), want)
    _, acc_only = hip.qgemm_w8a8(dx, xs, dw, None, None, 0, want_out=False)
    assert np.array_equal(acc_only.numpy(), a)
    for act in (0, 1):
        out_only, _ = hip.qgemm_w8a8(dx, xs, dw, dws, db, act, want_acc=False)
        assert np.array_equal(out_only.numpy(), np.maximum(want, 0) if act else want)
    out_nb, _ = hip.qgemm_w8a8(dx, xs, dw, dws, None, 0, want_acc=False)
    assert np.array_equal(out_nb.numpy(), oracle.w8a8_epilogue(a, xs, ws, None, 0))


# ------------------------------------------------------------------ fp32 GEMM
F32_SHAPES = [(1, 1, 1), (2, 3, 2), (37, 19, 73), (64, 32, 128), (9, 500, 300), (64, 64, 32),
              (128, 128, 64), (130, 260, 700), (256, 384, 512), (33, 40, 100), (96, 96, 96),
              (2048, 1024, 256),
              # shapes that take the 128x128 eight-wave tile, and ones just short of it in N or in tile count
              (2048, 4096, 64), (4096, 2176, 64), (4096, 1088, 32), (128, 64, 4096),
              # 64x64 tile counts with a nearly empty last round of one tile per CU: 32x64 tiles (NN and NT)
              (1152, 1152, 192), (1280, 960, 256),
              # few output tiles and a long K: the split-K route (bench_qgemm.c shapes among them)
              (32, 768, 768), (64, 1024, 4096), (128, 4096, 1024), (9, 100, 512), (16, 16, 8192), (70, 130, 1536),
              # few tiles and K short enough that one launch on 32x64 tiles beats the split, and their neighbours that split
              (1024, 256, 256), (64, 4096, 512), (256, 768, 768), (64, 768, 768), (1024, 512, 1536), (256, 1024, 1024),
              # up to 160 rows with an odd count of 32-row blocks: 32x64 tiles (whole and with clamped edges), alone and under the K split
              (32, 2048, 128), (96, 4096, 1024), (160, 3072, 768), (20, 2048, 512), (80, 1088, 256), (150, 260, 160), (130, 4096, 96),
              (24, 11008, 512),
              # one round of tiles over a long K: three stages (operands past the L2s), and the K split when a fifth of the CUs would idle
              (256, 3072, 2048), (192, 2816, 4096),
              # 64x64 tiles with the k split: two slabs per stage (K a multiple of 64; an odd and an even count of stages) and one (K = 160)
              (256, 512, 192), (320, 256, 448), (256, 256, 256), (256, 512, 160),
              # off the tile grid with a large interior: fast kernels inside, guarded kernel on the fringes
              (1032, 1100, 96), (2100, 4200, 64), (1024, 1092, 160),
              (130, 257, 1027), (67, 1001, 129),                  # rows off the 16-byte grid in every form
              (1024, 1088, 1045), (1030, 1100, 600),              # K off the 32 grid: main product, then the K tail on top
              # M or N off the 64 grid with K on the 32 grid and N % 4 == 0: direct-to-LDS tiles with guarded edges
              (65, 68, 64), (9, 4, 32), (63, 60, 96), (200, 36, 128), (500, 1000, 256), (12, 2052, 160),
              # K a multiple of 4 off the 32 grid: the last slab's tail is zero-filled in LDS
              (64, 4096, 784), (128, 64, 36), (64, 64, 4), (100, 132, 100), (256, 256, 44), (70, 64, 1000), (16, 256, 2076)]


@pytest.mark.parametrize("M,N,K", F32_SHAPES)
def test_sgemm_nn_nt_tn(hip, oracle, M, N, K):
    say("sgemm", M, N, K)
    oracle.seed(M + 31 * N + 977 * K)
    a, b = oracle.uniform((M, K), -1, 1), oracle.uniform((K, N), -1, 1)
    ref = oracle.gemm_opt(a, b)
    da, db = hip.array(a), hip.array(b)
    got = hip.sgemm(da, db).numpy()
    say("  nn", hip.last_kernel())
    check_fp32(oracle, got, a, b, ref=ref)
    bt = np.ascontiguousarray(b.T)
    got = hip.sgemm(da, hip.array(bt), transb=True).numpy()
    say("  nt", hip.last_kernel())
    check_fp32(oracle, got, a, bt, transb=True, ref=oracle.gemm_opt_nt(a, bt))
    at = np.ascontiguousarray(a.T)
    got = hip.sgemm(hip.array(at), db, transa=True).numpy()
    say("  tn", hip.last_kernel())
    check_fp32(oracle, got, a, b, ref=ref)


@pytest.mark.parametrize("M,N,K", [(16, 4096, 2304), (64, 8192, 1056), (40, 4100, 2112), (12, 11008, 1024)])
def test_sgemm_streaming_weight_tiles(hip, oracle, M, N, K):
    """A single row of tiles against 32 MiB of fp32 weights and more: the tiles of at most 64 rows fetch B with
    non-temporal loads (their own instantiation), whole and with clamped edges, alone and under the K split."""
    say("sgemm streaming tiles", M, N, K)
    oracle.seed(M + 31 * N + 977 * K)
    a, b = oracle.uniform((M, K), -1, 1), oracle.uniform((K, N), -1, 1)
    got = hip.sgemm(hip.array(a), hip.array(b)).numpy()
    say("  nn", hip.last_kernel())
    check_fp32(oracle, got, a, b, ref=oracle.gemm_opt(a, b))


@pytest.mark.parametrize("M,N,K,pad,off", [(256, 384, 128, 64, 32), (2048, 4096, 64, 128, 64),
                                           (256, 384, 128, 3, 1), (70, 50, 90, 5, 2)])
def test_sgemm_submatrix_views(hip, oracle, M, N, K, pad, off):
    """Operands and result are windows of larger row-major arrays (leading dimension > row
    length, first element `off` floats into the allocation): multiples of 4 keep the
    direct-to-LDS path, odd values must fall back to the guarded kernel; memory outside the C
    window must stay untouched."""
    oracle.seed(M + N + K + pad)
    big_a, big_b = oracle.uniform((M, K + pad), -1, 1), oracle.uniform((K, N + pad), -1, 1)
    big_bt = oracle.uniform((N, K + pad), -1, 1)
    big_c = oracle.uniform((M, N + pad), -1, 1)
    a, b = np.ascontiguousarray(big_a[:, off:off + K]), np.ascontiguousarray(big_b[:, off:off + N])
    bt = np.ascontiguousarray(big_bt[:, off:off + K])
    da, db, dbt = hip.array(big_a), hip.array(big_b), hip.array(big_bt)
    for transb, dbb, ldb, href in ((0, db, N + pad, b), (1, dbt, K + pad, bt)):
        dc = hip.array(big_c)
        hip.check(hip.L.axhip_sgemm(0, transb, M, N, K, 1.0, da.ptr + 4 * off, K + pad, dbb.ptr + 4 * off, ldb,
                                    0.0, dc.ptr + 4 * off, N + pad, None, 0))
        say("  view", (M, N, K, pad, off), "transb", transb, hip.last_kernel())
        got = dc.numpy()
        check_fp32(oracle, np.ascontiguousarray(got[:, off:off + N]), a, href, transb=bool(transb))
        mask = np.ones_like(big_c, bool)
        mask[:, off:off + N] = False
        assert np.array_equal(got[mask], big_c[mask])


def test_sgemm_known_answers(hip, golden):
    a = np.arange(1, 7, dtype=np.float32).reshape(2, 3)
    b = np.arange(7, 13, dtype=np.float32).reshape(3, 2)
    assert hip.sgemm(hip.array(a), hip.array(b)).numpy().reshape(-1).tolist() == [58, 64, 139, 154]
    c = hip.sgemm(hip.array(np.array([[1, 2], [3, 4]], np.float32)),
                  hip.array(np.array([[5, 6], [7, 8]], np.float32))).numpy()
    assert c.reshape(-1).tolist() == [19, 22, 43, 50]
    rng = np.random.default_rng(0)
    m = rng.uniform(-1, 1, (200, 200)).astype(np.float32)
    assert np.array_equal(hip.sgemm(hip.array(m), hip.array(np.eye(200, dtype=np.float32))).numpy(), m)
    assert not hip.sgemm(hip.array(np.zeros((70, 300), np.float32)), hip.array(m[:, :100].repeat(3, 0)[:300])).numpy().any()
    u, v = m[:33, :1].copy(), m[:1, :65].copy()
    assert np.array_equal(hip.sgemm(hip.array(u), hip.array(v)).numpy(), u * v)      # K = 1


@pytest.mark.parametrize("M,K,N", [(37, 73, 19), (64, 128, 32), (32, 2048, 16), (1, 784, 64), (7, 300, 130)])
def test_sgemm_against_reference_outputs(hip, oracle, golden, M, K, N):
    oracle.seed(M * 1000 + N)
    a, b = oracle.uniform((M, K), -1, 1), oracle.uniform((K, N), -1, 1)
    ref = golden[f"gemm_{M}x{K}x{N}_opt"]
    got = hip.sgemm(hip.array(a), hip.array(b)).numpy()
    # the reference's own GPU-vs-CPU gate is 1e-3 abs (tests/test_cuda.c:235); ours is tighter
    assert np.abs(got - ref).max() <= REL_FP32 * np.abs(ref).max()
    got = hip.sgemm(hip.array(a), hip.array(np.ascontiguousarray(b.T)), transb=True).numpy()
    assert np.abs(got - golden[f"gemm_nt_{M}x{K}x{N}_opt"]).max() <= REL_FP32 * np.abs(ref).max()


def test_sgemm_property_cases(hip, oracle, golden):
    for i in range(60):                                   # tests/test_property.c:176-208
        M, N, K, a, b = property_case(i)
        got = hip.sgemm(hip.array(a), hip.array(b)).numpy()
        cn = oracle.gemm_naive(a, b)
        assert (np.abs(got - cn) <= 1e-3 + 1e-4 * np.abs(cn)).all(), (i, M, N, K)
        assert abs(got.astype(np.float64).sum() - golden["prop_sums"][i, 1]) <= \
            1e-5 * max(1.0, golden["prop_sums"][i, 2])


def test_sgemm_config0_1024_cube(hip, oracle, golden):
    oracle.seed(0)
    a, b = oracle.uniform((1024, 1024), -1, 1), oracle.uniform((1024, 1024), -1, 1)
    da, db = hip.array(a), hip.array(b)
    dc = hip.sgemm(da, db)
    say("1024^3", hip.last_kernel())
    c = dc.numpy()
    check_fp32(oracle, c, a, b, ref=oracle.gemm_opt(a, b))
    assert np.abs(c[0] - golden["gemm_1024_row0"]).max() <= REL_FP32 * 60
    s, sabs = golden["gemm_1024_sums"]
    assert abs(c.astype(np.float64).sum() - s) <= 1e-6 * sabs
    # determinism (tests/test_optimization_paths.c:265-292): repeated runs are bit-identical
    for _ in range(5):
        assert np.array_equal(hip.sgemm(da, db).numpy(), c)


@pytest.mark.parametrize("M,N,K", [(130, 200, 96), (256, 320, 96), (2048, 4096, 32), (64, 128, 2048), (33, 70, 512), (1032, 1100, 96), (1024, 1088, 1045), (200, 260, 784)])
def test_sgemm_alpha_beta_bias_act(hip, oracle, M, N, K):
    say("sgemm epilogue", M, N, K)
    oracle.seed(21)
    a, b = oracle.uniform((M, K), -1, 1), oracle.uniform((K, N), -1, 1)
    c0 = oracle.uniform((M, N), -1, 1)
    bias = oracle.normal((N,), 0, 0.5)
    c64 = oracle.gemm_f64(a, b)
    da, db, dbias = hip.array(a), hip.array(b), hip.array(bias)
    got = hip.sgemm(da, db, alpha=0.5, beta=2.0, c=hip.array(c0)).numpy()
    assert np.abs(got - (0.5 * c64 + 2.0 * c0)).max() <= 1e-5 * K
    got = hip.sgemm(da, db, alpha=1.0, beta=1.0, c=hip.array(c0)).numpy()      # gemm_ex accumulate
    assert np.abs(got - (c64 + c0)).max() <= 1e-5 * K
    lin = hip.sgemm(da, db, bias=dbias).numpy()
    assert np.abs(lin - oracle.dense(a, b, bias, 0)).max() <= REL_FP32 * np.abs(c64).max()
    relu = hip.sgemm(da, db, bias=dbias, act=1).numpy()
    assert np.array_equal(relu, np.maximum(lin, 0))
    assert np.abs(relu - oracle.dense(a, b, bias, 1)).max() <= REL_FP32 * np.abs(c64).max()
    gelu = hip.sgemm(da, db, bias=dbias, act=2).numpy()
    assert np.abs(gelu - oracle.gelu(lin)).max() <= 1e-5 + 1e-5 * np.abs(lin).max()
    # beta = 0 must not read C: poison it with NaN
    poison = hip.array(np.full((M, N), np.nan, np.float32))
    assert np.isfinite(hip.sgemm(da, db, c=poison).numpy()).all()


# dimensions around every boundary the dispatch looks at (tile edges, vector widths, K slabs, split thresholds)
EDGY = [1, 2, 3, 4, 5, 7, 8, 9, 12, 15, 16, 17, 31, 32, 33, 36, 60, 63, 64, 65, 68, 96, 100, 127, 128, 129, 132, 160, 192,
        255, 256, 257, 260, 320, 384, 500, 512, 516, 640, 700, 768, 1000, 1024, 1028, 1100]


def test_sgemm_dispatch_sweep(hip, oracle):
    """120 seeded shapes drawn from the boundary dimensions, in a random form (NN / NT / TN), with a random
    alpha, beta, bias and activation: whichever route the dispatch takes, the result obeys the fp64 bound."""
    rng = np.random.default_rng(20240)
    seen = set()
    for case in range(120):
        M, N, K = (int(rng.choice(EDGY)) for _ in range(3))
        if case % 3 == 0:
            K = int(rng.choice([1024, 1536, 2048, 2052, 4096]))          # long K: split and K-tail routes
        form = int(rng.integers(0, 3))
        alpha = float(rng.choice([1.0, 1.0, 0.5, -2.0]))
        beta = float(rng.choice([0.0, 0.0, 1.0, 0.25]))
        use_bias, act = bool(rng.integers(0, 2)), int(rng.integers(0, 3))
        a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
        b = rng.uniform(-1, 1, (K, N)).astype(np.float32)
        c0 = rng.uniform(-1, 1, (M, N)).astype(np.float32)
        bias = rng.normal(0, 0.5, N).astype(np.float32)
        say("sweep", case, M, N, K, "form", form, "alpha", alpha, "beta", beta, "bias", use_bias, "act", act)
        da = hip.array(np.ascontiguousarray(a.T) if form == 2 else a)
        db = hip.array(np.ascontiguousarray(b.T) if form == 1 else b)
        got = hip.sgemm(da, db, transa=form == 2, transb=form == 1, alpha=alpha, beta=beta, c=hip.array(c0),
                        bias=hip.array(bias) if use_bias else None, act=act).numpy()
        seen.add(hip.last_kernel())
        pre = alpha * (a.astype(np.float64) @ b.astype(np.float64)) + beta * c0 + (bias if use_bias else 0.0)
        want = np.maximum(pre, 0) if act == 1 else oracle.gelu(pre.astype(np.float32)).astype(np.float64) if act == 2 else pre
        bound = BOUND_FP32 * (abs(alpha) * (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)) + abs(beta) + 1.0)
        assert (np.abs(got - want) <= bound + (2e-5 * (1 + np.abs(pre)) if act == 2 else 0)).all(), \
            (case, M, N, K, form, hip.last_kernel(), float(np.abs(got - want).max()))
    say("  routes:", sorted(seen))
    assert len(seen) >= 6


def test_w8a8_dispatch_sweep(hip, oracle):
    """100 seeded int8 shapes from the boundary dimensions (K also on and off the 16- and 128-byte grids):
    accumulators bit-exact and outputs equal to the oracle's epilogue whatever kernel ran."""
    rng = np.random.default_rng(20241)
    seen = set()
    for case in range(100):
        M, N = int(rng.choice(EDGY)), int(rng.choice(EDGY))
        K = int(rng.choice(EDGY + [1040, 2048, 2064, 4096, 4100]))
        act, use_bias = int(rng.integers(0, 2)), bool(rng.integers(0, 2))
        x = rng.integers(-127, 128, (M, K), dtype=np.int8)
        w = rng.integers(-127, 128, (N, K), dtype=np.int8)
        ws = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        bias = rng.normal(0, 0.02, N).astype(np.float32)
        xs = float(np.float32(0.0131))
        say("sweep i8", case, M, N, K, "act", act, "bias", use_bias)
        out, acc = hip.qgemm_w8a8(hip.array(x), xs, hip.array(w), hip.array(ws), hip.array(bias) if use_bias else None, act)
        seen.add(hip.last_kernel())
        want_acc = x.astype(np.int32) @ w.astype(np.int32).T
        assert np.array_equal(acc.numpy(), want_acc), (case, M, N, K, hip.last_kernel())
        assert np.array_equal(out.numpy(), oracle.w8a8_epilogue(want_acc, xs, ws, bias if use_bias else None, act)), \
            (case, M, N, K, hip.last_kernel())
    say("  routes:", sorted(seen))
    assert len(seen) >= 3


def test_forced_tiles_and_splits_keep_parity(hip, oracle):
    """The environment overrides change which kernel runs, never the result: W8A8 accumulators and outputs stay
    bit-exact and fp32 / skinny products stay inside their gates under every forced tile, split and block count."""
    names = ("AX_HIP_I8_TILE", "AX_HIP_I8_SPLITK", "AX_HIP_F32_TILE", "AX_HIP_F32_SPLITK", "AX_HIP_SKINNY_BLOCKS", "AX_HIP_I8_MFMA",
             "AX_HIP_SKINNY_FORM", "AX_HIP_SKINNY_KPS")
    saved = {n: os.environ.get(n) for n in names}
    rng = np.random.default_rng(77)
    M, N, K = 256, 512, 2048
    x, w = rng.integers(-127, 128, (M, K), dtype=np.int8), rng.integers(-127, 128, (N, K), dtype=np.int8)
    ws, bias = rng.uniform(1e-3, 1e-2, N).astype(np.float32), rng.normal(0, 0.02, N).astype(np.float32)
    want_acc = x.astype(np.int32) @ w.astype(np.int32).T
    want_out = oracle.w8a8_epilogue(want_acc, np.float32(0.02), ws, bias, 1)
    a, b = rng.uniform(-1, 1, (256, 1024)).astype(np.float32), rng.uniform(-1, 1, (1024, 512)).astype(np.float32)
    ref = oracle.gemm_opt(a, b)
    sa = rng.uniform(-1, 1, (3, 1024)).astype(np.float32)
    sref = oracle.gemm_opt(sa, b)
    dx, dw, dws, db, da, dbm, dsa = (hip.array(v) for v in (x, w, ws, bias, a, b, sa))
    seen = set()
    try:
        for tile, split in (("64x64", "1"), ("64x64", "4"), ("64x64k2", "1"), ("64x64k2", "3"), ("128x128", "2"),
                            ("128x64", "1"), ("128x64", "3"), ("256x256", "1"), ("", "16"), ("bogus", "99")):
            os.environ["AX_HIP_I8_TILE"], os.environ["AX_HIP_I8_SPLITK"] = tile, split
            hip.L.axhip_tuning_reload()
            say("forced i8", tile, split)
            out, acc = hip.qgemm_w8a8(dx, 0.02, dw, dws, db, 1)
            seen.add(hip.last_kernel())
            assert np.array_equal(acc.numpy(), want_acc), (tile, split, hip.last_kernel())
            assert np.array_equal(out.numpy(), want_out), (tile, split, hip.last_kernel())
        # the persistent 256x256 kernel on the other MFMA shape
        os.environ["AX_HIP_I8_TILE"], os.environ["AX_HIP_I8_SPLITK"], os.environ["AX_HIP_I8_MFMA"] = "256x256", "1", "32"
        hip.L.axhip_tuning_reload()
        say("forced i8 256x256 on 32x32x32")
        out, acc = hip.qgemm_w8a8(dx, 0.02, dw, dws, db, 1)
        seen.add(hip.last_kernel())
        assert np.array_equal(acc.numpy(), want_acc) and np.array_equal(out.numpy(), want_out)
        del os.environ["AX_HIP_I8_MFMA"]
        assert {"qgemm_w8a8_64x64_dma", "qgemm_w8a8_64x64_dma_splitk", "qgemm_w8a8_64x64k2_dma", "qgemm_w8a8_64x64k2_dma_splitk",
                "qgemm_w8a8_128x128_dma_splitk", "qgemm_w8a8_128x64_dma", "qgemm_w8a8_128x64_dma_splitk",
                "qgemm_w8a8_256x256_dma", "qgemm_w8a8_256x256_dma_mfma32x32x32"} <= seen, seen
        seen = set()
        for tile, split in (("64x64", "1"), ("64x64k2", "1"), ("128x128", "1"), ("", "4"), ("64x64", "8")):
            os.environ["AX_HIP_F32_TILE"], os.environ["AX_HIP_F32_SPLITK"] = tile, split
            hip.L.axhip_tuning_reload()
            say("forced f32", tile, split)
            got = hip.sgemm(da, dbm).numpy()
            seen.add(hip.last_kernel())
            check_fp32(oracle, got, a, b, ref=ref)
        assert {"sgemm_nn_64x64_dma", "sgemm_nn_64x64k2_dma", "sgemm_nn_128x128_dma", "sgemm_splitk"} <= seen, seen
        for blocks in ("8", "64", "4000"):
            os.environ["AX_HIP_SKINNY_BLOCKS"] = blocks
            hip.L.axhip_tuning_reload()
            say("forced skinny blocks", blocks)
            check_fp32(oracle, hip.sgemm_skinny(dsa, dbm).numpy(), sa, b, ref=sref)
        for form, kps in (("1", "64"), ("2", "1024"), ("3", "256"), ("3", "8192")):
            os.environ["AX_HIP_SKINNY_BLOCKS"], os.environ["AX_HIP_SKINNY_FORM"], os.environ["AX_HIP_SKINNY_KPS"] = "64", form, kps
            hip.L.axhip_tuning_reload()
            say("forced skinny form", form, kps)
            check_fp32(oracle, hip.sgemm_skinny(dsa, dbm).numpy(), sa, b, ref=sref)
    finally:
        for n, v in saved.items():
            if v is None:
                os.environ.pop(n, None)
            else:
                os.environ[n] = v
        hip.L.axhip_tuning_reload()


def test_w8a32_forced_tiles_keep_parity(hip):
    """AX_HIP_W8A32_TILE picks the matrix-core tile of the W8A32 product, whole or in its edge form; every choice stays
    inside the fp64 bound of a correct fp32 accumulation."""
    saved = os.environ.get("AX_HIP_W8A32_TILE")
    rng = np.random.default_rng(31)
    cases = []
    for (M, N, K) in ((256, 512, 320), (200, 260, 160)):
        a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
        w = rng.integers(-127, 128, (N, K), dtype=np.int8)
        ws = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        want = (a.astype(np.float64) @ w.astype(np.float64).T) * ws
        bound = BOUND_FP32 * (np.abs(a).astype(np.float64) @ np.abs(w).astype(np.float64).T) * ws + 1e-30
        cases.append((M, N, K, hip.array(a), hip.array(w), hip.array(ws), want, bound))
    try:
        for tile, form in (("128x256", "qgemm_w8a32_mfma_128x256_dma"), ("128x128", "qgemm_w8a32_mfma_128x128_dma"),
                           ("64x128", "qgemm_w8a32_mfma_64x128k2_dma"), ("32x128", "qgemm_w8a32_mfma_32x128k2_dma"),
                           ("32x64", "qgemm_w8a32_mfma_32x64k2_dma")):
            os.environ["AX_HIP_W8A32_TILE"] = tile
            assert hip.L.axhip_tuning_reload() == 1
            for (M, N, K, da, dw, ds, want, bound) in cases:
                say("forced w8a32", tile, M, N, K)
                got = hip.qgemm_w8a32(da, dw, ds).numpy()
                whole = M % int(tile.split("x")[0]) == 0 and N % int(tile.split("x")[1]) == 0
                assert hip.last_kernel() == form + ("" if whole else "_edge")
                assert (np.abs(got - want) <= bound).all(), (tile, M, N, K)
    finally:
        if saved is None:
            os.environ.pop("AX_HIP_W8A32_TILE", None)
        else:
            os.environ["AX_HIP_W8A32_TILE"] = saved
        hip.L.axhip_tuning_reload()


def test_w8a32_dispatch_sweep(hip, oracle):
    """80 seeded W8A32 shapes from the boundary dimensions: the weight-streaming form (M <= 6), the matrix-core form,
    its split over K and its K tail all obey the fp64 bound of a correct fp32 accumulation."""
    rng = np.random.default_rng(20243)
    seen = set()
    for case in range(80):
        M, N = int(rng.choice(EDGY[:34])), int(rng.choice(EDGY))
        K = int(rng.choice(EDGY + [1040, 2048, 2064, 4096, 4099]))
        a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
        w = rng.integers(-127, 128, (N, K), dtype=np.int8)
        ws = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        say("sweep w8a32", case, M, N, K)
        got = hip.qgemm_w8a32(hip.array(a), hip.array(w), hip.array(ws)).numpy()
        seen.add(hip.last_kernel())
        want = (a.astype(np.float64) @ w.astype(np.float64).T) * ws
        bound = BOUND_FP32 * (np.abs(a).astype(np.float64) @ np.abs(w).astype(np.float64).T) * ws + 1e-30
        assert (np.abs(got - want) <= bound).all(), (case, M, N, K, hip.last_kernel(), float((np.abs(got - want) / bound).max()))
    say("  routes:", sorted(seen))
    assert len(seen) >= 3


def test_config3_ffn_block(hip, oracle):
    """tokens 2048, d_model 1024, d_ff 4096: GEMM1 + bias + GELU -> GEMM2 + bias."""
    oracle.seed(3)
    x = oracle.normal((2048, 1024))
    w1, w2 = oracle.normal((1024, 4096), 0, 0.02), oracle.normal((4096, 1024), 0, 0.02)
    b1, b2 = oracle.normal((4096,), 0, 0.02), oracle.normal((1024,), 0, 0.02)
    say("ffn launch")
    dh = hip.sgemm(hip.array(x), hip.array(w1), bias=hip.array(b1), act=2)
    say("  ", hip.last_kernel())
    dy = hip.sgemm(dh, hip.array(w2), bias=hip.array(b2))
    h_ref = oracle.dense(x, w1, b1, 2)
    y_ref = oracle.dense(h_ref, w2, b2, 0)
    h, y = dh.numpy(), dy.numpy()
    assert np.abs(h - h_ref).max() <= 1e-5 + REL_FP32 * np.abs(h_ref).max()
    assert np.abs(y - y_ref).max() <= REL_FP32 * np.abs(y_ref).max()


# ------------------------------------------------------------------ skinny-M route
@pytest.mark.parametrize("M", list(range(1, 17)))
def test_skinny_against_oracle(hip, oracle, M):
    oracle.seed(100 + M)
    # (100, 3076) and (5000, 3072): a ragged last strip with K below one batch of rows, and splits longer
    # than the first staging pass of the activations
    for (K, N) in [(784, 4096), (4096, 4096), (4096, 10), (1, 5), (130, 67), (16, 64), (3000, 1000), (100, 3076),
                   (5000, 3072)]:
        say("skinny", M, K, N)
        a, b = oracle.uniform((M, K), 0, 1), oracle.kaiming((K, N), K)
        bias = oracle.normal((N,), 0, 0.1)
        da, db, dbias = hip.array(a), hip.array(b), hip.array(bias)
        got = hip.sgemm_skinny(da, db).numpy()
        check_fp32(oracle, got, a, b, ref=oracle.gemm_opt(a, b))
        fused = hip.sgemm_skinny(da, db, dbias, 1).numpy()
        assert np.array_equal(fused, np.maximum(got + bias[None, :], 0))
        via = hip.sgemm(da, db, bias=dbias, act=1).numpy()          # auto-routed
        if M >= 9 and K % 32 == 0 and N % 64 == 0:                  # whole tiles: the matrix-core tiles serve these rows
            assert not hip.last_kernel().startswith("sgemm_skinny")
            want = np.maximum(oracle.gemm_opt(a, b) + bias[None, :], 0)
            assert np.abs(via - want).max() <= REL_FP32 * max(np.abs(want).max(), 1e-30)
        else:
            assert hip.last_kernel().startswith("sgemm_skinny")
            assert np.array_equal(via, fused)
        assert np.array_equal(hip.sgemm_skinny(da, db).numpy(), got)  # deterministic


@pytest.mark.parametrize("M,K,N", [(1, 1030, 4096), (3, 2048, 3104), (8, 777, 4100), (13, 1500, 2052), (16, 4096, 1028)])
def test_skinny_padded_leading_dimensions(hip, oracle, M, K, N):
    """Sub-matrices of wider buffers (lda > K, ldb > N, ldc > N): the padding is neither read into
    the result nor written."""
    oracle.seed(300 + M + K + N)
    lda, ldb, ldc = K + 5, N + 8, N + 3
    abuf, bbuf = oracle.uniform((M, lda), 0, 1), oracle.kaiming((K, ldb), K)
    bias = oracle.normal((N,), 0, 0.1)
    a, b = np.ascontiguousarray(abuf[:, :K]), np.ascontiguousarray(bbuf[:, :N])
    da, db, dbias = hip.array(abuf), hip.array(bbuf), hip.array(bias)
    dc = hip.array(np.full((M, ldc), -3.0, np.float32))
    hip.check(hip.L.axhip_sgemm_skinny(M, N, K, da.ptr, lda, db.ptr, ldb, dc.ptr, ldc, dbias.ptr, 1))
    say("  kernel", hip.last_kernel())
    got = dc.numpy()
    assert (got[:, N:] == -3.0).all()
    want = np.maximum(hip.sgemm_skinny(hip.array(a), hip.array(b)).numpy() + bias[None, :], 0)
    assert np.array_equal(got[:, :N], want)
    check_fp32(oracle, hip.sgemm_skinny(hip.array(a), hip.array(b)).numpy(), a, b)


@pytest.mark.parametrize("M,K,N,NH,act,act2,keep,with_bias", [
    (1, 4096, 4096, 10, 1, 0, True, True), (8, 4096, 4096, 10, 1, 0, False, True), (16, 784, 4096, 16, 2, 1, True, True),
    (3, 100, 70, 1, 0, 0, True, False), (5, 64, 64, 7, 1, 1, True, True), (2, 2000, 1000, 3, 0, 2, False, False),
    (9, 300, 4100, 12, 1, 0, True, True), (4, 16, 8, 16, 0, 0, True, True)])
def test_skinny_with_head(hip, oracle, M, K, N, NH, act, act2, keep, with_bias):
    """A skinny layer with a narrow layer riding on it: the wide output is bit-identical to the plain route,
    the head's output is the oracle's dense layer on it (fp32 gate and fp64 bound), and calls in a row agree."""
    say("skinny+head", M, K, N, NH, act, act2, keep, with_bias)
    oracle.seed(M * 31 + K + N + NH)
    a, b = oracle.uniform((M, K), 0, 1), oracle.uniform((K, N), -0.05, 0.05)
    w2 = oracle.uniform((N, NH), -0.05, 0.05)
    bias, bias2 = oracle.normal((N,), 0, 0.1), oracle.normal((NH,), 0, 0.1)
    da, db, dw2 = hip.array(a), hip.array(b), hip.array(w2)
    dbias, dbias2 = (hip.array(bias), hip.array(bias2)) if with_bias else (None, None)
    want_c = hip.sgemm_skinny(da, db, dbias, act).numpy()
    c, o = hip.empty((M, N)), hip.empty((M, NH))
    outs = []
    for _ in range(2):
        hip.check(hip.L.axhip_memset(c.ptr, 0xFF, c.nbytes))
        hip.check(hip.L.axhip_memset(o.ptr, 0xFF, o.nbytes))
        hip.check(hip.L.axhip_sgemm_skinny_head(M, N, K, da.ptr, K, db.ptr, N, c.ptr if keep else None, N, hip._p(dbias), act,
                                                NH, dw2.ptr, hip._p(dbias2), act2, o.ptr))
        assert hip.last_kernel() == "sgemm_skinny_with_head"
        outs.append(o.numpy())
        if keep:
            assert np.array_equal(c.numpy(), want_c)
        else:
            assert np.isnan(c.numpy()).all()                     # never written
    assert np.array_equal(outs[0], outs[1])                      # deterministic
    ref = oracle.dense(want_c, w2, bias2 if with_bias else None, act2)
    assert np.abs(outs[0] - ref).max() <= REL_FP32 * max(np.abs(ref).max(), 1e-6)
    if act2 == 0:
        pre = outs[0] - (bias2[None, :] if with_bias else 0)
        check_fp32(oracle, pre.astype(np.float32), want_c, w2)
    assert hip.L.axhip_sgemm_skinny_head(M, N, K, da.ptr, K, db.ptr, N, None, N, None, 0, 17, dw2.ptr, None, 0, o.ptr) == 3
    assert hip.L.axhip_sgemm_skinny_head(M, N, K, da.ptr, K, db.ptr, N, None, N, None, 0, NH, None, None, 0, o.ptr) == 1


@pytest.mark.parametrize("M", [1, 2, 4, 8])
def test_config1_mlp_inference(hip, oracle, M):
    """x[M,784] -> dense 4096 -> ReLU -> dense 4096 -> ReLU -> dense 10; Kaiming-uniform weights
    drawn in layer order after seeding (src/core/layer.c:66-99), biases zero."""
    oracle.seed(1234)
    w1, w2, w3 = oracle.kaiming((784, 4096), 784), oracle.kaiming((4096, 4096), 4096), oracle.kaiming((4096, 10), 4096)
    z1, z2, z3 = np.zeros(4096, np.float32), np.zeros(4096, np.float32), np.zeros(10, np.float32)
    x = oracle.uniform((M, 784), 0, 1)
    ref = oracle.dense(oracle.dense(oracle.dense(x, w1, z1, 1), w2, z2, 1), w3, z3, 0)
    h1 = hip.sgemm(hip.array(x), hip.array(w1), bias=hip.array(z1), act=1)
    h2 = hip.sgemm(h1, hip.array(w2), bias=hip.array(z2), act=1)
    y = hip.sgemm(h2, hip.array(w3), bias=hip.array(z3)).numpy()
    assert y.shape == (M, 10)
    assert np.abs(y - ref).max() <= REL_FP32 * np.abs(ref).max()


# ------------------------------------------------------------------ strided batched
def test_strided_batched_qkt_and_pv(hip, oracle):
    oracle.seed(55)
    Bn, S, D = 6, 512, 64
    q, k, v = oracle.normal((Bn, S, D)), oracle.normal((Bn, S, D)), oracle.normal((Bn, S, D))
    dq, dk, dv = hip.array(q), hip.array(k), hip.array(v)
    ds = hip.sgemm_batched(dq, dk, transb=True, alpha=0.125)
    say("qkt", hip.last_kernel())
    s = ds.numpy()
    do = hip.sgemm_batched(ds, dv)
    say("pv", hip.last_kernel())
    o = do.numpy()
    for h in range(Bn):
        s_ref = oracle.gemm_opt_nt(q[h], k[h]) * np.float32(0.125)
        assert np.abs(s[h] - s_ref).max() <= REL_FP32 * np.abs(s_ref).max()
        o_ref = oracle.gemm_opt(s[h], v[h])
        assert np.abs(o[h] - o_ref).max() <= REL_FP32 * np.abs(o_ref).max()
    # ragged batch member shapes
    a, b = oracle.normal((3, 37, 29)), oracle.normal((3, 29, 41))
    c = hip.sgemm_batched(hip.array(a), hip.array(b)).numpy()
    for h in range(3):
        check_fp32(oracle, c[h], a[h], b[h])


def test_strided_batched_beyond_one_launch(hip, oracle):
    """More batch members than a launch's second grid dimension holds (65535): done in pieces."""
    oracle.seed(56)
    Bn = 70000
    a, b = oracle.normal((Bn, 4, 8)), oracle.normal((Bn, 8, 4))
    c = hip.sgemm_batched(hip.array(a), hip.array(b)).numpy()
    want = np.einsum("bik,bkj->bij", a.astype(np.float64), b.astype(np.float64))
    assert np.abs(c - want).max() <= 1e-5 * np.abs(want).max()
    assert np.abs(c[-1] - want[-1]).max() <= 1e-5 and np.abs(c[65535] - want[65535]).max() <= 1e-5


def test_config4b_attention_shapes_full_size(hip, oracle):
    """512 heads of [512,64]: sampled heads against the oracle, all heads by a linearity check."""
    oracle.seed(44)
    Bn, S, D = 512, 512, 64
    q, k, v = oracle.normal((Bn, S, D)), oracle.normal((Bn, S, D)), oracle.normal((Bn, S, D))
    dq, dk, dv = hip.array(q), hip.array(k), hip.array(v)
    ds = hip.sgemm_batched(dq, dk, transb=True)
    do = hip.sgemm_batched(ds, dv)
    s, o = ds.numpy(), do.numpy()
    for h in (0, 1, 255, 511):
        s_ref = oracle.gemm_opt_nt(q[h], k[h])
        assert np.abs(s[h] - s_ref).max() <= REL_FP32 * np.abs(s_ref).max()
        o_ref = oracle.gemm_opt(s[h], v[h])
        assert np.abs(o[h] - o_ref).max() <= REL_FP32 * np.abs(o_ref).max()
    # every head: row sums of S equal Q . (sum of K rows), to fp32 accumulation accuracy
    ksum = k.astype(np.float64).sum(axis=1)
    want = np.einsum("hsd,hd->hs", q.astype(np.float64), ksum)
    got = s.astype(np.float64).sum(axis=2)
    scale = np.einsum("hsd,hd->hs", np.abs(q).astype(np.float64), np.abs(k).astype(np.float64).sum(axis=1))
    assert (np.abs(got - want) <= 1e-5 * scale).all()


@pytest.mark.parametrize("walk", [0, 1, 2])
@pytest.mark.parametrize("Bn,M,N,K,alpha", [(600, 128, 256, 64, 1.0), (300, 256, 320, 32, 0.5), (130, 512, 512, 96, 0.125),
                                             (520, 128, 448, 128, 1.0), (1, 65536, 256, 64, 2.0), (513, 128, 256, 64, 1.0),
                                             (260, 160, 512, 128, 0.5), (300, 224, 512, 32, 1.0), (70, 1024, 2048, 96, 1.0), (512, 96 + 64, 512, 64, 1.0), (130, 256, 2048, 64, 0.25)])
def test_short_k_nt_row_blocks(hip, oracle, monkeypatch, Bn, M, N, K, alpha, walk):
    """A B^T with K of 32..128 and many output rows.  Walk 1: the kernel that keeps a 128-row block of A in
    LDS and walks the column blocks of B^T; walk 2: the one that keeps 256 rows of B in registers and walks
    A in blocks of 32 rows (taken when N is a multiple of 256, M of 32, and the workgroups fill the chip);
    walk 0: the library's own choice.
    Against the fp64 bound and, on sampled batch entries, the CPU path."""
    say("short-k nt", Bn, M, N, K, alpha, "walk", walk)
    oracle.seed(Bn + M + N + K)
    a, b = oracle.normal((Bn, M, K)), oracle.normal((Bn, N, K))
    da, db = hip.array(a), hip.array(b)
    c = hip.empty((Bn, M, N))
    hip.check(hip.L.axhip_memset(c.ptr, 0xFF, c.nbytes))                 # every output must be written
    if walk:
        monkeypatch.setenv("AX_HIP_NT_WALK", str(walk))
    assert hip.L.axhip_tuning_reload() == (1 if walk else 0)
    try:
        hip.check(hip.L.axhip_sgemm_strided_batched(0, 1, M, N, K, alpha, da.ptr, K, M * K, db.ptr, K, N * K, 0.0,
                                                    c.ptr, N, M * N, Bn))
        cols_route = walk != 1 and N % 256 == 0 and M % 32 == 0 and M >= (128 if walk == 2 else 256) and (N // 256) * Bn >= 512
        rows_route = M % 128 == 0 and N % 64 == 0 and N >= 256 and (M // 128) * Bn >= 512
        if cols_route:
            assert hip.last_kernel() == "sgemm_nt_cols256_dma"
        elif rows_route:
            assert hip.last_kernel() == "sgemm_nt_rows128_dma"
    finally:
        monkeypatch.delenv("AX_HIP_NT_WALK", raising=False)
        assert hip.L.axhip_tuning_reload() == 0
    got = c.numpy()
    assert not np.isnan(got).any()
    for h in sorted({0, Bn // 2, Bn - 1}):
        rows = slice(0, min(M, 1024))
        want = oracle.gemm_opt_nt(a[h][rows], b[h]) * np.float32(alpha)
        assert np.abs(got[h][rows] - want).max() <= REL_FP32 * np.abs(want).max()
    # every entry: row sums of C equal alpha * A . (sum of B's rows), to fp32 accumulation accuracy
    bsum = b.astype(np.float64).sum(axis=1)
    want = alpha * np.einsum("hmk,hk->hm", a.astype(np.float64), bsum)
    scale = abs(alpha) * np.einsum("hmk,hk->hm", np.abs(a).astype(np.float64), np.abs(b).astype(np.float64).sum(axis=1))
    assert (np.abs(got.astype(np.float64).sum(axis=2) - want) <= 1e-5 * scale).all()


@pytest.mark.parametrize("walk", [1, 2])
@pytest.mark.parametrize("Bn,M,N,K,alpha,pad", [(520, 256, 256, 64, 0.5, 4), (260, 384, 512, 96, 1.0, 8), (600, 128, 256, 32, 2.0, 12)])
def test_short_k_nt_padded_leading_dimensions(hip, oracle, monkeypatch, Bn, M, N, K, alpha, pad, walk):
    """The two short-K A B^T walks on operands and a result whose rows are `pad` floats longer than the
    matrices: pad columns are neither read into the sums nor written."""
    say("short-k nt padded", Bn, M, N, K, alpha, pad, "walk", walk)
    oracle.seed(3 * Bn + M + N + K)
    lda, ldb, ldc = K + pad, K + pad, N + pad
    a_full, b_full = oracle.normal((Bn, M, lda)), oracle.normal((Bn, N, ldb))
    a_full[:, :, K:] = np.float32(1e30)           # would wreck every sum it got into
    b_full[:, :, K:] = np.float32(-1e30)
    a, b = a_full[:, :, :K], b_full[:, :, :K]
    da, db = hip.array(a_full), hip.array(b_full)
    c = hip.empty((Bn, M, ldc))
    hip.check(hip.L.axhip_memset(c.ptr, 0xFF, c.nbytes))
    monkeypatch.setenv("AX_HIP_NT_WALK", str(walk))
    assert hip.L.axhip_tuning_reload() == 1
    try:
        hip.check(hip.L.axhip_sgemm_strided_batched(0, 1, M, N, K, alpha, da.ptr, lda, M * lda, db.ptr, ldb, N * ldb, 0.0,
                                                    c.ptr, ldc, M * ldc, Bn))
        assert hip.last_kernel() == ("sgemm_nt_cols256_dma" if walk == 2 else "sgemm_nt_rows128_dma")
    finally:
        monkeypatch.delenv("AX_HIP_NT_WALK", raising=False)
        assert hip.L.axhip_tuning_reload() == 0
    full = c.numpy()
    got = full[:, :, :N]
    assert not np.isnan(got).any() and np.isnan(full[:, :, N:]).all()
    for h in sorted({0, Bn // 2, Bn - 1}):
        want = oracle.gemm_opt_nt(np.ascontiguousarray(a[h]), np.ascontiguousarray(b[h])) * np.float32(alpha)
        assert np.abs(got[h] - want).max() <= REL_FP32 * np.abs(want).max()
    bsum = b.astype(np.float64).sum(axis=1)
    want = alpha * np.einsum("hmk,hk->hm", a.astype(np.float64), bsum)
    scale = abs(alpha) * np.einsum("hmk,hk->hm", np.abs(a).astype(np.float64), np.abs(b).astype(np.float64).sum(axis=1))
    assert (np.abs(got.astype(np.float64).sum(axis=2) - want) <= 1e-5 * scale).all()


@pytest.mark.parametrize("Bn,M,N,K,alpha,pad", [(200, 512, 64, 128, 1.0, 0), (67, 256, 384, 160, 0.5, 0), (280, 384, 64, 512, 1.0, 0),
                                                 (72, 512, 128, 1024, 0.25, 0), (264, 256, 64, 224, 2.0, 8), (9, 4096, 256, 192, 1.0, 4)])
def test_streamed_nn_tiles(hip, oracle, Bn, M, N, K, alpha, pad):
    """Batched A B with K of a few hundred and many 128 x 64 output tiles: the kernel whose workgroups walk
    a list of tiles with the K slabs of all of them in one stream; against the CPU path on sampled batch
    entries and, for every entry, a row-sum identity.  `pad`: extra floats in every leading dimension."""
    say("streamed nn", Bn, M, N, K, alpha, pad)
    oracle.seed(Bn + M + N + K)
    lda, ldb, ldc = K + pad, N + pad, N + pad
    a_full, b_full = oracle.normal((Bn, M, lda)), oracle.normal((Bn, K, ldb))
    a, b = a_full[:, :, :K], b_full[:, :, :N]
    da, db = hip.array(a_full), hip.array(b_full)
    c = hip.empty((Bn, M, ldc))
    hip.check(hip.L.axhip_memset(c.ptr, 0xFF, c.nbytes))                 # every output must be written, no pad column
    hip.check(hip.L.axhip_sgemm_strided_batched(0, 0, M, N, K, alpha, da.ptr, lda, M * lda, db.ptr, ldb, K * ldb, 0.0,
                                                c.ptr, ldc, M * ldc, Bn))
    assert hip.last_kernel() == "sgemm_nn_stream128x64_dma"
    full = c.numpy()
    got = full[:, :, :N]
    assert not np.isnan(got).any()
    if pad:
        assert np.isnan(full[:, :, N:]).all()
    for h in sorted({0, 7, Bn // 2, Bn - 1}):
        rows = slice(max(0, M - 1024), M)
        want = oracle.gemm_opt(np.ascontiguousarray(a[h][rows]), np.ascontiguousarray(b[h])) * np.float32(alpha)
        assert np.abs(got[h][rows] - want).max() <= REL_FP32 * np.abs(want).max()
    # every entry: row sums of C equal alpha * A . (row sums of B), to fp32 accumulation accuracy
    bsum = b.astype(np.float64).sum(axis=2)
    want = alpha * np.einsum("hmk,hk->hm", a.astype(np.float64), bsum)
    scale = abs(alpha) * np.einsum("hmk,hk->hm", np.abs(a).astype(np.float64), np.abs(b).astype(np.float64).sum(axis=2))
    assert (np.abs(got.astype(np.float64).sum(axis=2) - want) <= 1e-5 * scale).all()
    # and the same product on the one-tile-per-workgroup kernels
    os.environ["AX_HIP_F32_TILE"] = "642"
    try:
        hip.L.axhip_tuning_reload()
        c2 = hip.empty((Bn, M, ldc))
        hip.check(hip.L.axhip_sgemm_strided_batched(0, 0, M, N, K, alpha, da.ptr, lda, M * lda, db.ptr, ldb, K * ldb, 0.0,
                                                    c2.ptr, ldc, M * ldc, Bn))
        assert hip.last_kernel() != "sgemm_nn_stream128x64_dma"
        other = c2.numpy()[:, :, :N]
    finally:
        del os.environ["AX_HIP_F32_TILE"]
        hip.L.axhip_tuning_reload()
    assert np.abs(got - other).max() <= REL_FP32 * np.abs(other).max()


@pytest.mark.parametrize("M,N,K,splits", [(128, 4096, 2048, 0), (64, 2048, 2048, 0), (256, 1024, 2048, 4), (96, 1024, 4096, 16), (100, 1000, 2048, 2)])
def test_split_k_with_epilogue(hip, oracle, monkeypatch, M, N, K, splits):
    """A product whose K is split over workgroups (by the library's own rule, or a forced count), with alpha, beta, bias
    and an activation applied where the ranges meet, for fp32 operands (NN, NT, TN) and int8 weights: inside the fp64 bound."""
    say("split-k with epilogue", M, N, K, splits)
    oracle.seed(M + N + K)
    a, b = oracle.uniform((M, K), -1, 1), oracle.uniform((K, N), -1, 1)
    c0, bias = oracle.uniform((M, N), -1, 1), oracle.normal((N,), 0.0, 0.5)
    da, db, dat, dbt, dbias = hip.array(a), hip.array(b), hip.array(np.ascontiguousarray(a.T)), hip.array(np.ascontiguousarray(b.T)), hip.array(bias)
    w8 = np.random.default_rng(K).integers(-127, 128, (N, K), dtype=np.int8)
    ws = np.random.default_rng(N).uniform(1e-3, 1e-2, N).astype(np.float32)
    dw8, dws = hip.array(w8), hip.array(ws)
    alpha, beta = np.float32(0.5), np.float32(1.0)
    exact = alpha * (a.astype(np.float64) @ b.astype(np.float64)) + beta * c0 + bias
    want = np.maximum(exact, 0.0)
    bound = BOUND_FP32 * (abs(alpha) * (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)) + np.abs(c0) + np.abs(bias)) + 1e-30
    want8 = (a.astype(np.float64) @ w8.astype(np.float64).T) * ws
    bound8 = BOUND_FP32 * (np.abs(a).astype(np.float64) @ np.abs(w8).astype(np.float64).T) * ws + 1e-30
    try:
        if splits:
            monkeypatch.setenv("AX_HIP_F32_SPLITK", str(splits))
        hip.L.axhip_tuning_reload()
        for name, (ta, tb, pa, lda, pb, ldb) in {"nn": (0, 0, da, K, db, N), "nt": (0, 1, da, K, dbt, K), "tn": (1, 0, dat, M, db, N)}.items():
            c = hip.array(c0)
            hip.check(hip.L.axhip_sgemm(ta, tb, M, N, K, alpha, pa.ptr, lda, pb.ptr, ldb, beta, c.ptr, N, dbias.ptr, 1))
            say("  ", name, hip.last_kernel())
            assert hip.last_kernel() == "sgemm_splitk"
            got = c.numpy()
            assert (np.abs(got - want) <= bound).all(), (name, float((np.abs(got - want) / bound).max()))
        got8 = hip.qgemm_w8a32(da, dw8, dws).numpy()
        say("  ", "w8a32", hip.last_kernel())
        assert (np.abs(got8 - want8) <= bound8).all(), float((np.abs(got8 - want8) / bound8).max())
    finally:
        monkeypatch.delenv("AX_HIP_F32_SPLITK", raising=False)
        assert hip.L.axhip_tuning_reload() == 0


# ------------------------------------------------------------------ W8A32
W8A32_SHAPES = [(1, 8, 8), (4, 16, 32), (8, 64, 128), (32, 128, 512), (16, 256, 1024), (3, 17, 45),
                (1, 768, 3072), (1, 3072, 768), (8, 768, 768), (32, 768, 768), (128, 4096, 1024),
                (64, 1024, 4096), (1, 4096, 4096), (5, 33, 100),
                (2, 130, 256), (6, 67, 1040), (7, 5, 2064),
                (128, 1024, 512), (1024, 512, 1024), (256, 768, 768), (64, 768, 768),   # one launch on 32x64 tiles / split
                (20, 1024, 512), (150, 260, 160), (96, 2048, 1024), (160, 3072, 768),   # 32x64 tiles, whole and with clamped edges
                # the weight-streaming form: several row groups on one staging, 1 / 2 / 4 rows per wave, several slices of K,
                # a last window that ends inside a 16-byte step, rows that run past N
                (1, 20000, 520), (2, 16400, 300), (3, 8200, 1031), (6, 4100, 8200), (5, 4099, 2050), (4, 9000, 4100),
                (6, 33, 10000), (1, 70, 20000),
                (6, 4100, 8192), (5, 8192, 2048), (6, 64, 2048),   # five or six rows with a long K: the tiles
                (128, 4096, 192), (96, 2048, 320), (128, 3072, 160),   # 32x64 tiles: two slabs per stage (three and five stages), one
                (32, 128, 517), (70, 260, 1031), (3, 64, 1037),   # rows at odd byte offsets
                # seven and eight rows against a short K: the weight-streaming form again (one and two weight rows per wave)
                (7, 1024, 1024), (8, 3072, 768), (7, 2048, 2048), (8, 8192, 1024), (8, 2050, 1000), (7, 100, 517), (8, 40, 1024),
                (8, 16384, 768), (7, 768, 3072)]   # ... and past its limits: the tiles


@pytest.mark.parametrize("M,N,K", W8A32_SHAPES)
def test_w8a32_against_oracle(hip, oracle, golden, M, N, K):
    say("w8a32", M, N, K)
    a = xorshift32_unit(M * K, 7).reshape(M, K) if M * K < 70000 else None
    if a is None:
        oracle.seed(M + N + K)
        a, w = oracle.uniform((M, K), -1, 1), oracle.uniform((N, K), -1, 1)
    else:
        w = xorshift32_unit(N * K, 13).reshape(N, K)
    q, s = oracle.quantize_rows(w)
    got = hip.qgemm_w8a32(hip.array(a), hip.array(q), hip.array(s)).numpy()
    say("  ", hip.last_kernel())
    if M in (7, 8):
        streams = (K <= 1024 and N * K <= 8 << 20) or (K <= 2048 and N <= 2048)
        assert (hip.last_kernel() == "qgemm_w8a32_gemv") == streams
    ref = oracle.qgemm_w8a32(a, q, s)
    key = f"w8a32_{M}x{N}x{K}_out"
    if key in golden.files:
        assert np.array_equal(ref, golden[key])
    # the reference's own gate (tests/test_quantize.c:107-111) ...
    diff = np.abs(got - ref)
    assert not ((diff > 1e-2) & (diff / np.maximum(np.abs(ref), 1e-30) > 1e-3)).any()
    # ... and ours: fp32 accumulation-order noise only
    assert diff.max() <= REL_FP32 * max(np.abs(ref).max(), 1e-30)


W8A32_TILE_FORMS = [(2048, 8192, 160, "qgemm_w8a32_mfma_128x256_dma"), (2048, 4096, 192, "qgemm_w8a32_mfma_128x128_dma"),
                    (1024, 4096, 224, "qgemm_w8a32_mfma_64x128k2_dma"), (512, 4096, 288, "qgemm_w8a32_mfma_32x128k2_dma"),
                    (256, 4096, 160, "qgemm_w8a32_mfma_32x64k2_dma"), (256, 4096, 256, "qgemm_w8a32_mfma_32x64k2_dma"),
                    (512, 4096, 1056, "qgemm_w8a32_mfma_32x128k2_dma"), (512, 4096, 192, "qgemm_w8a32_mfma_32x128k2_dma"),
                    (256, 4096, 224, "qgemm_w8a32_mfma_32x64k2_dma"),
                    # off the tile grid: clamped fetches and a guarded write-back
                    (4000, 4000, 160, "qgemm_w8a32_mfma_128x256_dma_edge"), (2000, 4000, 192, "qgemm_w8a32_mfma_128x128_dma_edge"),
                    (1000, 4100, 224, "qgemm_w8a32_mfma_64x128k2_dma_edge"), (520, 4096, 288, "qgemm_w8a32_mfma_32x128k2_dma_edge"),
                    (220, 4100, 160, "qgemm_w8a32_mfma_32x64k2_dma_edge")]


@pytest.mark.parametrize("M,N,K,form", W8A32_TILE_FORMS)
def test_w8a32_tile_forms(hip, M, N, K, form):
    """The tile forms of the W8A32 product for many output tiles (fp32 activations cut into three bf16 terms, int8 weights
    as bf16, products on the bf16 matrix core): each obeys the fp64 bound of a correct fp32 accumulation, with slab counts
    that end the four-stage ring at every position."""
    say("w8a32 tiles", M, N, K)
    rng = np.random.default_rng(M + N + K)
    a = (rng.uniform(-1, 1, (M, K)) * 10.0 ** rng.integers(-3, 4, (M, 1))).astype(np.float32)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    ws = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    dout = hip.array(np.full((M + 1, N), np.nan, np.float32))          # a row past the output: never written
    da, dw, ds = hip.array(a), hip.array(w), hip.array(ws)
    hip.check(hip.L.axhip_qgemm_w8a32(da.ptr, dw.ptr, ds.ptr, dout.ptr, M, N, K))
    assert hip.last_kernel() == form
    full = dout.numpy()
    got = full[:M]
    assert np.isnan(full[M]).all()
    want = (a.astype(np.float64) @ w.astype(np.float64).T) * ws
    bound = BOUND_FP32 * (np.abs(a).astype(np.float64) @ np.abs(w).astype(np.float64).T) * ws + 1e-30
    assert (np.abs(got - want) <= bound).all(), float((np.abs(got - want) / bound).max())


def test_w8a32_three_bf16_terms_are_exact(hip, oracle):
    """Activations whose 24 significant bits are all in use, against weight rows with one non-zero: every output is a
    single product.  With a power of two as the weight the product is exact, so any bit the three-term split lost would
    show; with 3 or 127 the three exact partial products are rounded as they are added, within one unit in the last place."""
    M, N, K = 64, 128, 256
    rng = np.random.default_rng(5)
    a = rng.uniform(1, 2, (M, K)).astype(np.float32)
    a = np.nextafter(a, np.float32(3)) * rng.choice([-1, 1], (M, K)).astype(np.float32) * (2.0 ** rng.integers(-60, 60, (M, K))).astype(np.float32)
    w = np.zeros((N, K), np.int8)
    cols = rng.integers(0, K, N)
    vals = rng.choice([1, -1, 2, -64, 127, -128, 3], N)
    w[np.arange(N), cols] = vals
    s = np.ones(N, np.float32)
    got = hip.qgemm_w8a32(hip.array(a), hip.array(w), hip.array(s)).numpy()
    say("  ", hip.last_kernel())
    assert hip.last_kernel().startswith("qgemm_w8a32_mfma")
    want = a[:, cols].astype(np.float64) * vals
    pow2 = np.isin(vals, [1, -1, 2, -64, -128])
    assert np.array_equal(got[:, pow2].astype(np.float64), want[:, pow2])
    assert (np.abs(got - want) <= np.abs(want) * 2.0 ** -23).all()


@pytest.mark.parametrize("M,N,K", [(2, 10300, 4100), (1, 11008, 4096), (5, 10500, 4004), (4, 2000, 21000)])
def test_w8a32_streaming_loads(hip, M, N, K):
    """40 MiB of weights and more: the weight-streaming forms read them with non-temporal loads (rows at 4-byte alignment
    among them).  Same arithmetic, so the same fp64 bound as every other form."""
    say("w8a32 streaming", M, N, K)
    rng = np.random.default_rng(M * N + K)
    a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    ws = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    got = hip.qgemm_w8a32(hip.array(a), hip.array(w), hip.array(ws)).numpy()
    assert hip.last_kernel() == "qgemm_w8a32_gemv"
    want = (a.astype(np.float64) @ w.astype(np.float64).T) * ws
    bound = BOUND_FP32 * (np.abs(a).astype(np.float64) @ np.abs(w).astype(np.float64).T) * ws + 1e-30
    assert (np.abs(got - want) <= bound).all(), float((np.abs(got - want) / bound).max())


def test_w8a32_tiny_activations(hip):
    """The bf16 matrix core flushes denormal operands, so the low-order bf16 terms of activations below 2^-110 are
    dropped: the result stays within the fp32 bound plus K * 2^-118 per output, whatever the scale of the activations."""
    M, N, K = 64, 256, 512
    rng = np.random.default_rng(3)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    s = np.ones(N, np.float32)
    for scale in (1e-30, 1e-34, 1e-36, 1e-38, 1e-41):
        a = (rng.uniform(-1, 1, (M, K)) * scale).astype(np.float32)
        got = hip.qgemm_w8a32(hip.array(a), hip.array(w), hip.array(s)).numpy().astype(np.float64)
        assert hip.last_kernel().startswith("qgemm_w8a32_mfma")
        want = a.astype(np.float64) @ w.astype(np.float64).T
        bound = BOUND_FP32 * (np.abs(a).astype(np.float64) @ np.abs(w).astype(np.float64).T) + K * 2.0 ** -118
        assert (np.abs(got - want) <= bound).all(), (scale, float((np.abs(got - want) / bound).max()))


def test_w8a32_non_finite_activations(hip, oracle):
    """Infinities and NaNs among the activations come out as the reference's fp32 sum gives them (src/core/quantize.c:117-170, a plain fused multiply-add chain):
    +-inf where one sign of infinity meets non-zero weights, NaN where both signs meet, an infinity meets a zero weight,
    or a NaN is present; rows without them stay finite."""
    M, N, K = 40, 192, 320
    rng = np.random.default_rng(11)
    a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    w[:, 7] = np.where(np.arange(N) % 3 == 0, 0, w[:, 7])           # zero weights under an infinity
    a[1, 7] = np.inf
    a[2, 7], a[2, 100] = np.inf, -np.inf
    a[3, 200] = np.nan
    a[4, 7] = -np.inf
    a[5, 300] = np.float32(3.0e38)                                    # finite, overflows in the product
    a[6, 50] = np.array([0x7f800001], np.uint32).view(np.float32)[0]  # a NaN whose payload lies in the low 16 bits only
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    for rows in (M, 6):                                               # matrix-core form, weight-streaming form
        x = a[1:1 + rows] if rows == 6 else a
        got = hip.qgemm_w8a32(hip.array(x), hip.array(w), hip.array(s)).numpy()
        say("  ", hip.last_kernel())
        with np.errstate(all="ignore"):
            ref = oracle.qgemm_w8a32(x, w, s)
        assert np.array_equal(np.isnan(got), np.isnan(ref))
        assert np.array_equal(np.isinf(got), np.isinf(ref))
        inf = np.isinf(ref)
        assert np.array_equal(np.sign(got[inf]), np.sign(ref[inf]))
        fin = np.isfinite(ref)
        assert np.abs(got[fin] - ref[fin]).max() <= REL_FP32 * np.abs(ref[fin]).max()


def test_device_quantizer_bit_exact(hip, oracle, golden):
    for (N, K) in ((8, 8), (128, 128), (64, 1024), (5, 333)):
        w = xorshift32_unit(N * K, 42).reshape(N, K)
        dq, ds = hip.quantize_rows(hip.array(w))
        q, s = oracle.quantize_rows(w)
        assert np.array_equal(dq.numpy(), q) and np.array_equal(ds.numpy(), s)
    dq, ds = hip.quantize_rows(hip.array(golden["quant_ties_w"]))
    assert np.array_equal(dq.numpy(), golden["quant_ties_q"])
    dq, ds = hip.quantize_rows(hip.array(golden["quant_hand_w"]))
    assert np.array_equal(dq.numpy(), golden["quant_hand_q"]) and np.array_equal(ds.numpy(), golden["quant_hand_s"])


# ------------------------------------------------------------------ elementwise + errors
def test_elementwise_slots(hip, oracle, golden):
    oracle.seed(8)
    x = oracle.normal((37, 1001), 0, 2)
    dx = hip.array(x)
    out = hip.empty(x.shape)
    hip.check(hip.L.axhip_relu(dx.ptr, out.ptr, x.size))
    assert np.array_equal(out.numpy(), np.maximum(x, 0))
    hip.check(hip.L.axhip_gelu(dx.ptr, out.ptr, x.size))
    assert np.abs(out.numpy() - oracle.gelu(x)).max() <= 1e-6
    g = hip.array(golden["gelu_x"])
    go = hip.empty(g.shape)
    hip.check(hip.L.axhip_gelu(g.ptr, go.ptr, g.shape[0]))
    assert np.abs(go.numpy() - golden["gelu_y"]).max() <= 2e-6          # the reference's ax_gelu
    hip.check(hip.L.axhip_fill_f32(out.ptr, 2.5, x.size))
    assert (out.numpy() == 2.5).all()
    bias = oracle.normal((1001,), 0, 1)
    dbias = hip.array(bias)
    hip.check(hip.L.axhip_bias_add(dx.ptr, dbias.ptr, 37, 1001, 1, out.ptr))
    assert np.array_equal(out.numpy(), x + bias[None, :])
    rb = oracle.normal((37,), 0, 1)
    drb = hip.array(rb)
    hip.check(hip.L.axhip_bias_add(dx.ptr, drb.ptr, 1, 37, 1001, out.ptr))
    assert np.array_equal(out.numpy(), x + rb[:, None])
    z = hip.empty((1000,))                                               # zero-filled allocation
    assert not z.numpy().any()


def test_elementwise_in_place(hip, oracle):
    """Calls whose output is their input (the host core does this for fused activations, residual bias adds and
    the mean's final scale): same values as the out-of-place call."""
    oracle.seed(81)
    x = oracle.normal((513, 1027), 0, 2)            # odd row length: vector and element paths
    n = x.size
    bias = oracle.normal((1027,), 0, 1)
    dbias = hip.array(bias)

    def both(call):
        src, dst = hip.array(x), hip.empty(x.shape)
        call(src.ptr, dst.ptr)
        want = dst.numpy()
        call(src.ptr, src.ptr)
        assert np.array_equal(src.numpy(), want, equal_nan=True)

    both(lambda i, o: hip.check(hip.L.axhip_relu(i, o, n)))
    both(lambda i, o: hip.check(hip.L.axhip_gelu(i, o, n)))
    both(lambda i, o: hip.check(hip.L.axhip_unary(7, i, o, n, 0.0)))                  # tanh
    both(lambda i, o: hip.check(hip.L.axhip_unary(12, i, o, n, 0.25)))                # mul_scalar
    both(lambda i, o: hip.check(hip.L.axhip_bias_add(i, dbias.ptr, 513, 1027, 1, o)))
    both(lambda i, o: hip.check(hip.L.axhip_softmax_rows(i, o, 513, 1027)))
    import ctypes as C
    shape, dense = (C.c_int64 * 2)(513, 1027), (C.c_int64 * 2)(1027, 1)
    other = hip.array(oracle.normal((513, 1027), 0, 1))
    both(lambda i, o: hip.check(hip.L.axhip_binary(0, i, other.ptr, o, 2, shape, dense, dense)))


# ------------------------------------------------------------------ dense backward blocks
SUM_BOUND = 1e-5     # |gpu - sum64| <= SUM_BOUND * sum |x|   (fp32 sums in a fixed parallel order)


@pytest.mark.parametrize("shape,axis", [((37, 19), 0), ((37, 19), 1), ((4, 9, 10), 0), ((4, 9, 10), 1),
                                        ((4, 9, 10), 2), ((2048, 4096), 0), ((2048, 4096), 1),
                                        ((1000, 7), 0), ((3, 100003), 1), ((1, 64), 0), ((5000, 64), 0),
                                        ((16384, 772), 0), ((20000, 1000), 0), ((3000, 2044), 0), ((3000, 2052), 0),
                                        ((100003, 10), 1), ((70001, 33), 1), ((50001, 127), 1), ((1001, 3), 1)])
def test_sum_axis(hip, oracle, golden, shape, axis):
    say("sum", shape, axis)
    oracle.seed(4343 if shape in ((37, 19), (4, 9, 10)) else sum(shape) + axis)
    if shape == (4, 9, 10):
        oracle.uniform((37, 19), -1, 1)        # the golden vectors draw the 2-D case first
    x = oracle.uniform(shape, -1, 1)
    outer, inner = int(np.prod(shape[:axis])), int(np.prod(shape[axis + 1:]))
    out = hip.empty(shape[:axis] + shape[axis + 1:] or (1,))
    dx = hip.array(x)
    hip.check(hip.L.axhip_sum_axis(dx.ptr, outer, shape[axis], inner, out.ptr))
    got = out.numpy().reshape(shape[:axis] + shape[axis + 1:])
    s64, sabs = oracle.sum_axis_f64(x, axis)
    assert (np.abs(got - s64) <= SUM_BOUND * sabs + 1e-30).all()
    if axis == 0:
        ref = oracle.sum_axis0(x)              # the reference's own order, row by row
        assert np.abs(got - ref).max() <= SUM_BOUND * sabs.max()
    name = {(37, 19): "sum2d", (4, 9, 10): "sum3d"}.get(shape)
    if name:
        assert np.abs(got - golden[f"{name}_axis{axis}"]).max() <= SUM_BOUND * sabs.max()
    # run-to-run determinism
    hip.check(hip.L.axhip_sum_axis(dx.ptr, outer, shape[axis], inner, out.ptr))
    assert np.array_equal(out.numpy().reshape(got.shape), got)


@pytest.mark.parametrize("n", [1, 63, 4096, 4097, 1000003, 1 << 24])
def test_sum_all_and_axpy(hip, oracle, n):
    oracle.seed(n)
    x = oracle.uniform((n,), -1, 1)
    out = hip.empty((1,))
    dx = hip.array(x)
    hip.check(hip.L.axhip_sum_all(dx.ptr, n, out.ptr))
    exact = x.astype(np.float64).sum()
    assert abs(float(out.numpy()[0]) - exact) <= SUM_BOUND * np.abs(x).astype(np.float64).sum()
    y = oracle.uniform((n,), -1, 1)
    dy = hip.array(y)
    hip.check(hip.L.axhip_axpy(dx.ptr, 0.37, dy.ptr, n))
    assert np.array_equal(dy.numpy(), oracle.axpy(x, 0.37, y))        # one fused multiply-add: bit-exact


@pytest.mark.parametrize("M,K,N", [(48, 40, 24), (130, 70, 50), (2048, 1024, 4096)])
def test_dense_backward_blocks(hip, oracle, golden, M, K, N):
    """The three products of the dense layer's backward pass (src/core/autograd_ops.c:603-757)
    through the C ABI: dA = dY W^T (NT), dW = X^T dY (TN), dBias = sum(dY, 0); then the
    accumulate-into-an-existing-gradient forms (temp + axpy, and beta = 1)."""
    say("dense backward", M, K, N)
    oracle.seed(4242 if (M, K, N) == (48, 40, 24) else M + K + N)
    x, w, dy = oracle.uniform((M, K), -1, 1), oracle.uniform((K, N), -1, 1), oracle.uniform((M, N), -1, 1)
    dx_, dw_, ddy = hip.array(x), hip.array(w), hip.array(dy)
    dA = hip.sgemm(ddy, dw_, transb=True).numpy()                     # [M,N] x [K,N]^T -> [M,K]
    say("  dA", hip.last_kernel())
    check_fp32(oracle, dA, dy, w, transb=True, ref=oracle.gemm_opt_nt(dy, w))
    dW = hip.sgemm(dx_, ddy, transa=True).numpy()                     # [M,K]^T x [M,N] -> [K,N]
    say("  dW", hip.last_kernel())
    xt = np.ascontiguousarray(x.T)
    check_fp32(oracle, dW, xt, dy, ref=oracle.gemm_opt(xt, dy))
    db = hip.empty((N,))
    hip.check(hip.L.axhip_sum_axis(ddy.ptr, 1, M, N, db.ptr))
    s64, sabs = oracle.sum_axis_f64(dy, 0)
    assert (np.abs(db.numpy() - s64) <= SUM_BOUND * sabs).all()
    if (M, K, N) == (48, 40, 24):
        for got, key in ((dA, "dense_bwd_dA"), (dW, "dense_bwd_dW"), (db.numpy(), "dense_bwd_db")):
            assert np.abs(got - golden[key]).max() <= REL_FP32 * np.abs(golden[key]).max()
    # gradient that already exists: temp + axpy (what the reference does) == gemm with beta = 1
    g0 = oracle.uniform((K, N), -1, 1)
    acc1 = hip.array(g0)
    ddw = hip.array(dW)
    hip.check(hip.L.axhip_axpy(ddw.ptr, 1.0, acc1.ptr, K * N))
    assert np.array_equal(acc1.numpy(), g0 + dW)
    acc2 = hip.sgemm(dx_, ddy, transa=True, beta=1.0, c=hip.array(g0)).numpy()
    assert np.abs(acc2 - (g0 + dW)).max() <= 1e-6 * max(1.0, np.abs(dW).max())


# ------------------------------------------------------------------ attention forward
SDPA_TOL = 1e-5      # max |gpu - fp64 ground truth| on O (entries are convex combinations of V in [-0.5, 0.5))


def run_sdpa(hip, q, k, v, scale, causal, want_l=True):
    BH, S, dk = q.shape
    o = hip.empty((BH, S, dk))
    l = hip.empty((BH, S)) if want_l else None
    dq, dk_, dv = hip.array(q), hip.array(k), hip.array(v)      # named: they must outlive the call
    hip.check(hip.L.axhip_sdpa_fwd(dq.ptr, dk_.ptr, dv.ptr, o.ptr,
                                   l.ptr if l is not None else None, BH, S, dk, scale, int(causal)))
    return o.numpy(), (l.numpy() if l is not None else None)


@pytest.mark.parametrize("BH,S,dk,causal", [(6, 24, 16, 0), (2, 16, 8, 1), (3, 128, 64, 0), (3, 128, 64, 1),
                                            (2, 40, 32, 1), (5, 256, 64, 0), (5, 256, 64, 1), (2, 1, 64, 0),
                                            (1, 129, 64, 1), (3, 384, 64, 1), (2, 77, 128, 0), (4, 512, 64, 0),
                                            (3, 128, 32, 0), (2, 256, 32, 1), (3, 128, 128, 0), (2, 256, 128, 1),
                                            (2, 384, 128, 0), (11, 640, 64, 1), (19, 256, 32, 0), (9, 512, 128, 1),
                                            (17, 128, 64, 1), (3, 200, 64, 0), (2, 1000, 64, 1), (5, 63, 32, 0),
                                            (2, 191, 128, 1), (9, 65, 64, 0), (2, 64, 64, 1), (3, 127, 32, 1),
                                            (1, 897, 128, 0),
                                            # head sizes between the kernels' own (lanes past the row end load nothing)
                                            (3, 256, 96, 0), (2, 200, 80, 1), (5, 128, 40, 0), (2, 333, 100, 1),
                                            (3, 64, 4, 0), (2, 129, 124, 1), (4, 512, 48, 0), (2, 77, 20, 1),
                                            # and ones no fused kernel takes: batched GEMMs and a row softmax
                                            (2, 64, 6, 0), (2, 100, 256, 1), (3, 50, 130, 0)])
def test_sdpa_forward(hip, oracle, golden, BH, S, dk, causal):
    say("sdpa", BH, S, dk, causal)
    oracle.seed(5000 + BH * 100 + S + dk + causal)
    q, k, v = (oracle.uniform((BH, S, dk), -0.5, 0.5) for _ in range(3))
    scale = float(np.float32(1.0) / np.sqrt(np.float32(dk)))
    o, l = run_sdpa(hip, q, k, v, scale, causal)
    say("  kernel", hip.last_kernel())
    o64, l64 = oracle.sdpa(q, k, v, scale, causal, f64=True)
    assert np.abs(o - o64).max() <= SDPA_TOL, np.abs(o - o64).max()
    assert np.abs(l - l64).max() <= 1e-5 * max(1.0, np.abs(l64).max())
    o32, _ = oracle.sdpa(q, k, v, scale, causal)
    assert np.abs(o - o32).max() < 1e-4                                   # the reference test's own gate
    key = f"sdpa_{BH}x{S}x{dk}_c{causal}_O"
    if key in golden:
        assert np.abs(o - golden[key]).max() < 1e-4
        assert np.abs(l - golden[key[:-1] + "L"]).max() < 1e-4
    o2, none = run_sdpa(hip, q, k, v, scale, causal, want_l=False)        # L = NULL, and determinism
    assert none is None and np.array_equal(o2, o)


@pytest.mark.parametrize("B,H,S,dk,causal,pad_in,pad_out", [(2, 4, 128, 64, 0, 0, 0), (2, 4, 128, 64, 1, 0, 0),
                                                            (3, 2, 77, 32, 1, 8, 4), (1, 3, 200, 128, 0, 4, 12),
                                                            (2, 5, 256, 32, 0, 0, 8), (1, 2, 1, 64, 0, 0, 0),
                                                            (9, 4, 128, 64, 0, 0, 0), (2, 3, 321, 64, 1, 16, 0),
                                                            (2, 3, 200, 96, 0, 0, 0), (1, 5, 130, 40, 1, 4, 8),
                                                            (3, 2, 64, 12, 0, 0, 4)])
def test_sdpa_on_the_fused_projection_layout(hip, oracle, B, H, S, dk, causal, pad_in, pad_out):
    """Heads side by side in the rows of qkv [B*S, 3D (+ padding)]: the same numbers as the same
    heads handed over one matrix each, bit for bit, written into [B*S, D (+ padding)] with the
    padding columns untouched."""
    say("sdpa rows", B, H, S, dk, causal, pad_in, pad_out)
    D = H * dk
    ld, ldo = 3 * D + pad_in, D + pad_out
    oracle.seed(9000 + B * 1000 + H * 100 + S + dk + causal)
    qkv = oracle.uniform((B * S, ld), -0.5, 0.5)
    scale = float(np.float32(1.0) / np.sqrt(np.float32(dk)))
    heads = lambda third: np.ascontiguousarray(                       # noqa: E731  [B*H, S, dk]
        qkv[:, third * D:(third + 1) * D].reshape(B, S, H, dk).transpose(0, 2, 1, 3).reshape(B * H, S, dk))
    q, k, v = heads(0), heads(1), heads(2)
    want_o, want_l = run_sdpa(hip, q, k, v, scale, causal)
    o64, _ = oracle.sdpa(q, k, v, scale, causal, f64=True)
    assert np.abs(want_o - o64).max() <= SDPA_TOL
    dqkv = hip.array(qkv)
    out = hip.array(np.full((B * S, ldo), 7.0, np.float32))
    l = hip.empty((B * H, S))
    base = dqkv.ptr
    hip.check(hip.L.axhip_sdpa_fwd_rows(base, base + 4 * D, base + 8 * D, ld, out.ptr, ldo, l.ptr, B, H, S, dk,
                                        scale, int(causal)))
    got = out.numpy()
    assert (got[:, D:] == 7.0).all()
    got_heads = got[:, :D].reshape(B, S, H, dk).transpose(0, 2, 1, 3).reshape(B * H, S, dk)
    assert np.array_equal(got_heads, want_o)
    assert np.array_equal(l.numpy(), want_l)
    # refusals: a head size without a fused kernel, a pitch shorter than the heads, a pitch off the 16-byte grid
    assert hip.L.axhip_sdpa_fwd_rows(base, base, base, ld, out.ptr, ldo, None, B, H, S, 50, scale, 0) == 10
    assert hip.L.axhip_sdpa_fwd_rows(base, base, base, D - 4, out.ptr, ldo, None, B, H, S, dk, scale, 0) == 3
    assert hip.L.axhip_sdpa_fwd_rows(base, base, base, ld + 2, out.ptr, ldo, None, B, H, S, dk, scale, 0) == 3


def test_sdpa_shape_sweep(hip, oracle):
    """60 seeded (heads, S, dk, causal) draws over sequence lengths around the 64- and 128-row blocks and
    every kind of head size (native, padded to the next kernel, unfused)."""
    rng = np.random.default_rng(20242)
    lengths = [1, 2, 31, 63, 64, 65, 100, 127, 128, 129, 191, 192, 193, 255, 256, 257, 300, 384, 500, 513]
    sizes = [4, 8, 12, 16, 28, 32, 36, 40, 48, 60, 64, 68, 72, 80, 96, 100, 124, 128, 6, 130]
    for case in range(60):
        BH, S, dk, causal = int(rng.integers(1, 12)), int(rng.choice(lengths)), int(rng.choice(sizes)), int(rng.integers(0, 2))
        say("sdpa sweep", case, BH, S, dk, causal)
        q, k, v = (rng.uniform(-0.5, 0.5, (BH, S, dk)).astype(np.float32) for _ in range(3))
        scale = float(np.float32(1.0) / np.sqrt(np.float32(dk)))
        o, l = run_sdpa(hip, q, k, v, scale, causal)
        o64, l64 = oracle.sdpa(q, k, v, scale, causal, f64=True)
        assert np.abs(o - o64).max() <= SDPA_TOL, (case, BH, S, dk, causal, hip.last_kernel(), float(np.abs(o - o64).max()))
        assert np.abs(l - l64).max() <= 1e-5 * max(1.0, np.abs(l64).max()), (case, BH, S, dk, causal)


def test_sdpa_large_scores_and_full_size(hip, oracle):
    """Scores far from zero (the running maximum must absorb them), and the attention shape of
    the benchmark (512 heads of [512, 64]) checked on sampled heads."""
    oracle.seed(77)
    q, k, v = (oracle.uniform((2, 256, 64), -1, 1) for _ in range(3))
    q *= 30.0
    o, l = run_sdpa(hip, q, k, v, 1.0, False)
    o64, l64 = oracle.sdpa(q, k, v, 1.0, False, f64=True)
    # |score| reaches ~300 here: one fp32 rounding of a score moves its exponential by 300 * 2^-24 = 2e-5 relative
    assert np.isfinite(o).all() and np.abs(o - o64).max() <= 1e-4
    assert np.abs(l - l64).max() <= 1e-5 * np.abs(l64).max()
    BH, S, dk = 512, 512, 64
    q, k, v = (oracle.normal((BH, S, dk), 0, 1) for _ in range(3))
    scale = 0.125
    for causal in (False, True):
        o, l = run_sdpa(hip, q, k, v, scale, causal)
        say("  full size", hip.last_kernel())
        assert hip.last_kernel().startswith("sdpa_fused_dk64")
        heads = [0, 1, 255, 511]
        o64, l64 = oracle.sdpa(q[heads], k[heads], v[heads], scale, causal, f64=True)
        assert np.abs(o[heads] - o64).max() <= 5e-5      # V ~ N(0,1): entries up to ~4
        assert np.abs(l[heads] - l64).max() <= 1e-5 * np.abs(l64).max()
        # each output row is a convex combination of value rows
        assert (o.max(axis=1) <= v.max(axis=1) + 1e-4).all() and (o.min(axis=1) >= v.min(axis=1) - 1e-4).all()


def test_error_paths(hip):
    L = hip.L
    a = hip.empty((8, 8))
    assert L.axhip_sgemm(0, 0, 8, 8, 8, 1.0, None, 8, a.ptr, 8, 0.0, a.ptr, 8, None, 0) == 1
    assert L.axhip_sgemm(0, 0, 8, 8, 8, 1.0, a.ptr, 4, a.ptr, 8, 0.0, a.ptr, 8, None, 0) == 3
    assert L.axhip_sgemm(1, 1, 8, 8, 8, 1.0, a.ptr, 8, a.ptr, 8, 0.0, a.ptr, 8, None, 0) == 10
    assert L.axhip_sgemm_skinny(17, 8, 8, a.ptr, 8, a.ptr, 8, a.ptr, 8, None, 0) == 3
    assert L.axhip_qgemm_w8a8(a.ptr, 1.0, a.ptr, None, None, 0, None, None, 8, 8, 8) == 1
    assert L.axhip_qgemm_w8a8(a.ptr, 1.0, a.ptr, None, None, 7, None, a.ptr, 8, 8, 8) == 3
    assert "activation" in hip.last_error()
    assert L.axhip_sgemm(0, 0, 0, 8, 8, 1.0, a.ptr, 8, a.ptr, 8, 0.0, a.ptr, 8, None, 0) == 0   # empty
    hip.sync()


def test_matrix_core_probes_run_and_check_arguments(hip):
    """The measurement probes are no compute path, but they are exported: each shape launches, all-zero
    operands give all-zero checksums (the sink is written by every lane), and bad arguments are refused."""
    L = hip.L
    zeros8, sink32 = hip.empty((128 * 1024,), np.int8), hip.empty((512 * 1024,), np.int32)
    zerosf, sinkf = hip.empty((32 * 1024,)), hip.empty((512 * 1024,))
    cus = 256
    for shape in (32, 16):
        for reads in (0, 6):
            say("probe int8", shape, reads)
            hip.check(L.axhip_memset(sink32.ptr, 0xFF, sink32.nbytes))
            hip.check(L.axhip_probe_int8_matrix_core(shape, reads, zeros8.ptr, sink32.ptr))
            assert hip.last_kernel().startswith("probe_i8_mfma")
            assert not sink32.numpy()[: cus * 512].any()
        for reads in (0, 3):
            say("probe fp32", shape, reads)
            hip.check(L.axhip_memset(sinkf.ptr, 0xFF, sinkf.nbytes))
            hip.check(L.axhip_probe_fp32_matrix_core(shape, reads, zerosf.ptr, sinkf.ptr))
            assert hip.last_kernel().startswith("probe_f32_mfma")
            assert not sinkf.numpy()[: cus * 512].any()
    assert L.axhip_probe_int8_matrix_core(8, 0, zeros8.ptr, sink32.ptr) == 3
    assert L.axhip_probe_int8_matrix_core(32, 7, zeros8.ptr, sink32.ptr) == 3
    assert L.axhip_probe_int8_matrix_core(32, 0, None, sink32.ptr) == 1
    assert L.axhip_probe_fp32_matrix_core(16, 4, zerosf.ptr, sinkf.ptr) == 3
    assert L.axhip_probe_fp32_matrix_core(16, 0, zerosf.ptr, None) == 1
    assert L.axhip_device_free_bytes() > 0
    hip.sync()


# ---------------------------------------------------------------- elementwise / reduction / optimizer slots
import ctypes as C  # noqa: E402

import slot_cases as sc  # noqa: E402
from oracle_bind import Oracle as _O  # noqa: E402


def bcast_strides(shape, out_shape):
    """Element strides of a contiguous operand per output dimension, 0 where it is broadcast:
    the mapping of cpu_naive.c:48-62 resolved on the host."""
    shape = (1,) * (len(out_shape) - len(shape)) + tuple(shape)
    strides, st = [], 1
    for n in reversed(shape):
        strides.append(st if n > 1 else 0)
        st *= n
    return list(reversed(strides))


def run_binary(hip, name, a, b):
    out_shape = np.broadcast_shapes(a.shape, b.shape)
    nd = len(out_shape)
    arr = lambda v: (C.c_int64 * max(nd, 1))(*v)
    da, db, out = hip.array(a), hip.array(b), hip.empty(out_shape)
    hip.check(hip.L.axhip_binary(_O.BINARY[name], da.ptr, db.ptr, out.ptr, nd, arr(out_shape),
                                 arr(bcast_strides(a.shape, out_shape)), arr(bcast_strides(b.shape, out_shape))))
    return out.numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("case", range(len(sc.BCAST)))
def test_binary_broadcast_golden(hip, oracle, golden, case):
    """Single IEEE operations: bit-exact with the reference vectors."""
    say("binary golden", case)
    a, b = sc.binary_inputs(oracle, case)
    for name in sc.BINARY:
        assert np.array_equal(run_binary(hip, name, a, b), golden[f"bin_{name}_{case}"], equal_nan=True), name
    if a.shape == b.shape:
        assert np.array_equal(run_binary(hip, "add_relu", a, b), golden[f"bin_add_relu_{case}"])


@pytest.mark.gpu
@pytest.mark.parametrize("sa,sb", [((1024, 4096), (4096,)), ((1024, 4096), (1024, 1)), ((64, 33, 17), (33, 1)),
                                   ((7, 1, 5, 1, 3), (2, 1, 4, 3)), ((1,), (3, 5)), ((2048, 2048), (2048, 2048)),
                                   ((3, 1000003), (1,)), ((5, 6), (5, 6))])
def test_binary_broadcast_shapes(hip, oracle, sa, sb):
    say("binary", sa, sb)
    oracle.seed(sum(sa) + 7 * sum(sb))
    a, b = oracle.uniform(sa, -2, 2), oracle.uniform(sb, 0.5, 2)
    with np.errstate(all="ignore"):
        want = {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b, "greater": (a > b).astype(np.float32)}
    for name, w in want.items():
        assert np.array_equal(run_binary(hip, name, a, b), w), name
    if np.prod(np.broadcast_shapes(sa, sb)) <= 4096:           # the element-by-element restatement is slow
        assert np.array_equal(run_binary(hip, "mul", a, b), oracle.binary("mul", a, b))


# exp/log/tanh come from the device math library, not the host's: a few ulp apart
# (relative for large results, absolute below 1, where elu's exp(v) - 1 cancels)
UNARY_TOL = {"exp": 4e-7, "log": 4e-7, "sigmoid": 4e-7, "tanh": 1e-6, "elu": 4e-7, "swish": 4e-7}


def run_unary(hip, name, x, param=0.0):
    dx, out = hip.array(x), hip.empty(x.shape)
    hip.check(hip.L.axhip_unary(_O.UNARY[name], dx.ptr, out.ptr, x.size, param))
    return out.numpy()


@pytest.mark.gpu
def test_unary_golden_and_large(hip, oracle, golden):
    say("unary")
    params = {"leaky_relu": 0.1, "elu": 0.7, "add_scalar": 0.37, "mul_scalar": -1.7}
    x = sc.unary_input(oracle)
    oracle.seed(99)
    big = oracle.uniform((1 << 20) + 3, -4, 4)
    for name in _O.UNARY:
        p = params.get(name, 0.0)
        got, ref = run_unary(hip, name, x, p), golden[f"un_{name}"]
        tol = UNARY_TOL.get(name)
        if tol is None:
            assert np.array_equal(got, ref, equal_nan=True), name
        else:
            assert (np.abs(got - ref) <= tol * np.maximum(np.abs(ref), 1)).all(), name
        got, ref = run_unary(hip, name, big, p), oracle.unary(name, big, p)
        if tol is None:
            assert np.array_equal(got, ref), name
        else:
            assert (np.abs(got - ref) <= tol * np.maximum(np.abs(ref), 1)).all(), name


def run_reduce(hip, name, x, axis):
    dx = hip.array(x)
    if axis == -1:
        out = hip.empty((1,))
        hip.check(hip.L.axhip_reduce_all(_O.REDUCE[name], dx.ptr, x.size, out.ptr))
        return out.numpy()
    outer, inner = int(np.prod(x.shape[:axis])), int(np.prod(x.shape[axis + 1:]))
    out = hip.empty((outer * inner,))
    hip.check(hip.L.axhip_reduce_axis(_O.REDUCE[name], dx.ptr, outer, x.shape[axis], inner, out.ptr))
    return out.numpy().reshape(x.shape[:axis] + x.shape[axis + 1:])


def run_argmax(hip, x, axis):
    dx = hip.array(x)
    if axis == -1:
        outer, n, inner, shape = 1, x.size, 1, (1,)
    else:
        outer, n, inner = int(np.prod(x.shape[:axis])), x.shape[axis], int(np.prod(x.shape[axis + 1:]))
        shape = x.shape[:axis] + x.shape[axis + 1:]
    out = hip.empty((outer * inner,), np.int64)
    hip.check(hip.L.axhip_argmax_axis(dx.ptr, outer, n, inner, out.ptr))
    return out.numpy().reshape(shape)


@pytest.mark.gpu
def test_reductions_golden(hip, oracle, golden):
    say("reductions golden")
    for shp, arr in zip(sc.REDUCE_SHAPES, sc.reduce_inputs(oracle)):
        tag = "x".join(map(str, shp))
        for axis in range(-1, len(shp)):
            for name in ("max", "min"):                        # order-independent: bit-exact
                assert np.array_equal(run_reduce(hip, name, arr, axis), golden[f"red_{name}_{tag}_axis{axis}_naive"])
            assert np.abs(run_reduce(hip, "mean", arr, axis) - golden[f"red_mean_{tag}_axis{axis}_naive"]).max() < 2e-6
            assert np.array_equal(run_argmax(hip, arr, axis), golden[f"red_argmax_{tag}_axis{axis}"])


@pytest.mark.gpu
@pytest.mark.parametrize("shape,axis", [((4096, 4096), 0), ((4096, 4096), 1), ((3, 100000, 5), 1), ((64, 7, 64), 1),
                                        ((2, 3000001), 1), ((1 << 22,), 0), ((5, 4, 3, 130), 2), ((33, 1000), 0),
                                        ((1000, 33), 1), ((100000, 8), 0), ((17, 1), 0), ((20000, 1000), 0), ((16384, 772), 0),
                                        ((2048, 1024), 0), ((3, 9000, 36), 1), ((9001, 2050), 0),
                                        ((100003, 10), 1), ((70001, 32), 1), ((70001, 33), 1), ((50001, 128), 1),
                                        ((50001, 129), 1), ((1001, 3), 1), ((65, 17), 1), ((3001, 8), 1), ((3001, 7), 1)])
def test_reductions_shapes(hip, oracle, shape, axis):
    say("reduce", shape, axis)
    oracle.seed(sum(shape) + axis)
    x = oracle.uniform(shape, -1, 1)
    x.reshape(-1)[::97] = np.nan                               # passed over by max / min
    assert np.array_equal(run_reduce(hip, "max", x, axis), np.nanmax(x, axis=axis))
    assert np.array_equal(run_reduce(hip, "min", x, axis), np.nanmin(x, axis=axis))
    x = np.nan_to_num(x, nan=0.25)
    x64 = x.astype(np.float64)
    bound = SUM_BOUND * np.abs(x64).sum(axis=axis) + 1e-30
    assert (np.abs(run_reduce(hip, "sum", x, axis) - x64.sum(axis=axis)) <= bound).all()
    assert (np.abs(run_reduce(hip, "mean", x, axis) - x64.mean(axis=axis)) <= bound / shape[axis] + 1e-7).all()
    x.reshape(-1)[::5] = 0.75                                  # ties: the first index wins
    assert np.array_equal(run_argmax(hip, x, axis), np.argmax(x, axis=axis))
    # everything at once
    assert run_reduce(hip, "max", x, -1)[0] == x.max() and run_reduce(hip, "min", x, -1)[0] == x.min()
    assert run_argmax(hip, x, -1)[0] == int(np.argmax(x))
    got = float(run_reduce(hip, "mean", x, -1)[0])
    assert abs(got - x.astype(np.float64).mean()) <= SUM_BOUND * np.abs(x).astype(np.float64).mean() + 1e-7


@pytest.mark.gpu
def test_reduce_starting_values(hip):
    """cpu_naive.c:395-433: a row of NaN / -inf leaves the starting value -FLT_MAX."""
    x = np.array([[np.nan, -np.inf, np.nan], [1.0, np.nan, 2.0]], np.float32)
    assert np.array_equal(run_reduce(hip, "max", x, 1), np.array([-np.finfo(np.float32).max, 2.0], np.float32))
    assert np.array_equal(run_reduce(hip, "min", -x, 1), np.array([np.finfo(np.float32).max, -2.0], np.float32))


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols", [(1000, 37), (70, 300), (4099, 5), (63, 9)])
def test_argmax_down_columns_scan_rule(hip, oracle, rows, cols):
    """The reference's argmax scans from element 0 and replaces on strictly greater (opt_argmax,
    cpu_opt.c:7202-7249): NaNs are passed over, a NaN in element 0 is never replaced (answer 0),
    ties keep the first index.  Long axes are cut into slices on the GPU; the rule must survive."""
    say("argmax scan rule", rows, cols)
    oracle.seed(rows + cols)
    x = oracle.uniform((rows, cols), -1, 1)
    x[::7] = 0.5                                               # ties across slices
    x[0, 1] = np.nan                                           # NaN first: stays
    x[5:rows // 2, 2] = np.nan                                 # NaNs inside: skipped
    x[:, 3] = np.nan
    x[:, 4] = -np.inf
    x[rows - 1, 0] = 2.0                                       # maximum in the last slice
    want = np.zeros(cols, np.int64)
    for c in range(cols):
        bestv, best = x[0, c], 0
        for a in range(1, rows):
            if x[a, c] > bestv:
                bestv, best = x[a, c], a
        want[c] = best
    assert np.array_equal(run_argmax(hip, x, 0), want)


def run_softmax(hip, x):
    dx, out = hip.array(x), hip.empty(x.shape)
    hip.check(hip.L.axhip_softmax_rows(dx.ptr, out.ptr, x.shape[0], x.shape[1]))
    return out.numpy()


@pytest.mark.gpu
def test_softmax_rows(hip, oracle, golden):
    say("softmax")
    for (rows, cols), arr in zip(sc.SOFTMAX_SHAPES, sc.softmax_inputs(oracle)):
        assert np.abs(run_softmax(hip, arr) - golden[f"softmax_{rows}x{cols}_naive"]).max() < 1e-6
    # 4097 .. 36864 columns: the row held in LDS (rows start off the 16-byte grid when cols is odd);
    # beyond: two reads with the running-maximum form
    for (rows, cols) in [(1, 1), (7, 129), (1000, 512), (33, 513), (64, 1024), (5, 4096), (3, 4097), (2, 100000),
                         (8192, 512), (4097, 64), (5, 10001), (3, 36864), (3, 36865), (7, 50257), (2, 131075),
                         (300, 4100), (1, 36863), (9, 6144), (9, 6145), (17, 6143), (1003, 128), (33, 65), (35, 64),
                         (29, 33), (2, 256), (70, 200)]:
        oracle.seed(rows + cols)
        x = oracle.uniform((rows, cols), -8, 8)
        got = run_softmax(hip, x)
        e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
        want = e / e.sum(axis=1, keepdims=True)
        assert (np.abs(got - want) <= 2e-6 * want + 1e-12).all(), (rows, cols)
        if rows * cols <= 1 << 20:
            assert np.abs(got - oracle.softmax_rows(x)).max() < 1e-6
        if cols > 4096:                                   # in place (the slot allows in == out)
            dx = hip.array(x)
            hip.check(hip.L.axhip_softmax_rows(dx.ptr, dx.ptr, rows, cols))
            assert np.array_equal(dx.numpy(), got)


def run_layernorm(hip, x, gamma, beta, eps, save=True):
    rows, cols = int(np.prod(x.shape[:-1])), x.shape[-1]
    dx, dg, db = hip.array(x), hip.array(gamma), hip.array(beta)
    out, xh, inv = hip.empty(x.shape), hip.empty(x.shape), hip.empty((rows,))
    hip.check(hip.L.axhip_layernorm_fwd(dx.ptr, dg.ptr, db.ptr, out.ptr, xh.ptr if save else None,
                                        inv.ptr if save else None, rows, cols, eps))
    return out.numpy(), xh.numpy(), inv.numpy()


@pytest.mark.gpu
def test_layernorm_forward(hip, oracle, golden):
    say("layernorm")
    for shp, (x, gamma, beta) in zip(sc.LAYERNORM_SHAPES, sc.layernorm_inputs(oracle)):
        out, xh, inv = run_layernorm(hip, x, gamma, beta, 1e-5)
        assert np.abs(out - golden["layernorm_" + "x".join(map(str, shp))]).max() < 5e-6
        o_out, o_xh, o_inv = oracle.layernorm(x, gamma, beta, 1e-5)
        assert np.abs(out - o_out).max() < 5e-6 and np.abs(xh - o_xh).max() < 5e-6
        assert np.allclose(inv, o_inv, rtol=2e-6)
    for shp in [(4096, 1024), (2048, 768), (100, 4096), (3, 5000), (9, 1), (4097, 96), (5, 10001), (2, 36864),
                (3, 36867), (3, 50257), (130, 4099), (9, 6144), (9, 6145), (17, 6141), (1003, 128), (33, 65),
                (35, 64), (29, 33), (70, 200)]:
        oracle.seed(sum(shp))
        x, gamma, beta = oracle.uniform(shp, -3, 5), oracle.uniform((shp[-1],), 0.5, 1.5), oracle.uniform((shp[-1],), -1, 1)
        out, xh, inv = run_layernorm(hip, x, gamma, beta, 1e-5)
        x64 = x.astype(np.float64)
        want_xh = (x64 - x64.mean(axis=-1, keepdims=True)) / np.sqrt(x64.var(axis=-1, keepdims=True) + 1e-5)
        assert np.abs(xh - want_xh).max() < 2e-5 and np.abs(out - (gamma * want_xh + beta)).max() < 2e-5, shp
        out2, _, _ = run_layernorm(hip, x, gamma, beta, 1e-5, save=False)
        assert np.array_equal(out, out2)


@pytest.mark.gpu
@pytest.mark.parametrize("key", list(sc.OPTIMIZERS))
def test_optimizer_updates(hip, oracle, golden, key):
    say("optimizer", key)
    kind, kw = sc.OPTIMIZERS[key]
    w0, grads = sc.optimizer_inputs(oracle)
    dw, dm, dv = hip.array(w0), hip.array(np.zeros_like(w0)), hip.array(np.zeros_like(w0))
    w, m, v = w0.copy(), np.zeros_like(w0), np.zeros_like(w0)
    for step, g in enumerate(grads, 1):
        dg = hip.array(g)
        if kind == "sgd":
            use_m = kw["momentum"] > 0
            hip.check(hip.L.axhip_sgd_update(dw.ptr, dg.ptr, dm.ptr if use_m else None, w0.size, kw["lr"], kw["momentum"],
                                             kw["wd"], int(kw["nesterov"])))
            oracle.sgd_update(w, g, m if use_m else None, kw["lr"], kw["momentum"], kw["wd"], kw["nesterov"])
        else:
            bc1, bc2 = sc.bias_corrections(kw["beta1"], kw["beta2"], step)
            hip.check(hip.L.axhip_adam_update(dw.ptr, dg.ptr, dm.ptr, dv.ptr, w0.size, kw["lr"], kw["beta1"], kw["beta2"],
                                              kw["eps"], kw["wd"], bc1, bc2, int(kind == "adamw")))
            oracle.adam_update(w, g, m, v, kw["lr"], kw["beta1"], kw["beta2"], kw["eps"], kw["wd"], bc1, bc2, kind == "adamw")
        got = dw.numpy()
        assert np.abs(got - golden[key][step - 1]).max() < 2e-6, step        # the reference's CPU optimizer
        assert np.abs(got - w).max() < 5e-7, step                            # same formula; fma contraction apart


# ---------------------------------------------------------------- attention layout transforms
@pytest.mark.gpu
@pytest.mark.parametrize("B,S,H,dk", [(2, 3, 4, 5), (1, 1, 1, 1), (3, 7, 2, 8), (2, 128, 8, 64), (4, 33, 3, 20), (8, 512, 16, 64)])
def test_attention_layout_transforms(hip, oracle, B, S, H, dk):
    """Pure copies: bit-exact against numpy reshapes / transposes (the reference's index maps,
    src/core/attention/layout.c:134-148, 237-253)."""
    import attn_cases as ac
    say("attn layout", B, S, H, dk)
    D = H * dk
    oracle.seed(B * 1000 + S * 10 + H + dk)
    qkv, bias = oracle.uniform((B * S, 3 * D), -1, 1), oracle.uniform((3 * D,), -1, 1)
    dqkv, dbias = hip.array(qkv), hip.array(bias)
    q, k, v = (hip.empty((B * H, S, dk)) for _ in range(3))
    for use_bias in (False, True):
        hip.check(hip.L.axhip_head_split_qkv(dqkv.ptr, dbias.ptr if use_bias else None, q.ptr, k.ptr, v.ptr, B, S, H, dk, D))
        src = qkv + bias if use_bias else qkv
        for i, got in enumerate((q, k, v)):
            want = ac.split_heads(np.ascontiguousarray(src[:, i * D:(i + 1) * D]), B, S, H, dk)
            assert np.array_equal(got.numpy(), want), (use_bias, i)
    heads = oracle.uniform((B * H, S, dk), -1, 1)
    dh, merged, back = hip.array(heads), hip.empty((B * S, D)), hip.empty((B * H, S, dk))
    hip.check(hip.L.axhip_head_deinterleave(dh.ptr, merged.ptr, B, S, H, dk))
    assert np.array_equal(merged.numpy(), ac.merge_heads(heads, B, S, H, dk))
    hip.check(hip.L.axhip_head_interleave(merged.ptr, back.ptr, B, S, H, dk))
    assert np.array_equal(back.numpy(), heads)
    # fused projection panel [D, 3D] and bias [3D]
    wq, wk, wv = (oracle.uniform((D, D), -1, 1) for _ in range(3))
    dq, dk_, dv, panel = hip.array(wq), hip.array(wk), hip.array(wv), hip.empty((D, 3 * D))
    hip.check(hip.L.axhip_concat3_rows(panel.ptr, dq.ptr, dk_.ptr, dv.ptr, D, D))
    assert np.array_equal(panel.numpy(), np.concatenate([wq, wk, wv], axis=1))
    hip.check(hip.L.axhip_concat3_rows(panel.ptr, dq.ptr, dk_.ptr, dv.ptr, 1, D))
    assert np.array_equal(panel.numpy().reshape(-1)[:3 * D], np.concatenate([wq[0], wk[0], wv[0]]))


@pytest.mark.gpu
@pytest.mark.parametrize("N,M", [(65537, 32771), (262147, 32772)])
def test_binary_and_reductions_beyond_2_31_elements(hip, oracle, N, M):
    """An outer sum a[N,1] + b[1,M] whose work-item count passes 2^31 takes the 64-bit index path of
    the broadcasting kernel (one element per item for the odd M, four for the other: 8.6 and 34 GB
    of output).  The result is checked on the device: max and min are exact functions of the
    operands, the total is M*sum(a) + N*sum(b), and a window around flat index 2^31 is read back."""
    say("binary beyond 2^31", N, M)
    assert N * M // (4 if M % 4 == 0 else 1) > 2 ** 31
    oracle.seed(77)
    a, b = oracle.uniform((N, 1), -1, 1), oracle.uniform((1, M), -1, 1)
    out_shape = (C.c_int64 * 2)(N, M)
    da, db, out = hip.array(a), hip.array(b), hip.empty((N, M))
    hip.check(hip.L.axhip_binary(0, da.ptr, db.ptr, out.ptr, 2, out_shape, (C.c_int64 * 2)(1, 0), (C.c_int64 * 2)(0, 1)))
    one = hip.empty((1,))
    hip.check(hip.L.axhip_reduce_all(2, out.ptr, N * M, one.ptr))
    assert one.numpy()[0] == np.float32(a.max() + b.max())
    hip.check(hip.L.axhip_reduce_all(3, out.ptr, N * M, one.ptr))
    assert one.numpy()[0] == np.float32(a.min() + b.min())
    hip.check(hip.L.axhip_reduce_all(0, out.ptr, N * M, one.ptr))
    want = M * a.astype(np.float64).sum() + N * b.astype(np.float64).sum()
    bound = SUM_BOUND * (M * np.abs(a).astype(np.float64).sum() + N * np.abs(b).astype(np.float64).sum())
    assert abs(float(one.numpy()[0]) - want) <= bound
    rows = hip.empty((N,))
    hip.check(hip.L.axhip_reduce_axis(2, out.ptr, N, M, 1, rows.ptr))
    assert np.array_equal(rows.numpy(), (a + b.max()).reshape(-1))
    # rows around flat index 2^31
    r0 = 2 ** 31 // M - 1
    window = np.empty((3, M), np.float32)
    hip.check(hip.L.axhip_memcpy_d2h(window.ctypes.data, out.ptr + r0 * M * 4, window.nbytes))
    assert np.array_equal(window, a[r0:r0 + 3] + b)


@pytest.mark.gpu
@pytest.mark.parametrize("kind,M,N,K", [("f32", 66000, 33000, 8), ("f32", 65664, 32768, 64), ("i8", 65600, 32768, 128),
                                        ("i8", 66001, 33000, 64)])
def test_gemm_outputs_beyond_2_31_elements(hip, kind, M, N, K):
    """A product with more than 2^31 output elements (8.6 GB of fp32): element offsets into C must be
    64-bit in every kernel of the route (edge tiles, interior + fringes, the persistent int8 tiles).
    Operands are small integers, so every product and every row or column sum of C is an exact fp32
    integer whatever the order: row sums of C are A . rowsum(B), column sums are colsum(A) . B, and
    rows at the start, around flat index 2^31 and at the end are read back."""
    say("gemm beyond 2^31 outputs", kind, M, N, K)
    assert M * N > 2 ** 31
    rng = np.random.default_rng(M + N + K)
    a = rng.integers(-2, 3, (M, K))
    out = hip.empty((M, N))
    if kind == "f32":
        b = rng.integers(-2, 3, (K, N))
        da, db = hip.array(a.astype(np.float32)), hip.array(b.astype(np.float32))
        hip.check(hip.L.axhip_sgemm(0, 0, M, N, K, 1.0, da.ptr, K, db.ptr, N, 0.0, out.ptr, N, None, 0))
    else:
        w = rng.integers(-2, 3, (N, K))
        b = w.T
        da, dw = hip.array(a.astype(np.int8)), hip.array(w.astype(np.int8))
        ones = hip.array(np.ones(N, np.float32))
        hip.check(hip.L.axhip_qgemm_w8a8(da.ptr, 1.0, dw.ptr, ones.ptr, None, 0, out.ptr, None, M, N, K))
    rows, cols = hip.empty((M,)), hip.empty((N,))
    hip.check(hip.L.axhip_sum_axis(out.ptr, M, N, 1, rows.ptr))
    assert np.array_equal(rows.numpy(), (a @ b.sum(axis=1)).astype(np.float32))
    hip.check(hip.L.axhip_sum_axis(out.ptr, 1, M, N, cols.ptr))
    assert np.array_equal(cols.numpy(), (a.sum(axis=0) @ b).astype(np.float32))
    for r0 in (0, 2 ** 31 // N - 1, M - 3):
        window = np.empty((3, N), np.float32)
        hip.check(hip.L.axhip_memcpy_d2h(window.ctypes.data, out.ptr + r0 * N * 4, window.nbytes))
        assert np.array_equal(window, (a[r0:r0 + 3] @ b).astype(np.float32)), r0


@pytest.mark.gpu
def test_allocation_pool(hip):
    """Freed blocks come back for the next request of their size class, zero-filled, with earlier
    work on them finished first (one stream); foreign pointers and double frees are ignored."""
    say("allocation pool")
    a = hip.empty((1000,))
    p = a.ptr
    hip.check(hip.L.axhip_fill_f32(p, 3.0, 1000))
    del a                                                      # DeviceArray.__del__ -> axhip_free
    b = hip.empty((1024,))                                     # same 4 KiB class
    assert b.ptr == p and not b.numpy().any()
    c = hip.empty((1024,))
    assert c.ptr != p
    hip.L.axhip_free(p + 16)                                   # not a block of ours
    hip.L.axhip_free(None)
    big = [hip.empty((1 << 28,)) for _ in range(3)]            # 1 GiB each: still pooled
    ptrs = {x.ptr for x in big}
    del big
    again = [hip.empty((1 << 28,)) for _ in range(3)]
    assert {x.ptr for x in again} == ptrs
    assert not again[0].numpy()[::4097].any()
    del again
    huge = hip.empty(((1 << 28) + (1 << 20),))                 # above 1 GiB: not kept
    hp = huge.ptr
    hip.check(hip.L.axhip_fill_f32(hp, 1.0, 16))
    del huge
    out = hip.empty((16,))
    hip.check(hip.L.axhip_fill_f32(out.ptr, 2.0, 16))
    assert np.array_equal(out.numpy(), np.full(16, 2.0, np.float32))
    # a block freed twice is handed out once; the counters balance and tell pool hits from driver calls
    hip.L.axhip_reset_alloc_stats()
    x = hip.empty((3000,))
    xp = x.ptr
    hip.L.axhip_free(xp)
    hip.L.axhip_free(xp)                                       # second free: ignored
    x.ptr = None
    y, z = hip.empty((3000,)), hip.empty((3000,))
    assert y.ptr == xp and z.ptr != xp
    del y, z
    st = [C.c_int64() for _ in range(6)]
    hip.L.axhip_alloc_stats(*[C.byref(v) for v in st])
    allocs, frees, b_alloc, b_free, driver, cached = (v.value for v in st)
    assert allocs == 3 and frees == 3 and b_alloc == b_free == 3 * 16384 and driver <= 2 and cached >= 2 * 16384


def test_workspace_reserve_grows_once_and_never_shrinks(hip, oracle):
    """axhip_workspace_reserve sizes the shared workspace ahead of time: the size only grows, a split-K product
    that fits runs in the reserved block (same size afterwards) and still meets the fp32 gate."""
    import ctypes as C
    have = C.c_size_t(0)
    hip.check(hip.L.axhip_workspace_reserve(0, C.byref(have)))
    start = have.value
    want = max(start, 8 << 20) + (24 << 20)
    hip.check(hip.L.axhip_workspace_reserve(want, C.byref(have)))
    assert have.value >= want
    grown = have.value
    hip.check(hip.L.axhip_workspace_reserve(1 << 20, C.byref(have)))
    assert have.value == grown
    hip.check(hip.L.axhip_workspace_reserve(0, None))
    oracle.seed(5)
    a, b = oracle.uniform((64, 4096), -1, 1), oracle.uniform((4096, 1024), -1, 1)
    got = hip.sgemm(hip.array(a), hip.array(b)).numpy()
    assert hip.last_kernel() == "sgemm_splitk"
    check_fp32(oracle, got, a, b)
    hip.check(hip.L.axhip_workspace_reserve(0, C.byref(have)))
    assert have.value == grown
