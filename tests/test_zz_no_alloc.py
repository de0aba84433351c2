"""The allocation-free skinny-M entry point, axhip_sgemm_skinny_static, against axhip_sgemm_skinny
through the C ABI: the same kernels on the library's static device scratch must give bit-identical
results, on calls in a row that share the scratch (the later ones smaller), and shapes beyond the
scratch must be refused rather than run."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def both(hip, oracle, M, K, N, act, with_bias, seed):
    oracle.seed(seed)
    a, b = oracle.uniform((M, K), -1, 1), oracle.uniform((K, N), -1, 1)
    bias = oracle.normal((N,), 0.0, 0.5)
    da, db = hip.array(a), hip.array(b)
    dbias = hip.array(bias) if with_bias else None
    want = hip.sgemm_skinny(da, db, dbias, act).numpy()
    dc = hip.empty((M, N))
    hip.check(hip.L.axhip_memset(dc.ptr, 0xFF, dc.nbytes))          # NaN pattern: every output must be written
    hip.check(hip.L.axhip_sgemm_skinny_static(M, N, K, da.ptr, K, db.ptr, N, dc.ptr, N, hip._p(dbias), act))
    got = dc.numpy()
    # the oracle's dense layer on the same inputs, within the fp32 gate of the skinny route
    ref = oracle.dense(a, b, bias if with_bias else None, act)
    assert np.abs(want - ref).max() <= 1e-4 * max(np.abs(ref).max(), 1e-6)
    return got, want


def test_static_scratch_calls_in_a_row_match_the_allocating_entry_point(hip, oracle):
    # first call: 8 ranges of K over 64 strips through the tile join; then smaller ones that reuse the front of the scratch
    cases = [(8, 4096, 4096, 1, True), (3, 1000, 520, 0, False), (1, 784, 4096, 1, True),
             (16, 640, 260, 2, True), (1, 40, 10, 0, False), (8, 4096, 4096, 1, True)]
    for i, (M, K, N, act, with_bias) in enumerate(cases):
        say("skinny_static", M, K, N, act, with_bias)
        got, want = both(hip, oracle, M, K, N, act, with_bias, 100 + i)
        assert np.array_equal(got, want), f"call {i}: static-scratch result differs"
    assert hip.last_kernel().startswith("sgemm_skinny")


def test_static_scratch_back_to_back_without_host_waits(hip, oracle):
    """Two launches queued with nothing in between: the second (smaller) starts on the join slots the
    first one's workgroups emptied again."""
    oracle.seed(7)
    a1, b1 = oracle.uniform((4, 2048), -1, 1), oracle.uniform((2048, 1024), -1, 1)
    a2, b2 = oracle.uniform((2, 512), -1, 1), oracle.uniform((512, 256), -1, 1)
    d = [hip.array(x) for x in (a1, b1, a2, b2)]
    c1, c2 = hip.empty((4, 1024)), hip.empty((2, 256))
    say("skinny_static back to back")
    for _ in range(3):
        hip.check(hip.L.axhip_sgemm_skinny_static(4, 1024, 2048, d[0].ptr, 2048, d[1].ptr, 1024, c1.ptr, 1024, None, 0))
        hip.check(hip.L.axhip_sgemm_skinny_static(2, 256, 512, d[2].ptr, 512, d[3].ptr, 256, c2.ptr, 256, None, 0))
    assert np.array_equal(c1.numpy(), hip.sgemm_skinny(d[0], d[1]).numpy())
    assert np.array_equal(c2.numpy(), hip.sgemm_skinny(d[2], d[3]).numpy())


def test_static_scratch_refuses_what_does_not_fit(hip, monkeypatch):
    # No shape plans more than the scratch holds by itself (wide matrices get few ranges of K); with the
    # workgroup count forced up, M = 8 against 16448 columns plans 16 ranges: 8.4 MB of partial tiles
    # against 8 MiB of room.
    M, K, N = 8, 4096, 16448
    a, b, c = hip.empty((M, K)), hip.empty((K, N)), hip.empty((M, N))
    say("skinny_static refusal")
    monkeypatch.setenv("AX_HIP_SKINNY_BLOCKS", "65535")
    assert hip.L.axhip_tuning_reload() == 1
    try:
        rc = hip.L.axhip_sgemm_skinny_static(M, N, K, a.ptr, K, b.ptr, N, c.ptr, N, None, 0)
        assert rc == 3 and "static scratch" in hip.last_error()
        # the allocating entry point takes the same plan
        hip.check(hip.L.axhip_sgemm_skinny(M, N, K, a.ptr, K, b.ptr, N, c.ptr, N, None, 0))
        assert not c.numpy().any()
    finally:
        monkeypatch.delenv("AX_HIP_SKINNY_BLOCKS")
        assert hip.L.axhip_tuning_reload() == 0
    # argument checks are those of the allocating entry point
    assert hip.L.axhip_sgemm_skinny_static(17, 8, 8, a.ptr, 8, a.ptr, 8, a.ptr, 8, None, 0) == 3
    assert hip.L.axhip_sgemm_skinny_static(1, 8, 8, None, 8, a.ptr, 8, a.ptr, 8, None, 0) == 1


def test_static_scratch_calls_allocate_nothing(hip, oracle):
    """What the entry point is for: no device allocation, no pool traffic and no workspace growth across its
    calls — exchange-tree shapes (few rows) and tile-join shapes (M >= 5, many ranges) alike — and the
    reset call allocates nothing either."""
    import ctypes as C
    oracle.seed(11)
    shapes = [(1, 4096, 4096), (8, 4096, 4096), (4, 784, 4096), (6, 2048, 1024), (16, 640, 260)]
    ops = [(M, K, N, hip.array(oracle.uniform((M, K), -1, 1)), hip.array(oracle.uniform((K, N), -1, 1)), hip.empty((M, N)))
           for (M, K, N) in shapes]
    want = [hip.sgemm_skinny(a, b).numpy() for (_, _, _, a, b, _) in ops]        # also warms every allocating path
    hip.sync()

    def snapshot():
        have, st = C.c_size_t(0), [C.c_int64(0) for _ in range(6)]
        hip.check(hip.L.axhip_workspace_reserve(0, C.byref(have)))
        hip.L.axhip_alloc_stats(*[C.byref(x) for x in st])
        return have.value, [x.value for x in st], hip.L.axhip_device_free_bytes()

    before = snapshot()
    say("skinny_static allocation check")
    for _ in range(3):
        for (M, K, N, a, b, c) in ops:
            hip.check(hip.L.axhip_sgemm_skinny_static(M, N, K, a.ptr, K, b.ptr, N, c.ptr, N, None, 0))
        hip.check(hip.L.axhip_sgemm_skinny_reset())
    hip.sync()
    after = snapshot()
    assert after[0] == before[0], "workspace grew"
    assert after[1] == before[1], "pool counters moved"
    assert after[2] == before[2], "device memory in use changed"
    for (_, _, _, _, _, c), w in zip(ops, want):
        assert np.array_equal(c.numpy(), w)
