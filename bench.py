#!/usr/bin/env python3
"""Benchmark of the MI355X GEMM backend.  Prints ONE JSON line on stdout.

Headline workload (BASELINE.json configs[4], the shape the int8 target is quoted on): the
W8A8 quantized GEMM at M=N=K=8192 with its fused dequantize + bias write-back.  One "step"
is one such GEMM over inputs already resident in HBM; `value` is TOP/s (2*M*N*K per step).
The `secondary` object carries the other configurations the metric names: fp32 GEMM TFLOP/s
and the skinny-M route's GB/s, each with its own roofline fraction.  RESULT lines in the
reference's benchmark format (benchmarks/bench_common.h:25-42) go to stderr.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-secondary] [--no-cpu]
    python bench.py --counter-probe [headline|skinny|gemm1024|fp32|config2|attention|w8a32]
                                        # for hardware-counter runs: a few launches of one case's kernels and 3
                                        # launches of a copy-shaped kernel of known size, no output line
    python bench.py --sustain 8 [--operands zeros]   # back-to-back headline launches, for clock sampling
    python bench.py --hbm-ceiling                    # read / write / copy rates of this GPU on 2 GiB arrays, one JSON line
    python bench.py --dispatch-table                 # shape -> kernel -> us for a fixed list of shapes (fp32, W8A8, W8A32)

`secondary.configs` holds one record per BASELINE configuration in the reference's record shape
(benchmarks/bench_common.h:25-42 plus algorithmic work): workload, algorithmic_flops, algorithmic_bytes,
time_s, achieved, unit, roofline {bound, peak, achieved = achieved / peak}, kernel, and cpu = the
reference's own CPU path on the same shape, timed in this run on the host cores.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0      # MI355X dense int8 MFMA, TOP/s
PEAK_FP32_TFLOPS = 157.3     # MI355X fp32 matrix, TFLOP/s
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E, GB/s
# Bytes that cross the L2 boundary per headline launch come from the committed counter summary of
# `bench.py --counter-probe` (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, each scaled by what the same
# counter reads for the probe's copy-shaped kernel of known size).  The summary names the kernel
# variant it was taken on; for any other variant the figure is unknown and reported as null.
HEADLINE_COUNTERS = os.path.join(ROOT, "profiles", "qgemm_w8a8_256_8192cube_hbm_counters.txt")
PREHEAT_SECONDS = 0.6        # untimed launches before warm-up: the GPU leaves its idle clock only under load


def headline_traffic_bytes(kernel):
    """(bytes per launch, note) from the lines `bench_kernel: <name>` and `traffic_bytes_per_launch:
    <number>` of the counter summary; (None, why) when the file is missing or was taken on another
    kernel variant."""
    try:
        fields = {}
        for ln in open(HEADLINE_COUNTERS):
            key, sep, val = ln.partition(":")
            if sep and key.strip() in ("bench_kernel", "traffic_bytes_per_launch"):
                fields[key.strip()] = val.strip()
        if fields.get("bench_kernel") != kernel:
            return None, f"counter summary is for {fields.get('bench_kernel')!r}, this run used {kernel!r}"
        return float(fields["traffic_bytes_per_launch"]), os.path.relpath(HEADLINE_COUNTERS, ROOT)
    except (OSError, KeyError, ValueError) as e:
        return None, f"no usable counter summary: {e}"


def result_line(suite, case, metric, value):
    print(f"RESULT {suite} {case} {metric} {value:.6g}", file=sys.stderr, flush=True)


def rand_i8(rng, shape):
    return rng.integers(-127, 128, shape, dtype=np.int8)


def time_calls(hip, fn, steps=None, warmup=None, seconds=0.3):
    """(host ms per step between device syncs, event ms per step on the kernels' stream).
    Without explicit counts, warms up for `seconds` and times `seconds` worth of launches: the
    GPU raises its clock only after some tens of milliseconds of load and settles at its
    power-limited clock after a few hundred, and sustained throughput is what is reported."""
    if steps is None or warmup is None:
        for _ in range(3):
            fn()
        hip.sync()
        t0 = time.perf_counter()
        for _ in range(10):
            fn()
        hip.sync()
        per = max((time.perf_counter() - t0) / 10, 1e-6)
        n = int(min(max(seconds / per, 20), 20000))
        steps = n if steps is None else steps
        warmup = n if warmup is None else warmup
    for _ in range(warmup):
        fn()
    hip.sync()
    e0, e1 = hip.L.axhip_event_create(), hip.L.axhip_event_create()
    t0 = time.perf_counter()
    hip.check(hip.L.axhip_event_record(e0))
    for _ in range(steps):
        fn()
    hip.check(hip.L.axhip_event_record(e1))
    hip.sync()
    host_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms = C.c_float()
    hip.check(hip.L.axhip_event_elapsed_ms(e0, e1, C.byref(ms)))
    hip.L.axhip_event_destroy(e0)
    hip.L.axhip_event_destroy(e1)
    return host_ms, ms.value / steps


def time_each(hip, fn, steps, warmup, preheat_s):
    """Times `steps` calls one by one: an event on the kernels' stream before the first call and
    after every call, so each launch has its own duration (the reference's per-iteration samples,
    benchmarks/bench_comprehensive.c:90-95).  Before that, `preheat_s` seconds of untimed calls
    bring the GPU to its sustained clock, then `warmup` more untimed calls.  Returns (host ms per
    step between device syncs, per-launch event ms as an array, seconds actually pre-heated)."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < preheat_s:
        for _ in range(8):
            fn()
        hip.sync()
    preheated = time.perf_counter() - t0
    for _ in range(warmup):
        fn()
    hip.sync()
    ev = [hip.L.axhip_event_create() for _ in range(steps + 1)]
    t0 = time.perf_counter()
    hip.check(hip.L.axhip_event_record(ev[0]))
    for i in range(steps):
        fn()
        hip.check(hip.L.axhip_event_record(ev[i + 1]))
    hip.sync()
    host_ms = (time.perf_counter() - t0) * 1e3 / steps
    each = np.empty(steps)
    ms = C.c_float()
    for i in range(steps):
        hip.check(hip.L.axhip_event_elapsed_ms(ev[i], ev[i + 1], C.byref(ms)))
        each[i] = ms.value
    for e in ev:
        hip.L.axhip_event_destroy(e)
    return host_ms, each, preheated


def headline(hip, steps, warmup):
    M = N = K = 8192
    rng = np.random.default_rng(0)
    x, w = hip.array(rand_i8(rng, (M, K))), hip.array(rand_i8(rng, (N, K)))
    ws = hip.array(rng.uniform(1e-3, 1e-2, N).astype(np.float32))
    bias = hip.array(rng.normal(0.0, 0.02, N).astype(np.float32))
    out = hip.empty((M, N))

    def step():
        hip.check(hip.L.axhip_qgemm_w8a8(x.ptr, 0.01, w.ptr, ws.ptr, bias.ptr, 0, out.ptr, None, M, N, K))

    host_ms, each, preheated = time_each(hip, step, steps, warmup, PREHEAT_SECONDS)
    ops = 2.0 * M * N * K
    return {"M": M, "N": N, "K": K, "host_ms": host_ms, "event_ms": float(each.mean()),
            "median_ms": float(np.median(each)), "min_ms": float(each.min()), "max_ms": float(each.max()),
            "preheat_s": preheated, "ops": ops, "kernel": hip.last_kernel(),
            "algorithmic_bytes": M * K + N * K + 4 * M * N + 8 * N}


def config_record(workload, flops, nbytes, time_s, bound, kernel, **extra):
    """One BASELINE configuration in the reference's record shape.  `bound` picks the roofline the
    configuration is priced against: "hbm" (GB/s of algorithmic bytes), "mfma_fp32" (TFLOP/s) or
    "mfma_int8" (TOP/s); roofline.achieved is the fraction of that peak."""
    if bound == "hbm":
        achieved, unit, peak = nbytes / time_s / 1e9, "GB/s", PEAK_HBM_GBS
    elif bound == "mfma_fp32":
        achieved, unit, peak = flops / time_s / 1e12, "TFLOP/s", PEAK_FP32_TFLOPS
    else:
        achieved, unit, peak = flops / time_s / 1e12, "TOP/s", PEAK_INT8_TOPS
    rec = {"workload": workload, "algorithmic_flops": float(flops), "algorithmic_bytes": float(nbytes),
           "time_s": time_s, "achieved": achieved, "unit": unit,
           "roofline": {"bound": "hbm" if bound == "hbm" else "mfma", "peak": peak, "achieved": achieved / peak},
           "kernel": kernel, "cpu": None}
    rec.update(extra)
    return rec


def cpu_config_legs(budget_s=4.0):
    """The reference's own CPU path on each BASELINE configuration, on this box's host cores: a bounded
    sample per configuration (a few warm-up runs, then timed runs until `budget_s` seconds or the run
    count of the reference's own harness is reached).  Checker/baseline code only.  Returns
    {config key: {value, unit, cores, kind, sample}}; empty when only the CPU restatement is present
    (its legs are the two in cpu_baseline / cpu_baseline_fp32)."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_bind as ob
    if not ob.ref_available():
        return {}
    lib = ob.RefLib()
    L = lib.L
    lib.backend(lib.CPU_SIMD)
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    rng = np.random.default_rng(4)
    out = {}

    def timed(fn, warm, most):
        for _ in range(warm):
            fn()
        runs, t_end = [], time.perf_counter() + budget_s
        while len(runs) < most and (len(runs) < 3 or time.perf_counter() < t_end):
            t0 = time.perf_counter()
            fn()
            runs.append(time.perf_counter() - t0)
        return float(np.median(runs)), len(runs)

    # config 1: the 784-4096-4096-10 network through the reference's Sequential forward (src/core/layer.c:188-230)
    L.ax_set_seed(1)
    seq = L.ax_sequential_create()
    for (i, o, relu) in ((784, 4096, True), (4096, 4096, True), (4096, 10, False)):
        L.ax_sequential_add(seq, L.ax_dense_create(i, o, True))
        if relu:
            L.ax_sequential_add(seq, L.ax_relu_layer_create())
    weight_bytes = 4 * (784 * 4096 + 4096 * 4096 + 4096 * 10)
    for M in (1, 8):
        tx = lib.tensor(rng.uniform(0, 1, (M, 784)).astype(np.float32))

        def forward():
            y = L.ax_layer_forward(seq, tx)
            L.ax_tensor_destroy(y)
        dt, n = timed(forward, 5, 40)
        out[f"config1_M{M}"] = {"value": weight_bytes / dt / 1e9, "unit": "GB/s", "latency_us": dt * 1e6, "cores": cores,
                                "kind": "reference",
                                "sample": f"ax_layer_forward of Sequential(Dense 784-4096 + ReLU, Dense 4096-4096 + ReLU, Dense 4096-10) "
                                          f"at M={M}, median of {n} runs after 5 warm-up runs; weights {weight_bytes / 1e6:.1f} MB per pass"}
        lib.free(tx)
    L.ax_layer_destroy(seq)

    # config 2: the reference's quantized GEMM (W8A32: it has no int8 activations) at M=256, N=K=4096 (src/core/quantize.c:100)
    M, N, K = 256, 4096, 4096
    a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    qw = L.ax_qweight_create_from_fp32(np.ascontiguousarray(rng.uniform(-1, 1, (N, K)).astype(np.float32)), N, K)
    o = np.empty((M, N), np.float32)
    dt, n = timed(lambda: L.ax_qgemm_w8a32(a, qw, o, M), 3, 10)
    L.ax_qweight_destroy(qw)
    out["config2"] = {"value": 2.0 * M * N * K / dt / 1e12, "unit": "TOP/s", "latency_us": dt * 1e6, "cores": cores, "kind": "reference",
                      "sample": f"ax_qgemm_w8a32 (int8 weights x fp32 activations, fp32 accumulate) at M=256, N=K=4096, median of {n} runs "
                                f"after 3 warm-up runs (benchmarks/bench_qgemm.c:46-57)"}

    # config 3: the FFN block as the reference runs it: GEMM, GELU as its own pass, GEMM (benchmarks/bench_transformer.c:40-42)
    x = lib.tensor(rng.normal(0, 1, (2048, 1024)).astype(np.float32))
    w1 = lib.tensor(rng.normal(0, 0.02, (1024, 4096)).astype(np.float32))
    w2 = lib.tensor(rng.normal(0, 0.02, (4096, 1024)).astype(np.float32))
    h, y = lib.empty(2048, 4096), lib.empty(2048, 1024)

    def ffn():
        assert L.ax_compute_gemm(x, w1, h) == 0
        g = L.ax_gelu(h)
        assert L.ax_compute_gemm(g, w2, y) == 0
        L.ax_tensor_destroy(g)
    dt, n = timed(ffn, 3, 10)
    lib.free(x, w1, w2, h, y)
    out["config3"] = {"value": 2 * 2.0 * 2048 * 1024 * 4096 / dt / 1e12, "unit": "TFLOP/s", "latency_us": dt * 1e6, "cores": cores,
                      "kind": "reference",
                      "sample": f"ax_compute_gemm [2048,1024]x[1024,4096], ax_gelu, ax_compute_gemm [2048,4096]x[4096,1024] (cpu_opt), "
                                f"median of {n} runs after 3 warm-up runs; biases left out (the reference drops them without ReLU)"}

    # config 4b: 8 of the 512 heads, Q K^T through ax_compute_gemm_nt and P V through ax_compute_gemm
    heads, S, D = 8, 512, 64
    qs = [lib.tensor(rng.normal(0, 1, (S, D)).astype(np.float32)) for _ in range(heads)]
    ks = [lib.tensor(rng.normal(0, 1, (S, D)).astype(np.float32)) for _ in range(heads)]
    vs = [lib.tensor(rng.normal(0, 1, (S, D)).astype(np.float32)) for _ in range(heads)]
    ss = [lib.empty(S, S) for _ in range(heads)]
    os_ = [lib.empty(S, D) for _ in range(heads)]

    def qkt():
        for i in range(heads):
            assert L.ax_compute_gemm_nt(qs[i], ks[i], ss[i]) == 0

    def pv():
        for i in range(heads):
            assert L.ax_compute_gemm(ss[i], vs[i], os_[i]) == 0
    for name, fn in (("config4b_qkt", qkt), ("config4b_pv", pv)):
        dt, n = timed(fn, 3, 20)
        out[name] = {"value": heads * 2.0 * S * S * D / dt / 1e12, "unit": "TFLOP/s", "latency_us_512_heads": dt * 1e6 * 512 / heads,
                     "cores": cores, "kind": "reference",
                     "sample": f"{heads} of the 512 heads of [512,64], one {'ax_compute_gemm_nt' if name.endswith('qkt') else 'ax_compute_gemm'} "
                               f"per head (cpu_opt), median of {n} runs after 3 warm-up runs; time scaled by 512/{heads} for the whole batch"}
    for t in qs + ks + vs + ss + os_:
        lib.free(t)
    return out


def secondary(hip):
    """The metric's other configurations, each timed with HIP events on the kernels' stream."""
    rng = np.random.default_rng(1)
    res = {}
    configs = []          # one record per BASELINE configuration (config_record)

    def f32(a_shape, b_shape):
        return (hip.array(rng.uniform(-1, 1, a_shape).astype(np.float32)),
                hip.array(rng.uniform(-1, 1, b_shape).astype(np.float32)))

    # config 0: fp32 1024^3
    a, b = f32((1024, 1024), (1024, 1024))
    c = hip.empty((1024, 1024))
    _, ms = time_calls(hip, lambda: hip.check(hip.L.axhip_sgemm(
        0, 0, 1024, 1024, 1024, 1.0, a.ptr, 1024, b.ptr, 1024, 0.0, c.ptr, 1024, None, 0)))
    tf = 2 * 1024 ** 3 / ms / 1e9
    res["fp32_gemm_1024"] = {"us": ms * 1e3, "TFLOP/s": tf, "frac_of_fp32_mfma_peak": tf / PEAK_FP32_TFLOPS,
                             "kernel": hip.last_kernel()}
    result_line("axhip", "f32_nn_1024x1024x1024", "gflops", tf * 1e3)
    configs.append(config_record("configs[0]: fp32 GEMM C = A B, M=N=K=1024, row-major", 2 * 1024 ** 3, 3 * 4 * 1024 * 1024,
                                 ms * 1e-3, "mfma_fp32", hip.last_kernel(), key="config0"))

    # the same product at the sizes where the matrix cores, not the launch, set the time
    for n_ in (4096, 8192):
        a, b = f32((n_, n_), (n_, n_))
        c = hip.empty((n_, n_))
        _, ms = time_calls(hip, lambda: hip.check(hip.L.axhip_sgemm(
            0, 0, n_, n_, n_, 1.0, a.ptr, n_, b.ptr, n_, 0.0, c.ptr, n_, None, 0)), seconds=0.4)
        tf = 2 * n_ ** 3 / ms / 1e9
        res[f"fp32_gemm_{n_}"] = {"us": ms * 1e3, "TFLOP/s": tf, "frac_of_fp32_mfma_peak": tf / PEAK_FP32_TFLOPS,
                                  "kernel": hip.last_kernel()}
    del a, b, c

    # W8A32 with many rows (fp32 activations x int8 weights, fp32 accumulation): the tiles multiply on the bf16 matrix
    # core with three exact bf16 terms per activation, so the same product takes a fraction of the fp32 GEMM's time
    for (m_, n_, k_) in ((4096, 4096, 4096), (1024, 4096, 4096)):
        xa = hip.array(rng.normal(0, 1, (m_, k_)).astype(np.float32))
        wq = hip.array(rng.integers(-127, 128, (n_, k_), dtype=np.int8))
        wsc = hip.array(rng.uniform(1e-3, 1e-2, n_).astype(np.float32))
        wf = hip.array(rng.uniform(-1, 1, (k_, n_)).astype(np.float32))
        oq = hip.empty((m_, n_))
        _, ms = time_calls(hip, lambda: hip.check(hip.L.axhip_qgemm_w8a32(xa.ptr, wq.ptr, wsc.ptr, oq.ptr, m_, n_, k_)), seconds=0.4)
        kern = hip.last_kernel()
        _, ms32 = time_calls(hip, lambda: hip.check(hip.L.axhip_sgemm(
            0, 0, m_, n_, k_, 1.0, xa.ptr, k_, wf.ptr, n_, 0.0, oq.ptr, n_, None, 0)), seconds=0.4)
        tf = 2 * m_ * n_ * k_ / ms / 1e9
        res[f"w8a32_gemm_{m_}x{n_}x{k_}"] = {"us": ms * 1e3, "equivalent_TFLOP/s": tf, "fp32_gemm_us": ms32 * 1e3,
                                             "speedup_over_fp32": ms32 / ms,
                                             "frac_of_bf16_mfma_peak_at_3_terms": 3 * tf / 2500.0, "kernel": kern}
        del xa, wq, wsc, wf, oq

    # config 3: FFN block 2048 x 1024 x 4096, bias + GELU fused into GEMM1, bias into GEMM2
    x, w1 = f32((2048, 1024), (1024, 4096))
    w2 = hip.array(rng.normal(0, 0.02, (4096, 1024)).astype(np.float32))
    b1 = hip.array(rng.normal(0, 0.02, 4096).astype(np.float32))
    b2 = hip.array(rng.normal(0, 0.02, 1024).astype(np.float32))
    hbuf, y = hip.empty((2048, 4096)), hip.empty((2048, 1024))

    def ffn():
        hip.check(hip.L.axhip_sgemm(0, 0, 2048, 4096, 1024, 1.0, x.ptr, 1024, w1.ptr, 4096, 0.0,
                                    hbuf.ptr, 4096, b1.ptr, 2))
        hip.check(hip.L.axhip_sgemm(0, 0, 2048, 1024, 4096, 1.0, hbuf.ptr, 4096, w2.ptr, 1024, 0.0,
                                    y.ptr, 1024, b2.ptr, 0))
    _, ms = time_calls(hip, ffn)
    tf = 2 * 2 * 2048 * 1024 * 4096 / ms / 1e9
    res["fp32_ffn_2048x1024x4096"] = {"us": ms * 1e3, "TFLOP/s": tf,
                                      "frac_of_fp32_mfma_peak": tf / PEAK_FP32_TFLOPS}
    result_line("axhip", "f32_ffn_2048x1024x4096", "gflops", tf * 1e3)
    configs.append(config_record("configs[3]: fp32 FFN block, tokens 2048, d_model 1024, d_ff 4096: GEMM + bias + GELU fused, GEMM + bias",
                                 2 * 2 * 2048 * 1024 * 4096, 4 * (2048 * 1024 + 1024 * 4096 + 2 * 2048 * 4096 + 4096 * 1024 + 2048 * 1024),
                                 ms * 1e-3, "mfma_fp32", "two launches of " + hip.last_kernel(), key="config3"))

    # dense backward of the FFN block's first layer (X [2048,1024], W [1024,4096], dY [2048,4096]):
    # dA = dY W^T (NT), dW = X^T dY (TN), dBias = sum(dY, 0)
    dyb = hip.array(rng.normal(0, 1, (2048, 4096)).astype(np.float32))
    da, dw, dbias = hip.empty((2048, 1024)), hip.empty((1024, 4096)), hip.empty((4096,))
    L = hip.L
    _, ms = time_calls(hip, lambda: hip.check(L.axhip_sgemm(0, 1, 2048, 1024, 4096, 1.0, dyb.ptr, 4096, w1.ptr, 4096,
                                                           0.0, da.ptr, 1024, None, 0)))
    k_nt = hip.last_kernel()
    _, ms2 = time_calls(hip, lambda: hip.check(L.axhip_sgemm(1, 0, 1024, 4096, 2048, 1.0, x.ptr, 1024, dyb.ptr, 4096,
                                                            0.0, dw.ptr, 4096, None, 0)))
    k_tn = hip.last_kernel()
    _, ms3 = time_calls(hip, lambda: hip.check(L.axhip_sum_axis(dyb.ptr, 1, 2048, 4096, dbias.ptr)))
    fl = 2 * 2048 * 1024 * 4096
    res["fp32_dense_backward_2048x1024x4096"] = {
        "dA_nt_us": ms * 1e3, "dA_TFLOP/s": fl / ms / 1e9, "dA_kernel": k_nt,
        "dW_tn_us": ms2 * 1e3, "dW_TFLOP/s": fl / ms2 / 1e9, "dW_kernel": k_tn,
        "dBias_us": ms3 * 1e3, "dBias_GB/s": 4 * 2048 * 4096 / ms3 / 1e6,
        "frac_of_fp32_mfma_peak": 2 * fl / (ms + ms2) / 1e9 / PEAK_FP32_TFLOPS}
    del dyb, da, dw
    del x, w1, w2, hbuf, y

    # config 2: int8 M=256, N=K=4096 (HBM/latency-bound)
    xi, wi = hip.array(rand_i8(rng, (256, 4096))), hip.array(rand_i8(rng, (4096, 4096)))
    ws = hip.array(rng.uniform(1e-3, 1e-2, 4096).astype(np.float32))
    bi = hip.array(rng.normal(0, 0.02, 4096).astype(np.float32))
    oi = hip.empty((256, 4096))
    _, ms = time_calls(hip, lambda: hip.check(hip.L.axhip_qgemm_w8a8(
        xi.ptr, 0.01, wi.ptr, ws.ptr, bi.ptr, 0, oi.ptr, None, 256, 4096, 4096)))
    nbytes = 4096 * 4096 + 256 * 4096 + 4 * 256 * 4096 + 8 * 4096
    res["int8_qgemm_256x4096x4096"] = {"us": ms * 1e3, "TOP/s": 2 * 256 * 4096 * 4096 / ms / 1e9,
                                       "GB/s": nbytes / ms / 1e6,
                                       "frac_of_hbm_peak": nbytes / ms / 1e6 / PEAK_HBM_GBS,
                                       "kernel": hip.last_kernel()}
    # the same with 36 weight matrices in rotation (604 MB), so that every launch meets its weights in HBM
    # rather than in the 256 MB Infinity Cache, as a layer of a large model does
    wsets = [wi] + [hip.array(rand_i8(rng, (4096, 4096))) for _ in range(35)]
    turn = [0]

    def config2_rotating():
        turn[0] = (turn[0] + 1) % len(wsets)
        hip.check(hip.L.axhip_qgemm_w8a8(xi.ptr, 0.01, wsets[turn[0]].ptr, ws.ptr, bi.ptr, 0, oi.ptr, None, 256, 4096, 4096))
    _, ms = time_calls(hip, config2_rotating)
    res["int8_qgemm_256x4096x4096"]["weights_from_hbm_us"] = ms * 1e3
    configs.append(config_record("configs[2]: int8 W8A8 GEMM M=256, N=K=4096, dequantize + bias epilogue; weights read from HBM "
                                 "(36 weight matrices in rotation)", 2 * 256 * 4096 * 4096, nbytes, ms * 1e-3, "hbm",
                                 res["int8_qgemm_256x4096x4096"]["kernel"], key="config2",
                                 time_s_weights_in_cache=res["int8_qgemm_256x4096x4096"]["us"] * 1e-6))
    del xi, wi, oi, wsets

    # one round of fp32 tiles over a long K (256 tiles, K = 4096), operands cached and in rotation (9 x 67 MB)
    a1 = hip.array(rng.normal(0, 1, (256, 4096)).astype(np.float32))
    bsets = [hip.array(rng.normal(0, 0.02, (4096, 4096)).astype(np.float32)) for _ in range(9)]
    c1 = hip.empty((256, 4096))
    _, ms = time_calls(hip, lambda: hip.check(hip.L.axhip_sgemm(0, 0, 256, 4096, 4096, 1.0, a1.ptr, 4096, bsets[0].ptr, 4096, 0.0,
                                                                c1.ptr, 4096, None, 0)))

    def one_round_rotating():
        turn[0] = (turn[0] + 1) % len(bsets)
        hip.check(hip.L.axhip_sgemm(0, 0, 256, 4096, 4096, 1.0, a1.ptr, 4096, bsets[turn[0]].ptr, 4096, 0.0, c1.ptr, 4096, None, 0))
    _, ms2 = time_calls(hip, one_round_rotating)
    fl = 2 * 256 * 4096 * 4096
    res["fp32_gemm_256x4096x4096"] = {"us": ms * 1e3, "TFLOP/s": fl / ms / 1e9, "weights_from_hbm_us": ms2 * 1e3,
                                      "weights_from_hbm_TFLOP/s": fl / ms2 / 1e9, "kernel": hip.last_kernel()}
    del a1, bsets, c1

    # config 1: bs=1 MLP 784 -> 4096 -> 4096 -> 10 through the skinny-M route, M in {1,2,4,8}.
    # 8 rotating weight sets (641 MB) so every pass streams from HBM, not the 256 MB Infinity Cache.
    sets = []
    for _ in range(8):
        sets.append((hip.array(rng.uniform(-0.09, 0.09, (784, 4096)).astype(np.float32)),
                     hip.array(rng.uniform(-0.04, 0.04, (4096, 4096)).astype(np.float32)),
                     hip.array(rng.uniform(-0.04, 0.04, (4096, 10)).astype(np.float32))))
    zeros = hip.empty((4096,))
    weight_bytes = 4 * (784 * 4096 + 4096 * 4096 + 4096 * 10)
    mlp = {}
    for M in (1, 2, 4, 8):
        xin = hip.array(rng.uniform(0, 1, (M, 784)).astype(np.float32))
        h1, h2, yo = hip.empty((M, 4096)), hip.empty((M, 4096)), hip.empty((M, 10))
        it = [0]

        def mlp_step():
            # what Sequential's forward issues for this network: the first layer, then the second with the
            # 10-wide output layer riding on it (two launches)
            w1_, w2_, w3_ = sets[it[0] % 8]
            it[0] += 1
            L = hip.L
            hip.check(L.axhip_sgemm(0, 0, M, 4096, 784, 1.0, xin.ptr, 784, w1_.ptr, 4096, 0.0, h1.ptr, 4096, zeros.ptr, 1))
            hip.check(L.axhip_sgemm_skinny_head(M, 4096, 4096, h1.ptr, 4096, w2_.ptr, 4096, None, 4096, zeros.ptr, 1,
                                                10, w3_.ptr, zeros.ptr, 0, yo.ptr))

        def mlp_step_by_layer():
            w1_, w2_, w3_ = sets[it[0] % 8]
            it[0] += 1
            L = hip.L
            hip.check(L.axhip_sgemm(0, 0, M, 4096, 784, 1.0, xin.ptr, 784, w1_.ptr, 4096, 0.0, h1.ptr, 4096, zeros.ptr, 1))
            hip.check(L.axhip_sgemm(0, 0, M, 4096, 4096, 1.0, h1.ptr, 4096, w2_.ptr, 4096, 0.0, h2.ptr, 4096, zeros.ptr, 1))
            hip.check(L.axhip_sgemm(0, 0, M, 10, 4096, 1.0, h2.ptr, 4096, w3_.ptr, 10, 0.0, yo.ptr, 10, zeros.ptr, 0))

        def layer2_only():
            _, w2_, _ = sets[it[0] % 8]
            it[0] += 1
            hip.check(hip.L.axhip_sgemm(0, 0, M, 4096, 4096, 1.0, h1.ptr, 4096, w2_.ptr, 4096, 0.0, h2.ptr, 4096, zeros.ptr, 1))

        _, ms = time_calls(hip, mlp_step)
        _, ms3 = time_calls(hip, mlp_step_by_layer)
        _, ms2 = time_calls(hip, layer2_only)
        gbs, gbs2 = weight_bytes / ms / 1e6, 4 * 4096 * 4096 / ms2 / 1e6
        mlp[f"M{M}"] = {"mlp_us": ms * 1e3, "mlp_GB/s": gbs, "mlp_frac_of_hbm_peak": gbs / PEAK_HBM_GBS,
                        "mlp_three_launches_us": ms3 * 1e3,
                        "layer2_us": ms2 * 1e3, "layer2_GB/s": gbs2,
                        "layer2_frac_of_hbm_peak": gbs2 / PEAK_HBM_GBS}
        result_line("axhip", f"mlp3_bs{M}", "latency_us", ms * 1e3)
        if M in (1, 8):
            configs.append(config_record(f"configs[1]: fp32 MLP 784-4096-4096-10 at M={M} through the skinny-M route, weights read from "
                                         f"HBM (8 weight sets in rotation); two launches, the 10-wide layer rides on the second",
                                         2 * M * (784 * 4096 + 4096 * 4096 + 4096 * 10), weight_bytes + 4 * M * (784 + 2 * 4096 + 10),
                                         ms * 1e-3, "hbm", "sgemm_skinny_vec4 + sgemm_skinny_with_head", key=f"config1_M{M}",
                                         layer2_alone_time_s=ms2 * 1e-3,
                                         layer2_alone_frac_of_hbm_peak=gbs2 / PEAK_HBM_GBS))
    res["skinny_mlp_784_4096_4096_10"] = mlp
    del sets

    # the same route on one large layer (8192 x 8192 fp32, 268 MB of weights, 4 rotating sets): what the
    # kernel streams at once a launch's fixed cost (start-up, split-K join, about 5 us) is small beside its traffic
    big_sets = [hip.array(rng.uniform(-0.03, 0.03, (8192, 8192)).astype(np.float32)) for _ in range(4)]
    bias8k = hip.empty((8192,))
    big = {}
    for M in (1, 8):
        xin = hip.array(rng.uniform(0, 1, (M, 8192)).astype(np.float32))
        yb = hip.empty((M, 8192))
        it = [0]

        def big_step():
            w_ = big_sets[it[0] % 4]
            it[0] += 1
            hip.check(hip.L.axhip_sgemm(0, 0, M, 8192, 8192, 1.0, xin.ptr, 8192, w_.ptr, 8192, 0.0, yb.ptr, 8192, bias8k.ptr, 1))

        _, ms = time_calls(hip, big_step)
        gbs = 4 * 8192 * 8192 / ms / 1e6
        big[f"M{M}"] = {"us": ms * 1e3, "GB/s": gbs, "frac_of_hbm_peak": gbs / PEAK_HBM_GBS, "kernel": hip.last_kernel()}
    res["skinny_layer_8192x8192"] = big
    del big_sets

    # what a skinny launch costs before and beyond its bytes: time against K at N = 4096, M = 1 (weights from
    # HBM, rotating sets of at least 600 MB), least-squares line  time = fixed + bytes / rate
    pts = []
    for K in (512, 1024, 2048, 4096, 8192, 16384):
        nset = max(3, int(600e6 / (K * 4096 * 4)) + 1)
        base = rng.uniform(-0.03, 0.03, (K, 4096)).astype(np.float32)      # the same values in every set: only the addresses differ
        wsets = [hip.array(base) for _ in range(nset)]
        xin, yo_ = hip.array(rng.uniform(0, 1, (1, K)).astype(np.float32)), hip.empty((1, 4096))
        it = [0]

        def line_step():
            w_ = wsets[it[0] % nset]
            it[0] += 1
            hip.check(hip.L.axhip_sgemm(0, 0, 1, 4096, K, 1.0, xin.ptr, K, w_.ptr, 4096, 0.0, yo_.ptr, 4096, zeros.ptr, 1))

        _, ms = time_calls(hip, line_step, seconds=0.15)
        pts.append((K * 4096 * 4, ms * 1e3))
        del wsets
    xs_, ys_ = np.array([p[0] for p in pts], np.float64), np.array([p[1] for p in pts], np.float64)
    slope, fixed = np.polyfit(xs_, ys_, 1)
    res["skinny_time_vs_bytes_M1_N4096"] = {
        "points_MB_us": [[b / 1e6, t] for b, t in pts], "fixed_us": float(fixed), "marginal_GB/s": float(1e-3 / slope),
        "marginal_frac_of_hbm_peak": float(1e-3 / slope / PEAK_HBM_GBS), "launch_floor_us": None}

    # config 4b: strided-batched attention-shaped products, 512 heads of [512,64]
    Bn, S, D = 512, 512, 64
    q = hip.array(rng.normal(0, 1, (Bn, S, D)).astype(np.float32))
    k = hip.array(rng.normal(0, 1, (Bn, S, D)).astype(np.float32))
    v = hip.array(rng.normal(0, 1, (Bn, S, D)).astype(np.float32))
    s, o = hip.empty((Bn, S, S)), hip.empty((Bn, S, D))
    _, ms = time_calls(hip, lambda: hip.check(hip.L.axhip_sgemm_strided_batched(
        0, 1, S, S, D, 1.0, q.ptr, D, S * D, k.ptr, D, S * D, 0.0, s.ptr, S, S * S, Bn)))
    nbytes = 4 * (2 * Bn * S * D + Bn * S * S)
    res["fp32_batched_qkt"] = {"us": ms * 1e3, "TFLOP/s": 2 * Bn * S * S * D / ms / 1e9,
                               "GB/s": nbytes / ms / 1e6, "frac_of_hbm_peak": nbytes / ms / 1e6 / PEAK_HBM_GBS,
                               "kernel": hip.last_kernel()}
    _, ms = time_calls(hip, lambda: hip.check(hip.L.axhip_sgemm_strided_batched(
        0, 0, S, D, S, 1.0, s.ptr, S, S * S, v.ptr, D, S * D, 0.0, o.ptr, D, S * D, Bn)))
    res["fp32_batched_pv"] = {"us": ms * 1e3, "TFLOP/s": 2 * Bn * S * S * D / ms / 1e9,
                              "GB/s": nbytes / ms / 1e6, "frac_of_hbm_peak": nbytes / ms / 1e6 / PEAK_HBM_GBS}
    res["fp32_batched_pv"]["kernel"] = hip.last_kernel()
    # arithmetic intensity 25.6 flop/byte against a machine balance of 19.7: the roofline prices both at the matrix cores
    # (109 us); the time the bytes alone take at 8 TB/s (84 us) is given beside it
    for key, name, what in (("config4b_qkt", "fp32_batched_qkt", "S = Q K^T, [512,64] x [512,64]^T"),
                            ("config4b_pv", "fp32_batched_pv", "O = S V, [512,512] x [512,64]")):
        t = res[name]["us"] * 1e-6
        configs.append(config_record(f"configs[4] (b): strided-batched fp32 GEMM over 512 heads, {what}", 2 * Bn * S * S * D, nbytes, t,
                                     "mfma_fp32", res[name]["kernel"], key=key, frac_of_hbm_peak=nbytes / t / 1e9 / PEAK_HBM_GBS))
    # fused attention forward over the same heads (both products and the softmax in one kernel,
    # no [512,512] score matrix in memory); flops counted as the two GEMMs'
    l = hip.empty((Bn, S))
    _, ms = time_calls(hip, lambda: hip.check(hip.L.axhip_sdpa_fwd(q.ptr, k.ptr, v.ptr, o.ptr, l.ptr, Bn, S, D,
                                                                  0.125, 0)))
    res["fp32_sdpa_fwd_512x512x64"] = {"us": ms * 1e3, "TFLOP/s": 4 * Bn * S * S * D / ms / 1e9,
                                       "frac_of_fp32_mfma_peak": 4 * Bn * S * S * D / ms / 1e9 / PEAK_FP32_TFLOPS,
                                       "kernel": hip.last_kernel(),
                                       "unfused_us": res["fp32_batched_qkt"]["us"] + res["fp32_batched_pv"]["us"]}
    _, ms = time_calls(hip, lambda: hip.check(hip.L.axhip_sdpa_fwd(q.ptr, k.ptr, v.ptr, o.ptr, l.ptr, Bn, S, D,
                                                                  0.125, 1)))
    res["fp32_sdpa_fwd_causal_512x512x64"] = {"us": ms * 1e3, "useful_TFLOP/s": 2 * Bn * S * S * D / ms / 1e9,
                                              "kernel": hip.last_kernel()}
    del q, k, v, s, o, l

    # the HBM-bound slots around the FFN (an encoder block's residual add, layer norm, softmax) and
    # the optimizer pass: algorithmic bytes = every operand read once + every result written once
    stream = {}
    R, Dm = 16384, 4096                                     # 268 MB per [R, Dm] tensor
    xa, xb = hip.array(rng.normal(0, 1, (R, Dm)).astype(np.float32)), hip.array(rng.normal(0, 1, (R, Dm)).astype(np.float32))
    xo, vec = hip.empty((R, Dm)), hip.array(rng.normal(1, 0.1, (Dm,)).astype(np.float32))
    rowv, colv = hip.empty((R,)), hip.empty((Dm,))
    full = 4 * R * Dm
    shape2 = (C.c_int64 * 2)(R, Dm)
    dense2, bcast2 = (C.c_int64 * 2)(Dm, 1), (C.c_int64 * 2)(0, 1)

    def rate(name, nbytes, fn):
        _, ms = time_calls(hip, fn)
        stream[name] = {"us": ms * 1e3, "GB/s": nbytes / ms / 1e6, "frac_of_hbm_peak": nbytes / ms / 1e6 / PEAK_HBM_GBS}

    rate("add_same_shape", 3 * full, lambda: hip.check(hip.L.axhip_binary(0, xa.ptr, xb.ptr, xo.ptr, 2, shape2, dense2, dense2)))
    rate("add_row_vector", 2 * full, lambda: hip.check(hip.L.axhip_binary(0, xa.ptr, vec.ptr, xo.ptr, 2, shape2, dense2, bcast2)))
    rate("tanh", 2 * full, lambda: hip.check(hip.L.axhip_unary(7, xa.ptr, xo.ptr, R * Dm, 0.0)))
    rate("max_axis0", full, lambda: hip.check(hip.L.axhip_reduce_axis(2, xa.ptr, 1, R, Dm, colv.ptr)))
    rate("max_axis1", full, lambda: hip.check(hip.L.axhip_reduce_axis(2, xa.ptr, R, Dm, 1, rowv.ptr)))
    rate("sum_axis0", full, lambda: hip.check(hip.L.axhip_reduce_axis(0, xa.ptr, 1, R, Dm, colv.ptr)))
    rate("softmax_rows_4096", 2 * full, lambda: hip.check(hip.L.axhip_softmax_rows(xa.ptr, xo.ptr, R, Dm)))
    rate("softmax_rows_512", 2 * full, lambda: hip.check(hip.L.axhip_softmax_rows(xa.ptr, xo.ptr, R * 8, Dm // 8)))
    rate("layernorm_4096", 2 * full, lambda: hip.check(hip.L.axhip_layernorm_fwd(xa.ptr, vec.ptr, vec.ptr, xo.ptr, None, None,
                                                                                 R, Dm, 1e-5)))
    rate("layernorm_1024", 2 * full, lambda: hip.check(hip.L.axhip_layernorm_fwd(xa.ptr, vec.ptr, vec.ptr, xo.ptr, None, None,
                                                                                 R * 4, Dm // 4, 1e-5)))
    hip.check(hip.L.axhip_fill_f32(xo.ptr, 0.0, R * Dm))
    m2 = hip.array(np.zeros((R, Dm), np.float32))
    rate("adam_update", 7 * full, lambda: hip.check(hip.L.axhip_adam_update(xa.ptr, xb.ptr, xo.ptr, m2.ptr, R * Dm, 1e-3, 0.9,
                                                                            0.999, 1e-8, 0.01, 0.1, 0.001, 1)))
    res["streaming_slots_16384x4096"] = stream
    del xa, xb, xo, vec, rowv, colv, m2

    # what this box charges per launch, whatever the kernel does: back-to-back fills of 64 floats on the
    # stream.  The latency-bound figures above and below (bs=1 layers, few-tile GEMMs, the encoder) are
    # read against it, as the streaming ones are against the read / copy rates measured just above.
    tiny = hip.empty((64,))
    _, ms = time_calls(hip, lambda: hip.check(hip.L.axhip_fill_f32(tiny.ptr, 1.0, 64)))
    res["launch_floor_us"] = ms * 1e3
    res["skinny_time_vs_bytes_M1_N4096"]["launch_floor_us"] = ms * 1e3
    del tiny

    # the seven shapes of the reference's benchmarks/bench_qgemm.c:76-82 (fp32 GEMM against W8A32 on the
    # same weights), on device-resident operands, plus W8A8 with the activations quantized per tensor
    qshapes = {}
    for (M, N, K) in ((1, 768, 3072), (1, 3072, 768), (8, 768, 768), (32, 768, 768), (128, 4096, 1024),
                      (64, 1024, 4096), (1, 4096, 4096)):
        a = hip.array(rng.uniform(-1, 1, (M, K)).astype(np.float32))
        wt = hip.array(rng.uniform(-1, 1, (K, N)).astype(np.float32))          # [K, N] for the fp32 GEMM
        wq = hip.array(rand_i8(rng, (N, K)))
        ws = hip.array(rng.uniform(1e-3, 1e-2, N).astype(np.float32))
        xq = hip.array(rand_i8(rng, (M, K)))
        out = hip.empty((M, N))
        _, t_fp = time_calls(hip, lambda: hip.check(hip.L.axhip_sgemm(0, 0, M, N, K, 1.0, a.ptr, K, wt.ptr, N, 0.0, out.ptr, N,
                                                                      None, 0)))
        _, t_q = time_calls(hip, lambda: hip.check(hip.L.axhip_qgemm_w8a32(a.ptr, wq.ptr, ws.ptr, out.ptr, M, N, K)))
        _, t_8 = time_calls(hip, lambda: hip.check(hip.L.axhip_qgemm_w8a8(xq.ptr, 0.02, wq.ptr, ws.ptr, None, 0, out.ptr, None,
                                                                         M, N, K)))
        qshapes[f"{M}x{N}x{K}"] = {"fp32_us": t_fp * 1e3, "w8a32_us": t_q * 1e3, "w8a8_us": t_8 * 1e3,
                                   "w8a32_speedup_over_fp32": t_fp / t_q, "w8a8_kernel": hip.last_kernel()}
        # the same two with the weights in rotation (about 600 MB of each kind), i.e. read from HBM on every call as the
        # reference's CPU benchmark reads them from DRAM: the case a quarter of the weight bytes is for
        nset = max(2, min(64, int(600e6 // (4 * N * K))))
        wts = [wt] + [hip.array(rng.uniform(-1, 1, (K, N)).astype(np.float32)) for _ in range(nset - 1)]
        wqs = [wq] + [hip.array(rand_i8(rng, (N, K))) for _ in range(4 * nset - 1)]
        turn = [0, 0]

        def fp_rot():
            turn[0] = (turn[0] + 1) % len(wts)
            hip.check(hip.L.axhip_sgemm(0, 0, M, N, K, 1.0, a.ptr, K, wts[turn[0]].ptr, N, 0.0, out.ptr, N, None, 0))

        def q_rot():
            turn[1] = (turn[1] + 1) % len(wqs)
            hip.check(hip.L.axhip_qgemm_w8a32(a.ptr, wqs[turn[1]].ptr, ws.ptr, out.ptr, M, N, K))
        _, t_fp = time_calls(hip, fp_rot, seconds=0.2)
        _, t_q = time_calls(hip, q_rot, seconds=0.2)
        qshapes[f"{M}x{N}x{K}"].update({"fp32_weights_from_hbm_us": t_fp * 1e3, "w8a32_weights_from_hbm_us": t_q * 1e3,
                                        "w8a32_speedup_weights_from_hbm": t_fp / t_q})
        del wts, wqs
    res["bench_qgemm_shapes"] = qshapes

    # config 1 again, end to end through the public API the reference's users call: ax_layer_forward of a
    # Sequential (Dense 784-4096-4096-10 with ReLU) on a device tensor, output tensor created and destroyed
    # every call — so this figure includes the host code and the device allocator, not only the kernels
    from axiom_amd.axiom import Axiom
    ax = Axiom()
    L = ax.L
    if L.ax_init() == 0:
        L.ax_set_default_device(2)
        L.ax_set_seed(1)
        seq = L.ax_sequential_create()
        for (i, o, relu) in ((784, 4096, True), (4096, 4096, True), (4096, 10, False)):
            L.ax_sequential_add(seq, L.ax_dense_create(i, o, True))
            if relu:
                L.ax_sequential_add(seq, L.ax_relu_layer_create())
        api = {}
        for M in (1, 8):
            tx = ax.from_numpy(rng.uniform(0, 1, (M, 784)).astype(np.float32))

            def forward():
                y = L.ax_layer_forward(seq, tx)
                L.ax_tensor_destroy(y)

            for _ in range(50):
                forward()
            hip.sync()
            n = 2000
            t0 = time.perf_counter()
            for _ in range(n):
                forward()
            hip.sync()
            api[f"M{M}_us_per_forward"] = (time.perf_counter() - t0) * 1e6 / n
            ax.free(tx)
        L.ax_layer_destroy(seq)
        res["mlp3_through_ax_layer_forward"] = api

        # the encoder of the reference's bench_transformer.c (:20-53): 6 x [LayerNorm, MHA(4 heads),
        # LayerNorm, Dense 256-1024, GELU, Dense 1024-256], LayerNorm, Dense 256-1024 on [8,128,256];
        # forward only, every layer on the device (LayerNorm, fused attention, GEMM epilogues)
        enc = L.ax_sequential_create()
        for _ in range(6):
            L.ax_sequential_add(enc, L.ax_layernorm_create(256, 1e-5))
            L.ax_sequential_add(enc, L.ax_mha_create(256, 4, True, False))
            L.ax_sequential_add(enc, L.ax_layernorm_create(256, 1e-5))
            L.ax_sequential_add(enc, L.ax_dense_create(256, 1024, True))
            L.ax_sequential_add(enc, L.ax_gelu_layer_create())
            L.ax_sequential_add(enc, L.ax_dense_create(1024, 256, True))
        L.ax_sequential_add(enc, L.ax_layernorm_create(256, 1e-5))
        L.ax_sequential_add(enc, L.ax_dense_create(256, 1024, True))
        tx = ax.from_numpy(rng.uniform(-0.1, 0.1, (8, 128, 256)).astype(np.float32))

        def enc_forward():
            y = L.ax_layer_forward(enc, tx)
            if not y:
                raise RuntimeError("encoder forward failed: %s" % (ax.err(),))
            L.ax_tensor_destroy(y)

        for _ in range(20):
            enc_forward()
        hip.sync()
        n = 300
        t0 = time.perf_counter()
        for _ in range(n):
            enc_forward()
        hip.sync()
        res["encoder6_forward_8x128x256"] = {"us_per_forward": (time.perf_counter() - t0) * 1e6 / n,
                                             "layers": 38}
        ax.free(tx)
        L.ax_layer_destroy(enc)
        L.ax_set_default_device(0)
    res["configs"] = configs
    return res


def counter_probe(hip, case, repeat=1):
    """Workloads for per-dispatch hardware counters and kernel traces: a few launches of the kernels of
    one case, then for scale the elementwise ReLU kernel over 64 Mi floats, which reads 256 MiB and
    writes 256 MiB exactly once (a plain copy as far as memory traffic goes).
      headline  W8A8 8192^3
      skinny    the 4096 x 4096 layer of the bs=1 MLP at M = 1 and M = 8 over 8 rotating weight sets
                (537 MB, so every launch streams its 67.1 MB from HBM and not from the Infinity Cache)
      gemm1024  fp32 1024^3
      fp32      the FFN pair 2048 x 1024 x 4096 (bias + GELU fused into the first GEMM) and back
      config2   W8A8 M = 256, N = K = 4096
      attention batched Q K^T and P V over 512 heads of [512, 64], then the fused forward
      w8a32     W8A32 with many rows, 4096^3 and 1024 x 4096 x 4096 (bf16 matrix core, three terms per activation)"""
    rng = np.random.default_rng(0)
    L = hip.L
    reps = 3 * repeat                # `repeat` > 1 (--probe-repeat): long enough for sustained clocks, for kernel traces
    if case == "headline":
        M = N = K = 8192
        x, w = hip.array(rand_i8(rng, (M, K))), hip.array(rand_i8(rng, (N, K)))
        ws = hip.array(rng.uniform(1e-3, 1e-2, N).astype(np.float32))
        bias = hip.array(rng.normal(0.0, 0.02, N).astype(np.float32))
        out = hip.empty((M, N))
        for _ in range(reps):
            hip.check(L.axhip_qgemm_w8a8(x.ptr, 0.01, w.ptr, ws.ptr, bias.ptr, 0, out.ptr, None, M, N, K))
        what = f"{reps} x qgemm_w8a8 8192^3 ({hip.last_kernel()})"
    elif case == "skinny":
        sets = [hip.array(rng.uniform(-0.04, 0.04, (4096, 4096)).astype(np.float32)) for _ in range(8)]
        zeros = hip.empty((4096,))
        what = ""
        for M in (1, 8):
            xin, h2 = hip.array(rng.uniform(0, 1, (M, 4096)).astype(np.float32)), hip.empty((M, 4096))
            for i in range(16 * repeat):
                hip.check(L.axhip_sgemm(0, 0, M, 4096, 4096, 1.0, xin.ptr, 4096, sets[i % 8].ptr, 4096, 0.0,
                                        h2.ptr, 4096, zeros.ptr, 1))
            what += f"{16 * repeat} x sgemm M={M} 4096x4096 ({hip.last_kernel()}) "
    elif case == "gemm1024":
        a = hip.array(rng.uniform(-1, 1, (1024, 1024)).astype(np.float32))
        b = hip.array(rng.uniform(-1, 1, (1024, 1024)).astype(np.float32))
        c = hip.empty((1024, 1024))
        for _ in range(16 * repeat):
            hip.check(L.axhip_sgemm(0, 0, 1024, 1024, 1024, 1.0, a.ptr, 1024, b.ptr, 1024, 0.0, c.ptr, 1024, None, 0))
        what = f"{16 * repeat} x sgemm 1024^3 ({hip.last_kernel()})"
    elif case == "fp32":
        what = ""
        x = hip.array(rng.normal(0, 1, (2048, 1024)).astype(np.float32))
        w1 = hip.array(rng.normal(0, 0.02, (1024, 4096)).astype(np.float32))
        w2 = hip.array(rng.normal(0, 0.02, (4096, 1024)).astype(np.float32))
        b1 = hip.array(rng.normal(0, 0.02, 4096).astype(np.float32))
        b2 = hip.array(rng.normal(0, 0.02, 1024).astype(np.float32))
        hbuf, y = hip.empty((2048, 4096)), hip.empty((2048, 1024))
        for _ in range(8 * repeat):
            hip.check(L.axhip_sgemm(0, 0, 2048, 4096, 1024, 1.0, x.ptr, 1024, w1.ptr, 4096, 0.0, hbuf.ptr, 4096, b1.ptr, 2))
            k1 = hip.last_kernel()
            hip.check(L.axhip_sgemm(0, 0, 2048, 1024, 4096, 1.0, hbuf.ptr, 4096, w2.ptr, 1024, 0.0, y.ptr, 1024, b2.ptr, 0))
        what += f"{8 * repeat} x FFN pair ({k1}, {hip.last_kernel()})"
    elif case == "config2":
        xi, wi = hip.array(rand_i8(rng, (256, 4096))), hip.array(rand_i8(rng, (4096, 4096)))
        ws = hip.array(rng.uniform(1e-3, 1e-2, 4096).astype(np.float32))
        bi = hip.array(rng.normal(0, 0.02, 4096).astype(np.float32))
        oi = hip.empty((256, 4096))
        for _ in range(16 * repeat):
            hip.check(L.axhip_qgemm_w8a8(xi.ptr, 0.01, wi.ptr, ws.ptr, bi.ptr, 0, oi.ptr, None, 256, 4096, 4096))
        what = f"{16 * repeat} x qgemm_w8a8 256x4096x4096 ({hip.last_kernel()})"
    elif case == "attention":
        Bn, S, D = 512, 512, 64
        q, k, v = (hip.array(rng.normal(0, 1, (Bn, S, D)).astype(np.float32)) for _ in range(3))
        sc, o, l = hip.empty((Bn, S, S)), hip.empty((Bn, S, D)), hip.empty((Bn, S))
        for _ in range(reps):
            hip.check(L.axhip_sgemm_strided_batched(0, 1, S, S, D, 1.0, q.ptr, D, S * D, k.ptr, D, S * D, 0.0,
                                                    sc.ptr, S, S * S, Bn))
            k1 = hip.last_kernel()
            hip.check(L.axhip_sgemm_strided_batched(0, 0, S, D, S, 1.0, sc.ptr, S, S * S, v.ptr, D, S * D, 0.0,
                                                    o.ptr, D, S * D, Bn))
            k2 = hip.last_kernel()
            hip.check(L.axhip_sdpa_fwd(q.ptr, k.ptr, v.ptr, o.ptr, l.ptr, Bn, S, D, 0.125, 0))
        what = f"{reps} x (QK^T {k1}, PV {k2}, fused {hip.last_kernel()}) over 512 heads of [512, 64]"
    elif case == "w8a32":
        what = ""
        for (M, N, K) in ((4096, 4096, 4096), (1024, 4096, 4096)):
            xa = hip.array(rng.normal(0, 1, (M, K)).astype(np.float32))
            wq = hip.array(rand_i8(rng, (N, K)))
            ws = hip.array(rng.uniform(1e-3, 1e-2, N).astype(np.float32))
            out = hip.empty((M, N))
            for _ in range(reps):
                hip.check(L.axhip_qgemm_w8a32(xa.ptr, wq.ptr, ws.ptr, out.ptr, M, N, K))
            what += f"{reps} x qgemm_w8a32 {M}x{N}x{K} ({hip.last_kernel()}) "
    else:
        sys.exit(f"unknown counter-probe case {case!r}")
    hip.sync()
    n = 64 << 20
    src, dst = hip.empty((n,)), hip.empty((n,))
    for _ in range(3):
        hip.check(L.axhip_relu(src.ptr, dst.ptr, n))
    hip.sync()
    print(f"counter probe: {what}, then 3 x ReLU (k_unary<0>) over {n} floats", file=sys.stderr, flush=True)


DISPATCH_FP32 = [   # (M, N, K): the configurations, bench_qgemm.c:76-82, then one shape on each side of every tile / route rule
    (1024, 1024, 1024), (2048, 4096, 1024), (2048, 1024, 4096), (1, 4096, 784), (1, 4096, 4096), (8, 4096, 4096), (1, 10, 4096),
    (1, 768, 3072), (1, 3072, 768), (8, 768, 768), (32, 768, 768), (128, 4096, 1024), (64, 1024, 4096),
    (8, 8192, 8192), (9, 4096, 4096), (16, 4096, 4096), (17, 4096, 4096), (32, 4096, 4096), (33, 4096, 4096),
    (160, 11008, 4096), (224, 11008, 4096), (512, 1024, 1024), (576, 1024, 1024), (1280, 960, 2048), (1024, 256, 256),
    (128, 4096, 2048), (768, 1024, 4096), (1024, 1024, 4096), (256, 4096, 4096), (2048, 2048, 2048), (1920, 2048, 2048),
    (4096, 4096, 4096), (500, 4096, 4096), (256, 4096, 784), (4000, 4000, 4000)]
DISPATCH_W8A8 = [
    (256, 4096, 4096), (8192, 8192, 8192), (1, 768, 3072), (1, 3072, 768), (8, 768, 768), (32, 768, 768), (128, 4096, 1024),
    (64, 1024, 4096), (1, 4096, 4096), (4, 4096, 4096), (5, 4096, 4096), (100, 4096, 4096), (128, 4096, 4096), (128, 16384, 4096),
    (512, 4096, 4096), (1024, 4096, 4096), (1024, 4096, 1024), (2048, 2048, 4096), (2048, 2048, 8192), (2048, 4096, 4096),
    (2304, 2304, 8192), (4096, 4096, 4096), (64, 64, 8192), (256, 2048, 8192), (8000, 8000, 8192), (2000, 2000, 2000)]
DISPATCH_W8A32 = [
    (1, 768, 3072), (1, 3072, 768), (8, 768, 768), (32, 768, 768), (128, 4096, 1024), (64, 1024, 4096), (1, 4096, 4096),
    (4, 4096, 4096), (5, 4096, 4096), (6, 4096, 4096), (7, 4096, 4096), (8, 4096, 4096), (4, 11008, 4096), (6, 1024, 4096),
    (32, 4096, 4096), (256, 4096, 4096), (512, 4096, 4096), (768, 11008, 4096), (1024, 4096, 4096), (4096, 4096, 4096),
    (1000, 4096, 4096)]


def dispatch_table(hip):
    """Shape -> kernel -> microseconds for a fixed list of shapes, one line each: the five configurations, the seven shapes
    of the reference's benchmarks/bench_qgemm.c:76-82 and one shape on each side of the rules that pick a tile, a split or
    a route (the counterpart of benchmarks/bench_gemm_suite.c:44-63).  Operands stay the same from launch to launch (cached
    where they fit the caches).  Re-run after any change to a rule: on one box, a line that moves by more than 5 % is a
    finding."""
    rng = np.random.default_rng(7)
    L = hip.L
    print(f"# device {L.axhip_device_name().decode()}; us per launch, sustained over >= 0.1 s of launches", flush=True)
    print(f"# {'kind':6s} {'M':>5s} {'N':>6s} {'K':>6s}  {'us':>9s}  kernel", flush=True)

    def line(kind, M, N, K, fn):
        fn()
        kern = hip.last_kernel()
        _, ms = time_calls(hip, fn, seconds=0.1)
        print(f"  {kind:6s} {M:5d} {N:6d} {K:6d}  {ms * 1e3:9.2f}  {kern}", flush=True)

    for (M, N, K) in DISPATCH_FP32:
        a = hip.array(rng.uniform(-1, 1, (M, K)).astype(np.float32))
        b = hip.array(rng.uniform(-1, 1, (K, N)).astype(np.float32))
        c = hip.empty((M, N))
        line("fp32", M, N, K, lambda: hip.check(L.axhip_sgemm(0, 0, M, N, K, 1.0, a.ptr, K, b.ptr, N, 0.0, c.ptr, N, None, 0)))
        del a, b, c
    Bn, S, D = 512, 512, 64
    q, k, v = (hip.array(rng.normal(0, 1, (Bn, S, D)).astype(np.float32)) for _ in range(3))
    sc, o = hip.empty((Bn, S, S)), hip.empty((Bn, S, D))
    line("fp32nt", S, S, D, lambda: hip.check(L.axhip_sgemm_strided_batched(0, 1, S, S, D, 1.0, q.ptr, D, S * D, k.ptr, D, S * D, 0.0,
                                                                         sc.ptr, S, S * S, Bn)))
    line("fp32b", S, D, S, lambda: hip.check(L.axhip_sgemm_strided_batched(0, 0, S, D, S, 1.0, sc.ptr, S, S * S, v.ptr, D, S * D, 0.0,
                                                                        o.ptr, D, S * D, Bn)))
    del q, k, v, sc, o
    for (M, N, K) in DISPATCH_W8A8:
        x, w = hip.array(rand_i8(rng, (M, K))), hip.array(rand_i8(rng, (N, K)))
        ws = hip.array(rng.uniform(1e-3, 1e-2, N).astype(np.float32))
        out = hip.empty((M, N))
        line("w8a8", M, N, K, lambda: hip.check(L.axhip_qgemm_w8a8(x.ptr, 0.01, w.ptr, ws.ptr, None, 0, out.ptr, None, M, N, K)))
        del x, w, ws, out
    for (M, N, K) in DISPATCH_W8A32:
        a = hip.array(rng.uniform(-1, 1, (M, K)).astype(np.float32))
        w = hip.array(rand_i8(rng, (N, K)))
        ws = hip.array(rng.uniform(1e-3, 1e-2, N).astype(np.float32))
        out = hip.empty((M, N))
        line("w8a32", M, N, K, lambda: hip.check(L.axhip_qgemm_w8a32(a.ptr, w.ptr, ws.ptr, out.ptr, M, N, K)))
        del a, w, ws, out


def hbm_ceiling(hip):
    """What this GPU's memory delivers to the library's plainest streaming kernels, on arrays far larger than the 256 MB
    Infinity Cache (2 GiB each): a read-only pass (sum of all elements), a write-only pass (fill), a copy (ReLU: one read,
    one write per element).  The figures the bandwidth-bound kernels' fractions of the 8 TB/s datasheet peak are to be
    read against.  One JSON line."""
    n = 512 << 20
    src, dst, one = hip.empty((n,)), hip.empty((n,)), hip.empty((1,))
    hip.check(hip.L.axhip_fill_f32(src.ptr, 0.25, n))
    res = {}
    # the same 2 GiB read as a [65536, 8192] matrix by the skinny-M route at M = 1, whose weight loads are non-temporal
    # 16-byte loads: the rate the bandwidth-bound GEMM kernels themselves can reach
    xk, yk = hip.empty((1, 65536)), hip.empty((1, 8192))
    for name, fn, nbytes in (("read_sum_all", lambda: hip.check(hip.L.axhip_sum_all(src.ptr, n, one.ptr)), 4 * n),
                             ("read_nontemporal_skinny_m1", lambda: hip.check(hip.L.axhip_sgemm(
                                 0, 0, 1, 8192, 65536, 1.0, xk.ptr, 65536, src.ptr, 8192, 0.0, yk.ptr, 8192, None, 0)), 4 * n),
                             ("write_fill", lambda: hip.check(hip.L.axhip_fill_f32(dst.ptr, 1.0, n)), 4 * n),
                             ("copy_relu", lambda: hip.check(hip.L.axhip_relu(src.ptr, dst.ptr, n)), 8 * n)):
        fn()
        _, ms = time_calls(hip, fn, seconds=0.5)
        res[name] = {"us": ms * 1e3, "GB/s": nbytes / ms / 1e6, "frac_of_8TBs": nbytes / ms / 1e6 / PEAK_HBM_GBS}
    print(json.dumps({"hbm_ceiling_2GiB_arrays": res, "device": hip.L.axhip_device_name().decode()}), flush=True)


def sample_sclk(stop, out, first_after_s=2.5, every_s=0.6):
    """Shader clock as rocm-smi reports it, sampled beside a running loop (a child process per sample, which
    only reads the driver's counters); appends MHz figures to `out` until `stop` is set."""
    import re
    import subprocess
    time.sleep(first_after_s)
    while not stop.is_set():
        try:
            txt = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=10).stdout
            m = re.search(r"sclk clock level[^(]*\((\d+)Mhz\)", txt)
            if m:
                out.append(int(m.group(1)))
        except Exception as e:                      # no rocm-smi on the box: the times are still printed
            out.append(f"rocm-smi: {e}")
            return
        time.sleep(every_s)


def sustain(hip, seconds, operands, clocks=False):
    """One kernel launched back to back for `seconds`, so that clock and power can be sampled while it runs
    (--sample-clocks does it from a thread of this process with rocm-smi): the headline over random int8
    operands or all-zero ones (same instruction stream, no switching activity in the matrix core), the
    fp32 8192^3 product over random / zero operands ("fp32", "fp32zeros"), the batched attention products
    ("qkt", "pv", each also with "zeros"), or the int8 matrix-core probe ("probe<shape>r<reads>[zeros]",
    e.g. probe32r6: the headline's MFMAs and LDS fragment reads with nothing else, axhip_probe_int8_matrix_core;
    "fprobe<shape>r<reads>[zeros]": the fp32 counterpart, axhip_probe_fp32_matrix_core).
    Prints the average time per launch about once a second."""
    M = N = K = 8192
    rng = np.random.default_rng(0)
    import threading
    stop, mhz = threading.Event(), []
    sampler = threading.Thread(target=sample_sclk, args=(stop, mhz), daemon=True) if clocks else None
    if operands.startswith("fprobe"):
        import re
        m = re.fullmatch(r"fprobe(16|32)r([0-3])(zeros)?", operands)
        if not m:
            sys.exit("fp32 probe operands are fprobe<16|32>r<0..3>[zeros]")
        shape, reads = int(m.group(1)), int(m.group(2))
        src = hip.empty((32 * 1024,)) if m.group(3) else hip.array(rng.normal(0, 1, (32 * 1024,)).astype(np.float32))
        sink = hip.empty((512 * 1024,))
        per_print = 500

        def launch():
            hip.check(hip.L.axhip_probe_fp32_matrix_core(shape, reads, src.ptr, sink.ptr))
    elif operands.startswith("probe"):
        import re
        m = re.fullmatch(r"probe(16|32)r([0-6])(zeros)?", operands)
        if not m:
            sys.exit("probe operands are probe<16|32>r<0..6>[zeros] | fprobe<16|32>r<0..3>[zeros]")
        shape, reads = int(m.group(1)), int(m.group(2))
        src = hip.empty((128 * 1024,), np.int8) if m.group(3) else hip.array(rand_i8(rng, (128 * 1024,)))
        sink = hip.empty((512 * 1024,), np.int32)
        per_print = 2000

        def launch():
            hip.check(hip.L.axhip_probe_int8_matrix_core(shape, reads, src.ptr, sink.ptr))
    elif operands.startswith("qkt") or operands.startswith("pv"):
        # the attention-shaped products of 512 heads of [512, 64]: Q K^T (writes 537 MB) or P V (reads it)
        Bn, S, D = 512, 512, 64
        zeros = operands.endswith("zeros")
        mk = (lambda shape: hip.empty(shape)) if zeros else (lambda shape: hip.array(rng.normal(0, 1, shape).astype(np.float32)))
        if operands.startswith("qkt"):
            q, k_, s_ = mk((Bn, S, D)), mk((Bn, S, D)), hip.empty((Bn, S, S))

            def launch():
                hip.check(hip.L.axhip_sgemm_strided_batched(0, 1, S, S, D, 1.0, q.ptr, D, S * D, k_.ptr, D, S * D, 0.0,
                                                            s_.ptr, S, S * S, Bn))
        else:
            p_, v_, o_ = mk((Bn, S, S)), mk((Bn, S, D)), hip.empty((Bn, S, D))

            def launch():
                hip.check(hip.L.axhip_sgemm_strided_batched(0, 0, S, D, S, 1.0, p_.ptr, S, S * S, v_.ptr, D, S * D, 0.0,
                                                            o_.ptr, D, S * D, Bn))
        per_print = 4000
    elif operands.startswith("fp32"):
        if operands == "fp32zeros":
            a, b = hip.empty((M, K)), hip.empty((K, N))
        else:
            a = hip.array(rng.standard_normal((M, K), dtype=np.float32))
            b = hip.array(rng.standard_normal((K, N), dtype=np.float32))
        out = hip.empty((M, N))
        per_print = 120

        def launch():
            hip.check(hip.L.axhip_sgemm(0, 0, M, N, K, 1.0, a.ptr, K, b.ptr, N, 0.0, out.ptr, N, None, 0))
    elif operands in ("random", "zeros"):
        if operands == "zeros":
            x, w = hip.empty((M, K), np.int8), hip.empty((N, K), np.int8)
        else:
            x, w = hip.array(rand_i8(rng, (M, K))), hip.array(rand_i8(rng, (N, K)))
        ws = hip.array(rng.uniform(1e-3, 1e-2, N).astype(np.float32))
        bias = hip.array(rng.normal(0.0, 0.02, N).astype(np.float32))
        out = hip.empty((M, N))
        per_print = 2000

        def launch():
            hip.check(hip.L.axhip_qgemm_w8a8(x.ptr, 0.01, w.ptr, ws.ptr, bias.ptr, 0, out.ptr, None, M, N, K))
    if sampler:
        sampler.start()
    t_end = time.perf_counter() + seconds
    while time.perf_counter() < t_end:
        t0 = time.perf_counter()
        for _ in range(per_print):
            launch()
        hip.sync()
        print(f"sustain {operands}: {(time.perf_counter() - t0) / per_print * 1e6:.1f} us per launch "
              f"({hip.last_kernel()})", flush=True)
    if sampler:
        stop.set()
        sampler.join(timeout=15)
        print(f"sustain {operands}: sclk MHz while the loop ran: {' '.join(str(x) for x in mhz)}", flush=True)


def cpu_baseline():
    """The reference's own CPU path on this box's host cores.  Checker/baseline code only."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_bind as ob
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    rng = np.random.default_rng(2)
    M, N, K = 8192, 8192, 8192          # the headline shape itself: ~4 s a run on 16 cores
    a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    q = rand_i8(rng, (N, K))
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    if ob.ref_available():
        lib, kind = ob.RefLib(), "reference"
    else:
        lib, kind = ob.Oracle(), "port"
    runs, spent = [], 0.0
    while len(runs) < 3 and spent < 20.0:                # a bounded sample: three runs, 20 s at most
        t0 = time.perf_counter()
        lib.qgemm_w8a32(a, q, s)
        runs.append(time.perf_counter() - t0)
        spent += runs[-1]
    dt = min(runs)
    tops = 2.0 * M * N * K / dt / 1e12
    result_line("cpu", f"q8a32_{M}x{N}x{K}", "gflops", tops * 1e3)
    return {"value": tops, "unit": "TOP/s", "cores": cores, "kind": kind,
            "sample": f"ax_qgemm_w8a32 (the reference's only quantized GEMM: int8 weights x fp32 "
                      f"activations, fp32 accumulate; it has no W8A8) on the headline shape M=N=K=8192, "
                      f"best of {len(runs)} runs ({', '.join('%.1f' % r for r in runs)} s)"}


def cpu_baseline_fp32():
    """The fp32 half of the metric on the host cores: the reference's cpu_opt GEMM
    (src/compute/backends/cpu_opt.c:3446) at M=N=K=1024, configs[0], with the harness shape of
    benchmarks/bench_comprehensive.c:26-36 (5 warm + 40 timed runs, per-run samples)."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_bind as ob
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    rng = np.random.default_rng(3)
    n = 1024
    a = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    b = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    if ob.ref_available():
        lib, kind = ob.RefLib(), "reference"
        lib.backend(lib.CPU_SIMD)
        ta, tb, to = lib.tensor(a), lib.tensor(b), lib.empty(n, n)       # operands placed once, outside the timing

        def run():
            assert lib.L.ax_compute_gemm(ta, tb, to) == 0
    else:
        lib, kind = ob.Oracle(), "port"
        c = np.empty((n, n), np.float32)

        def run():
            lib.L.axo_gemm_opt(a, b, c, n, n, n)
    for _ in range(5):
        run()
    runs = []
    for _ in range(40):
        t0 = time.perf_counter()
        run()
        runs.append(time.perf_counter() - t0)
    runs = np.array(runs)
    tf = 2.0 * n ** 3 / np.median(runs) / 1e12
    result_line("cpu", f"f32_nn_{n}x{n}x{n}", "gflops", tf * 1e3)
    return {"value": tf, "unit": "TFLOP/s", "cores": cores, "kind": kind,
            "median_ms": float(np.median(runs) * 1e3), "min_ms": float(runs.min() * 1e3),
            "sample": f"cpu_opt fp32 GEMM (opt_gemm through ax_compute_gemm) at M=N=K={n}, operands in place, "
                      f"median of 40 runs after 5 warm-up runs"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--no-secondary", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--counter-probe", nargs="?", const="headline", default=None,
                    choices=["headline", "skinny", "gemm1024", "fp32", "config2", "attention", "w8a32"])
    ap.add_argument("--probe-repeat", type=int, default=1, help="multiplies the launch counts of --counter-probe")
    ap.add_argument("--sustain", type=float, default=0.0, help="seconds of back-to-back headline launches")
    ap.add_argument("--hbm-ceiling", action="store_true", help="read / write / copy rates of this GPU on 2 GiB arrays")
    ap.add_argument("--dispatch-table", action="store_true", help="shape -> kernel -> us for a fixed list of shapes")
    ap.add_argument("--cpu-legs", action="store_true", help="only the reference's CPU path on the configurations (no GPU), one JSON line")
    ap.add_argument("--operands", default="random",
                    help="random | zeros | fp32 | fp32zeros | qkt | qktzeros | pv | pvzeros | probe<16|32>r<0..6>[zeros]")
    ap.add_argument("--sample-clocks", action="store_true", help="with --sustain: sample the shader clock with rocm-smi while the loop runs")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if args.cpu_legs:
        print(json.dumps({"cpu_baseline": cpu_baseline(), "cpu_baseline_fp32": cpu_baseline_fp32(),
                          "legs": {} if args.no_secondary else cpu_config_legs()}), flush=True)
        return

    from axiom_amd import AxHip
    hip = AxHip()
    hip.init()
    if args.counter_probe:
        counter_probe(hip, args.counter_probe, args.probe_repeat)
        return
    if args.sustain > 0:
        sustain(hip, args.sustain, args.operands, args.sample_clocks)
        return
    if args.hbm_ceiling:
        hbm_ceiling(hip)
        return
    if args.dispatch_table:
        dispatch_table(hip)
        return

    h = headline(hip, args.steps, args.warmup)
    tops = h["ops"] / h["host_ms"] / 1e9
    achieved = h["ops"] / h["event_ms"] / 1e9
    traffic, traffic_source = headline_traffic_bytes(h["kernel"])
    result_line("axhip", "q8a8_8192x8192x8192", "gflops", tops * 1e3)
    line = {
        "metric": "int8 qgemm TOP/s on 1 MI355X (W8A8, M=N=K=8192, fused dequant+bias)",
        "value": tops, "unit": "TOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": h["host_ms"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8 (int32 accumulate, fp32 epilogue)", "data": "synthetic",
        "config": {"workload": "configs[4]: int8 qgemm M=N=K=8192, W int8 [N,K] + per-channel fp32 "
                               "scales, X int8 + per-tensor scale, bias, fp32 out",
                   "M": h["M"], "N": h["N"], "K": h["K"], "device": hip.L.axhip_device_name().decode()},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                     "frac": achieved / PEAK_INT8_TOPS,
                     "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": h["kernel"],
                     "kernel_us": h["event_ms"] * 1e3, "median_us": h["median_ms"] * 1e3,
                     "min_us": h["min_ms"] * 1e3, "max_us": h["max_ms"] * 1e3,
                     "algorithmic_ops": h["ops"], "algorithmic_bytes": h["algorithmic_bytes"]},
        "preheat_s": round(h["preheat_s"], 3),
    }
    if not args.no_secondary:
        line["secondary"] = secondary(hip)
        line["secondary"]["configs"].append(config_record(
            "configs[4] (a): int8 W8A8 GEMM M=N=K=8192, dequantize + bias epilogue (the headline)", h["ops"], h["algorithmic_bytes"],
            h["event_ms"] * 1e-3, "mfma_int8", h["kernel"], key="config4a"))
    hip.sync()
    if not args.no_cpu:
        # The CPU legs run in a process of their own that never touches the GPU: this process has the HIP host library
        # loaded, which exports the reference's own function names (it mirrors its API), and the reference library's
        # internal calls would bind to those.
        import subprocess
        child = subprocess.run([sys.executable, os.path.abspath(__file__), "--cpu-legs"] + (["--no-secondary"] if args.no_secondary else []),
                               capture_output=True, text=True, timeout=600)
        sys.stderr.write(child.stderr)
        if child.returncode != 0:
            sys.exit(f"cpu legs failed with status {child.returncode}")
        cpu = json.loads(child.stdout.strip().splitlines()[-1])
        line["cpu_baseline"] = cpu["cpu_baseline"]
        line["cpu_baseline_fp32"] = cpu["cpu_baseline_fp32"]
        if not args.no_secondary:
            legs = cpu["legs"]
            legs["config4a"] = line["cpu_baseline"]
            legs["config0"] = line["cpu_baseline_fp32"]
            for rec in line["secondary"]["configs"]:
                rec["cpu"] = legs.get(rec["key"])
    if not args.no_secondary:
        line["secondary"]["configs"].sort(key=lambda r: r["key"])
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
