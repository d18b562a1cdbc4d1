#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

Headline (BASELINE.json metric): int4 decode tokens/s on the 7B-shape Llama-style decoder
(32 layers, d_model 4096, 32 q / 8 kv heads, head_dim 128, SwiGLU 14336, vocab 32000, every linear
int4 with group size 32 and fp16 scales, fp16 KV cache pre-filled to context 2048), greedy, batch 1.
One "step" = one decode step of the whole batch.  Weights are random-initialised on the device,
inputs are synthetic, everything is resident in HBM before the timed region.

The single JSON line also carries
  roofline      -- the dominant kernel against the 8 TB/s HBM peak.  At batch 1 that is the single-launch
                   decode kernel (one cooperative launch runs all timed steps): algorithmic bytes per launch
                   (per step: packed weights + scales once, plus the KV cache rows read) / the launch duration
                   measured with HIP events on the launch stream.  With --graph-path or batch > 1 it is the
                   skinny int4 GEMV of the multi-kernel path, timed around the projections of whole steps;
  cpu_baseline  -- the restated reference CPU kernels timed on this host (bounded sample);
  extra         -- batch-16 decode and the stand-alone kernels of the other BASELINE configs.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_BF16_PEAK = 2500.0     # TFLOP/s dense (fp16 shares the rate)
MFMA_I8_PEAK = 5000.0       # TOP/s dense
# HBM bytes per skinny-kernel launch from rocprofv3 --pmc runs of this benchmark (fetch 15 306 KiB x 2.0, the factor a
# plain 256 MiB copy gives for FETCH_SIZE on this GPU, + write 38 KiB x 1.0): profiles/int4_skinny_decode7b_graph_path.md
SKINNY_TRAFFIC_BYTES = 31_385_000
# HBM bytes per decode step of the single-launch kernel from the same kind of counter runs (None until measured)
PERSIST_TRAFFIC_BYTES_PER_STEP = 4_429_000_000  # fetch 4.337 GB (x2.0 scale) + write 0.092 GB: profiles/decode_persistent_7b.md

CFG7B = dict(n_layers=32, d_model=4096, n_heads=32, n_kv_heads=8, head_dim=128, d_ff=14336, vocab=32000,
             group_size=32, max_batch=16, max_ctx=2048 + 512, max_steps=1024, rope_theta=10000.0, rms_eps=1e-5)
PREFILL = 2048


def decode_bytes_per_step(cfg):
    """Algorithmic bytes the projections of one decode step read: packed nibbles + fp16 scales."""
    D, hd, g = cfg["d_model"], cfg["head_dim"], cfg["group_size"]
    hq, hkv, ff = cfg["n_heads"] * hd, cfg["n_kv_heads"] * hd, cfg["d_ff"]
    per_layer = (hq + 2 * hkv) * D + D * hq + 2 * ff * D + D * ff
    params = cfg["n_layers"] * per_layer + cfg["vocab"] * D
    return params // 2 + (params // g) * 2, params


def event_time_ms(fn, torch):
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e)


def bench_decode(dec, torch, batch, steps, warmup, stream_ptr, persistent=False):
    """Wall time of `steps` decode steps after `warmup` untimed ones.  persistent: every run() call is ONE
    cooperative launch that executes all its steps on the device; otherwise one HIP-graph replay per step."""
    import numpy as np

    dec.reset(np.arange(1, batch + 1, dtype=np.int32), PREFILL)
    dec.run(warmup, use_graph=True, stream=stream_ptr, persistent=persistent)
    torch.cuda.synchronize()
    s_ev, e_ev = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    s_ev.record()
    dec.run(steps, use_graph=True, stream=stream_ptr, persistent=persistent)
    e_ev.record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    toks = dec.tokens(warmup, steps)
    assert toks.shape == (steps, batch) and (toks >= 0).all() and (toks < dec.cfg["vocab"]).all()
    return dt, s_ev.elapsed_time(e_ev) * 1e-3


def check_single_launch(dec, torch, steps=8):
    """The single-launch kernel against the multi-kernel path from the benchmark's own start state: the last step's
    logits agree to 2e-2 of max|logit| (two implementations with different fp16 rounding points) and a token differs
    only where the other path's logits of the two picks are within that difference.  Raises if not."""
    import numpy as np

    start = np.arange(1, 2, dtype=np.int32)
    dec.reset(start, PREFILL)
    dec.run(steps, use_graph=True)
    tg, lg = dec.tokens(0, steps)[:, 0].copy(), dec.logits()[0].copy()
    dec.reset(start, PREFILL)
    dec.run(steps, persistent=True)
    tp, lp = dec.tokens(0, steps)[:, 0].copy(), dec.logits()[0].copy()
    same = bool(np.array_equal(tg, tp))
    rel = float(np.abs(lg - lp).max() / np.abs(lg).max())
    assert np.isfinite(lp).all() and (same or rel < 2e-2), "single-launch decode disagrees with the multi-kernel path"
    assert not same or rel < 2e-2, "same tokens but logits differ by %g of max|logit|" % rel
    return {"steps": steps, "tokens_equal_multi_kernel_path": same, "max_rel_logit_diff_last_step": round(rel, 6)}


def bench_projections(dec, torch, batch, stream_ptr, reps=6):
    """Average duration of one skinny-kernel launch over the projections of whole decode steps."""
    import numpy as np

    dec.reset(np.arange(1, batch + 1, dtype=np.int32), PREFILL)
    dec.run_projections(2, stream=stream_ptr)
    torch.cuda.synchronize()
    ms = event_time_ms(lambda: dec.run_projections(reps, stream=stream_ptr), torch)
    launches = reps * (4 * dec.cfg["n_layers"] + 1)
    return ms * 1e-3 / launches, launches


def cpu_baseline(cfg, seconds_budget=20.0):
    """Restated reference CPU kernels (AVX-512 / AVX2 / scalar picked at run time, as the reference's
    dispatchers do) on the projections of one decode step, batch 1, one thread -- what the reference
    runs for MatMul-routed int4 weights.  Sample: one layer's seven projections + a 1/8 slice of lm_head."""
    import numpy as np

    from oracle import oracle as orc

    orc.build()
    D, hd, g = cfg["d_model"], cfg["head_dim"], cfg["group_size"]
    hq, hkv, ff = cfg["n_heads"] * hd, cfg["n_kv_heads"] * hd, cfg["d_ff"]
    shapes = [(hq, D), (hkv, D), (hkv, D), (D, hq), (ff, D), (ff, D), (D, ff)]
    rng = np.random.default_rng(7)
    ws = []
    for (n, k) in shapes + [(cfg["vocab"] // 8, D)]:
        ws.append((rng.integers(0, 256, n * k // 2, dtype=np.uint8), rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float32),
                   rng.standard_normal(k).astype(np.float32), n, k))

    def one_pass(threads):
        t0 = time.perf_counter()
        for (p, s, x, n, k) in ws[:-1]:
            orc.simd_packed_int4_gemv_dispatch(p, s, x, n, k, g, threads=threads)
        t_layer = time.perf_counter() - t0
        p, s, x, n, k = ws[-1]
        t0 = time.perf_counter()
        orc.simd_packed_int4_gemv_dispatch(p, s, x, n, k, g, threads=threads)
        t_head = (time.perf_counter() - t0) * 8
        return t_layer * cfg["n_layers"] + t_head

    one_pass(1)  # warm-up (page faults)
    times, t_start = [], time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < seconds_budget / 2 and len(times) < 15):
        times.append(one_pass(1))
    t1 = sorted(times)[len(times) // 2]
    model, usable, nthreads = host_cpu()
    one_pass(nthreads)
    tm = sorted(one_pass(nthreads) for _ in range(3))[1]
    paths = orc.simd_paths(g)
    return {
        "value": round(1.0 / t1, 3), "unit": "tok/s", "cores": 1, "kind": "port",
        "sample": "projections of 1 of 32 layers + 1/8 of lm_head at batch 1, median of %d, extrapolated to a "
                  "full step; attention/norm glue not included (favours the CPU)" % len(times),
        "kernel": "restated packed_int4_gemv_dispatch -> " + paths["int4_gemv"],
        "cpu_model": model,
        "all_cores": {"value": round(1.0 / tm, 3), "threads": nthreads, "usable_logical_cpus": usable,
                      "note": "one thread per physical core, N-row partition; not present in the reference for MatMul"},
        "other_configs": cpu_baseline_kernels(),
    }


def lcg_states(seed, n):
    """s_1 .. s_n of s <- s * 6364136223846793005 + 1442695040888963407 (mod 2^64), the generator of the reference's
    micro-benchmark (apps/llm-bench/src/bin/kernel_bench.rs:28-50), vectorised: s_i = a^i s_0 + c (1 + a + .. + a^(i-1))."""
    import numpy as np

    a, c = np.uint64(6364136223846793005), np.uint64(1442695040888963407)
    with np.errstate(over="ignore"):
        pw = np.multiply.accumulate(np.full(n, a, np.uint64))            # a^1 .. a^n (wraps mod 2^64)
        geo = np.cumsum(np.concatenate([np.ones(1, np.uint64), pw[:-1]]))  # 1 + a + .. + a^(i-1)
        return pw * np.uint64(seed) + c * geo


def lcg_i8(seed, n):
    import numpy as np

    return ((lcg_states(seed, n) >> np.uint64(33)).astype(np.int64) % 256 - 128).astype(np.int8)


def lcg_f32(seed, n):
    import numpy as np

    return ((lcg_states(seed, n) >> np.uint64(33)).astype(np.int64) % 2001 - 1000).astype(np.float32) * np.float32(0.001)


def host_cpu():
    """(model name, logical CPUs this process may use, physical cores among them)."""
    model, cores = "unknown", set()
    try:
        phys = core = None
        for line in open("/proc/cpuinfo"):
            key, _, val = line.partition(":")
            key, val = key.strip(), val.strip()
            if key == "model name":
                model = val
            elif key == "physical id":
                phys = val
            elif key == "core id":
                core = val
            elif key == "processor":
                cur = int(val)
            if not line.strip() and phys is not None and core is not None:
                cores.add((phys, core))
                phys = core = None
    except OSError:
        pass
    usable = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    physical = min(usable, len(cores)) if cores else usable
    return model, usable, max(1, physical)


def cpu_baseline_kernels(budget_s=12.0):
    """The restated reference CPU kernels (runtime-dispatched AVX-512 / AVX2 / VNNI, oracle/yscv_cpu_simd.c) on the
    stand-alone BASELINE configs, inputs from the reference micro-benchmark's generator and seeds
    (kernel_bench.rs:159-160, 304-306, 343-345); one thread (what the reference runs) and all physical cores."""
    import numpy as np

    from oracle import oracle as orc

    orc.build()
    model, usable, physical = host_cpu()
    out = {"cpu_model": model, "usable_logical_cpus": usable, "physical_cores_used": physical,
           "kernels": orc.simd_paths(32)}

    def med(fn, iters, warm=1):
        for _ in range(warm):
            fn()
        ts = []
        for _ in range(iters):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2]

    # config 1: int4 GEMV 4096 x 4096, group 32 (kernel_bench bench_int4_gemv: weights 0x100, activation 0x200)
    n = k = 4096
    packed, scales = orc.pack_int4_symmetric_per_group(lcg_f32(0x100, n * k), n, k, 32)
    x = lcg_f32(0x200, k)
    byt = n * k // 2 + n * (k // 32) * 4 + k * 4 + n * 4
    t1 = med(lambda: orc.simd_packed_int4_gemv_dispatch(packed, scales, x, n, k, 32), 20, 2)
    tm = med(lambda: orc.simd_packed_int4_gemv_dispatch(packed, scales, x, n, k, 32, threads=physical), 20, 2)
    out["config1_gemv_m1_k4096_n4096"] = {"us_1_thread": round(t1 * 1e6, 1), "GB/s_1_thread": round(byt / t1 / 1e9, 2),
                                          "us_all_cores": round(tm * 1e6, 1), "GB/s_all_cores": round(byt / tm / 1e9, 2)}
    # config 2: int8 GEMM 512 x 4096 x 4096 (bench_int8_gemm: A 0xAA, B 0xBB), prepacked dispatch
    m, k, n = 512, 4096, 4096
    a, b = lcg_i8(0xAA, m * k), lcg_i8(0xBB, k * n)
    pb = orc.SimdPackedI8B(b, k, n)
    ops = 2.0 * m * k * n
    t1 = med(lambda: pb.matmul(a, m), 3)
    tm = med(lambda: pb.matmul(a, m, threads=physical), 3)
    out["config2_int8_m512_k4096_n4096"] = {"ms_1_thread": round(t1 * 1e3, 2), "GOP/s_1_thread": round(ops / t1 / 1e9, 1),
                                            "ms_all_cores": round(tm * 1e3, 2), "GOP/s_all_cores": round(ops / tm / 1e9, 1),
                                            "note": "M-row blocks over the cores (the split of runner/conv/quantized.rs:410-445; "
                                                    "the reference's MatMul runs one thread)"}
    del pb, a, b
    # config 3: int4 GEMM 2048 x 4096 -> 14336, group 128: a 64-row sample of the 2048 rows (the kernel unpacks a group once
    # and loops over the rows, so time grows linearly in M), symmetric weights (the reference kernel has no zero points)
    m_full, m, k, n, g = 2048, 64, 4096, 14336, 128
    rng = np.random.default_rng(3)
    packed = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float32)
    x = lcg_f32(0x300 + m, m * k)
    fl = 2.0 * m * k * n
    t1 = med(lambda: orc.simd_packed_int4_gemm_dispatch(packed, scales, x, m, n, k, g), 1, 0)
    tm = med(lambda: orc.simd_packed_int4_gemm_dispatch(packed, scales, x, m, n, k, g, threads=physical), 2, 0)
    out["config3_int4_prefill_m2048_k4096_n14336"] = {
        "sample": "64 of the 2048 rows, full weight", "GFLOP/s_1_thread": round(fl / t1 / 1e9, 1),
        "GFLOP/s_all_cores": round(fl / tm / 1e9, 1), "s_full_shape_1_thread_extrapolated": round(t1 * m_full / m, 2),
        "s_full_shape_all_cores_extrapolated": round(tm * m_full / m, 2)}
    # config 5: LM-head shape 4096 -> 128256, group 32: m = 1 (GEMV) and m = 16 (GEMM, the reference switches at m >= 8)
    k, n, g = 4096, 128256, 32
    packed = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float32)
    wbytes = n * k // 2 + n * (k // g) * 4
    x1, x16 = lcg_f32(0x200, k), lcg_f32(0x300 + 16, 16 * k)
    t1 = med(lambda: orc.simd_packed_int4_gemv_dispatch(packed, scales, x1, n, k, g), 3)
    tm = med(lambda: orc.simd_packed_int4_gemv_dispatch(packed, scales, x1, n, k, g, threads=physical), 3)
    t16 = med(lambda: orc.simd_packed_int4_gemm_dispatch(packed, scales, x16, 16, n, k, g), 1, 0)
    t16m = med(lambda: orc.simd_packed_int4_gemm_dispatch(packed, scales, x16, 16, n, k, g, threads=physical), 1, 0)
    out["config5_lm_head_k4096_n128256"] = {
        "m1": {"ms_1_thread": round(t1 * 1e3, 2), "weight_GB/s_1_thread": round(wbytes / t1 / 1e9, 2),
               "ms_all_cores": round(tm * 1e3, 2), "weight_GB/s_all_cores": round(wbytes / tm / 1e9, 2)},
        "m16": {"ms_1_thread": round(t16 * 1e3, 1), "GFLOP/s_1_thread": round(2.0 * 16 * k * n / t16 / 1e9, 1),
                "ms_all_cores": round(t16m * 1e3, 1), "GFLOP/s_all_cores": round(2.0 * 16 * k * n / t16m / 1e9, 1)}}
    return out


def measured_peaks(torch):
    """What this GPU sustains on a plain 1 GiB HBM read stream and on back-to-back MFMAs held in registers
    (yscv_hip_measure_peaks).  The roofline fractions stay priced against the published peaks; these figures say how
    much of a published peak is within reach of any kernel on this machine."""
    import ctypes as C

    from yscv_amd import capi

    torch.cuda.synchronize()
    r, f, i = C.c_double(), C.c_double(), C.c_double()
    capi.lib().measure_peaks(C.byref(r), C.byref(f), C.byref(i))
    l2, far = C.c_double(), C.c_double()
    capi.lib().measure_fill(C.byref(l2), C.byref(far))  # operand path of the GEMMs: LDS-direct loads, per CU
    return {"hbm_read_GB/s": round(r.value, 1), "frac_of_8TB/s": round(r.value / HBM_PEAK_GBS, 3),
            "mfma_f16_TFLOP/s": round(f.value, 1), "frac_of_2.5PFLOP/s": round(f.value / 2500.0, 3),
            "mfma_i8_TOP/s": round(i.value, 1), "frac_of_5POP/s": round(i.value / 5000.0, 3),
            "lds_direct_fill_from_L2_GB/s_per_CU": round(l2.value, 1),
            "lds_direct_fill_from_16MiB_region_GB/s_per_CU": round(far.value, 1)}


def extra_kernels(torch, stream_ptr):
    """Stand-alone kernels of BASELINE configs 1-3 and 5 (short runs; the parity tests cover correctness).
    Each call sequence is captured into a HIP graph and replayed, so the figures are device time per call
    without the Python / launch overhead of the caller."""
    import numpy as np

    from yscv_amd import kernels as K

    out = {}
    rng = np.random.default_rng(1)
    side = torch.cuda.Stream()

    def tavg(fn, calls_per_graph, replays=10):
        """Average device time of one fn() call: calls_per_graph calls captured once, replayed `replays` times."""
        with torch.cuda.stream(side):
            for _ in range(2):
                fn()
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                for _ in range(calls_per_graph):
                    fn()
            g.replay()
            torch.cuda.synchronize()
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            for _ in range(replays):
                g.replay()
            e.record()
            torch.cuda.synchronize()
        return s.elapsed_time(e) * 1e-3 / (replays * calls_per_graph)

    # config 1: GEMV M1 K4096 N4096 g32, f32 scales, f32 activations.  "cold": a ring of 56 distinct weight copies
    # (587 MB, more than twice the 256 MB Infinity Cache) so every call streams from HBM; "hot": one copy, cache-resident
    n = k = 4096
    ring = []
    for _ in range(56):
        ring.append(K.PackedInt4Weight(rng.integers(0, 256, n * k // 2, dtype=np.uint8),
                                       rng.uniform(0.005, 0.02, n * (k // 32)).astype(np.float32), 32, n, k,
                                       nibble_format=K.NIBBLE_UNSIGNED))
    i = [0]
    byt = n * k // 2 + n * (k // 32) * 4 + k * 4 + n * 4
    c1 = {}
    for name, dt in (("f32_activations", torch.float32), ("f16_activations", torch.float16)):
        x = torch.randn(1, k, device="cuda").to(dt)
        y = torch.empty(1, n, device="cuda", dtype=dt)

        def gemv():
            ring[i[0] % len(ring)].matmul(x, out=y)
            i[0] += 1

        def gemv_hot():
            ring[0].matmul(x, out=y)

        t = tavg(gemv, 56)
        th = tavg(gemv_hot, 56)
        c1[name] = {"us_per_call_whole_op": round(t * 1e6, 2), "GB/s_whole_op": round(byt / t / 1e9, 1),
                    "hot_us_per_call": round(th * 1e6, 2), "hot_GB/s": round(byt / th / 1e9, 1)}
    from yscv_amd.capi import lib as _lib
    import ctypes as _C

    def empty():
        _lib().launch_empty(_C.c_void_p(torch.cuda.current_stream().cuda_stream))

    c1["launch_floor_us"] = round(tavg(empty, 200) * 1e6, 2)
    c1["note"] = ("launch_floor_us = an empty kernel of the same grid timed the same way (nodes of one graph); cold = 56 rotating weight copies (587 MB, > 2x the 256 MB Infinity Cache), hot = one copy; one kernel per "
                  "call, the f32 input is normalised and split inside it")
    out["config1_gemv_m1_k4096_n4096"] = c1
    del ring
    # config 2: int8 M512 K4096 N4096
    m, k, n = 512, 4096, 4096
    pb = K.pack_i8_b_for_matmul(rng.integers(-127, 128, (k, n), dtype=np.int8), k, n)
    a = torch.randint(0, 256, (m, k), device="cuda", dtype=torch.uint8)
    o32 = torch.empty(m, n, device="cuda", dtype=torch.int32)
    q8 = torch.empty(m, n, device="cuda", dtype=torch.uint8)
    t = tavg(lambda: pb.matmul(a, a_zp=128, out=o32), 20)
    t2 = tavg(lambda: pb.matmul_requant(a, 128, 1.0 / 4096, 128.0, K.ROUND_HALF_AWAY, 0, 255, out=q8), 20)
    ops = 2.0 * m * k * n
    out["config2_int8_m512_k4096_n4096"] = {"us_i32": round(t * 1e6, 2), "TOP/s_i32": round(ops / t / 1e12, 1),
                                            "us_fused_requant": round(t2 * 1e6, 2), "TOP/s_fused_requant": round(ops / t2 / 1e12, 1),
                                            "frac_of_i8_mfma_peak": round(ops / t / 1e12 / MFMA_I8_PEAK, 4),
                                            # one 64 x 128 tile per CU: (64 + 128) * K operand bytes through LDS-direct loads
                                            "operand_KB_per_CU": round((64 + 128) * k / 1024.0, 0),
                                            "operand_fill_GB/s_per_CU_whole_kernel": round((64 + 128) * k / t / 1e9, 1),
                                            "note": "compare with extra.measured_peaks.lds_direct_fill_from_L2_GB/s_per_CU: the tiling "
                                                    "that fills 256 CUs with 512 x 4096 outputs is bound by the L2 -> LDS path"}
    del pb
    # config 3: int4 prefill M2048 K4096 N14336 g128, zero points 6..10, bf16
    m, k, n, g = 2048, 4096, 14336, 128
    zq = rng.integers(6, 11, (n, k // g))
    zp = (zq[:, 0::2] | (zq[:, 1::2] << 4)).astype(np.uint8)
    w = K.PackedInt4Weight(rng.integers(0, 256, n * k // 2, dtype=np.uint8), rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16),
                           g, n, k, zero_points=zp, nibble_format=K.NIBBLE_UNSIGNED)
    xb = torch.randn(m, k, device="cuda").bfloat16()
    yb = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
    # caller-provided scratch for the fp16 copy of the activations (yscv_hip_int4_matmul_ws): nothing is allocated per call
    ws = torch.empty(max(w.workspace_bytes(m, torch.bfloat16), 256), dtype=torch.uint8, device="cuda")
    t = tavg(lambda: w.matmul(xb, out=yb, workspace=ws), 4, replays=5)
    fl = 2.0 * m * k * n
    out["config3_int4_prefill_m2048_k4096_n14336"] = {"us_whole_op": round(t * 1e6, 1), "TFLOP/s": round(fl / t / 1e12, 1),
                                                      "frac_of_bf16_mfma_peak": round(fl / t / 1e12 / MFMA_BF16_PEAK, 4),
                                                      "note": "activation pass (bf16 -> normalised fp16) + GEMM kernel, scratch from the caller"}
    del ws
    w.close()
    del w, xb, yb
    # config 5: LM-head shape K4096 N128256 g32, bf16 activations, M = 1 .. 256
    k, n, g = 4096, 128256, 32
    w = K.PackedInt4Weight(rng.integers(0, 256, n * k // 2, dtype=np.uint8), rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16),
                           g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
    wbytes = n * k // 2 + n * (k // g) * 2
    sweep = {}
    for m in (1, 2, 4, 8, 16, 32, 64, 128, 256):
        xb = torch.randn(m, k, device="cuda").bfloat16()
        yb = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
        ws = torch.empty(max(w.workspace_bytes(m, torch.bfloat16), 256), dtype=torch.uint8, device="cuda")
        t = tavg(lambda: w.matmul(xb, out=yb, workspace=ws), 4, replays=4)
        fl = 2.0 * m * k * n
        sweep["m%d" % m] = {"us": round(t * 1e6, 1), "weight_GB/s": round(wbytes / t / 1e9, 0),
                            "frac_of_hbm_peak": round(wbytes / t / 1e9 / HBM_PEAK_GBS, 3),
                            "TFLOP/s": round(fl / t / 1e12, 1), "frac_of_mfma_peak": round(fl / t / 1e12 / MFMA_BF16_PEAK, 4),
                            "kernel": "int4_skinny_kernel" if m <= 16 else ("int4_mid_kernel" if m <= 32 else "int4_gemm_ring_kernel")}
    out["config5_lm_head_sweep_k4096_n128256"] = sweep

    # where the skinny kernel hands over to the MFMA GEMM: both kernels on either side of m = 16 (event-timed eager
    # calls: the forced modes take their scratch from the stream-ordered allocator)
    def teager(fn, reps=20):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        s_, e_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s_.record()
        for _ in range(reps):
            fn()
        e_.record()
        torch.cuda.synchronize()
        return s_.elapsed_time(e_) * 1e-3 / reps

    x16, x32 = torch.randn(16, k, device="cuda").bfloat16(), torch.randn(32, k, device="cuda").bfloat16()
    x17 = torch.randn(17, k, device="cuda").bfloat16()
    y16 = torch.empty(16, n, device="cuda", dtype=torch.bfloat16)
    y17 = torch.empty(17, n, device="cuda", dtype=torch.bfloat16)
    y32 = torch.empty(32, n, device="cuda", dtype=torch.bfloat16)

    def two_passes():
        w.matmul(x32[:16], out=y32[:16], mode="gemv")
        w.matmul(x32[16:], out=y32[16:], mode="gemv")

    out["switch_skinny_to_gemm_lm_head"] = {
        "m16_skinny_us": round(teager(lambda: w.matmul(x16, out=y16, mode="gemv")) * 1e6, 1),
        "m17_gemm_us": round(teager(lambda: w.matmul(x17, out=y17, mode="gemm")) * 1e6, 1),
        "m32_two_skinny_passes_us": round(teager(two_passes) * 1e6, 1),
        "m32_gemm_us": round(teager(lambda: w.matmul(x32, out=y32, mode="gemm")) * 1e6, 1),
        "note": "yscv_hip_int4_matmul switches at m = 16: one skinny pass up to 16 rows, 17 .. 32 rows on the kernel that keeps "
                "all rows' activations in registers (int4_mid.hip; the forced GEMM mode takes it too), above that the "
                "LDS-ring MFMA GEMM"}
    w.close()
    return out


def bench_prefill(dec, torch, cfg, n_tokens, params):
    """The prompt phase llm-bench times apart from the decode phase (apps/llm-bench/src/main.rs:403-470): n_tokens prompt
    tokens through yscv_hip_decoder_prefill in one pass (MFMA GEMM projections, causal attention, cache filled)."""
    import numpy as np

    prompt = np.random.default_rng(11).integers(0, cfg["vocab"], n_tokens).astype(np.int32)
    dec.prefill(prompt)  # warm-up: kernel images, the stream-ordered pool's first allocations
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    reps = 3
    for _ in range(reps):
        dec.prefill(prompt)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / reps
    fl = 2.0 * (params - cfg["vocab"] * cfg["d_model"]) * n_tokens  # the LM head sees the last row only
    return {"ms": round(t * 1e3, 2), "prompt_tok/s": round(n_tokens / t, 0), "TFLOP/s_projections": round(fl / t / 1e12, 1),
            "frac_of_mfma_peak": round(fl / t / 1e12 / MFMA_BF16_PEAK, 4),
            "note": "host-timed whole call (token upload, per-call scratch from the stream-ordered pool, every launch), "
                    "one pass over all 32 layers; feeding the same prompt through the decode step takes n x ms_per_step"}


def bench_reference_model(torch):
    """The model the reference publishes its own llm-bench numbers on (apps/llm-bench/COMPARISON.md:9-12: 24 layers,
    hidden 1024, 2 kv heads of 64, a 43-token prompt, 16 greedy tokens; there on a 12-thread Zen 4 with int4 group 32:
    prefill 1939 ms, decode 3.53 tok/s), random weights of that shape: head_dim 64 with eight query heads per kv head
    runs on the general attention kernel."""
    import numpy as np

    from yscv_amd.decoder import Decoder

    cfg = dict(n_layers=24, d_model=1024, n_heads=16, n_kv_heads=2, head_dim=64, d_ff=2816, vocab=151936, group_size=32,
               max_batch=1, max_ctx=256, max_steps=32, rope_theta=1000000.0, rms_eps=1e-6)
    dec = Decoder(**cfg)
    dec.init_random(seed=3, nibbles=(1, 15))
    prompt = np.random.default_rng(12).integers(0, cfg["vocab"], 43).astype(np.int32)
    out = {}
    for _ in range(2):  # the first round warms up (graph capture, kernel images)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dec.prefill(prompt)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        dec.run(16, auto=True)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        out = {"prefill_ms_43_tokens": round((t1 - t0) * 1e3, 3), "decode_ms_16_tokens": round((t2 - t1) * 1e3, 3),
               "decode_tok/s": round(16 / (t2 - t1), 1), "decode_path": {1: "one HIP-graph replay per step", 2: "single launch"}[dec.last_path()]}
    out["note"] = "host-timed like llm-bench (prefill and decode apart); random weights, FFN width 2816 assumed"
    dec.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--no-extra", action="store_true", help="skip the stand-alone kernels and the batch-16 run")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--extra-only", action="store_true",
                    help="run only the stand-alone kernels of BASELINE configs 1, 2, 3 and 5 and print their figures "
                         "(the run the rocprofv3 summaries of those kernels are taken from)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the prompt phase (2048 tokens through yscv_hip_decoder_prefill) and print its figures "
                         "(the run the rocprofv3 summary of the prompt pass is taken from)")
    ap.add_argument("--prefill-tokens", type=int, nargs="+", default=[2048],
                    help="prompt lengths for --prefill-only (default 2048; several lengths give one entry each)")
    ap.add_argument("--graph-path", action="store_true",
                    help="time the multi-kernel path (one HIP-graph replay per step) instead of the single-launch kernel")
    ap.add_argument("--no-check", action="store_true",
                    help="skip the comparison of the single-launch kernel with the multi-kernel path (timing experiments)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (torch copy_ kernel, 3 launches): the known-size "
                         "kernel that FETCH_SIZE / WRITE_SIZE counter runs are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (every config of the metric fits one "
              "MI355X); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import numpy as np  # noqa: F401
    import torch

    from yscv_amd.decoder import Decoder

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    assert 1 <= args.batch <= 16
    cfg = dict(CFG7B)
    need = PREFILL + args.steps + args.warmup
    if need > cfg["max_ctx"]:
        cfg["max_ctx"] = ((need + 127) // 128) * 128
    cfg["max_steps"] = max(cfg["max_steps"], args.steps + args.warmup)
    stream_ptr = torch.cuda.current_stream().cuda_stream
    if args.extra_only:
        extra = extra_kernels(torch, stream_ptr)
        extra["measured_peaks"] = measured_peaks(torch)
        print(json.dumps({"extra": extra}))
        return

    if args.calib_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    dec = Decoder(**cfg)
    dec.init_random(seed=1)
    dec.fill_kv_random(seed=2)
    w_bytes, params = decode_bytes_per_step(cfg)
    assert dec.weight_bytes() >= w_bytes
    if args.prefill_only:
        print(json.dumps({"extra": {"prefill_%d_tokens" % n: bench_prefill(dec, torch, cfg, n, params) for n in args.prefill_tokens}}))
        return

    persistent = args.batch == 1 and not args.graph_path
    check = check_single_launch(dec, torch) if persistent and not args.no_check else None
    dt, dt_events = bench_decode(dec, torch, args.batch, args.steps, args.warmup, stream_ptr, persistent=persistent)
    tok_s = args.batch * args.steps / dt
    kv_row_bytes = 2 * cfg["n_layers"] * cfg["n_kv_heads"] * cfg["head_dim"] * 2  # K + V bytes one cached position adds
    kv_bytes_per_seq = kv_row_bytes * PREFILL
    ideal_step_s = (w_bytes + args.batch * kv_bytes_per_seq) / (HBM_PEAK_GBS * 1e9)
    if persistent:
        # dominant kernel = the single-launch decode kernel: one launch runs all timed steps.  Algorithmic bytes
        # per launch = per step, the packed weights + scales (read once) + the KV cache rows attended to.
        first = PREFILL + args.warmup
        kv_bytes = sum(kv_row_bytes * (first + i) for i in range(args.steps))
        bytes_per_launch = w_bytes * args.steps + kv_bytes
        launch_s, launches = dt_events, 1
        kernel = "decode_persistent_kernel (one launch = %d decode steps)" % args.steps
        traffic = PERSIST_TRAFFIC_BYTES_PER_STEP * args.steps if PERSIST_TRAFFIC_BYTES_PER_STEP else None
    else:
        launch_s, launches = bench_projections(dec, torch, args.batch, stream_ptr)
        n_proj = 4 * cfg["n_layers"] + 1
        bytes_per_launch = w_bytes / n_proj  # activations are < 0.1 % of the traffic and are left out
        kernel = "int4_skinny_kernel (all %d projections of a decode step)" % n_proj
        traffic = SKINNY_TRAFFIC_BYTES
    achieved = bytes_per_launch / launch_s / 1e9

    result = {
        "metric": "int4 decode tok/s (7B-shape) + matmul GB/s and % HBM/MFMA roofline, 1 GPU",
        "value": round(tok_s, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(dt / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic (random-init int4 weights, random fp16 KV cache)",
        "config": {"workload": "BASELINE configs[3]: Llama-style decoder 32L d4096 32q/8kv hd128 ffn14336 vocab32000, "
                               "int4 g32 fp16 scales, fp16 KV ctx %d, greedy decode" % PREFILL,
                   "batch": args.batch, "tokens_per_step": args.batch,
                   "path": "single cooperative launch for all steps" if persistent else "one HIP-graph replay per step",
                   "arithmetic": "int4 weights (exact in fp16) x fp16 activations on v_mfma_f32_16x16x32_f16, fp32 accumulate"},
        "roofline": {
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
            "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this benchmark (profiles/), scaled to this "
                              "run's launch; not re-measured in this run",
            "kernel": kernel, "bytes_per_launch": int(bytes_per_launch), "avg_launch_us": round(launch_s * 1e6, 3),
            "launches_timed": launches,
        },
        "hbm_roofline_whole_step": {"ideal_ms": round(ideal_step_s * 1e3, 4), "frac": round(ideal_step_s / (dt / args.steps), 4),
                                    "bytes_weights": w_bytes, "bytes_kv_per_seq": kv_bytes_per_seq},
    }
    if check is not None:
        result["config"]["checked_before_timing"] = check
    extra = {}
    if not args.no_extra:
        n_proj = 4 * cfg["n_layers"] + 1
        if persistent:
            dtg, _ = bench_decode(dec, torch, 1, min(args.steps, 64), 4, stream_ptr)
            avg1, _ = bench_projections(dec, torch, 1, stream_ptr)
            extra["decode_batch1_graph_path"] = {"tok/s": round(min(args.steps, 64) / dtg, 1),
                                                 "ms_per_step": round(dtg / min(args.steps, 64) * 1e3, 4),
                                                 "skinny_kernel_GB/s": round(w_bytes / n_proj / avg1 / 1e9, 1)}
        if args.batch != 16:
            dt16, _ = bench_decode(dec, torch, 16, min(args.steps, 64), 4, stream_ptr)
            avg16, _ = bench_projections(dec, torch, 16, stream_ptr, reps=3)
            extra["decode_batch16"] = {"tok/s": round(16 * min(args.steps, 64) / dt16, 1),
                                       "ms_per_step": round(dt16 / min(args.steps, 64) * 1e3, 4),
                                       "path": "one HIP-graph replay per step",
                                       "skinny_kernel_GB/s": round(w_bytes / n_proj / avg16 / 1e9, 1)}
            # the batches between the two the metric names, same path (fp16 cache, one graph replay per step)
            sweep = {}
            for bsz in (2, 4, 8):
                dtb, _ = bench_decode(dec, torch, bsz, min(args.steps, 64), 4, stream_ptr)
                sweep[f"batch{bsz}"] = {"tok/s": round(bsz * min(args.steps, 64) / dtb, 1),
                                        "ms_per_step": round(dtb / min(args.steps, 64) * 1e3, 4)}
            extra["decode_batch_sweep"] = sweep
    if not args.no_extra:
        extra["prefill_2048_tokens"] = bench_prefill(dec, torch, cfg, 2048, params)
        # shorter prompts (llm-bench's own prompt has 43 tokens): below ~512 rows the projections have fewer output
        # tiles than CUs and the GEMM is cut along K as well
        extra["prefill_short_prompts"] = {"%d_tokens" % n_tok: {kk: vv for kk, vv in bench_prefill(dec, torch, cfg, n_tok, params).items()
                                                                if kk in ("ms", "prompt_tok/s")} for n_tok in (43, 128, 512)}
    del dec
    torch.cuda.empty_cache()
    if not args.no_extra:
        extra["reference_bench_model_24L_h1024_16q2kv_hd64"] = bench_reference_model(torch)
    if not args.no_extra and args.batch != 16:
        # the same batch-16 run with the int8 KV cache (llm-bench --kv-dtype i8): half the cache bytes per step
        dec8 = Decoder(kv_dtype="i8", **cfg)
        dec8.init_random(seed=1)
        dec8.fill_kv_random(seed=2)
        dt8, _ = bench_decode(dec8, torch, 16, min(args.steps, 64), 4, stream_ptr)
        extra["decode_batch16_kv_i8"] = {"tok/s": round(16 * min(args.steps, 64) / dt8, 1),
                                         "ms_per_step": round(dt8 / min(args.steps, 64) * 1e3, 4),
                                         "path": "one HIP-graph replay per step, int8 KV cache with one scale per position"}
        del dec8
        torch.cuda.empty_cache()
    if not args.no_extra:
        extra.update(extra_kernels(torch, stream_ptr))
        extra["measured_peaks"] = measured_peaks(torch)
        result["extra"] = extra
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
