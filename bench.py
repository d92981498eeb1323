#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

Default workload (the configuration the headline metric is quoted on): the W4A16 matmul chain of a Llama-7B
decoder block at decode, M = 1 -- q/k/v/o [4096->4096], gate/up [4096->11008], down [11008->4096], uint4
weights in groups of 128 with bf16 scales and uint4 zero points.  One step = one pass over the seven matmuls
of one layer; the layers rotate over enough distinct weight copies to exceed the 256 MB Infinity Cache, so the
weights stream from HBM.  Inputs are resident in HBM before the timed region starts.

Prints ONE JSON line: whole-job throughput (`value`, GB/s of algorithmic bytes), the roofline of the dominant
kernel measured with HIP events on the launch stream, the INT8 requant GEMM figure, and the CPU baseline (the
restated reference algorithm on the host cores).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from __graft_entry__ import load_package  # noqa: E402

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, AMD's published figure
INT8_PEAK_TOPS = 5000.0      # dense INT8 MFMA
BF16_PEAK_TFLOPS = 2500.0    # dense bf16 MFMA
HBM_TRAFFIC_RATIO = 1.022    # measured HBM bytes / algorithmic bytes of the decode chain (see roofline.traffic_source)


def _dev_bf16(torch, bits):
    return torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)


def host_chain(S, M):
    """Seeded host operands of the seven matmuls (generated once; every weight copy is a distinct HBM allocation)."""
    return [S.w4a16(M, K, N, 128, seed=mi) for mi, (name, K, N) in enumerate(S.LLAMA7B_CHAIN)]


def build_chain(pkg, S, torch, M, n_layers, cfgs):
    """Packed weights for n_layers decoder blocks plus one activation/output pair per matmul."""
    layers = []
    for li in range(n_layers):
        mats = []
        for cfg, (name, K, N) in zip(cfgs, S.LLAMA7B_CHAIN):
            w = pkg.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=4,
                              q_group_size=128)
            mats.append((name, K, N, w))
        layers.append(mats)
    acts = {}
    for name, K, N in S.LLAMA7B_CHAIN:
        if K not in acts:
            x = S.bf16_round(np.random.default_rng(K).standard_normal((M, K), dtype=np.float32))
            acts[K] = _dev_bf16(torch, x)
    outs = {(name): torch.empty((M, N), dtype=torch.bfloat16, device="cuda") for name, K, N in S.LLAMA7B_CHAIN}
    return layers, acts, outs


# steps captured into one HIP graph at most (4 launches each; a 32-layer decoder's graph holds 32 steps' worth per token)
MAX_STEPS_PER_GRAPH = 256
# Before the W warm-up steps the timed graph is replayed for this long, untimed: a GPU that has idled for a few
# milliseconds (graph capture is host work) runs its first milliseconds at lower clocks, and a decode loop is a
# loop that is already running.  The read-only ceiling the result is compared with gets the same treatment.
PREROLL_S = 0.02

# sibling projections that read the same activations go out as one grouped launch
CHAIN_GROUPS = [("q_proj", "k_proj", "v_proj"), ("o_proj",), ("gate_proj", "up_proj"), ("down_proj",)]


def run_chain(pkg, mats, acts, outs, grouped=True):
    """One pass over the seven matmuls; returns the number of kernel launches."""
    if not grouped:
        for name, K, N, w in mats:
            pkg.a16mm_launch(w, acts[K], outs[name])
        return len(mats)
    by_name = {name: (K, w) for name, K, N, w in mats}
    for grp in CHAIN_GROUPS:
        K = by_name[grp[0]][0]
        if len(grp) == 1:
            pkg.a16mm_launch(by_name[grp[0]][1], acts[K], outs[grp[0]])
        else:
            pkg.a16mm_launch_group([by_name[n][1] for n in grp], acts[K], [outs[n] for n in grp])
    return len(CHAIN_GROUPS)


def bench_chain(pkg, S, torch, M, steps, warmup, n_layers, cfgs, grouped=True, graph_steps=None):
    """Times exactly `steps` steps (one step = the seven matmuls of one layer).  The launches are replayed from HIP
    graphs, as few as possible: one graph holds up to MAX_STEPS_PER_GRAPH steps back to back, step i on weight copy
    i % n_layers (as a decoder's graph holds all of its layers), a second one the steps left over, so that a graph
    launch's own cost is spread over many steps as it is in a real decode step.  graph_steps: steps per graph when
    that is to be something else."""
    layers, acts, outs = build_chain(pkg, S, torch, M, n_layers, cfgs)
    per_graph = graph_steps or min(steps, MAX_STEPS_PER_GRAPH)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for mats in layers:  # eager pass first: loads the code objects before capture
            launches = run_chain(pkg, mats, acts, outs, grouped)
        stream.synchronize()

        def capture(count):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for i in range(count):
                    run_chain(pkg, layers[i % n_layers], acts, outs, grouped)
            return g

        full = capture(per_graph)
        rest = capture(steps % per_graph) if steps % per_graph else None
        warm = capture(min(max(warmup, 1), per_graph))
        t_end = time.perf_counter() + PREROLL_S
        while time.perf_counter() < t_end:
            for _ in range(4):
                full.replay()
            stream.synchronize()
        for i in range(max(1, -(-warmup // per_graph))):
            warm.replay()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        ev0.record(stream)
        t0 = time.perf_counter()
        for i in range(steps // per_graph):
            full.replay()
        if rest is not None:
            rest.replay()
        ev1.record(stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    wall_s = t1 - t0
    gpu_s = ev0.elapsed_time(ev1) * 1e-3
    chain_bytes = sum(S.w4_gemv_bytes(M, K, N, 128) for _, K, N in S.LLAMA7B_CHAIN)
    res = {
        "wall_s": wall_s, "gpu_s": gpu_s, "chain_bytes": chain_bytes, "launches_per_step": launches,
        "weight_set_mb": sum(w.nbytes for m in layers for *_, w in m) / 1e6,
    }
    for mats in layers:
        for *_, w in mats:
            w.destroy()
    return res


def bench_int8(pkg, S, torch, clib, n, steps, warmup, M=None, graph=False):
    """INT8 requant GEMM, N = K = n and M rows (default n), per-channel Q31 multiplier + right shift, int8 output.
    graph: replay the launches from a HIP graph -- for launches of a few microseconds, which issued one by one from
    Python would be timed by the host's call rate."""
    M = n if M is None else M
    c = S.int8_matmul(M, n, n, seed=7, right_transpose=True)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    a, b, bias = dev(c["a"]), dev(c["b"]), dev(c["bias"])
    rq = pkg.RequantDesc(clib.RQ_QDM, clib.ROUND_HALF_AWAY_FROM_ZERO, out_dtype=clib.DT_I8,
                         multiplier=dev(c["mult"]), shift=dev(c["shift"]))
    out = torch.empty((M, n), dtype=torch.int8, device="cuda")
    def run():
        pkg.i8mm_launch(a, b, bias, right_transpose=True, rq=rq, out=out)

    def run10():
        for _ in range(10):
            run()

    if graph:
        sec = _time_graph(torch, run10, max(3, steps // 10)) / 10
    else:
        sec = _time_launches(torch, run, steps, warmup=warmup)
    tops = 2.0 * M * n * n / sec / 1e12
    rec = {"workload": "int8_requant_gemm_M%d_N%d_K%d_qdm_per_channel" % (M, n, n), "tops": round(tops, 2),
           "us_per_launch": round(sec * 1e6, 2), "frac_of_int8_mfma_peak": round(tops / INT8_PEAK_TOPS, 4),
           "dtype": "int8*int8->int32->int8"}
    if M <= 32:  # a stream over the right operand (one buffer here: it stays in the 256 MB memory-side cache)
        rec["right_operand_GBps"] = round(n * n / sec / 1e9, 1)
        rec["right_operand"] = "one %d MB buffer, cache-resident" % (n * n // 1000000)
    return rec


def _time_launches(torch, fn, steps, warmup=5, preroll_s=PREROLL_S / 2):
    """Average device time of fn() (which enqueues on the current stream), by HIP events, in seconds.  preroll_s: fn is
    first repeated for that long, untimed (see PREROLL_S)."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        t_end = time.perf_counter() + preroll_s
        while preroll_s and time.perf_counter() < t_end:
            for _ in range(4):
                fn()
            stream.synchronize()
        for _ in range(warmup):
            fn()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        stream.synchronize()
        ev0.record(stream)
        for _ in range(steps):
            fn()
        ev1.record(stream)
        stream.synchronize()
    return ev0.elapsed_time(ev1) * 1e-3 / steps


def bench_int8_context(pkg, S, torch, clib, n, launches=100):
    """What bounds the INT8 figure on this machine, measured in the same run: the vendor library's int8 GEMM
    (torch._int_mm: int32 output, no requantization) on the same random operands, and both kernels on all-zero operands.
    The matrix cores' clock under load depends on the data (power): the gap between the random and the zero rows is
    that effect, and no kernel here reaches the nominal 5 POPS (2.4 GHz) on random int8 data."""
    out = {}
    dev = lambda x: torch.from_numpy(np.ascontiguousarray(x)).cuda()
    c = S.int8_matmul(8, 8, n, seed=7)
    rq = pkg.RequantDesc(clib.RQ_QDM, clib.ROUND_HALF_AWAY_FROM_ZERO, out_dtype=clib.DT_I8,
                         multiplier=dev(c["mult"]), shift=dev(c["shift"]))
    bias = torch.zeros(n, dtype=torch.int32, device="cuda")
    y = torch.empty((n, n), dtype=torch.int8, device="cuda")
    for label in ("random", "zeros"):
        if label == "random":
            a = torch.randint(-128, 128, (n, n), dtype=torch.int8, device="cuda")
            b = torch.randint(-128, 128, (n, n), dtype=torch.int8, device="cuda")
        else:
            a = torch.zeros((n, n), dtype=torch.int8, device="cuda")
            b = torch.zeros((n, n), dtype=torch.int8, device="cuda")
        ours = _time_launches(torch, lambda: pkg.i8mm_launch(a, b, bias, right_transpose=True, rq=rq, out=y), launches)
        rec = {"this_kernel_us": round(ours * 1e6, 2), "this_kernel_tops": round(2.0 * n ** 3 / ours / 1e12, 1)}
        if hasattr(torch, "_int_mm"):
            try:
                ven = _time_launches(torch, lambda: torch._int_mm(a, b.t()), launches)
                rec["vendor_int_mm_us"] = round(ven * 1e6, 2)
                rec["vendor_int_mm_tops"] = round(2.0 * n ** 3 / ven / 1e12, 1)
            except Exception as e:  # the vendor path is a reference point only
                rec["vendor_int_mm_error"] = str(e)[:80]
        out[label] = rec
    out["launches_each"] = launches
    return out


def cpu_baseline_int8(S, budget_s=8.0):
    """The restated reference algorithm of the quantized tpu.MatMul on the host cores (oracle: int8 operands widened to
    f32, f32 GEMM, per-channel MultiplyByQuantizedMultiplier in a scalar loop -- MatMul.cpp:598-604, :696-707), on a
    bounded sample: M = 256 rows of the 4096 x 4096 product per pass."""
    from oracle import pyoracle as O  # CPU baseline leg only
    M, K, N = 256, 4096, 4096
    c = S.int8_matmul(M, K, N, seed=7, right_transpose=True)
    a, b = c["a"].astype(np.float32), c["b"].astype(np.float32)
    bias, multi = c["bias"].astype(np.float32), c["mult"].astype(np.float32)
    passes, t0 = 0, time.perf_counter()
    while True:
        O.matmul_int8(a, b, bias, multi, M=M, K=K, N=N, right_transpose=True, quant_mode=O.RQ_TFLITE,
                      multipliers=[int(c["mult"][0])], rshifts=[int(c["shift"][0])], gemm_kind=O.GEMM_FAST)
        passes += 1
        el = time.perf_counter() - t0
        if el > budget_s or passes >= 20:
            break
    return {"value": round(2.0 * M * K * N * passes / el / 1e12, 4), "unit": "TOPS", "cores": O.num_threads(),
            "kind": "port", "sample": "%d passes of a 256 x 4096 x 4096 slice in %.1f s (f32 GEMM on the host cores, "
                                      "scalar requantization loop)" % (passes, el)}


def _time_graph(torch, fn, replays, warmup=2, preroll_s=PREROLL_S / 2):
    """Average device time of one fn() when fn's launches are replayed from a HIP graph (fn runs eagerly first, so
    that whatever it allocates on its stream exists before the capture): a launch of a few microseconds issued from
    Python would otherwise be timed by the host's call rate."""
    stream = torch.cuda.Stream()
    g_ = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        fn()
        stream.synchronize()
        with torch.cuda.graph(g_, stream=stream):
            fn()
    return _time_launches(torch, g_.replay, replays, warmup=warmup, preroll_s=preroll_s)


def bench_read_ceiling(pkg, torch, sizes, steps=60, pool_mb=1024):
    """What a single launch that only READS n bytes from HBM costs on this machine (mi_bench_read_launch: one 16-byte
    load per lane, every load of a wave requested up front), timed exactly as the GEMVs are: launches replayed from
    a HIP graph, each on a different region of a pool larger than the 256 MB cache.  The best of 2 / 4 / 8 chunks per
    wave is kept.  Returns {n_bytes: {"us": .., "GBps": ..}}."""
    pool = torch.empty(pool_mb << 20, dtype=torch.uint8, device="cuda").fill_(1)
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    out = {}
    for nbytes in sizes:
        stride = (nbytes + 4095) & ~4095
        copies = max(2, min(64, (pool_mb << 20) // stride))
        best = None
        for cpw in (2, 4, 8):
            def run():
                for c in range(copies):
                    pkg.bench_read_launch(pool[c * stride:], nbytes, sink, chunks_per_wave=cpw)
            sec = _time_graph(torch, run, max(3, steps // copies)) / copies
            best = sec if best is None else min(best, sec)
        out[int(nbytes)] = {"us": round(best * 1e6, 2), "GBps": round(nbytes / best / 1e9, 1)}
    del pool
    return out


def bench_launch_floor(pkg, torch, launch_bytes, replays=20, copies=16):
    """What one step's launches cost when their kernels touch no memory: the same grids as the read-only ceiling's
    launches (one per entry of launch_bytes), every wave returning at once, replayed from a HIP graph that holds
    `copies` such steps.  Returns microseconds per step and per launch."""
    pool = torch.empty(max(launch_bytes), dtype=torch.uint8, device="cuda")
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")

    def run():
        for _ in range(copies):
            for b in launch_bytes:
                pkg.bench_read_launch(pool, b, sink, chunks_per_wave=0)
    sec = _time_graph(torch, run, replays) / copies
    return {"us_per_step": round(sec * 1e6, 2), "us_per_launch": round(sec * 1e6 / len(launch_bytes), 2),
            "launches_per_step": len(launch_bytes)}


def bench_single_matmuls(pkg, S, torch, steps=60):
    """Per-matmul figures of the secondary configurations: decode GEMVs (HBM GB/s of algorithmic bytes) and
    prefill GEMMs (TFLOP/s).  Each case rotates over enough weight copies to stay out of the 256 MB cache when the
    weights are small enough for that to matter."""
    out = []

    def one(tag, bits, M, K, N, g, copies):
        cfg = S.w4a16(1, K, N, g, seed=31) if bits == 4 else S.w8a16(1, K, N, g, seed=31)
        ws = [pkg.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=bits, q_group_size=g)
              for _ in range(copies)]
        x = _dev_bf16(torch, S.bf16_round(np.random.default_rng(5).standard_normal((M, K), dtype=np.float32)))
        y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        g_ = torch.cuda.CUDAGraph()
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            for w in ws:
                pkg.a16mm_launch(w, x, y)
            stream.synchronize()
            with torch.cuda.graph(g_, stream=stream):
                for w in ws:
                    pkg.a16mm_launch(w, x, y)
        # prefill launches are timed warm: the first ten milliseconds after a pause read 5-15 % slow on this machine
        sec = _time_launches(torch, g_.replay, max(3, steps // copies), warmup=5 if M <= 32 else 40) / copies
        nbytes = S.w4_gemv_bytes(M, K, N, g) if bits == 4 else S.w8_gemv_bytes(M, K, N, g)
        rec = {"case": tag, "bits": bits, "M": M, "K": K, "N": N, "g": g, "us": round(sec * 1e6, 2)}
        if M <= 32:
            rec["GBps"] = round(nbytes / sec / 1e9, 1)
            rec["frac_hbm_peak"] = round(nbytes / sec / 1e9 / HBM_PEAK_GBS, 4)
        else:
            rec["TFLOPs"] = round(2.0 * M * N * K / sec / 1e12, 1)
            rec["frac_bf16_peak"] = round(2.0 * M * N * K / sec / 1e12 / BF16_PEAK_TFLOPS, 4)
        out.append(rec)
        for w in ws:
            w.destroy()

    # decode GEMVs at K = 4096 (weights from HBM: 32 x 8.8 MB / 12 x 23.6 MB exceed the cache)
    one("w4_g128_q_proj", 4, 1, 4096, 4096, 128, 32)
    one("w4_g128_gate_proj", 4, 1, 4096, 11008, 128, 12)
    one("w4_g128_down_proj", 4, 1, 11008, 4096, 128, 12)
    one("w4_g128_lm_head", 4, 1, 4096, 32000, 128, 5)
    for M in (1, 4, 16):
        one("w4_g64_2048x6144", 4, M, 2048, 6144, 64, 40)
    for M in (1, 32):
        one("w8_pc_11008x4096", 8, M, 4096, 11008, 0, 6)
    # prefill
    for M in (128, 1024, 2048):
        one("w4_g128_prefill_4096x4096", 4, M, 4096, 4096, 128, 2)
    one("w8_pc_prefill_11008x4096", 8, 512, 4096, 11008, 0, 2)
    return out


def bench_f16_prefill_forms(pkg, S, torch, clib, launches=10):
    """W4 g128 prefill on f16 activations, 4096 x 4096: the exact kernel (the reference's unrounded fp32 weights) beside
    the tolerance form (weights rounded to f16 first, mi_a16mm_launch_tol: about 2e-3 of the output RMS away from the
    reference at the worst output).  The tolerance form is opt-in and offered for f16 only."""
    K = N = 4096
    cfg = S.w4a16(1, K, N, 128, seed=31)
    scale16 = np.ascontiguousarray(S.bf16_to_f32(cfg["scale"]).astype(np.float16)).view(np.uint16)  # bf16 values fit f16
    w = pkg.A16Weight(cfg["weight"], scale16, cfg["zp"], None, K=K, N=N, weight_bits=4, q_group_size=128,
                      dtype=clib.DT_F16)
    out = []
    for M in (2048, 4096):
        x = torch.randn((M, K), device="cuda").to(torch.float16)
        y = torch.empty((M, N), dtype=torch.float16, device="cuda")
        rec = {"M": M, "K": K, "N": N}
        for label, tol in (("exact", False), ("tolerance", True)):
            sec = _time_launches(torch, lambda: pkg.a16mm_launch(w, x, y, tolerance=tol), launches, warmup=2)
            rec[label + "_us"] = round(sec * 1e6, 1)
            rec[label + "_TFLOPs"] = round(2.0 * M * N * K / sec / 1e12, 1)
        rec["tolerance_frac_f16_peak"] = round(rec["tolerance_TFLOPs"] / BF16_PEAK_TFLOPS, 4)
        out.append(rec)
    w.destroy()
    return out


def bench_dynamic_quant(pkg, S, torch, steps=40):
    """tpu.A16MatMul with dynamic integer activation quantization (activation quantizer + integer product per call),
    weights rotating through HBM; launches replayed from a HIP graph."""
    out = []
    for M, K, N, copies in ((1, 4096, 4096, 32), (16, 4096, 4096, 32), (1, 4096, 11008, 12), (128, 4096, 4096, 32)):
        cfg = S.w4a16(1, K, N, 128, seed=33)
        ws = [pkg.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=4, q_group_size=128)
              for _ in range(copies)]
        x = _dev_bf16(torch, S.bf16_round(np.random.default_rng(6).standard_normal((M, K), dtype=np.float32)))
        y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")

        def run():
            for w in ws:
                pkg.a16mm_dq_launch(w, x, y)

        sec = _time_graph(torch, run, max(3, steps // copies)) / copies
        nbytes = S.w4_gemv_bytes(M, K, N, 128)
        out.append({"case": "w4_g128_dynamic_int", "M": M, "K": K, "N": N, "us": round(sec * 1e6, 2),
                    "GBps": round(nbytes / sec / 1e9, 1)})
        for w in ws:
            w.destroy()
    # the float code types: E2M1 codes in 4-bit and E4M3 codes in 8-bit weights (weights: random codes, scales as above)
    K = N = 4096
    for case, bits, dq, cfg in (("w4_g128_dynamic_f4", 4, "DQ_F4", S.w4a16(1, K, N, 128, seed=34)),
                                ("w8_g128_dynamic_f8e4m3", 8, "DQ_F8E4M3", S.w8a16(1, K, N, 128, seed=35, signed=False))):
        if bits == 8:
            cfg["weight"] = cfg["weight"] & np.uint8(0x77)  # finite E4M3 codes
        cfg["zp"] = np.zeros_like(cfg["zp"])
        copies = 16
        ws = [pkg.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=bits, q_group_size=128)
              for _ in range(copies)]
        for M in (1, 16):
            x = _dev_bf16(torch, S.bf16_round(np.random.default_rng(6).standard_normal((M, K), dtype=np.float32)))
            y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")

            def run():
                for w in ws:
                    pkg.a16mm_dq_launch(w, x, y, dq_type=getattr(pkg, dq))

            sec = _time_graph(torch, run, max(3, steps // copies)) / copies
            nbytes = S.w4_gemv_bytes(M, K, N, 128) + (N * K // 2 if bits == 8 else 0)
            out.append({"case": case, "M": M, "K": K, "N": N, "us": round(sec * 1e6, 2),
                        "GBps": round(nbytes / sec / 1e9, 1)})
        for w in ws:
            w.destroy()
    return out


def bench_f8_matmul(pkg, torch, clib, steps=20, shapes=((4096, 4096, 4096), (256, 1024, 1024))):
    """tpu.MatMul on E4M3 codes with per-channel F8 output requantization (codes out), random finite codes."""
    out = []
    rng = np.random.default_rng(12)
    for M, K, N in shapes:
        a = torch.from_numpy((rng.integers(0, 256, size=(M, K)).astype(np.uint8) & np.uint8(0xD7))).cuda()
        b = torch.from_numpy((rng.integers(0, 256, size=(N, K)).astype(np.uint8) & np.uint8(0xD7))).cuda()
        bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).cuda()
        scales = torch.from_numpy(rng.uniform(0.5, 2.0, size=N) * 0.01).cuda()

        y = torch.empty((M, N), dtype=torch.uint8, device="cuda")

        def run():
            pkg.f8mm_launch(a, b, bias, right_transpose=True, out_scales=scales, out=y)

        def run10():
            for _ in range(10):
                run()

        # the small shape from a graph: issued one by one from Python it would be timed by the host's call rate
        sec = _time_launches(torch, run, steps, warmup=3) if M >= 2048 else _time_graph(torch, run10, 4) / 10
        tf = 2.0 * M * N * K / sec / 1e12
        out.append({"case": "f8e4m3_matmul_requant_M%d_N%d_K%d" % (M, N, K), "us": round(sec * 1e6, 2),
                    "TFLOPs": round(tf, 1), "frac_fp8_peak": round(tf / 5000.0, 4)})
    return out


def bench_mfma_kernels(pkg, S, torch, clib, launches=10):
    """The three MFMA-bound kernels alone, a few eager launches each: the short command the hardware-counter profiles
    of these kernels are taken with (--only-mfma)."""
    out = {"int8_4096": bench_int8(pkg, S, torch, clib, 4096, launches, 2)}
    K = N = 4096
    cfg = S.w4a16(1, K, N, 128, seed=31)
    w = pkg.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=4, q_group_size=128)
    x = _dev_bf16(torch, S.bf16_round(np.random.default_rng(5).standard_normal((2048, K), dtype=np.float32)))
    y = torch.empty((2048, N), dtype=torch.bfloat16, device="cuda")
    sec = _time_launches(torch, lambda: pkg.a16mm_launch(w, x, y), launches, warmup=2)
    out["w4_g128_prefill_M2048_4096x4096"] = {"us": round(sec * 1e6, 2),
                                              "TFLOPs": round(2.0 * 2048 * N * K / sec / 1e12, 1)}
    w.destroy()
    # the wide-tile kernel: W8 per-channel prefill (cfg4, M = 512) and the f16 tolerance form of the W4 product
    K, N = 4096, 11008
    cfg = S.w8a16(1, K, N, 0, seed=31)
    w = pkg.A16Weight(cfg["weight"], cfg["scale"], cfg["zp"], None, K=K, N=N, weight_bits=8, q_group_size=0)
    x = _dev_bf16(torch, S.bf16_round(np.random.default_rng(5).standard_normal((512, K), dtype=np.float32)))
    y = torch.empty((512, N), dtype=torch.bfloat16, device="cuda")
    sec = _time_launches(torch, lambda: pkg.a16mm_launch(w, x, y), launches, warmup=2)
    out["w8_pc_prefill_M512_11008x4096"] = {"us": round(sec * 1e6, 2), "TFLOPs": round(2.0 * 512 * N * K / sec / 1e12, 1)}
    w.destroy()
    out["prefill_f16_exact_vs_tolerance"] = bench_f16_prefill_forms(pkg, S, torch, clib, launches=launches)
    out["f8_matmul"] = bench_f8_matmul(pkg, torch, clib, steps=launches, shapes=((4096, 4096, 4096),))
    return out


def bench_operator_boundary(pkg, S, steps=200):
    """The same q_proj GEMV through the reference's operator interface (float32-expanded host tensors in and out,
    like InferenceParameter): includes the host<->device transfers and conversions, so it is NOT a roofline figure.
    us_per_call times the C entry point with a prepared parameter block, as the interpreter's C++ walk would call it;
    python_wrapper_us_per_call goes through the numpy front end (which allocates the output and builds the block)."""
    import ctypes
    clib = load_package("clib")
    K = N = 4096
    cfg = S.w4a16(1, K, N, 128, seed=41)
    x, w, s, z, _ = S.f32_valued_a16(cfg)
    op = pkg.A16MatMul(K=K, N=N, weight_bits=4, q_group_size=128).init(w, s, z, None)
    for _ in range(50):  # an idle GPU answers the first calls slowly
        op.inference(x)
    t0 = time.perf_counter()
    for _ in range(steps):
        op.inference(x)
    sec_py = (time.perf_counter() - t0) / steps
    y = np.empty((1, N), dtype=np.float32)
    fp = ctypes.POINTER(ctypes.c_float)
    ins = (fp * 5)(x.ctypes.data_as(fp), w.ctypes.data_as(fp), s.ctypes.data_as(fp), z.ctypes.data_as(fp), None)
    outs = (fp * 1)(y.ctypes.data_as(fp))
    prm = clib.InferParam(ins, 5, outs, 1, op.param.c.handle)
    op.attr.M = 1
    fn, a_ref, p_ref = clib.lib().mi_a16mm_inference, ctypes.byref(op.attr), ctypes.byref(prm)
    for _ in range(10):
        fn(a_ref, p_ref)
    t0 = time.perf_counter()
    for _ in range(steps):
        rc = fn(a_ref, p_ref)
    sec = (time.perf_counter() - t0) / steps
    assert rc == 0 and np.array_equal(y, op.inference(x))
    op.deinit()
    return {"case": "A16MatMul.inference, float32 host tensors, M=1 4096x4096", "us_per_call": round(sec * 1e6, 1),
            "python_wrapper_us_per_call": round(sec_py * 1e6, 1),
            "GBps_algorithmic": round(S.w4_gemv_bytes(1, K, N, 128) / sec / 1e9, 1)}


def bench_operator_boundary_int8(pkg, S, clib, steps=100):
    """The quantized tpu.MatMul of cfg1 (256 x 1024 x 1024, int8 weights on the right) through the reference's operator
    interface: float32-expanded host tensors in and out (1 MiB each way), per-channel multipliers with one common right
    shift (the fused BM168x requantization, MatMul.cpp:708-716).  Times the C entry point with a prepared parameter
    block; includes the float <-> 8-bit conversions and both transfers, so it is NOT a roofline figure."""
    import ctypes
    M, K, N = 256, 1024, 1024
    c = S.int8_matmul(M, K, N, seed=9, right_transpose=False, qdm=False)
    x = c["a"].astype(np.float32)
    right = c["b"].astype(np.float32)
    bias = c["bias"].astype(np.float32)
    multi = c["mult"].astype(np.float32)
    op = pkg.MatMulInt8(K, N, quant_mode=clib.RQ_MULTIPLIER_SHIFT, fuse_rq=True, multipliers=[1],
                        rshifts=[int(c["shift"][0])], out_dtype=clib.DT_I8, right_is_weight=True)
    op.init(x, right, bias, multi)
    want = op.inference(x)
    y = np.empty((M, N), dtype=np.float32)
    fp = ctypes.POINTER(ctypes.c_float)
    ins = (fp * 5)(x.ctypes.data_as(fp), right.ctypes.data_as(fp), bias.ctypes.data_as(fp), multi.ctypes.data_as(fp), None)
    outs = (fp * 1)(y.ctypes.data_as(fp))
    prm = clib.InferParam(ins, 5, outs, 1, op.param.c.handle)
    op.attr.M = M
    fn, a_ref, p_ref = clib.lib().mi_i8mm_inference, ctypes.byref(op.attr), ctypes.byref(prm)
    for _ in range(10):
        fn(a_ref, p_ref)
    t0 = time.perf_counter()
    for _ in range(steps):
        rc = fn(a_ref, p_ref)
    sec = (time.perf_counter() - t0) / steps
    assert rc == 0 and np.array_equal(y, want)
    op.deinit()
    return {"case": "tpu.MatMul int8 inference, float32 host tensors, 256x1024x1024, fused per-channel requant",
            "us_per_call": round(sec * 1e6, 1), "host_bytes_per_call": int(4 * (M * K + M * N))}


def bench_module_block(pkg, S, clib, cfgs, steps=50):
    """The decode block as a device-resident op list (float32 in through set_tensor, Cast to bf16, the seven
    matmuls chained q/k/v <- x, o <- q, gate/up <- o, down <- gate, float32 out through get_tensor): wall time of
    invoke() alone (graph replay + stream sync) and of the whole set_tensor/invoke/get_tensor round trip."""
    by = {name: cfg for cfg, (name, K, N) in zip(cfgs, S.LLAMA7B_CHAIN)}
    m = pkg.Module()
    m.add_tensor("x", clib.ST_F32, (1, 4096)).add_tensor("xb", clib.ST_BF16, (1, 4096))
    for name, K, N in S.LLAMA7B_CHAIN:
        m.add_tensor(name, clib.ST_BF16, (1, N))
    m.add_cast("x", "xb", in_type=clib.ST_F32, out_type=clib.ST_BF16)
    src = {"q_proj": "xb", "k_proj": "xb", "v_proj": "xb", "o_proj": "q_proj", "gate_proj": "o_proj",
           "up_proj": "o_proj", "down_proj": "gate_proj"}
    for name, K, N in S.LLAMA7B_CHAIN:
        c = by[name]
        m.add_a16matmul(src[name], name, c["weight"], c["scale"], c["zp"], None, K=K, N=N, weight_bits=4,
                        q_group_size=128)
    x = np.random.default_rng(3).standard_normal((1, 4096)).astype(np.float32)
    m.set_tensor("x", x)
    for _ in range(5):
        m.invoke()
    t0 = time.perf_counter()
    for _ in range(steps):
        m.invoke()
    t_inv = (time.perf_counter() - t0) / steps
    t0 = time.perf_counter()
    for _ in range(steps):
        m.set_tensor("x", x)
        m.invoke()
        m.get_tensor("down_proj")
    t_all = (time.perf_counter() - t0) / steps
    graph = m.uses_graph()
    m.destroy()
    return {"case": "llama7b decode block as mi_module (cast + 7 A16MatMul, one weight copy)",
            "invoke_us": round(t_inv * 1e6, 1), "set_invoke_get_us": round(t_all * 1e6, 1), "graph_replay": graph}


def cpu_baseline_chain(S, M, cfgs, budget_s=20.0):
    """The restated reference algorithm (oracle) on the host cores: per call dequantize [N,K] to f32,
    transpose to [K,N], f32 GEMM, round to bf16 -- what A16MatMul.cpp:172-245 + Dnnl/MatMul.cpp:167-227 do."""
    from oracle import pyoracle as O  # CPU baseline leg only
    ops = []
    for cfg, (name, K, N) in zip(cfgs, S.LLAMA7B_CHAIN):
        ops.append((K, N, S.bf16_to_f32(cfg["x"]), cfg["weight"].astype(np.float32), S.bf16_to_f32(cfg["scale"]),
                    cfg["zp"].astype(np.float32)))
    chain_bytes = sum(S.w4_gemv_bytes(M, K, N, 128) for _, K, N in S.LLAMA7B_CHAIN)
    passes, t0 = 0, time.perf_counter()
    while True:
        for K, N, x, w, s, z in ops:
            O.a16matmul(x, w, s, z, None, M=M, K=K, N=N, weight_bits=4, q_group_size=128, gemm_kind=O.GEMM_FAST)
        passes += 1
        el = time.perf_counter() - t0
        if el > budget_s or passes >= 50:
            break
    # second variant: weights dequantized and transposed once, outside the timed loop (only the sgemm and the output
    # rounding per call) -- what a CPU path that cached its f32 weights would do; the reference does not
    pre = [(x, np.ascontiguousarray(O.a16_dequant(w, s, z, N, K, 4, 128).T)) for K, N, x, w, s, z in ops]
    p2, t1 = 0, time.perf_counter()
    while True:
        for x, w_kn in pre:
            O.BF16(O.sgemm(x, w_kn, None, kind=O.GEMM_FAST))
        p2 += 1
        el2 = time.perf_counter() - t1
        if el2 > budget_s / 4 or p2 >= 200:
            break
    del pre
    return {"value": round(chain_bytes * passes / el / 1e9, 4), "unit": "GB/s", "cores": O.num_threads(),
            "kind": "port",
            "weights_predequantized": {"value": round(chain_bytes * p2 / el2 / 1e9, 4), "unit": "GB/s",
                                       "sample": "%d passes in %.1f s, f32 [K,N] weights kept (sgemm + rounding only); "
                                                 "same W4 byte count as the numerator" % (p2, el2)},
            "sample": "%d passes of the same 7-matmul chain (M=%d) in %.1f s; weights dequantized and transposed "
                      "on every call as the reference interpreter does; dequant loop serial, sgemm OpenMP" %
                      (passes, M, el)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the first milliseconds after a pause run at lower clocks (200 steps after 20: 3770-3860 GB/s; 1000 after 100:
    # 4030-4040; 2000 after 200: 4057): the defaults time a 26 ms stretch of a loop that is already running
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--batch", type=int, default=1, help="activation rows M of the decode chain")
    ap.add_argument("--layers", type=int, default=4, help="distinct weight copies rotated through (4 x 101 MB); one "
                    "HIP graph replay covers one step on each of them")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-int8", action="store_true")
    ap.add_argument("--no-group", action="store_true",
                    help="one launch per matmul (7) instead of grouping q/k/v and gate/up (4 launches)")
    ap.add_argument("--int8-size", type=int, default=4096)
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the secondary figures (other M, single matmuls, prefill, cache-resident chain)")
    ap.add_argument("--only-mfma", action="store_true",
                    help="run only the three MFMA-bound kernels (INT8 4096^3, W4A16 prefill M=2048, F8 4096^3), a few "
                         "launches each, and print their figures: the command for hardware-counter profiles")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; every GPU box of this run has one. Use --gpus 1.")

    import torch
    pkg = load_package()
    S = load_package("synth")
    clib = load_package("clib")
    if not torch.cuda.is_available() or pkg.device_count() < 1:
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    torch.cuda.set_device(0)

    # one plain device copy of known size (256 MiB read + 256 MiB written): the reference point that scales the
    # FETCH_SIZE / WRITE_SIZE counters when this command runs under rocprofv3 --pmc
    cal_src = torch.empty(64 << 20, dtype=torch.float32, device="cuda").fill_(1.0)
    cal_dst = torch.empty_like(cal_src)
    cal_dst.copy_(cal_src)
    torch.cuda.synchronize()
    del cal_src, cal_dst

    if args.only_mfma:
        print(json.dumps({"only_mfma": bench_mfma_kernels(pkg, S, torch, clib)}), flush=True)
        return

    M = args.batch
    cfgs = host_chain(S, M)
    r = bench_chain(pkg, S, torch, M, args.steps, args.warmup, args.layers, cfgs, grouped=not args.no_group)
    value = r["chain_bytes"] * args.steps / r["wall_s"] / 1e9
    n_launch = args.steps * r["launches_per_step"]
    avg_launch_s = r["gpu_s"] / n_launch
    bytes_per_launch = r["chain_bytes"] / r["launches_per_step"]
    achieved = bytes_per_launch / avg_launch_s / 1e9
    # The ceiling for a launch of n bytes on this machine: a kernel that only reads n bytes, timed the same way in the
    # same run.  The four launches of a step move these byte counts (q+k+v, o, gate+up, down):
    by = {name: S.w4_gemv_bytes(M, K, N, 128) for name, K, N in S.LLAMA7B_CHAIN}
    launch_bytes = [sum(by[n] for n in grp) for grp in CHAIN_GROUPS] if not args.no_group else list(by.values())
    ceil = bench_read_ceiling(pkg, torch, sorted(set(launch_bytes + [8 << 20, 512 << 20])))
    ceil_step_us = sum(ceil[b]["us"] for b in launch_bytes)
    step_us = r["gpu_s"] / args.steps * 1e6
    line = {
        "metric": "W4A16 decode GEMV HBM GB/s (% peak); INT8 requant GEMM TOPS (% MFMA peak)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(r["wall_s"] / args.steps * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u4*bf16->f32->bf16", "data": "synthetic",
        "config": {"workload": "llama7b_w4a16_g128_decode_chain_M%d (q,k,v,o 4096x4096; gate,up 11008x4096; "
                               "down 4096x11008)" % M,
                   "bytes_per_step": r["chain_bytes"], "launches_per_step": r["launches_per_step"],
                   "weight_copies": args.layers, "resident_weight_mb": round(r["weight_set_mb"], 1),
                   "launch": ("one HIP graph replay per %d steps (step i on weight copy i %% %d); "
                              % (min(args.steps, MAX_STEPS_PER_GRAPH), args.layers)) +
                             ("q/k/v and gate/up each as one grouped launch" if not args.no_group
                              else "one launch per matmul"),
                   "timing": "value: host wall clock around the timed region; roofline: HIP events on the launch stream",
                   "preroll_ms": PREROLL_S * 1e3,
                   "preroll": "the timed graph is replayed for preroll_ms, untimed, before the warm-up steps (and the "
                              "launches of the read-only ceiling and of every figure under extras for half as long "
                              "before each of their timings): the first milliseconds after an idle stretch run at "
                              "lower clocks"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE of this command
                     # (profiles/hbm_traffic_pmc_*.md): a ratio to the algorithmic bytes measured once under the
                     # profiler at M = 1 with grouped launches, applied here; this run does not re-measure it
                     "traffic": int(bytes_per_launch * HBM_TRAFFIC_RATIO) if (M == 1 and not args.no_group) else None,
                     "traffic_source": "profiles/hbm_traffic_pmc_decode_chain_and_int8_gemm.md (ratio %.3f)"
                                       % HBM_TRAFFIC_RATIO,
                     "kernel": "a16_decode_kernel<4-bit, bf16, 1 group per tile> (both instances: 8 waves x 4 tiles, "
                               "16 waves x 6 tiles)",
                     "bytes_per_launch": int(bytes_per_launch),
                     "avg_launch_us": round(avg_launch_s * 1e6, 3),
                     "timing": "HIP events on the launch stream around the whole timed region / launches",
                     # the same step made of read-only launches of the same byte counts, measured in this run
                     "read_only_ceiling_us_per_step": round(ceil_step_us, 2),
                     "frac_of_measured_ceiling": round(ceil_step_us / step_us, 4)},
        "frac_of_hbm_peak_whole_job": round(value / HBM_PEAK_GBS, 4),
    }
    if not args.no_int8:
        # at least 100 launches whatever --steps says: short runs flatter a kernel whose clock sags under load
        line["int8_requant_gemm"] = bench_int8(pkg, S, torch, clib, args.int8_size, max(100, args.steps // 2), 10)
        line["int8_requant_gemm"]["launches_timed"] = max(100, args.steps // 2)
        if not args.no_cpu_baseline:
            line["int8_requant_gemm"]["cpu_baseline"] = cpu_baseline_int8(S)
    if not args.no_extras:
        ex = {}
        ex["read_ceiling"] = {str(k): v for k, v in ceil.items()}
        # the step's launches with kernels that touch no memory: what remains of a step when no byte moves
        ex["launch_floor_us"] = bench_launch_floor(pkg, torch, launch_bytes)
        if not args.no_int8:
            ex["int8_context"] = bench_int8_context(pkg, S, torch, clib, args.int8_size)
        # the same chain with one weight copy (101 MB: resident in the 256 MB cache after the first pass)
        r1 = bench_chain(pkg, S, torch, M, max(20, args.steps // 2), 5, 1, cfgs, grouped=not args.no_group,
                         graph_steps=args.layers)
        ex["chain_cache_resident_GBps"] = round(r1["chain_bytes"] / (r1["gpu_s"] / max(20, args.steps // 2)) / 1e9, 1)
        # one launch per matmul, for comparison with the grouped default
        r7 = bench_chain(pkg, S, torch, M, max(20, args.steps // 2), 5, args.layers, cfgs, grouped=False)
        ex["chain_7_launches_GBps"] = round(r7["chain_bytes"] / (r7["gpu_s"] / max(20, args.steps // 2)) / 1e9, 1)
        for m in (8, 32):
            cm = host_chain(S, m)
            rm = bench_chain(pkg, S, torch, m, 40, 5, args.layers, cm, grouped=not args.no_group)
            ex["chain_M%d_GBps" % m] = round(rm["chain_bytes"] / (rm["gpu_s"] / 40) / 1e9, 1)
        ex["single_matmuls"] = bench_single_matmuls(pkg, S, torch)
        ex["prefill_f16_exact_vs_tolerance"] = bench_f16_prefill_forms(pkg, S, torch, clib)
        ex["dynamic_quant"] = bench_dynamic_quant(pkg, S, torch)
        ex["int8_256x1024x1024"] = bench_int8(pkg, S, torch, clib, 1024, 40, 5, M=256, graph=True)
        ex["int8_1x4096x4096"] = bench_int8(pkg, S, torch, clib, 4096, 40, 5, M=1, graph=True)
        ex["f8_matmul"] = bench_f8_matmul(pkg, torch, clib)
        ex["operator_boundary"] = bench_operator_boundary(pkg, S)
        ex["operator_boundary_int8"] = bench_operator_boundary_int8(pkg, S, clib)
        ex["device_resident_block"] = bench_module_block(pkg, S, clib, cfgs)
        line["extras"] = ex
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline_chain(S, M, cfgs)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
