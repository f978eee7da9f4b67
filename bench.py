#!/usr/bin/env python3
"""Benchmark of the W8A8 linear hot path on one MI355X.

A "step" is one W8A8 linear over one batch of synthetic, HBM-resident input:

  headline  M=K=N=4096 prefill GEMM (the prefill benchmark shape): int8 A x prepacked
            int8 B, int32 accumulation, per-token x per-channel scale, f32
            bias, requantization to int8 at output scale 0.05 (ties to even).
            Reported as int8 TOPS and as a fraction of the int8 MFMA peak.
  gemv      M=1, K=4096, N=14336 decode GEMV (the decode benchmark shape): dequant +
            bias to f32.  Reported as GB/s of algorithmic bytes and as a
            fraction of HBM peak, rotating over enough weight copies that the
            256 MB Infinity Cache cannot serve them.

The timed region is the K steps recorded once into a HIP graph, replayed back to back
until at least 200 ms of device time have passed (short bursts run at a clock the device
does not sustain under matrix load), timed with HIP events on the launch stream; the
mean over all replays is the figure, the fastest replay is reported beside it
(`ms_per_step_launched_singly` gives the same K steps launched one by one).

Prints ONE JSON line.  The CPU column times the reference's own native CPU
route (oracle/_ref, compiled from the reference sources) on the host cores
with a bounded sample; it is a reported baseline, never part of the GPU path.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

METRIC = "W8A8 linear int8 TOPS (%MFMA peak) at 4096³; GB/s (%HBM) at M=1"
PEAK_INT8_TOPS = 5000.0   # dense int8 MFMA, MI355X
PEAK_HBM_GBS = 8000.0     # HBM3E, MI355X
# HBM-side bytes per launch from the FETCH_SIZE / WRITE_SIZE counter runs summarised under
# profiles/ (each counter scaled by what it reads for a 512 MiB copy kernel).  A counter run
# cannot share a process with the timed run, so `roofline.traffic` is NOT measured by this run: the
# values are carried here from those profiles, and the JSON line says so (`traffic_source`).
MEASURED_TRAFFIC_BYTES = {
    "gemm_4096x4096x4096": 101_186_560 + 18_155_622,
    "gemv_1x4096x14336": 60_708_098 + 57_344,
}


def gemv_algorithmic_bytes(m, k, n):
    # weights once + activations + per-channel scales + bias + per-token scales + f32 output
    return n * k + m * k + 4 * n + 4 * n + 4 * m + 4 * m * n


MIN_TIMED_MS = 200.0


def timed_region(fn, steps, torch, stream):
    """ms per step of fn(0..steps-1), two ways.  (1) The `steps` launches recorded once into a HIP
    graph and replayed back to back until MIN_TIMED_MS of device time have passed: one HIP event
    pair on `stream` around the whole run gives the mean, one pair per replay the fastest replay.
    The recording and the first replay (which uploads the graph) are not timed.  (2) The same
    launches issued one by one, over the same minimum time.  Returns a dict; graph figures are
    None if capture is refused."""
    def event():
        return torch.cuda.Event(enable_timing=True)

    res = {"graph_ms": None, "graph_min_ms": None, "graph_replays": 0}
    with torch.cuda.stream(stream):
        # launched singly
        stream.synchronize()
        e0, e1 = event(), event()
        e0.record(stream)
        for i in range(steps):
            fn(i)
        e1.record(stream)
        stream.synchronize()
        once = max(e0.elapsed_time(e1), 1e-3)
        singly_rounds = max(1, int(np.ceil(MIN_TIMED_MS / once)))
        e0.record(stream)
        for _ in range(singly_rounds):
            for i in range(steps):
                fn(i)
        e1.record(stream)
        stream.synchronize()
        res["singly_ms"] = e0.elapsed_time(e1) / (singly_rounds * steps)
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(steps):
                fn(i)
        stream.synchronize()
        with torch.cuda.stream(stream):
            graph.replay()
            stream.synchronize()
            # the replay count comes from a timed replay of the graph itself (a replayed step is shorter
            # than a singly launched one), with a margin, so that MIN_TIMED_MS are really timed
            e0.record(stream)
            graph.replay()
            e1.record(stream)
            stream.synchronize()
            rounds = max(1, int(np.ceil(1.2 * MIN_TIMED_MS / max(e0.elapsed_time(e1), 1e-3))))
            marks = [event() for _ in range(rounds + 1)]
            marks[0].record(stream)
            for r in range(rounds):
                graph.replay()
                marks[r + 1].record(stream)
            stream.synchronize()
        per = [marks[r].elapsed_time(marks[r + 1]) / steps for r in range(rounds)]
        res.update(graph_ms=marks[0].elapsed_time(marks[-1]) / (rounds * steps), graph_min_ms=min(per),
                   graph_replays=rounds)
    except RuntimeError as e:  # capture refused: report the singly launched figure only
        print(f"bench.py: HIP graph capture failed ({e}); timing single launches", file=sys.stderr)
    res["timed_ms_total"] = (res["graph_ms"] * res["graph_replays"] if res["graph_ms"] is not None
                             else res["singly_ms"] * singly_rounds) * steps
    return res


def time_events(fn, steps, torch, stream):
    """Device time of fn() in ms from one event pair per launch on `stream` (mean, median, min).
    Each pair adds the events' own cost (about 2 us), so these bound the kernel time from above."""
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(steps):
        starts[i].record(stream)
        fn(i)
        stops[i].record(stream)
    stream.synchronize()
    t = np.array([s.elapsed_time(e) for s, e in zip(starts, stops)])
    return float(t.mean()), float(np.median(t)), float(t.min())


def host_cpu():
    """(model string, logical CPUs the process may use, threads to run the baseline on).  A GPU box
    gives one GPU's share of its host to a job (16 workers, the value its OMP_NUM_THREADS carries);
    elsewhere every CPU the process is allowed on is used."""
    model = "unknown"
    try:
        for line in Path("/proc/cpuinfo").read_text().splitlines():
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    allowed = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    share = int(os.environ.get("OMP_NUM_THREADS", "0")) or allowed
    return model, allowed, max(1, min(allowed, share))


def host_physical_cores():
    """Physical cores of the host as /proc/cpuinfo lists them (distinct (physical id, core id) pairs);
    None if it does not say.  The baseline runs on this job's share of them, not on all."""
    try:
        cores, phys = set(), None
        for line in Path("/proc/cpuinfo").read_text().splitlines():
            if line.startswith("physical id"):
                phys = line.split(":", 1)[1].strip()
            elif line.startswith("core id"):
                cores.add((phys, line.split(":", 1)[1].strip()))
        return len(cores) or None
    except OSError:
        return None


def _time_calls(call, seconds):
    call()
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < seconds or reps < 2:
        result = call()
        reps += 1
    return (time.perf_counter() - t0) / reps, result


def cpu_baseline_gemm(rows, k, n, seed):
    """The reference's native CPU route (its policy picks the packed or the raw kernel) on the
    headline workload at full size, all rows, with one input scale (the reference's QLinear has no
    per-token form): on the host cores this job may use, and on one thread."""
    from oracle.pyoracle import Reference, Oracle, DTYPE_I8
    model, allowed, cores = host_cpu()
    rng = np.random.default_rng(seed)
    x = rng.integers(-127, 128, (rows, k)).astype(np.int8)
    w = rng.integers(-127, 128, (n, k)).astype(np.int8)
    sw = (rng.uniform(0.002, 0.01, n) / np.sqrt(k) * 4).astype(np.float32)
    zps = np.zeros(n, np.int32)
    bias = np.zeros(n, np.int32)
    args = (0.03, 0, 0.05, 0, DTYPE_I8, DTYPE_I8, DTYPE_I8)
    ops = 2.0 * rows * k * n
    if Reference.available():
        ref = Reference()
        packed_route = ref.packed_preferred(rows, k, n, DTYPE_I8, True)
        packed = ref.pack_q8(w, DTYPE_I8) if packed_route else None
        call = (lambda: ref.qlinear_packed(x, packed, bias, sw, zps, *args)) if packed_route else \
               (lambda: ref.qlinear_native(x, w, bias, sw, zps, *args))
        threads = ref.enter_pool(cores)
        dt, (ok, _) = _time_calls(call, 8.0)
        ref.leave_pool()
        ref.enter_pool(1)
        dt1, _ = _time_calls(call, 6.0)
        ref.leave_pool()
        kind = "reference"
        route = "vx_qlinear_i8u8_packed" if packed_route else "vx_qlinear_i8u8_native"
        sample = (f"{route}, all {rows} rows at K=N={k}, one input scale: {dt * 1e3:.1f} ms per call on {threads} "
                  f"threads, {dt1 * 1e3:.1f} ms on 1 thread")
        one = {"value": ops / dt1 / 1e12, "unit": "TOPS", "cores": 1, "ms_per_call": dt1 * 1e3}
    else:
        orc = Oracle()
        threads = 1
        t0 = time.perf_counter()
        ok, _ = orc.qlinear(x[:8], w, bias, sw, zps, *args)
        dt = (time.perf_counter() - t0) * rows / 8
        kind = "port"
        sample = f"vxo_qlinear_i8u8 (scalar restatement), 8 of {rows} rows timed and scaled: {dt * 1e3:.0f} ms per call"
        one = None
    assert ok == 1
    return {"value": ops / dt / 1e12, "unit": "TOPS", "cores": threads, "kind": kind, "sample": sample,
            "ms_per_call": dt * 1e3, "single_thread": one, "cpu_model": model, "logical_cpus_allowed": allowed,
            "host_physical_cores": host_physical_cores(),
            "cores_note": "cores = the threads the baseline ran on: this job's share of the host (its OMP_NUM_THREADS), "
                          "not every physical core of the host"}


def cpu_baseline_gemv(k, n, seed):
    from oracle.pyoracle import Reference, Oracle
    import _cases as cases
    model, allowed, cores = host_cpu()
    c = cases.decode_case(1, k, n, 128, seed)
    orc = Oracle()
    words = orc.pack_w8_words(c["w"])
    x = (c["a8"].astype(np.float32) * c["row_scales"][:, None]).astype(np.float32)
    gb = gemv_algorithmic_bytes(1, k, n)
    one = None
    if Reference.available():
        ref = Reference()
        call = lambda: ref.packed_linear(x, words, c["scales"], c["bias"], n, 128)
        threads = ref.enter_pool(cores)
        dt, _ = _time_calls(call, 3.0)
        ref.leave_pool()
        ref.enter_pool(1)
        dt1, _ = _time_calls(call, 3.0)
        ref.leave_pool()
        kind, route = "reference", "vx_llm_forward_f32 (PackedLinear, DYNAMIC_I8)"
        one = {"value": gb / dt1 / 1e9, "unit": "GB/s", "cores": 1, "ms_per_call": dt1 * 1e3}
    else:
        threads = 1
        dt, _ = _time_calls(lambda: orc.packed_linear(x, words, c["scales"], c["bias"], n, 128), 3.0)
        kind, route = "port", "vxo_packed_linear_forward"
    return {"value": gb / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": kind,
            "sample": f"{route}, M=1 K={k} N={n} full size, {dt * 1e3:.2f} ms per call on {threads} threads",
            "ms_per_call": dt * 1e3, "single_thread": one, "cpu_model": model, "logical_cpus_allowed": allowed,
            "host_physical_cores": host_physical_cores()}


def region_ms(fn, steps, torch, warmup=5):
    """ms per call over `steps` calls replayed from one HIP graph on the current stream (launched
    one by one if capture is refused); see timed_region."""
    for i in range(warmup):
        fn(i)
    r = timed_region(fn, steps, torch, torch.cuda.current_stream())
    return r["graph_ms"] if r["graph_ms"] is not None else r["singly_ms"]


def bench_other_configs(torch, vx, cases, ctx):
    """configs[1] at M=4,8,16, configs[2] at M=512,2048 and configs[4] (M=2048, K=14336, N=4096,
    dynamic per-token scales, f32 dequant+bias): time per call with inputs resident."""
    from volvoxai_amd.decoder import pack_w8_words
    from volvoxai_amd.w8a8 import operand_order_codes
    res = {}
    # decode GEMV, M = 4 and 16 (rotating weight copies as for M = 1)
    Kg, Ng, G, copies = 4096, 14336, 128, 6
    d = cases.decode_case(16, Kg, Ng, G, 14336)
    words = pack_w8_words(d["w"])
    pls = [vx.PackedLinear(words, d["scales"], d["bias"], Kg, Ng, G) for _ in range(copies)]
    # With more than one row the int8 codes are handed over the way the library's preparation
    # kernels write them for a decode context: the rows' 16-byte chunks interleaved (operand
    # order), which the GEMV loads as whole cache lines.  The row-major figure stays beside it.
    octx = vx.Context(0, torch.cuda.current_stream())
    octx.set_activation_layout(True)
    for m in (4, 8, 16):
        a8 = torch.from_numpy(d["a8"][:m]).cuda()
        o8 = torch.from_numpy(operand_order_codes(d["a8"][:m])).cuda()
        ars = torch.from_numpy(d["row_scales"][:m]).cuda()
        y = torch.empty((m, Ng), dtype=torch.float32, device="cuda")
        y_rows = torch.empty((m, Ng), dtype=torch.float32, device="cuda")
        ms = region_ms(lambda i: pls[i % copies].forward_a8(octx, o8, ars, out=y), 100, torch)
        ms_rows = region_ms(lambda i: pls[i % copies].forward_a8(ctx, a8, ars, out=y_rows), 100, torch)
        gb = gemv_algorithmic_bytes(m, Kg, Ng)
        res[f"gemv_M{m}_K4096_N14336"] = {"ms": ms, "GBs": gb / (ms * 1e-3) / 1e9, "frac_hbm": gb / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                           "variant": octx.last_variant, "activations": "operand order",
                                           "ms_with_row_major_activations": ms_rows,
                                           "same_bits_either_way": bool(torch.equal(y.view(torch.int32), y_rows.view(torch.int32)))}
    # one f32 row through the reference's own call shape (the row is quantized inside the call:
    # vx_packed_linear_forward, packed_linear_ops.inc:1545-1621): one launch, the GEMV preparing the row
    x1 = torch.from_numpy((d["a8"][:1].astype(np.float32) * d["row_scales"][:1, None]).astype(np.float32)).cuda()
    y1 = torch.empty((1, Ng), dtype=torch.float32, device="cuda")
    ms = region_ms(lambda i: pls[i % copies].forward_f32(ctx, x1, out=y1), 100, torch)
    res["packed_linear_f32_row_M1_K4096_N14336"] = {"ms": ms, "variant": ctx.last_variant,
                                                    "includes": "activation preparation, in the same launch"}
    for p in pls:
        p.close()
    # the same decode shape with four-bit weights: half the weight bytes, same scales and output
    from volvoxai_amd.decoder import pack_w4_words
    w4words = pack_w4_words((d["w"] >> 4).astype(np.int8))
    # (twelve copies: six of these 29 MB matrices would fit the 256 MB Infinity Cache)
    w4copies = 2 * copies
    pls = [vx.PackedLinear(w4words, d["scales"], d["bias"], Kg, Ng, G, weight_bits=4) for _ in range(w4copies)]
    for m in (1, 4, 16):
        o8 = torch.from_numpy(operand_order_codes(d["a8"][:m])).cuda()
        ars = torch.from_numpy(d["row_scales"][:m]).cuda()
        y = torch.empty((m, Ng), dtype=torch.float32, device="cuda")
        ms = region_ms(lambda i: pls[i % w4copies].forward_a8(octx, o8, ars, out=y), 100, torch)
        gb = gemv_algorithmic_bytes(m, Kg, Ng) - Kg * Ng // 2
        res[f"w4a8_gemv_M{m}_K4096_N14336"] = {"ms": ms, "GBs": gb / (ms * 1e-3) / 1e9,
                                                "frac_hbm": gb / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                                "variant": octx.last_variant, "activations": "operand order"}
    octx.close()
    a8 = torch.from_numpy(np.tile(d["a8"], (128, 1))).cuda()
    ars = torch.from_numpy(np.tile(d["row_scales"], 128)).cuda()
    y = torch.empty((2048, Ng), dtype=torch.float32, device="cuda")
    ms = region_ms(lambda i: pls[0].forward_a8(ctx, a8, ars, out=y), 30, torch)
    ops = 2.0 * 2048 * Kg * Ng
    res["w4a8_gemm_f32out_M2048_K4096_N14336"] = {"ms": ms, "TOPS": ops / (ms * 1e-3) / 1e12,
                                                   "frac_mfma": ops / (ms * 1e-3) / 1e12 / PEAK_INT8_TOPS,
                                                   "variant": ctx.last_variant}
    for p in pls:
        p.close()
    # prefill GEMM, M = 512 and 2048
    c = cases.rowscale_case(2048, 4096, 4096, 4096)
    lin = vx.QLinear(c["w"], c["scales"], c["zps"], None, vx.DTYPE_I8)
    bd = torch.from_numpy(c["bias_f32"]).cuda()
    for m in (512, 2048):
        xd = torch.from_numpy(c["x"][:m]).cuda()
        rs = torch.from_numpy(c["row_scales"][:m]).cuda()
        yd = torch.empty((m, 4096), dtype=torch.int8, device="cuda")
        ms = region_ms(lambda i: lin.forward_rowscale(ctx, xd, rs, c["s_out"], 0, bias_f32=bd, out=yd), 100, torch)
        ops = 2.0 * m * 4096 * 4096
        res[f"gemm_M{m}_K4096_N4096"] = {"ms": ms, "TOPS": ops / (ms * 1e-3) / 1e12, "frac_mfma": ops / (ms * 1e-3) / 1e12 / PEAK_INT8_TOPS,
                                          "variant": ctx.last_variant}
    lin.close()
    # QuantizeLinear -> QLinear -> DequantizeLinear on one f32 row (static scales), as one call
    q = cases.qlinear_random_case(1, 4096, 4096, 4097, vx.DTYPE_I8, vx.DTYPE_I8, vx.DTYPE_I8, True)
    lins = [vx.QLinear(q["w"], q["scales"], q["zps"], q["bias"], vx.DTYPE_I8) for _ in range(24)]  # 24 x 16 MiB: past the Infinity Cache
    xq = torch.from_numpy(np.random.default_rng(9).normal(0, 40 * q["s_in"], (1, 4096)).astype(np.float32)).cuda()
    ms = region_ms(lambda i: lins[i % 24].forward_f32(ctx, xq, q["s_in"], q["zp_in"], q["s_out"], q["zp_out"]), 96, torch)
    res["qlinear_sandwich_f32_row_M1_K4096_N4096"] = {"ms": ms, "variant": ctx.last_variant,
                                                      "includes": "QuantizeLinear and DequantizeLinear, in the same launch"}
    # QLinear with the DequantizeLinear behind it at the prompt shape: 4096 int8 rows in, f32 out, one launch
    xb = torch.from_numpy(np.random.default_rng(10).integers(-127, 128, (4096, 4096)).astype(np.int8)).cuda()
    yf = torch.empty((4096, 4096), dtype=torch.float32, device="cuda")
    ms = region_ms(lambda i: lins[0].forward_dequantized(ctx, xb, q["s_in"], q["zp_in"], q["s_out"], q["zp_out"], out=yf), 40, torch)
    ops = 2.0 * 4096 ** 3
    res["qlinear_dequantized_M4096_K4096_N4096"] = {"ms": ms, "TOPS": ops / (ms * 1e-3) / 1e12,
                                                    "frac_mfma": ops / (ms * 1e-3) / 1e12 / PEAK_INT8_TOPS,
                                                    "variant": ctx.last_variant,
                                                    "includes": "DequantizeLinear, in the GEMM's epilogue (f32 output)"}
    for l in lins:
        l.close()
    # outlier-heavy large-K GEMM: f32 activations, dynamic per-token quantization, f32 out
    rows, k, n = 2048, 14336, 4096
    rng = np.random.default_rng(55)
    x = rng.normal(0, 1, (rows, k)).astype(np.float32)
    x[:, rng.choice(k, k // 100, replace=False)] *= 20.0
    w = rng.integers(-127, 128, (n, k)).astype(np.int8)
    chan = rng.uniform(0.002, 0.01, n).astype(np.float32)
    pl = vx.PackedLinear(pack_w8_words(w), np.repeat(chan[:, None], k // G, axis=1).copy(),
                         rng.normal(0, 0.1, n).astype(np.float32), k, n, G)
    xd = torch.from_numpy(x).cuda()
    y = torch.empty((rows, n), dtype=torch.float32, device="cuda")
    ms = region_ms(lambda i: pl.forward_f32(ctx, xd, out=y), 20, torch)
    ops = 2.0 * rows * k * n
    res["gemm_f32out_M2048_K14336_N4096"] = {"ms": ms, "TOPS": ops / (ms * 1e-3) / 1e12,
                                             "frac_mfma": ops / (ms * 1e-3) / 1e12 / PEAK_INT8_TOPS,
                                             "variant": ctx.last_variant,
                                             "includes": "activation preparation (f32 -> int8 codes + per-token scales)"}
    pl.close()
    return res


def bench_gemm_budget(torch, vx, cases, ctx):
    """Where the headline GEMM's time goes, from the product's own launches only (no instrumented
    build): the M=N=4096 kernel at K = 1024 .. 8192 on random bytes gives a fixed part and a part per
    k-byte (least squares over the four K); the same kernel on constant operands (all weights and
    activations 1: the datapath does not toggle) against random ones separates what the data costs
    from what the structure costs; the register-only MFMA loop of the same operation count is the
    ceiling beside both."""
    res = {"shape": "M=N=4096, per-token requantizing epilogue, f32 bias"}
    rng = np.random.default_rng(4096)
    M = N = 4096
    scales = (rng.uniform(0.002, 0.01, N) / np.sqrt(4096) * 4).astype(np.float32)
    row_scales = torch.from_numpy(rng.uniform(0.01, 0.05, M).astype(np.float32)).cuda()
    bias = torch.from_numpy(rng.normal(0, 0.1, N).astype(np.float32)).cuda()
    y = torch.empty((M, N), dtype=torch.int8, device="cuda")
    times = {}
    for label, constant in (("random", False), ("constant", True)):
        for K in ((1024, 2048, 4096, 8192) if not constant else (4096,)):
            w = np.ones((N, K), np.int8) if constant else rng.integers(-127, 128, (N, K)).astype(np.int8)
            x = np.ones((M, K), np.int8) if constant else rng.integers(-127, 128, (M, K)).astype(np.int8)
            lin = vx.QLinear(w, scales, np.zeros(N, np.int32), None, vx.DTYPE_I8)
            xd = torch.from_numpy(x).cuda()
            ms = region_ms(lambda i: lin.forward_rowscale(ctx, xd, row_scales, 0.05, 0, bias_f32=bias, out=y), 20, torch)
            times[(label, K)] = ms * 1e3
            res[f"{label}_operands_K{K}_us"] = ms * 1e3
            res.setdefault("variants", {})[f"{label}_K{K}"] = ctx.last_variant
            lin.close()
            del xd
    ks = np.array([1024, 2048, 4096, 8192], dtype=np.float64)
    ts = np.array([times[("random", int(k))] for k in ks])
    slope, fixed = np.polyfit(ks, ts, 1)
    res["fit_random_operands"] = {"fixed_us": float(fixed), "us_per_k_block_of_128": float(slope * 128),
                                  "loop_us_at_K4096": float(slope * 4096),
                                  "loop_int8_TOPS_at_K4096": 2.0 * M * N * 4096 / (slope * 4096 * 1e-6) / 1e12,
                                  "residuals_us": [float(v) for v in ts - (fixed + slope * ks)]}
    res["register_only_mfma_same_operation_count"] = {
        "random_operands": ctx.probe_mfma_rate(128, True, k64=True),
        "constant_operands": ctx.probe_mfma_rate(128, False, k64=True)}
    return res


def bench_config5(torch, vx, ctx):
    """configs[4] alone (M=2048, K=14336, N=4096, f32 rows in, f32 out): the call, its two launches
    apart, and the probe that says what bounds the GEMM: matrix and vector instructions of a SIMD
    take turns, so the MFMAs and the exact per-group fold add up."""
    from volvoxai_amd.decoder import pack_w8_words
    from volvoxai_amd.w8a8 import packed_prepare_i8
    rows, k, n, G = 2048, 14336, 4096, 128
    rng = np.random.default_rng(55)
    x = rng.normal(0, 1, (rows, k)).astype(np.float32)
    x[:, rng.choice(k, k // 100, replace=False)] *= 20.0
    w = rng.integers(-127, 128, (n, k)).astype(np.int8)
    chan = rng.uniform(0.002, 0.01, n).astype(np.float32)
    pl = vx.PackedLinear(pack_w8_words(w), np.repeat(chan[:, None], k // G, axis=1).copy(),
                         rng.normal(0, 0.1, n).astype(np.float32), k, n, G)
    xd = torch.from_numpy(x).cuda()
    y = torch.empty((rows, n), dtype=torch.float32, device="cuda")
    ops = 2.0 * rows * k * n
    ms = region_ms(lambda i: pl.forward_f32(ctx, xd, out=y), 20, torch)
    a8, rs = packed_prepare_i8(ctx, xd)
    ms_gemm = region_ms(lambda i: pl.forward_a8(ctx, a8, rs, out=y), 20, torch)
    variant = ctx.last_variant
    ms_prep = region_ms(lambda i: packed_prepare_i8(ctx, xd), 20, torch)
    pl.close()
    groups = k // G
    return {"workload": "configs[4]: M=2048, K=14336, N=4096, dynamic per-token quantization, f32 dequant + bias",
            "ms": ms, "TOPS": ops / (ms * 1e-3) / 1e12, "frac_mfma": ops / (ms * 1e-3) / 1e12 / PEAK_INT8_TOPS,
            "ms_gemm_alone": ms_gemm, "ms_preparation_alone": ms_prep, "variant": variant,
            "per_simd": {"mfma_16x16x64": rows * n * k / (16 * 16 * 64) / 1024,
                         "fold_vector_instructions": rows * n * groups * 3 / 64 / 1024},
            "mfma_valu_overlap_probe": ctx.probe_mfma_valu_overlap(2000),
            "mfma_valu_overlap_probe_constant_operands": ctx.probe_mfma_valu_overlap(2000, constant_operands=True)}


def bench_single_row(torch, prompt_len=128, new_tokens=128):
    """The decoder benchmark's model at one row (a single stream): a step through the fused single-row
    linears, five launches per layer, beside the nine-launch layer the 32 rows take."""
    from volvoxai_amd.decoder import DecoderConfig, W8A8Decoder, init_weights
    cfg = DecoderConfig()
    single = {}
    weights = init_weights(cfg, 2024)
    one = torch.from_numpy(np.random.default_rng(8).integers(0, cfg.vocab, (1, prompt_len))).cuda()
    one_tokens = {}
    for name, fuse in (("fused_linears", True), ("separate_launches", False)):
        d1 = W8A8Decoder(cfg, weights, 1, fuse_rows=fuse)
        d1.prefill(one)
        d1.capture()
        d1.stream.synchronize()
        t0 = time.perf_counter()
        one_tokens[name] = d1.decode(new_tokens - 1).cpu().numpy()
        single[name] = {"ms_per_decode_step": (time.perf_counter() - t0) * 1e3 / (new_tokens - 1),
                        "last_linear_variant": d1.ctx.last_variant}
        d1.close()
    single["tokens_equal"] = bool((one_tokens["fused_linears"] == one_tokens["separate_launches"]).all())
    return single


def bench_decoder(torch, rows=32, prompt_len=128, new_tokens=128, single_row=True):
    """The decoder benchmark: random-init W8A8 decoder, every linear on the PackedLinear kernels,
    greedy decode of 32 concurrent rows, 128-token prompts, 128 new tokens each."""
    from volvoxai_amd.decoder import DecoderConfig, W8A8Decoder, init_weights
    cfg = DecoderConfig()
    dec = W8A8Decoder(cfg, init_weights(cfg, 2024), rows)
    prompt = torch.from_numpy(np.random.default_rng(7).integers(0, cfg.vocab, (rows, prompt_len))).cuda()
    torch.cuda.synchronize()
    dec.prefill(prompt)  # warm-up of the prefill shapes
    dec.stream.synchronize()
    t0 = time.perf_counter()
    dec.prefill(prompt)
    dec.stream.synchronize()
    prefill_s = time.perf_counter() - t0
    prefill_variant = dec.ctx.last_variant
    dec.capture()
    t0 = time.perf_counter()
    tokens = dec.decode(new_tokens - 1)
    decode_s = time.perf_counter() - t0
    step_variant = dec.ctx.last_variant
    # the same decode without the graph, for the launch-overhead comparison
    dec.prefill(prompt)
    dec.stream.synchronize()
    graph, dec.graph = dec.graph, None
    t0 = time.perf_counter()
    eager_tokens = dec.decode(new_tokens - 1)
    eager_s = time.perf_counter() - t0
    same = bool((tokens == eager_tokens).all().item())
    weight_bytes = sum(L[k].resident_bytes for L in dec.layers for k in ("qkv", "o", "gate_up", "down")) + \
        dec.lm_head.resident_bytes
    dec.graph = graph
    dec.close()
    total_s = prefill_s + decode_s
    single = bench_single_row(torch, prompt_len, new_tokens) if single_row else {}
    return {"workload": "configs[3]: 28-layer W8A8 decoder (hidden 1024, 16q/8kv x128, SwiGLU 3072, vocab 32000), "
                        "32 rows, prompt 128, 128 new tokens, greedy",
            "value": rows * new_tokens / total_s, "unit": "tokens/s",
            "decode_tokens_per_s": rows * (new_tokens - 1) / decode_s,
            "prefill_tokens_per_s": rows * prompt_len / prefill_s,
            "ms_per_decode_step": decode_s * 1e3 / (new_tokens - 1),
            "ms_per_decode_step_without_graph": eager_s * 1e3 / (new_tokens - 1),
            "prefill_ms": prefill_s * 1e3, "graph_and_eager_tokens_equal": same,
            "decode_linear_variant": step_variant, "prefill_linear_variant": prefill_variant,
            "weight_bytes_read_per_step": weight_bytes,
            "decode_hbm_GBs": weight_bytes / (decode_s / (new_tokens - 1)) / 1e9,
            "single_row": single,
            "glue": "HIP kernels of the same library (embedding gather, residual+RMSNorm+prepare, RoPE+KV append, "
                    "prompt and decode GQA attention, SwiGLU+prepare, argmax+advance); "
                    "one HIP graph per decode step"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-single-row", action="store_true",
                    help="decoder leg: the 32-row workload only (keeps a kernel profile of it unmixed)")
    ap.add_argument("--only", choices=["gemm", "gemv", "decoder", "decoder_single_row", "copy", "other", "gemm_budget", "config5"], default=None,
                    help="run one leg only (for profiling a single kernel); 'copy' runs a plain "
                         "device copy of known size, the yardstick for the HBM traffic counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU only (one kernel on one GPU's share of the "
                 "work); --gpus N with N > 1 is not supported.")

    import torch
    import volvoxai_amd as vx
    import _cases as cases
    from oracle.pyoracle import Oracle

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    if args.only == "copy":
        nbytes = 512 << 20
        src = torch.empty(nbytes, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": nbytes, "copy_bytes_written": nbytes, "launches": args.steps}))
        return
    stream = torch.cuda.Stream()
    ctx = vx.Context(0, stream)
    out = {"metric": METRIC, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
           "data": "synthetic (seeded; random-init weights)"}

    # ---- headline: 4096^3 prefill GEMM ------------------------------------------
    if args.only in (None, "gemm"):
        M = K = N = 4096
        c = cases.rowscale_case(M, K, N, 4096)
        lin = vx.QLinear(c["w"], c["scales"], c["zps"], None, vx.DTYPE_I8)
        xd = torch.from_numpy(c["x"]).cuda()
        rs = torch.from_numpy(c["row_scales"]).cuda()
        bd = torch.from_numpy(c["bias_f32"]).cuda()
        yd = torch.empty((M, N), dtype=torch.int8, device="cuda")

        def step(_i=0):
            ok, _ = lin.forward_rowscale(ctx, xd, rs, c["s_out"], 0, bias_f32=bd, out=yd)
            assert ok == 1, vx.library().vxhip_last_error()

        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            for _ in range(args.warmup):
                step()
        reg = timed_region(step, args.steps, torch, stream)
        wall_ms = reg["graph_ms"] if reg["graph_ms"] is not None else reg["singly_ms"]
        with torch.cuda.stream(stream):
            ev_mean, ev_med, ev_min = time_events(step, max(args.steps, 50), torch, stream)
        ops = 2.0 * M * K * N
        out.update(value=ops / (wall_ms * 1e-3) / 1e12, ms_per_step=wall_ms, ms_per_step_fastest_replay=reg["graph_min_ms"],
                   ms_per_step_launched_singly=reg["singly_ms"], graph_replays=reg["graph_replays"],
                   timed_ms_total=reg["timed_ms_total"],
                   launch=f"the {args.steps} steps recorded into one HIP graph, replayed {reg['graph_replays']} times back to back"
                   if reg["graph_ms"] is not None else "single launches",
                   config={"workload": "configs[2]: prefill GEMM M=K=N=4096, int8 x int8 -> int32, per-token x "
                                       "per-channel scale + f32 bias, requant to int8 (scale 0.05, ties-even)",
                           "M": M, "K": K, "N": N, "variant": ctx.last_variant,
                           "epilogue": "per-token scale and f32 bias: an extension of the reference's QLinear "
                                       "(per-tensor scale, int32 bias), pinned by closed forms in tests/test_oracle.py"})
        # The kernel's average duration is the sustained per-step time of the replayed graph: one
        # launch per step, so it bounds the kernel time from above by the ~1 us between graph nodes.
        out["roofline"] = {"bound": "mfma", "achieved": ops / (wall_ms * 1e-3) / 1e12, "peak": PEAK_INT8_TOPS,
                           "unit": "TOP/s", "frac": ops / (wall_ms * 1e-3) / 1e12 / PEAK_INT8_TOPS,
                           "traffic": MEASURED_TRAFFIC_BYTES["gemm_4096x4096x4096"],
                           "traffic_source": "carried from profiles/gemm_k64_rowscale_4096x4096x4096.md (separate rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs), not measured in this run",
                           "kernel": ctx.last_variant, "ops_per_launch": ops,
                           "avg_kernel_ms": wall_ms, "fastest_replay_kernel_ms": reg["graph_min_ms"],
                           "event_pair_per_launch_ms": {"mean": ev_mean, "median": ev_med, "min": ev_min},
                           "note": "int8 TOP/s against the 5.0 POP/s dense int8 MFMA peak; avg_kernel_ms is the mean "
                                   "step of >= 200 ms of graph replays, timed with HIP events on the launch stream"}
        # What the matrix pipes reach with nothing in their way (register-only MFMA loop, as many
        # MFMAs per SIMD as this GEMM issues): with random operand bytes the device lowers its
        # clock, and that rate, not the 5.0 POP/s peak, is what a GEMM on +-127 data can approach.
        out["mfma_ceiling_probe"] = {
            "same_mfma_count_random_operands": ctx.probe_mfma_rate(128, True),
            "same_mfma_count_constant_operands": ctx.probe_mfma_rate(128, False),
            "sustained_random_operands": ctx.probe_mfma_rate(2000, True),
            "sustained_constant_operands": ctx.probe_mfma_rate(2000, False),
            # the instruction the benchmarked tile runs on
            "k64_same_mfma_count_random_operands": ctx.probe_mfma_rate(128, True, k64=True),
            "k64_sustained_random_operands": ctx.probe_mfma_rate(2000, True, k64=True),
            "k64_sustained_constant_operands": ctx.probe_mfma_rate(2000, False, k64=True)}
        # spot parity on the benchmarked output itself
        orc = Oracle()
        ridx, cidx = np.arange(0, M, 257)[:12], np.arange(3, N, 131)[:24]
        ok2, want, _ = orc.qlinear_rowscale(c["x"][ridx], c["w"][cidx], c["scales"][cidx], c["zps"][cidx],
                                            c["row_scales"][ridx], c["s_out"], 0, bias_f32=c["bias_f32"][cidx])
        got = yd.cpu().numpy()[np.ix_(ridx, cidx)]
        out["parity_spot_check"] = bool(ok2 == 1 and (got == want).all())
        lin.close()
        del xd, yd

    # ---- decode GEMV: M=1, K=4096, N=14336 -------------------------------------
    if args.only in (None, "gemv"):
        Mg, Kg, Ng, G = 1, 4096, 14336, 128
        from volvoxai_amd.decoder import pack_w8_words
        d = cases.decode_case(Mg, Kg, Ng, G, 14336)
        orc = Oracle()  # (the checker of the spot parity below, never part of what is timed)
        words = pack_w8_words(d["w"])
        copies = 6  # 6 x 56 MiB > 256 MB Infinity Cache
        pls = [vx.PackedLinear(words, d["scales"], d["bias"], Kg, Ng, G) for _ in range(copies)]
        a8 = torch.from_numpy(d["a8"]).cuda()
        ars = torch.from_numpy(d["row_scales"]).cuda()
        yg = torch.empty((Mg, Ng), dtype=torch.float32, device="cuda")

        def gstep(i=0):
            st, _ = pls[i % copies].forward_a8(ctx, a8, ars, out=yg)
            assert st == 0, vx.library().vxhip_last_error()

        def gstep_hot(_i=0):
            gstep(0)

        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            for i in range(args.warmup):
                gstep(i)
        # a multiple of the copy count per graph, so every replay rotates through all copies
        gsteps = max(copies, (args.steps + copies - 1) // copies * copies)
        greg = timed_region(gstep, gsteps, torch, stream)
        gwall_ms = greg["graph_ms"] if greg["graph_ms"] is not None else greg["singly_ms"]
        with torch.cuda.stream(stream):
            gmean, gmed, gmin = time_events(gstep, max(gsteps, 60), torch, stream)
        # the same launch on one weight copy (served by the Infinity Cache), timed like the rotated one
        # (not when this leg runs alone, which is how its kernel profile is taken: the profile then holds
        # the rotated launches only)
        hot_ms = None
        if args.only is None:
            hreg = timed_region(gstep_hot, gsteps, torch, stream)
            hot_ms = hreg["graph_ms"] if hreg["graph_ms"] is not None else hreg["singly_ms"]
        gb = gemv_algorithmic_bytes(Mg, Kg, Ng)
        _, want, _ = orc.packed_linear_a8(d["a8"], d["row_scales"], words, d["scales"], d["bias"], Ng, G)
        out["gemv"] = {"workload": "configs[1]: decode GEMV M=1, K=4096, N=14336, dequant + bias to f32",
                       "value": gb / (gwall_ms * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": gwall_ms,
                       "ms_per_step_fastest_replay": greg["graph_min_ms"],
                       "ms_per_step_launched_singly": greg["singly_ms"], "steps_per_graph": gsteps,
                       "graph_replays": greg["graph_replays"], "timed_ms_total": greg["timed_ms_total"],
                       "variant": ctx.last_variant, "weight_copies_rotated": copies,
                       "hot_in_cache_GBs": gb / (hot_ms * 1e-3) / 1e9 if hot_ms else None,
                       "hot_in_cache_ms_per_step": hot_ms,
                       "parity_bit_exact": bool((yg.cpu().numpy().view(np.uint32) == want.view(np.uint32)).all())}
        out["roofline_gemv"] = {"bound": "hbm", "achieved": gb / (gwall_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                                "unit": "GB/s", "frac": gb / (gwall_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                "traffic": MEASURED_TRAFFIC_BYTES["gemv_1x4096x14336"],
                                "traffic_source": "carried from profiles/gemv_fit_1x4096x14336.md (separate rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs), not measured in this run",
                                "kernel": ctx.last_variant, "bytes_per_launch": gb, "avg_kernel_ms": gwall_ms,
                                "fastest_replay_kernel_ms": greg["graph_min_ms"],
                                "event_pair_per_launch_ms": {"mean": gmean, "median": gmed, "min": gmin},
                                "note": "algorithmic bytes over the mean step of >= 200 ms of graph replays"}
        # What the memory system gives a kernel of this size that only reads (same bytes, buffers
        # rotated the same way): the practical ceiling next to the 8 TB/s on the data sheet.
        plain = [torch.randint(0, 255, (Kg * Ng,), dtype=torch.uint8, device="cuda") for _ in range(copies)]
        torch.cuda.synchronize()
        probe = ctx.probe_stream_read(plain, launches=60)
        probe["gemv_rate_over_plain_read"] = out["roofline_gemv"]["achieved"] / probe["GBs"]
        out["hbm_ceiling_probe"] = probe
        del plain
        if args.only == "gemv":
            out.update(value=out["gemv"]["value"], unit="GB/s", ms_per_step=gwall_ms, steps=gsteps,
                       config={"workload": out["gemv"]["workload"]}, roofline=out["roofline_gemv"])
        for p in pls:
            p.close()

    if args.only == "gemm_budget":
        with torch.cuda.stream(stream):
            out["gemm_budget"] = bench_gemm_budget(torch, vx, cases, ctx)
        out.update(value=None, config={"workload": "where the M=K=N=4096 GEMM's time goes (fixed part, loop, data)"})

    if args.only == "config5":
        with torch.cuda.stream(stream):
            out["config5"] = bench_config5(torch, vx, ctx)
        out.update(value=out["config5"]["TOPS"], ms_per_step=out["config5"]["ms"], config={"workload": out["config5"]["workload"]})

    # ---- the other benchmark sizes, timed only (their parity is in tests/) -----
    if args.only in (None, "other"):
        with torch.cuda.stream(stream):
            out["other_configs"] = bench_other_configs(torch, vx, cases, ctx)

    # ---- config 4: 28-layer decoder, 32 rows, greedy decode ------------------------
    if args.only == "decoder_single_row":
        out["decoder_single_row"] = bench_single_row(torch)
        out.update(value=1e3 / out["decoder_single_row"]["fused_linears"]["ms_per_decode_step"], unit="tokens/s",
                   ms_per_step=out["decoder_single_row"]["fused_linears"]["ms_per_decode_step"],
                   config={"workload": "configs[3]'s model at one row, prompt 128, 128 new tokens, greedy"})
    if args.only in (None, "decoder"):
        out["decoder"] = bench_decoder(torch, single_row=not args.no_single_row)
        if args.only == "decoder":
            out.update(value=out["decoder"]["value"], unit="tokens/s", ms_per_step=out["decoder"]["ms_per_decode_step"],
                       config={"workload": out["decoder"]["workload"]})

    if not args.no_cpu_baseline:
        if args.only in (None, "gemm"):
            out["cpu_baseline"] = cpu_baseline_gemm(4096, 4096, 4096, 7)
        if args.only in (None, "gemv"):
            out["cpu_baseline_gemv"] = cpu_baseline_gemv(4096, 14336, 8)
            if args.only == "gemv":
                out["cpu_baseline"] = out["cpu_baseline_gemv"]
    ctx.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
