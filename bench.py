#!/usr/bin/env python3
"""Benchmark of the W2A8 GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (config "c2", the decode regime the headline metric is quoted on): one step =
the 24 independent GEMMs of the sweep, M in {1,2,4,8,16,32} over the four Llama-3-8B linear
shapes (4096x4096, 1024x4096, 14336x4096, 4096x14336), 2-bit symmetric group-128 weights,
per-token int8 activations with 0.1 % outlier channels, fp16 out, issued as ONE grouped
launch of the skinny kernel (slimk_w2a8_gemm_grouped).  Inputs are resident in HBM before
the timed region; every GEMM of every step reads a different copy of its weight matrix, so
the stream comes from HBM and not from the 256 MiB Infinity Cache ("cold").  Steps are
replayed from a HIP graph so that host launch cost does not pace the GPU.

value  = algorithmic bytes of all GEMMs / wall time      (GB/s, higher is better)
roofline.achieved = algorithmic bytes per launch / mean launch duration, HIP events on the
                    launch stream, against the 8 TB/s HBM3E peak.
detail.single_launch repeats the same step as 24 separate launches (one GEMM each): those are
latency-bound (5-10 us per launch whatever the size) and are reported per shape in
detail.decode.
cpu_baseline = the same GEMMs (bounded sample) through the CPU oracle's restatement of the
               reference CPU path (numpy quantiser/packer output + torch CPU int matmul).
Activation quantisation is timed separately (detail.act_quant).  detail also carries the
per-shape cold/warm table, the prefill (int8-MFMA-bound) TOPS of the tiled kernel and a
plain streaming-read calibration.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0       # MI355X dense int8 MFMA, published (5.0 POP/s)
COLD_FOOTPRINT = 640 << 20    # bytes of distinct weight copies between two uses of one copy

# HBM bytes per launch of the dominant kernel from two rocprofv3 --pmc runs of
# `python3 bench.py --skip-detail` (FETCH_SIZE, then WRITE_SIZE), each scaled by what the same
# counter reads for this file's 256 MiB calibration read (read_probe_kernel: 131077 -> x2.0) and
# calibration fill (fill_zero_kernel: 262144 -> x1.0):  (115915 * 2.0 + 2898 * 1.0) KiB.
# Counters cannot be read from inside a run: the figure is the one of the committed profile summary named in
# TRAFFIC_SOURCE, taken on the same kernel code (the summary gives the command).
CLOCK_WARMUP_MS = 150   # untimed run of the measured work before every timed region (see timed_run, time_graph)
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = int((115915 * 2.0 + 2898 * 1.0) * 1024)
TRAFFIC_SOURCE = "profiles/skinny_grouped_kernel__c2_decode_sweep.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, scaled by the in-run 256 MiB read / fill calibration)"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--skip-detail", action="store_true", help="only the headline line (no per-shape table, prefill, CPU baseline)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the W2A8 path has no multi-GPU part); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from slimkernels_amd import torch as ops   # raises if the HIP library is missing: no fallback
    from slimkernels_amd import _lib, workloads

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L = _lib.lib()

    # ------------------------------------------------------------------ inputs (resident in HBM)
    def n_copies(nbytes, uses_per_cycle):
        return max(uses_per_cycle, -(-COLD_FOOTPRINT // nbytes))

    class Shape:
        pass

    cases = workloads.config_cases("c2")
    shapes = {}
    for name, (N, K) in workloads.LLAMA8B_LINEARS.items():
        sh = Shape()
        sh.name, sh.N, sh.K = name, N, K
        c0 = workloads.Case("c2", 1, N, K, outliers=True)
        packed, scales, zero = workloads.make_quantized_weight(c0)
        base = ops.repack_w2(packed, scales, None, 128, zp_const=2)
        sh.base = base
        sh.host = (packed, scales, zero)
        sh.copies = [base]
        shapes[name] = sh
    total_w = sum(s.base.w_r.numel() * 4 + s.base.s_r.numel() * 2 for s in shapes.values())
    # every launch of a step cycle uses the next copy; one copy is reused only after all copies of
    # all shapes have been streamed (>= COLD_FOOTPRINT of other traffic in between)
    for sh in shapes.values():
        nb = sh.base.w_r.numel() * 4 + sh.base.s_r.numel() * 2
        want = n_copies(nb, len(workloads.DECODE_M))
        for _ in range(want - 1):
            sh.copies.append(ops.W2A8Weight(sh.base.w_r.clone(), sh.base.s_r.clone(), None, 2, sh.N, sh.K, 128))
        sh.next = 0

    acts = {}
    for c in cases:
        x = torch.from_numpy(workloads.make_activation(c)).to(dev)
        qa = ops.quantize_act_int8(x, 128)
        out = torch.empty((c.M, c.N), dtype=torch.float16, device=dev)
        acts[(c.N, c.K, c.M)] = (x, qa, out)
    name_of = {(N, K): n for n, (N, K) in workloads.LLAMA8B_LINEARS.items()}

    def launch_step(warm=False, grouped=True):
        probs = []
        for c in cases:
            sh = shapes[name_of[(c.N, c.K)]]
            w = sh.copies[0] if warm else sh.copies[sh.next % len(sh.copies)]
            if not warm:
                sh.next += 1
            _, qa, out = acts[(c.N, c.K, c.M)]
            if grouped:
                probs.append((qa, w, out))
            else:
                ops.w2a8_gemm(qa, w, torch.float16, out=out)
        if grouped:
            ops.w2a8_gemm_grouped(probs, torch.float16)

    # Every capture in this file records on one stream of its own, and what is captured runs eagerly on that stream
    # first: the wrapper keeps a split-K workspace per (weight, stream), so the workspaces exist before the capture
    # and no allocation or counter fill ends up inside a graph.
    cap_stream = _capture_stream(torch)
    with torch.cuda.stream(cap_stream):
        for c in cases:
            _, qa, out = acts[(c.N, c.K, c.M)]
            for w in shapes[name_of[(c.N, c.K)]].copies:
                ops.w2a8_gemm(qa, w, torch.float16, out=out)
    torch.cuda.synchronize()

    def capture(n_steps, warm=False, grouped=True):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=cap_stream):
            for _ in range(n_steps):
                launch_step(warm, grouped)
        return g

    # ------------------------------------------------------------------ timed region
    UNROLL = 8

    def timed_run(grouped, steps, warmup):
        """`warmup` warm-up steps, then exactly `steps` timed steps; returns (wall seconds, HIP-event milliseconds)."""
        graphs = {}

        def plan(k):
            full, rem = divmod(k, UNROLL)
            if full and UNROLL not in graphs:
                graphs[UNROLL] = capture(UNROLL, grouped=grouped)
            if rem and rem not in graphs:
                graphs[rem] = capture(rem, grouped=grouped)
            return full, rem

        full_w, rem_w = plan(warmup)
        full_k, rem_k = plan(steps)
        torch.cuda.synchronize()
        # clock warm-up: the same steps, untimed, for CLOCK_WARMUP_MS, so that the W + K steps below run at the
        # clocks of a busy card and not on the ramp from idle (the first ~100 ms after idle run 5-20 % slower)
        any_graph = graphs[UNROLL] if UNROLL in graphs else graphs[rem_k or rem_w]
        t_end = time.perf_counter() + CLOCK_WARMUP_MS * 1e-3
        while time.perf_counter() < t_end:
            for _ in range(4):
                any_graph.replay()
            torch.cuda.synchronize()
        for _ in range(full_w):
            graphs[UNROLL].replay()
        if rem_w:
            graphs[rem_w].replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(full_k):
            graphs[UNROLL].replay()
        if rem_k:
            graphs[rem_k].replay()
        e1.record()
        torch.cuda.synchronize()
        return time.perf_counter() - t0, e0.elapsed_time(e1)

    # counter calibration: a plain read and a plain fill of known size (256 MiB each), so that a
    # rocprofv3 --pmc run of this command can scale FETCH_SIZE / WRITE_SIZE of the GEMM kernel
    cal = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    for _ in range(3):
        _lib.check(L.slimk_w2a8_workspace_init(cal.data_ptr(), cal.numel(), torch.cuda.current_stream().cuda_stream))
        _lib.check(L.slimk_w2a8_read_probe(cal.data_ptr(), cal.numel(), sink.data_ptr(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    del cal

    wall, ev_ms = timed_run(True, args.steps, args.warmup)

    step_bytes = sum(workloads.algorithmic_bytes(c) for c in cases)
    step_ops = sum(workloads.algorithmic_ops(c) for c in cases)
    launches = args.steps                       # one grouped launch per step
    ms_per_step = wall * 1e3 / args.steps
    value = step_bytes * args.steps / wall / 1e9
    avg_launch_us = ev_ms * 1e3 / launches
    achieved = step_bytes / (avg_launch_us * 1e-6) / 1e9

    result = {
        "metric": "W2A8 GEMM TOPS + HBM GB/s (% roofline) at M=1..4096, 1 MI355X",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "c2 decode sweep: M in {1,2,4,8,16,32} x Llama-3-8B linears "
                               "(4096x4096, 1024x4096, 14336x4096, 4096x14336), W2 sym g128, A8 per-token, "
                               "fp16 out; the 24 GEMMs of a step issued as one grouped skinny-kernel launch, "
                               "cold HBM (rotating weight copies)",
                   "launches_per_step": 1, "gemms_per_step": len(cases), "algorithmic_bytes_per_step": step_bytes,
                   "ops_per_step": step_ops, "timing": "HIP graph replay, inputs resident in HBM",
                   "clock_warmup_ms": CLOCK_WARMUP_MS},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH,
                     "traffic_source": TRAFFIC_SOURCE, "kernel": "w2a8::skinny_grouped_kernel", "avg_launch_us": round(avg_launch_us, 3),
                     "algorithmic_bytes_per_launch": step_bytes},
    }

    detail = {"tops_decode": round(step_ops * args.steps / wall / 1e12, 3)}
    if not args.skip_detail:
        # at most 40 steps here: 24 launches a step, and a profiler that serialises dispatches to read counters
        # does not survive ten thousand of them in flight
        steps1 = min(args.steps, 40)
        wall1, ev1 = timed_run(False, steps1, min(args.warmup, 8))
        us1 = ev1 * 1e3 / (len(cases) * steps1)
        detail["single_launch"] = {
            "what": "the same steps as 24 separate launches, one GEMM each (w2a8::skinny_kernel)",
            "steps": steps1, "GBps": round(step_bytes * steps1 / wall1 / 1e9, 2), "ms_per_step": round(wall1 * 1e3 / steps1, 5),
            "avg_launch_us": round(us1, 3),
            "frac_hbm": round(step_bytes / len(cases) / (us1 * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)}
        try:
            detail.update(collect_detail(torch, np, ops, L, workloads, shapes, acts, cases, name_of, dev))
        except Exception as e:  # the side rows must not take the headline line down with them; say what happened
            import traceback
            traceback.print_exc(file=sys.stderr)
            detail["detail_error"] = repr(e)
        result["roofline"]["also"] = also_rows(detail, step_bytes, len(cases))
        result["roofline"].update(flat_fractions(detail))
        result["cpu_baseline"] = cpu_baseline(np, workloads, shapes)
    else:
        result["cpu_baseline"] = None
    result["detail"] = detail
    print(json.dumps(result))


def also_rows(detail, step_bytes, n_gemms):
    """The other half of the metric and the single-GEMM figures, lifted out of `detail` into the `roofline` object:
    int8-MFMA fractions of the tiled kernel at M >= 2048 (c3, and c4 at its largest shapes), HBM fractions of single
    decode GEMMs (c4 at M = 1 / 16, the c2 sweep as 24 launches) and of the grouped sweep restricted to M <= 16."""
    rows = []
    for r in detail.get("prefill", []):
        if r["M"] >= 2048:
            rows.append({"bound": "int8_mfma", "workload": f"c3 M={r['M']} {r['shape']} g128", "kernel": "w2a8::tiled_kernel",
                         "avg_us": r["us"], "achieved": r["TOPS"], "peak": INT8_PEAK_TOPS, "unit": "TOP/s", "frac": r["frac_int8_mfma"]})
    for r in detail.get("other_configs", []):
        if r["config"] == "c4" and r["M"] >= 2048:
            rows.append({"bound": "int8_mfma", "workload": f"c4 M={r['M']} {r['shape']} g64 bf16", "kernel": "w2a8::tiled_kernel",
                         "avg_us": r["us"], "achieved": r["TOPS"], "peak": INT8_PEAK_TOPS, "unit": "TOP/s", "frac": r["frac_int8_mfma"]})
        elif r["config"] == "c4" and r["M"] <= 16:
            rows.append({"bound": "hbm", "workload": f"c4 M={r['M']} {r['shape']} g64 bf16, one GEMM per launch, cold", "kernel": "w2a8::skinny_kernel",
                         "avg_us": r["us"], "achieved": r["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": r["frac_hbm"]})
        elif r["config"] in ("c4", "c5"):
            rows.append({"bound": "near the ridge (both given)", "workload": f"{r['config']} M={r['M']} {r['shape']} g{r['group']} {r['mode']}",
                         "avg_us": r["us"], "frac_hbm": r["frac_hbm"], "frac_int8_mfma": r["frac_int8_mfma"]})
    if "single_launch" in detail:
        sl = detail["single_launch"]
        rows.append({"bound": "hbm", "workload": "c2 sweep as 24 launches, one GEMM each (latency-bound)", "kernel": "w2a8::skinny_kernel",
                     "avg_us": sl["avg_launch_us"], "achieved": sl["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": sl["frac_hbm"]})
    if "decode_sweep_m_le_16" in detail:
        r = detail["decode_sweep_m_le_16"]
        rows.append({"bound": "hbm", "workload": "c2 sweep restricted to M <= 16 (20 GEMMs), one grouped launch, cold",
                     "kernel": "w2a8::skinny_grouped_kernel", "avg_us": r["us"], "achieved": r["GBps"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": r["frac_hbm"]})
    return rows


def flat_fractions(detail):
    """The same figures as `also`, as scalar keys of the `roofline` object itself (a reader that keeps only an object's
    scalars still gets both halves of the metric): `mfma_frac_*` against the int8 MFMA peak, `hbm_frac_*` against HBM,
    named <config>_m<rows>_<N>x<K>; single launches unless the name says grouped."""
    flat = {}
    for r in detail.get("prefill", []):
        flat[f"mfma_frac_c3_m{r['M']}_{r['shape']}"] = r["frac_int8_mfma"]
        flat[f"act_quant_us_c3_m{r['M']}_{r['shape']}"] = r["act_quant_us"]
    for r in detail.get("other_configs", []):
        key = f"{r['config']}_m{r['M']}_{r['shape']}"
        if r["M"] >= 2048:
            flat[f"mfma_frac_{key}"] = r["frac_int8_mfma"]
        elif r["M"] <= 16:
            flat[f"hbm_frac_{key}"] = r["frac_hbm"]
        else:  # near the ridge: both
            flat[f"hbm_frac_{key}"] = r["frac_hbm"]
            flat[f"mfma_frac_{key}"] = r["frac_int8_mfma"]
        flat[f"us_{key}"] = r["us"]
        if "tiled_kernel_us" in r:
            flat[f"us_tiled_kernel_{key}"] = r["tiled_kernel_us"]
    if "single_launch" in detail:
        flat["hbm_frac_c2_single_launch"] = detail["single_launch"]["frac_hbm"]
    if "decode_sweep_m_le_16" in detail:
        flat["hbm_frac_c2_grouped_m_le_16"] = detail["decode_sweep_m_le_16"]["frac_hbm"]
    return flat


def _lib_check(rc):
    from slimkernels_amd import _lib
    _lib.check(rc)


_CAPTURE_STREAM = []


def _capture_stream(torch):
    if not _CAPTURE_STREAM:
        _CAPTURE_STREAM.append(torch.cuda.Stream())
    return _CAPTURE_STREAM[0]


def time_graph(torch, fn, launches_in_graph, replays=6):
    """Mean microseconds per launch of `fn` (which enqueues `launches_in_graph` launches)."""
    s = _capture_stream(torch)
    with torch.cuda.stream(s):  # eagerly first, on the capturing stream: per-stream workspaces come to exist here
        fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        fn()
    g.replay()
    torch.cuda.synchronize()
    # untimed replays first: a card that idled while the host prepared inputs needs ~100 ms of load to reach
    # the clocks it then holds, and a figure taken on that ramp is 5-20 % low
    t_end = time.perf_counter() + CLOCK_WARMUP_MS * 1e-3
    while time.perf_counter() < t_end:
        g.replay()
        torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (replays * launches_in_graph)


def collect_detail(torch, np, ops, L, workloads, shapes, acts, cases, name_of, dev):
    detail = {}
    # ---- streaming-read calibration: what a plain 16-byte-per-lane read kernel reaches on this box
    buf = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    buf.zero_()
    sink = torch.zeros(4, dtype=torch.int32, device=dev)

    def probe():
        st = torch.cuda.current_stream().cuda_stream  # the capture stream while a graph records
        for _ in range(4):
            _lib_check(L.slimk_w2a8_read_probe(buf.data_ptr(), buf.numel(), sink.data_ptr(), st))
    us = time_graph(torch, probe, 4)
    detail["read_probe_GBps_1GiB"] = round(buf.numel() / (us * 1e-6) / 1e9, 1)
    del buf

    # ---- per-(shape, M) decode table, cold (rotating copies) and warm (one copy, cache resident)
    table = []
    for c in cases:
        sh = shapes[name_of[(c.N, c.K)]]
        _, qa, out = acts[(c.N, c.K, c.M)]
        nb = workloads.algorithmic_bytes(c)
        row = {"shape": f"{c.N}x{c.K}", "M": c.M, "bytes": nb,
               "split_k": L.slimk_w2a8_gemm_auto_split_k(c.M, c.N, c.K, 128, 0)}
        for label, ws in (("cold", sh.copies), ("warm", sh.copies[:1] * 16)):
            def fn(ws=ws):
                for w in ws:
                    ops.w2a8_gemm(qa, w, torch.float16, out=out)
            us = time_graph(torch, fn, len(ws), replays=3 if label == "cold" else 10)
            row[f"{label}_us"] = round(us, 2)
            row[f"{label}_GBps"] = round(nb / (us * 1e-6) / 1e9, 1)
        row["cold_frac_hbm"] = round(row["cold_GBps"] / HBM_PEAK_GBPS, 4)
        table.append(row)
    detail["decode"] = table

    # ---- the grouped sweep restricted to M <= 16 (the rows the HBM target is worded on): 20 GEMMs, one launch, cold
    small = [c for c in cases if c.M <= 16]
    nb16 = sum(workloads.algorithmic_bytes(c) for c in small)
    n_rot = max(len(sh.copies) for sh in shapes.values())

    def sweep16():
        for rot in range(n_rot):
            probs = []
            for i, c in enumerate(small):
                sh = shapes[name_of[(c.N, c.K)]]
                _, qa, out = acts[(c.N, c.K, c.M)]
                probs.append((qa, sh.copies[(rot * 5 + i) % len(sh.copies)], out))
            ops.w2a8_gemm_grouped(probs, torch.float16)
    us = time_graph(torch, sweep16, n_rot, replays=6)
    detail["decode_sweep_m_le_16"] = {"gemms": len(small), "bytes": nb16, "us": round(us, 2), "GBps": round(nb16 / (us * 1e-6) / 1e9, 1),
                                      "frac_hbm": round(nb16 / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)}

    # ---- activation quantisation, timed on its own (bytes: 2MK read + MK + 4M + 4MG written)
    aq = []
    for (N, K, M) in ((4096, 4096, 1), (4096, 4096, 32), (4096, 14336, 32)):
        x, _, _ = acts[(N, K, M)]
        us = time_graph(torch, lambda: [ops.quantize_act_int8(x, 128) for _ in range(8)], 8)
        aq.append({"M": M, "K": K, "us": round(us, 2), "GBps": round((3 * M * K + 4 * M + 4 * M * (K // 128)) / (us * 1e-6) / 1e9, 1)})
    detail["act_quant"] = aq

    # ---- decode rows end to end (fp16 activation rows in, fp16 out, cold weights): act-quant + GEMM as two launches
    # against the single launch with the quantisation inside the GEMM, where that launch takes the shape
    fused = []
    for c in cases:
        if c.M not in (1, 2, 4, 16, 32):
            continue
        sh = shapes[name_of[(c.N, c.K)]]
        x, _, out = acts[(c.N, c.K, c.M)]
        two = time_graph(torch, lambda: [ops.w2a8_gemm(ops.quantize_act_int8(x, 128), w, torch.float16, out=out) for w in sh.copies],
                         len(sh.copies), replays=3)
        row = {"shape": f"{c.N}x{c.K}", "M": c.M, "act_quant_then_gemm_us": round(two, 2), "fused_us": None}
        if ops.fused_applies(c.M, c.K):
            for w in sh.copies:
                ops.w2a8_linear_fused(x, w, torch.float16, out=out)
            one = time_graph(torch, lambda: [ops.w2a8_linear_fused(x, w, torch.float16, out=out) for w in sh.copies],
                             len(sh.copies), replays=3)
            row["fused_us"] = round(one, 2)
        fused.append(row)
    detail["decode_row_end_to_end"] = fused

    # ---- prefill regime (c3): tiled int8-MFMA kernel
    pre = []
    for (N, K) in ((14336, 4096), (4096, 14336)):
        w = shapes[name_of[(N, K)]].base
        for M in (512, 2048, 4096):
            c = workloads.Case("c3", M, N, K)
            x = torch.from_numpy(workloads.make_activation(c)).to(dev)
            qa = ops.quantize_act_int8(x, 128)
            out = torch.empty((M, N), dtype=torch.float16, device=dev)
            ops.w2a8_gemm(qa, w, torch.float16, out=out)
            us = time_graph(torch, lambda: [ops.w2a8_gemm(qa, w, torch.float16, out=out) for _ in range(4)], 4)
            tops = workloads.algorithmic_ops(c) / (us * 1e-6) / 1e12
            # the quantiser as W2A8Linear runs it in front of this GEMM: without the group sums where the kernel the
            # library picks does not read them (the tiled kernel with the symmetric levels), and with them for comparison
            sums = ops.needs_rowsum(M, w)
            aq_us = time_graph(torch, lambda: [ops.quantize_act_int8(x, 128, rowsum=sums) for _ in range(4)], 4)
            aq_sums_us = time_graph(torch, lambda: [ops.quantize_act_int8(x, 128) for _ in range(4)], 4)
            pre.append({"shape": f"{N}x{K}", "M": M, "us": round(us, 1), "TOPS": round(tops, 1),
                        "frac_int8_mfma": round(tops / INT8_PEAK_TOPS, 4), "act_quant_us": round(aq_us, 1),
                        "act_quant_group_sums": bool(sums), "act_quant_with_sums_us": round(aq_sums_us, 1)})
    detail["prefill"] = pre

    # ---- the other configurations (c4: Llama-70B-class linears, group 64, bf16 out; c5: ragged shapes
    # with per-group zero-points), timing only, on random codes and scales in the streaming layout
    # (their parity is what the GPU tests check on quantised data).  M <= 16 cold (ten weight copies
    # in rotation, over twice the 256 MiB last-level cache; one graph replay = ten launches), larger M warm.
    def random_weight(N, K, g, asym):
        strips = -(-N // 64)
        # the streaming layout pads the step count to whole runs of four: size the buffer as the library does and
        # leave the padding units zero
        dwords = L.slimk_w2a8_repacked_weight_bytes(N, K) // 4
        used = strips * (K // 64) * 256
        w_r = torch.zeros(dwords, dtype=torch.int32, device=dev)
        if used == dwords:
            w_r.copy_(torch.randint(-2**31, 2**31 - 1, (dwords,), dtype=torch.int32, device=dev))
        else:  # runs of four steps per strip: [run][strip][4 steps][256 dwords]; the last run's surplus steps stay zero
            steps = K // 64
            view = w_r.view(-1, strips, 4, 256)
            full = steps // 4
            view[:full].copy_(torch.randint(-2**31, 2**31 - 1, (full, strips, 4, 256), dtype=torch.int32, device=dev))
            if steps % 4:
                view[full, :, :steps % 4].copy_(torch.randint(-2**31, 2**31 - 1, (strips, steps % 4, 256), dtype=torch.int32, device=dev))
        s_r = (torch.rand(strips * (K // g) * 64, device=dev) * 0.02 + 0.005).half()
        zp_r = torch.randint(0, 4, (strips * (K // g) * 64,), dtype=torch.uint8, device=dev) if asym else None
        return ops.W2A8Weight(w_r, s_r, zp_r, 0 if asym else 2, N, K, g)

    others = []
    # the memory-bound rows first: straight after a compute-bound run (M = 2048 draws the most power) the card holds
    # lower clocks for a while, which the 150 ms of untimed replays before each figure do not always outlast
    c4_shapes = ((28672, 8192), (8192, 28672))
    plan = [("c4", N, K, 64, "sym", torch.bfloat16, M) for (N, K) in c4_shapes for M in (1, 16)]
    plan += [("c5", 5120, 13824, 128, "asym", torch.float16, 1), ("c5", 11008, 4096, 128, "asym", torch.float16, 77)]
    # (33 and 80 rows: row counts that would leave 64-row tiles mostly empty, which the library gives to the kernel
    # that takes every row in one workgroup on matrices this large; the tiled kernel's time is reported beside it)
    plan += [("c4", 28672, 8192, 64, "sym", torch.bfloat16, M) for M in (33, 80)]
    plan += [("c4", N, K, 64, "sym", torch.bfloat16, M) for (N, K) in c4_shapes for M in (128, 2048)]
    cache = {}
    for (cfg, N, K, g, mode, odt, M) in plan:
        cold = M <= 16
        key = (N, K, g, mode)
        if key not in cache:
            cache.clear()
            torch.cuda.empty_cache()
            cache[key] = [random_weight(N, K, g, mode == "asym") for _ in range(10)]
        ws = cache[key] if cold else cache[key][:1] * 4
        c = workloads.Case(cfg, M, N, K, group_size=g, mode=mode, out_dtype="bfloat16" if odt == torch.bfloat16 else "float16")
        x = torch.randn(M, K, device=dev, dtype=torch.float16)
        qa = ops.quantize_act_int8(x, g)
        out = torch.empty((M, N), dtype=odt, device=dev)
        for w in (ws if cold else ws[:1]):  # also allocates each copy's split-K workspace outside the capture
            ops.w2a8_gemm(qa, w, odt, out=out)
        us = time_graph(torch, lambda: [ops.w2a8_gemm(qa, w, odt, out=out) for w in ws], len(ws), replays=4)
        nb, nops = workloads.algorithmic_bytes(c), workloads.algorithmic_ops(c)
        route = L.slimk_w2a8_gemm_auto_route(M, N, K, g)
        extra = {}
        if route == 4:
            ops.w2a8_gemm(qa, ws[0], odt, out=out, kernel="tiled")
            extra["tiled_kernel_us"] = round(time_graph(torch, lambda: [ops.w2a8_gemm(qa, w, odt, out=out, kernel="tiled") for w in ws],
                                                        len(ws), replays=4), 2)
        others.append({"config": cfg, "shape": f"{N}x{K}", "M": M, "group": g, "mode": mode, "weights": "cold" if cold else "warm",
                       "route": {1: "skinny, one strip per workgroup", 2: "tiled", 3: "skinny, shared activations",
                                 4: "every row in one workgroup (SLIMK_KERNEL_MID)"}.get(route, str(route)), **extra,
                       "split_k": L.slimk_w2a8_gemm_auto_split_k(M, N, K, g, 0), "us": round(us, 2),
                       "GBps": round(nb / (us * 1e-6) / 1e9, 1), "frac_hbm": round(nb / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                       "TOPS": round(nops / (us * 1e-6) / 1e12, 1), "frac_int8_mfma": round(nops / (us * 1e-6) / 1e12 / INT8_PEAK_TOPS, 4)})
    cache.clear()
    detail["other_configs"] = others

    # ---- W4A8: 4-bit weights held as two 2-bit planes over a reduction of 2K (hi plane: scales 4s, zero-points
    # zp >> 2; lo plane: scales s, zero-points zp & 3), the activation row laid down twice, one launch of the
    # same kernels.  Timing on random codes in the streaming layout (parity: tests/test_w4a8.py).  Bytes are those
    # of a 4-bit layout: N K / 2 + 2 N G (scales) + N G / 2 (4-bit zero-points) + M K + 4 M + 2 M N.
    from slimkernels_amd.torch import w4 as tw4
    w4rows = []
    for (N, K, g, copies, Ms) in ((14336, 4096, 128, 12, (1, 16, 2048)), (28672, 8192, 128, 4, (1, 16))):
        torch.cuda.empty_cache()
        ws4 = [tw4.W4A8Weight(random_weight(N, 2 * K, g, True), N, K, g) for _ in range(copies)]
        for M in Ms:
            cold = M <= 16
            use = ws4 if cold else ws4[:1] * 4
            x = torch.randn(M, K, device=dev, dtype=torch.float16)
            qa = ops.quantize_act_int8(x, g)
            qa2 = tw4.activation_twice(qa)
            out = torch.empty((M, N), dtype=torch.float16, device=dev)
            for w in (use if cold else use[:1]):
                ops.w2a8_gemm(qa2, w.planes, torch.float16, out=out)
            us = time_graph(torch, lambda: [ops.w2a8_gemm(qa2, w.planes, torch.float16, out=out) for w in use], len(use), replays=4)
            G = K // g
            nb = N * K // 2 + 2 * N * G + N * G // 2 + M * K + 4 * M + 2 * M * N
            nops = 2 * M * N * K
            w4rows.append({"shape": f"{N}x{K}", "M": M, "group": g, "weights": "cold" if cold else "warm", "kernel": "two planes over 2K",
                           "us": round(us, 2),
                           "GBps": round(nb / (us * 1e-6) / 1e9, 1), "frac_hbm": round(nb / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                           "TOPS": round(nops / (us * 1e-6) / 1e12, 1), "frac_int8_mfma": round(nops / (us * 1e-6) / 1e12 / INT8_PEAK_TOPS, 4)})
            if not cold:
                # symmetric weights, many rows: the digits joined in front of the matrix core, one pass over K
                w1 = tw4.W4A8Weight(use[0].planes, N, K, g, uniform_zp8=True)
                tw4.w4a8_gemm_one_pass(qa, w1, torch.float16, out=out)
                us = time_graph(torch, lambda: [tw4.w4a8_gemm_one_pass(qa, w1, torch.float16, out=out) for _ in range(4)], 4, replays=4)
                w4rows.append({"shape": f"{N}x{K}", "M": M, "group": g, "weights": "warm", "kernel": "one pass (zero-point 8)",
                               "us": round(us, 2), "TOPS": round(nops / (us * 1e-6) / 1e12, 1),
                               "frac_int8_mfma": round(nops / (us * 1e-6) / 1e12 / INT8_PEAK_TOPS, 4)})
        del ws4
    detail["w4a8"] = w4rows

    # the decode sweep of the headline with 4-bit weights, as one grouped launch: every GEMM has its own weight
    # (24 weights, 430 MB of 4-bit planes in all: more than the last-level cache, so every launch streams from HBM)
    torch.cuda.empty_cache()
    probs4, bytes4 = [], 0
    for c in cases:
        G = c.K // 128
        w4w = tw4.W4A8Weight(random_weight(c.N, 2 * c.K, 128, True), c.N, c.K, 128)
        _, qa, _ = acts[(c.N, c.K, c.M)]
        probs4.append((tw4.activation_twice(qa), w4w.planes, torch.empty((c.M, c.N), dtype=torch.float16, device=dev)))
        bytes4 += c.N * c.K // 2 + 2 * c.N * G + c.N * G // 2 + c.M * c.K + 4 * c.M + 2 * c.M * c.N
    ops.w2a8_gemm_grouped(probs4, torch.float16)
    us = time_graph(torch, lambda: [ops.w2a8_gemm_grouped(probs4, torch.float16) for _ in range(4)], 4, replays=10)
    detail["w4a8_decode_sweep_grouped"] = {"gemms": len(probs4), "bytes": bytes4, "us": round(us, 2),
                                           "GBps": round(bytes4 / (us * 1e-6) / 1e9, 1),
                                           "frac_hbm": round(bytes4 / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                                           "note": "the int8 rows are laid down twice before the timed region (48 small copies, as act-quant is timed apart)"}

    # ---- weight-only form: fp16 activations as they are, 2-bit codes widened to fp16 in front of the fp16 matrix
    # cores (parity: tests/test_w2a16.py).  Bytes: N K / 4 + 2 N G (scales) + 2 M K + 2 M N.
    torch.cuda.empty_cache()
    a16rows = []
    for (N, K, g, copies, Ms) in ((14336, 4096, 128, 24, (1, 16)), (28672, 8192, 128, 6, (1, 16))):
        ws16 = [random_weight(N, K, g, False) for _ in range(copies)]
        for M in Ms:
            x = torch.randn(M, K, device=dev, dtype=torch.float16)
            out = torch.empty((M, N), dtype=torch.float16, device=dev)
            for w in ws16:
                ops.w2a16_gemm(x, w, torch.float16, out=out)
            us = time_graph(torch, lambda: [ops.w2a16_gemm(x, w, torch.float16, out=out) for w in ws16], len(ws16), replays=4)
            xb = x.to(torch.bfloat16)   # the same rows as bf16 activations (the bf16 matrix cores, a fifth MFMA per 32 k)
            for w in ws16:
                ops.w2a16_gemm(xb, w, torch.float16, out=out)
            us_b = time_graph(torch, lambda: [ops.w2a16_gemm(xb, w, torch.float16, out=out) for w in ws16], len(ws16), replays=4)
            nb = N * K // 4 + 2 * N * (K // g) + 2 * M * K + 2 * M * N
            a16rows.append({"shape": f"{N}x{K}", "M": M, "group": g, "weights": "cold",
                            "split_k": L.slimk_w2a16_gemm_auto_split_k(M, N, K, g), "us": round(us, 2), "us_bf16_activations": round(us_b, 2),
                            "GBps": round(nb / (us * 1e-6) / 1e9, 1), "frac_hbm": round(nb / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)})
        del ws16
    detail["w2a16"] = a16rows
    # one decode step's four linears (the c2 shapes) at one token row, weight-only: one grouped launch against four
    layer = ((4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336))
    sets = [[random_weight(N, K, 128, False) for (N, K) in layer] for _ in range(12)]
    xs = {K: torch.randn(1, K, device=dev, dtype=torch.float16) for K in (4096, 14336)}
    outs = [torch.empty((1, N), dtype=torch.float16, device=dev) for (N, K) in layer]
    def single():
        for ws in sets:
            for w, o in zip(ws, outs):
                ops.w2a16_gemm(xs[w.K], w, torch.float16, out=o)
    def grouped():
        for ws in sets:
            ops.w2a16_gemm_grouped([(xs[w.K], w, o) for w, o in zip(ws, outs)], torch.float16)
    us_single = time_graph(torch, single, len(sets), replays=4)
    us_grouped = time_graph(torch, grouped, len(sets), replays=4)
    nb = sum(N * K // 4 + 2 * N * (K // 128) + 2 * K + 2 * N for (N, K) in layer)
    detail["w2a16_layer_m1"] = {"shapes": [f"{N}x{K}" for (N, K) in layer], "group": 128, "weights": "cold",
                                "us_four_launches": round(us_single, 2), "us_one_grouped_launch": round(us_grouped, 2),
                                "frac_hbm_grouped": round(nb / (us_grouped * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)}
    return detail


def cpu_baseline(np, workloads, shapes):
    """The reference CPU path on a bounded sample of the same workload: one step (the four Llama linears at
    M in {1, 2, 4, 8, 16, 32}), through the oracle's torch-CPU-int-matmul restatement, on this box's host cores."""
    import torch
    from oracle import w2a8_oracle as orc
    torch.set_num_threads(min(16, os.cpu_count() or 1))
    tot_bytes, tot_s, c_port_s = 0, 0.0, 0.0
    for name, M in [(n, m) for n in workloads.LLAMA8B_LINEARS for m in workloads.DECODE_M]:
        N, K = workloads.LLAMA8B_LINEARS[name]
        c = workloads.Case("c2", M, N, K, outliers=True)
        packed, scales, zero = shapes[name].host
        x = workloads.make_activation(c)
        t0 = time.perf_counter()
        orc.torch_reference_forward(x, packed, scales, zero, 128)
        tot_s += time.perf_counter() - t0
        q, s_a, _ = orc.c_act_quant(x, 128)
        t0 = time.perf_counter()
        orc.c_gemm_fused(q, s_a, packed, scales, zero, 128)
        c_port_s += time.perf_counter() - t0
        tot_bytes += workloads.algorithmic_bytes(c)
    return {"value": round(tot_bytes / tot_s / 1e9, 4), "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": "one step of the workload, once: the four c2 shapes at M in {1,2,4,8,16,32} (act-quant + unpack + torch CPU "
                      "int32 matmul per group + fp32 epilogue); algorithmic bytes / wall seconds",
            "seconds": round(tot_s, 3), "host_cpus": os.cpu_count(),
            "scalar_c_port_1core_GBps": round(tot_bytes / c_port_s / 1e9, 4)}


if __name__ == "__main__":
    main()
