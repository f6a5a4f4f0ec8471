#!/usr/bin/env python3
"""Benchmark of the NF4 decode-shape dequant-GEMV path on one MI355X.

One "step" = one pass of the hot path over BASELINE.json's config 2: the five Llama-3-8B
projection shapes as standalone NF4 linears (blocksize 64, fp32 absmax), x bf16 with
M in {1, 4, 16}: 15 calls of nf4hip_gemv through the C ABI, all operands resident in HBM.
Every call of a step reads a different copy of its weight from a ring larger than the 256 MB
Infinity Cache, so the reported rate is an HBM rate.

Prints ONE JSON line:
  value     = algorithmic bytes of a step * steps / wall time of the timed region  (GB/s)
  roofline  = the kernel that takes the largest share of a step (the three decode kernels are
              timed group by group): algorithmic bytes per launch / average launch duration, from
              HIP events recorded inside the timed region on the launch stream, against the
              8 TB/s HBM peak; config.kernels lists all three groups, each with the time of a
              launch that only reads the same weights (pure_read_launch_us, frac_of_pure_read);
              config.by_kernel: the same calls grouped by the kernel the library launches for them (nf4hip_gemv_plan),
              timed after the timed region
  config.prefill = BASELINE config 3 (M in {512, 2048, 8192}) run after the timed region: TFLOP/s of the fused GEMM
              kernel, of HIP dequantize + the hand-written dense kernel and of HIP dequantize + the library GEMM, vs
              the bf16 MFMA peak; which of them the router picks
  config.llama70b_double_quant = BASELINE config 5 (nested absmax, M in {1, 16, 2048}) run after the timed region
  config.decode = BASELINE config 4 (full Llama-3-8B architecture, greedy decode, batch 1 and 8)
              run after the timed region: decode tokens/s, the second half of the metric
  cpu_baseline = the reference's CPU-side route (torch-eager dequantize + linear, restated in
              oracle/nf4_oracle.py) timed on this box's host cores on a bounded sample
"""

from __future__ import annotations

import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SHAPES = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (128256, 4096)]  # [N, K]
MS = (1, 4, 16)
BLOCKSIZE = 64
HBM_PEAK_GBS = 8000.0
RING_BYTES = 640 << 20  # per shape: more than twice the 256 MB Infinity Cache


def algorithmic_bytes(M: int, N: int, K: int) -> int:
    """codes + fp32 absmax + code book + x + out, each moved once."""
    n = N * K
    return n // 2 + 4 * (n // BLOCKSIZE) + 64 + 2 * M * K + 2 * M * N


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (defaults: a timed region of ~55 ms behind ~15 ms of the same work; the first few milliseconds after an idle
    # GPU run 15-20 % slower -- clocks, first touch of every weight copy -- and a 5 + 20 step run measures mostly that)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="bound on the CPU baseline sample (0 disables)")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill-regime section (BASELINE config 3) and the quantize/dequantize bandwidth section")
    ap.add_argument("--section-warm-seconds", type=float, default=0.08,
                    help="warm-up ahead of every timing of the prefill / double-quant / codec sections (0: three calls, for counter runs)")
    ap.add_argument("--decode-tokens", type=int, default=128,
                    help="tokens of the Llama-3-8B greedy decode that follows the GEMV pass (0 disables)")
    args = ap.parse_args()
    global SECTION_WARM_SECONDS
    SECTION_WARM_SECONDS = args.section_warm_seconds
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only; --gpus {args.gpus} is not supported "
              "(the path would shard like a dense linear: by rows of W for q/k/v/gate/up/lm_head, by columns for o/down)", file=sys.stderr)
        return 2

    import torch

    ta = importlib.import_module("lightning-thunder_amd")
    lib = ta._lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    code = ta.nf4_code(dev)

    # ---- synthetic weights: seeded bf16 N(0, 0.02), quantized by the HIP kernel, `ncopy` copies ----
    # Copy 0 of every ring is the canonical tensor of the configuration, drawn on the CPU (weight seed 2000 + index
    # of the shape, activation seed 200000 + 100 * shape + index of M) and fingerprinted with SHA-256 so that runs on
    # different boxes can be compared; the other copies only exist to defeat the Infinity Cache and are drawn on the
    # GPU.
    import hashlib

    def sha(t):
        return hashlib.sha256(t.contiguous().view(torch.int16).numpy().tobytes()).hexdigest()[:16]

    fingerprints = {}
    weights = {}
    for si, (N, K) in enumerate(SHAPES):
        n = N * K
        per_copy = n // 2 + 4 * (n // BLOCKSIZE)
        ncopy = max(2, -(-RING_BYTES // per_copy))
        ring = []
        for c in range(ncopy):
            if c == 0:
                w_cpu = (torch.randn(N, K, generator=torch.Generator().manual_seed(2000 + si), dtype=torch.float32) * 0.02).to(torch.bfloat16)
                fingerprints[f"W[{N},{K}] seed {2000 + si}"] = sha(w_cpu)
                w = w_cpu.to(dev)
                del w_cpu
            else:
                g = torch.Generator(device=dev).manual_seed(2000 + 100 * si + c)
                w = (torch.randn(N, K, generator=g, device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16)
            qw, absmax, _ = ta.quantize_nf4(w, BLOCKSIZE)
            ring.append((qw, absmax))
            del w
        weights[(N, K)] = ring
    xs, outs = {}, {}
    for mi, M in enumerate(MS):
        for si, (N, K) in enumerate(SHAPES):
            seed = 200000 + 100 * si + mi
            x_cpu = torch.randn(M, K, generator=torch.Generator().manual_seed(seed), dtype=torch.float32).to(torch.bfloat16)
            fingerprints[f"x[{M},{K}] seed {seed}"] = sha(x_cpu)
            xs[(M, N, K)] = x_cpu.to(dev)
            outs[(M, N, K)] = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    ws_bytes = max(lib.nf4hip_gemv_workspace_bytes(M, N, K) for M in MS for (N, K) in SHAPES)
    ws = torch.zeros(max(ws_bytes, 1 << 20), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream()
    sptr = stream.cuda_stream

    def launch(M, N, K, it):
        qw, absmax = weights[(N, K)][it % len(weights[(N, K)])]
        rc = lib.nf4hip_gemv(xs[(M, N, K)].data_ptr(), ta._lib.BF16, M, qw.data_ptr(), absmax.data_ptr(), code.data_ptr(),
                             None, N, K, BLOCKSIZE, outs[(M, N, K)].data_ptr(), ws.data_ptr(), ws.numel(), sptr)
        if rc:
            ta._lib.check(rc)

    # the calls of a step grouped by rows of x, each group timed with HIP events on the launch stream (which kernel
    # serves a call is the library's choice: profiles/bench_gemv_kernel_trace.txt lists them per shape)
    groups = [
        (f"nf4hip_gemv M={M}", f"M = {M}: the five shapes, one launch each", [(M, N, K) for (N, K) in SHAPES]) for M in MS
    ]
    group_bytes = [sum(algorithmic_bytes(*c) for c in calls) for _, _, calls in groups]
    bytes_step = sum(group_bytes)

    # one chain of events over the timed region: event s * G + g opens group g of step s and closes
    # the group before it (a record between two launches costs a few microseconds of the stream)
    def step(it, ev=None, s=0):
        for gi, (_, _, calls) in enumerate(groups):
            if ev:
                ev[s * len(groups) + gi].record(stream)
            for c in calls:
                launch(*c, it)

    # A plain device copy of known size (256 MiB read + 256 MiB written), outside the timed region:
    # hardware-counter runs (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) are scaled by what the same
    # counter reads for this kernel.
    calib_src = torch.empty(64 << 20, dtype=torch.float32, device=dev).normal_()
    calib_dst = torch.empty_like(calib_src)
    calib_dst.copy_(calib_src)
    del calib_src, calib_dst

    for it in range(args.warmup):
        step(it)
    events = [torch.cuda.Event(enable_timing=True) for _ in range(len(groups) * args.steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for it in range(args.steps):
        step(args.warmup + it, events, it)
    events[-1].record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    wall = t1 - t0
    ms_per_step = wall * 1e3 / args.steps
    value = bytes_step * args.steps / wall / 1e9

    # the same calls on ONE copy of every weight (it = 0 throughout): what the Infinity Cache makes of them; reported
    # next to the cold numbers, never as the metric
    warm_events = [torch.cuda.Event(enable_timing=True) for _ in range(len(groups) * 10 + 1)]
    for s_ in range(10):
        step(0, warm_events, s_)
    warm_events[-1].record(stream)
    torch.cuda.synchronize()

    # By KERNEL, after the timed region (which kernel serves a call is the library's answer, nf4hip_gemv_plan): the same
    # 15 calls, cold, issued in four segments with an event between them -- the calls with one row of x that the kernel
    # with the largest share of the bytes (the staged kernel, where in use) does not serve, those it serves, then the same
    # for the remaining calls.  An event record costs about 3 us of the stream and launches of the staged kernel that
    # follow each other directly run a few per cent slower than in the order of the timed region, so these figures are a
    # little pessimistic.
    import ctypes

    KERNEL_NAMES = {1: "gemv_rows_kernel", 2: "gemv_quad_kernel", 3: "gemv_quad_kernel on two halves of x", 4: "gemv_tiles_kernel",
                    5: "gemv_stage_kernel"}

    def kernel_of(M, N, K):
        plan = (ctypes.c_int * 4)()
        ta._lib.check(lib.nf4hip_gemv_plan(M, N, K, BLOCKSIZE, 0, ctypes.byref(plan)))
        return plan[0]

    calls_all = [(M, N, K) for M in MS for (N, K) in SHAPES]
    kern = {c: kernel_of(*c) for c in calls_all}
    weight_of = {}
    for c in calls_all:
        weight_of[kern[c]] = weight_of.get(kern[c], 0) + algorithmic_bytes(*c)
    main_kernel = max(weight_of, key=weight_of.get)
    segments = [[c for c in calls_all if (c[0] == MS[0]) == first and (kern[c] == main_kernel) == is_main]
                for first in (True, False) for is_main in (False, True)]
    segments = [seg for seg in segments if seg]
    k_events = [torch.cuda.Event(enable_timing=True) for _ in range(len(segments) * args.steps + 1)]
    for st in range(args.steps):
        for si_, seg in enumerate(segments):
            k_events[st * len(segments) + si_].record(stream)
            for c in seg:
                launch(*c, args.warmup + args.steps + st)
    k_events[-1].record(stream)
    torch.cuda.synchronize()
    by_kernel = {}
    for si_, seg in enumerate(segments):
        name = " + ".join(KERNEL_NAMES[k] for k in sorted({kern[c] for c in seg}))
        ms = sum(k_events[st * len(segments) + si_].elapsed_time(k_events[st * len(segments) + si_ + 1]) for st in range(args.steps)) / args.steps
        e = by_kernel.setdefault(name, {"calls": [], "ms": 0.0})
        e["calls"] += seg
        e["ms"] += ms
    by_kernel_rows = []
    for name, e in by_kernel.items():
        byts = sum(algorithmic_bytes(*c) for c in e["calls"])
        by_kernel_rows.append({
            "kernel": name, "calls": "; ".join(f"M={M} [{N},{K}]" for (M, N, K) in e["calls"]), "launches_per_step": len(e["calls"]),
            "algorithmic_bytes_per_launch": byts // len(e["calls"]), "avg_launch_us": round(e["ms"] * 1e3 / len(e["calls"]), 3),
            "achieved_GBs": round(byts / (e["ms"] * 1e-3) / 1e9, 1), "frac_of_hbm_peak": round(byts / (e["ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        })

    def pct(sorted_vals, q):
        return sorted_vals[min(len(sorted_vals) - 1, int(q * len(sorted_vals)))]

    # What one launch that only reads the same bytes takes (codes and absmax of a weight, cold, from the same rings;
    # libnf4hip_probe.so: 16 bytes per lane, whole lines, non-temporal, nothing computed): per shape the average of 20
    # launches back to back between two events -- the same protocol as the groups above, launch gaps included.
    pure_read_us = {}
    probe_path = os.path.join(ROOT, "lightning-thunder_amd", "libnf4hip_probe.so")
    if os.path.exists(probe_path):
        probe = ctypes.CDLL(probe_path)
        probe.nf4hip_probe_stream_read.restype = ctypes.c_int
        probe.nf4hip_probe_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
        sink = torch.zeros(4, dtype=torch.int32, device=dev)
        for (N, K) in SHAPES:
            ring = weights[(N, K)]

            def read(i):
                qw, absmax = ring[i % len(ring)]
                rc = probe.nf4hip_probe_stream_read(qw.data_ptr(), qw.numel() // 16 * 16, absmax.data_ptr(), absmax.numel() * 4 // 16 * 16,
                                                    sink.data_ptr(), sptr)
                assert rc == 0, rc

            for i in range(3):
                read(i)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for i in range(20):
                read(3 + i)
            e1.record(stream)
            torch.cuda.synchronize()
            pure_read_us[(N, K)] = e0.elapsed_time(e1) * 1e3 / 20

    kernels = []
    for gi, (name, what, calls) in enumerate(groups):
        G = len(groups)
        per_step = sorted(events[st * G + gi].elapsed_time(events[st * G + gi + 1]) for st in range(args.steps))
        ms = sum(per_step) / args.steps
        warm = sorted(warm_events[st * G + gi].elapsed_time(warm_events[st * G + gi + 1]) for st in range(10))
        per_launch = 1e3 / len(calls)
        kernels.append({
            "kernel": name, "calls": what, "launches_per_step": len(calls),
            "algorithmic_bytes_per_launch": group_bytes[gi] // len(calls),
            "avg_launch_us": round(ms * per_launch, 3),
            "median_launch_us": round(pct(per_step, 0.5) * per_launch, 3),
            "p10_launch_us": round(pct(per_step, 0.1) * per_launch, 3),
            "p90_launch_us": round(pct(per_step, 0.9) * per_launch, 3),
            "warm_median_launch_us": round(pct(warm, 0.5) * per_launch, 3),
            "achieved_GBs": round(group_bytes[gi] / (ms * 1e-3) / 1e9, 1),
            "share_of_step_time": round(ms / ms_per_step, 3),
        })
        if pure_read_us:
            # a launch that only reads each weight of the group, and how close the group's launches come to it
            pr = sum(pure_read_us[(N, K)] for (_, N, K) in calls) / len(calls)
            kernels[-1]["pure_read_launch_us"] = round(pr, 3)
            kernels[-1]["frac_of_pure_read"] = round(pr / (ms * per_launch), 4)
    dom = max(kernels, key=lambda k: k["share_of_step_time"])

    # HBM traffic per launch of that group: counter figures (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE) cannot be taken
    # inside this run; the committed summary of the same command is quoted and named as the source
    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", "gemv_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic = json.load(f).get(dom["kernel"], {}).get("hbm_bytes_per_launch")
        if traffic is not None:
            traffic_source = "profiles/gemv_traffic.json (rocprofv3 --pmc runs of this command, not measured in this run)"

    result = {
        "metric": "NF4 dequant-GEMV HBM GB/s (% of peak) + decode tok/s, Llama-3-8B shapes, 1 GPU",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic (CPU-seeded bf16 N(0,0.02) weights quantized to NF4 by the HIP kernel, x bf16 N(0,1); fingerprints in config.inputs_sha256_16)",
        "config": {
            "workload": "BASELINE config 2: Llama-3-8B projection shapes [4096,4096],[1024,4096],[14336,4096],"
                        "[4096,14336],[128256,4096] as NF4 linears (blocksize 64, fp32 absmax), M in {1,4,16}; "
                        "15 nf4hip_gemv calls per step, weights rotated through >= 640 MB rings",
            "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
            "algorithmic_bytes_per_step": bytes_step,
            "kernels": kernels,
            "by_kernel": by_kernel_rows,
            "pure_read_us_by_shape": {f"[{N},{K}]": round(t, 2) for (N, K), t in pure_read_us.items()},
            "inputs_sha256_16": fingerprints,
        },
        "roofline": {
            "kernel": f"{dom['kernel']} (the {dom['launches_per_step']} calls per step that take the most time)",
            "bound": "hbm",
            "achieved": dom["achieved_GBs"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(dom["achieved_GBs"] / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "traffic_source": traffic_source,
            "algorithmic_bytes_per_launch": dom["algorithmic_bytes_per_launch"],
            "avg_launch_us": dom["avg_launch_us"],
        },
    }

    del weights, xs, outs, ws
    torch.cuda.empty_cache()
    if not args.no_prefill:
        result["config"]["prefill"] = prefill_section(torch, ta)
        result["config"]["llama70b_double_quant"] = double_quant_section(torch, ta)
        result["config"]["codec"] = codec_section(torch, ta)
    if args.decode_tokens > 1:
        result["config"]["decode"] = llama_decode(torch, ta, args.decode_tokens)
    if args.cpu_seconds > 0:
        result["cpu_baseline"] = cpu_baseline(torch, args.cpu_seconds)
    print(json.dumps(result))
    return 0


MFMA_BF16_PEAK_TFLOPS = 2516.6  # 256 CUs x 2.4 GHz x 4096 flop/clk/CU


SECTION_WARM_SECONDS = 0.08  # (--section-warm-seconds)


def _timed(torch, fn, reps, warm=3, warm_seconds=None):
    """Seconds per call: the median of three event-bracketed batches of ``reps`` calls after at least ``warm`` untimed
    ones and ``warm_seconds`` of them.  (Every case of the sections below starts on a GPU that sat idle while the
    host drew its inputs; for tens of milliseconds after that the same kernel runs 10-15 % slower -- a 250 us GEMM
    39 % of the MFMA peak after three calls, 41 % after thirty, 44 % after three hundred -- and three calls measured
    that, not the kernel.)"""
    if warm_seconds is None:
        warm_seconds = SECTION_WARM_SECONDS
    t0, n = time.perf_counter(), 0
    while n < warm or time.perf_counter() - t0 < warm_seconds:
        for _ in range(max(1, reps)):
            fn()
        torch.cuda.synchronize()
        n += max(1, reps)
    per = []
    for _ in range(3):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        per.append(e0.elapsed_time(e1) * 1e-3 / reps)
    return sorted(per)[1]


def _cpu_seeded(torch, shape, seed, std):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float32) * std).to(torch.bfloat16)


def prefill_section(torch, ta) -> dict:
    """BASELINE config 3, outside the timed region of the GEMV metric: the five Llama-3-8B projection shapes (and the
    fused gate/up weight [28672, 4096]) with M in {512, 2048, 8192} rows of x.  Every case is timed on THREE routes
    -- the hand-written fused kernel (nf4hip_gemm: NF4 codes expanded on chip straight into MFMA operands),
    nf4hip_dequantize + the hand-written dense MFMA kernel (nf4hip_linear), and nf4hip_dequantize + the vendor
    library's GEMM -- and ``router_pick`` marks the one ``matmul_nf4`` picks (it times all three on its first call of a
    shape; the library has to win by more than 3 %).  TFLOP/s = 2 M N K / time against the bf16 MFMA peak; HIP events
    bracket 10 calls (4 beyond 4 TFLOP per call) after 80 ms of warm-up calls.  ``dense_kernel_alone``: nf4hip_linear and the
    library GEMM on the already dequantized weight.
    ``rows64``: the same weights with 64 rows of x (fused kernel with K split over workgroups vs the dense route)."""
    dev = torch.device("cuda:0")
    F = ta.functional
    L, lib = ta._lib, ta._lib.load()
    code = ta.nf4_code(dev)
    sptr = torch.cuda.current_stream().cuda_stream
    names = {"dequant+gemm": "nf4hip_dequantize + nf4hip_linear", "gemm": "nf4hip_gemm (fused)",
             "dequant+libgemm": "nf4hip_dequantize + library GEMM"}
    rows, mid, alone = [], [], []
    shapes = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (128256, 4096), (28672, 4096)]
    for si, (N, K) in enumerate(shapes):
        w = _cpu_seeded(torch, (N, K), 2000 + si if si < 5 else 2900, 0.02).to(dev)  # configs 2 and 3 share their weights
        qw, absmax, _ = ta.quantize_nf4(w, BLOCKSIZE)
        del w
        for mi, M in enumerate((512, 2048, 8192)):
            x = _cpu_seeded(torch, (M, K), 300000 + 100 * si + mi, 1.0).to(dev)
            out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
            flops = 2.0 * M * N * K
            reps = 10 if flops < 4e12 else 4
            need = lib.nf4hip_gemm_workspace_bytes(M, N, K)
            ws = torch.zeros(max(need, 16), dtype=torch.uint8, device=dev)

            def fused():
                L.check(lib.nf4hip_gemm(x.data_ptr(), L.BF16, M, qw.data_ptr(), absmax.data_ptr(), code.data_ptr(), None, N, K, BLOCKSIZE,
                                        out.data_ptr(), ws.data_ptr(), ws.numel(), sptr))

            def dense():
                return F.linear_bf16(x, F.dequantize_nf4(qw, absmax, code, BLOCKSIZE, torch.bfloat16, (N, K)))

            def dense_lib():
                return torch.nn.functional.linear(x, F.dequantize_nf4(qw, absmax, code, BLOCKSIZE, torch.bfloat16, (N, K)))

            tf, td, tl = _timed(torch, fused, reps), _timed(torch, dense, reps), _timed(torch, dense_lib, reps)
            # the router's pick: matmul_nf4 times the routes itself on its first call of a shape on this device
            ta.matmul_nf4(x, qw, None, absmax, code, BLOCKSIZE, torch.bfloat16, (N, K))
            router = names[F.fused_route(x, None, BLOCKSIZE, torch.bfloat16, (N, K))]
            for route, t in ((names["gemm"], tf), (names["dequant+gemm"], td), (names["dequant+libgemm"], tl)):
                rows.append({"N": N, "K": K, "M": M, "route": route, "router_pick": route == router, "us": round(t * 1e6, 1),
                             "tflops": round(flops / t / 1e12, 1), "frac_of_mfma_peak": round(flops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)})
            if M >= 2048:
                wd = F.dequantize_nf4(qw, absmax, code, BLOCKSIZE, torch.bfloat16, (N, K))
                ta_, tb_ = _timed(torch, lambda: F.linear_bf16(x, wd), reps), _timed(torch, lambda: torch.nn.functional.linear(x, wd), reps)
                alone.append({"N": N, "K": K, "M": M, "nf4hip_linear_us": round(ta_ * 1e6, 1),
                              "nf4hip_linear_frac_of_mfma_peak": round(flops / ta_ / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                              "library_us": round(tb_ * 1e6, 1),
                              "library_frac_of_mfma_peak": round(flops / tb_ / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)})
                del wd
            del x, out
        # 64 rows of x (between the decode and the prefill regime): the router's choice, which is the fused
        # kernel with K split over workgroups, next to the dense route (dequantize + library GEMM) forced
        x = _cpu_seeded(torch, (64, K), 390000 + si, 1.0).to(dev)
        route = F.fused_route(x, None, BLOCKSIZE, torch.bfloat16, (N, K))
        t = _timed(torch, lambda: ta.matmul_nf4(x, qw, None, absmax, code, BLOCKSIZE, torch.bfloat16, (N, K)), 20)
        td = _timed(torch, lambda: torch.nn.functional.linear(x, F.dequantize_nf4(qw, absmax, code, BLOCKSIZE, torch.bfloat16, (N, K))), 20)
        mid.append({"N": N, "K": K, "M": 64, "route": route, "us": round(t * 1e6, 1), "dense_route_us": round(td * 1e6, 1)})
        del qw, absmax
    return {"peak_tflops": MFMA_BF16_PEAK_TFLOPS, "cases": rows, "dense_kernel_alone": alone, "rows64": mid}


def double_quant_section(torch, ta) -> dict:
    """BASELINE config 5, outside the timed region of the GEMV metric: Llama-3-70B layer shapes with double-quantised
    statistics (NF4 blocksize 64, absmax in 8 bits over nested blocks of 256 plus an fp32 offset), M in {1, 16, 2048},
    through ``matmul_nf4`` on the nested form.  Decode rows are rated against the HBM peak over their algorithmic bytes
    (codes + 8-bit absmax + nested statistics + x + out), cold (weights rotated through a ring larger than the Infinity
    Cache); M = 2048 against the bf16 MFMA peak."""
    dev = torch.device("cuda:0")
    F = ta.functional
    code = ta.nf4_code(dev)
    lib = ta._lib.load()
    dq_shapes = [(8192, 8192), (1024, 8192), (28672, 8192), (8192, 28672)]
    ws = torch.zeros(max(1 << 20, max(lib.nf4hip_gemv_workspace_bytes(M, N, K) for M in (1, 16) for (N, K) in dq_shapes)),
                     dtype=torch.uint8, device=dev)
    sptr = torch.cuda.current_stream().cuda_stream
    cases = []
    for si, (N, K) in enumerate(dq_shapes):
        n = N * K
        per_copy = n // 2 + n // BLOCKSIZE
        ncopy = max(2, -(-RING_BYTES // per_copy))
        ring = []
        for c in range(ncopy):
            if c == 0:
                w = _cpu_seeded(torch, (N, K), 5000 + si, 0.02).to(dev)
            else:
                g = torch.Generator(device=dev).manual_seed(5000 + 100 * si + c)
                w = (torch.randn(N, K, generator=g, device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16)
            qw, absmax, _ = ta.quantize_nf4(w, BLOCKSIZE)
            ring.append((qw, ta.compress_absmax(absmax)))
            del w, absmax
        nested_bytes = n // BLOCKSIZE + 4 * -(-(n // BLOCKSIZE) // 256) + 1024 + 4
        for mi, M in enumerate((1, 16, 2048)):
            x = _cpu_seeded(torch, (M, K), 500000 + 100 * si + mi, 1.0).to(dev)
            if M > 16:
                ta.matmul_nf4(x, ring[0][0], None, ring[0][1], code, BLOCKSIZE, torch.bfloat16, (N, K))  # lets the router time both routes
            route = F.fused_route(x, None, BLOCKSIZE, torch.bfloat16, (N, K), nested=True)
            it = [0]
            out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)

            def call():
                qw, nq = ring[it[0] % ncopy]
                it[0] += 1
                if M > 16:
                    return ta.matmul_nf4(x, qw, None, nq, code, BLOCKSIZE, torch.bfloat16, (N, K))
                # decode rows go straight to the C ABI, as the GEMV metric's own launches do
                rc = lib.nf4hip_gemv_dq(x.data_ptr(), ta._lib.BF16, M, qw.data_ptr(), nq.q.data_ptr(), nq.absmax2.data_ptr(),
                                        nq.map256.data_ptr(), float(nq.offset), nq.blocksize, code.data_ptr(), None, N, K,
                                        BLOCKSIZE, out.data_ptr(), ws.data_ptr(), ws.numel(), sptr)
                if rc:
                    ta._lib.check(rc)

            t = _timed(torch, call, 20 if M <= 16 else 6, warm=ncopy if M <= 16 else 3)
            row = {"N": N, "K": K, "M": M, "route": route, "us": round(t * 1e6, 1)}
            if M <= 16:
                byts = n // 2 + nested_bytes + 64 + 2 * M * K + 2 * M * N
                row.update({"algorithmic_bytes": byts, "GBs": round(byts / t / 1e9, 1), "frac_of_hbm_peak": round(byts / t / 1e9 / HBM_PEAK_GBS, 4)})
            else:
                flops = 2.0 * M * N * K
                row.update({"tflops": round(flops / t / 1e12, 1), "frac_of_mfma_peak": round(flops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)})
            cases.append(row)
        del ring
    return {"note": "decode rows (M <= 16) call nf4hip_gemv_dq through the C ABI; M = 2048 goes through matmul_nf4 and its router", "cases": cases}


def codec_section(torch, ta) -> dict:
    """The two HBM-bound conversion kernels, outside the timed region of the GEMV metric: quantize
    (bf16 -> NF4) and dequantize (NF4 -> bf16) of one Llama-3-8B FFN weight and of the lm_head, cold
    (a ring of distinct buffers larger than the 256 MB Infinity Cache).  GB/s over the algorithmic
    bytes: 2n read + n/2 + n/16 written, and n/2 + n/16 + 64 read + 2n written."""
    dev = torch.device("cuda:0")
    code = ta.nf4_code(dev)
    out = {}
    for N, K in [(14336, 4096), (128256, 4096)]:
        n = N * K
        ncopy = max(2, (640 << 20) // (2 * n) + 1)
        g = torch.Generator(device=dev).manual_seed(N)
        ws = [(torch.randn(N, K, generator=g, device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16) for _ in range(ncopy)]
        packed = [ta.quantize_nf4(w, BLOCKSIZE) for w in ws]
        torch.cuda.synchronize()

        def timed(fn, reps=2 * ncopy):
            t0 = time.perf_counter()
            while True:  # (as in _timed: past the slow first milliseconds after an idle GPU)
                for i in range(ncopy):
                    fn(i)
                torch.cuda.synchronize()
                if time.perf_counter() - t0 >= SECTION_WARM_SECONDS:
                    break
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(reps):
                fn(i % ncopy)
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e-3 / reps

        # through the C ABI with preallocated outputs: the kernels, not the allocator
        lib = ta._lib.load()
        sptr = torch.cuda.current_stream().cuda_stream
        qout = torch.empty(n // 2, dtype=torch.uint8, device=dev)
        aout = torch.empty(n // BLOCKSIZE, dtype=torch.float32, device=dev)
        wout = torch.empty(N, K, dtype=torch.bfloat16, device=dev)

        def quant(i):
            ta._lib.check(lib.nf4hip_quantize(ws[i].data_ptr(), ta._lib.BF16, n, BLOCKSIZE, qout.data_ptr(), aout.data_ptr(), sptr))

        def dequant(i):
            ta._lib.check(lib.nf4hip_dequantize(packed[i][0].data_ptr(), packed[i][1].data_ptr(), code.data_ptr(), n, BLOCKSIZE,
                                                wout.data_ptr(), ta._lib.BF16, sptr))

        tq = timed(quant)
        td = timed(dequant)
        bq = 2 * n + n // 2 + 4 * (n // BLOCKSIZE)
        bd = n // 2 + 4 * (n // BLOCKSIZE) + 64 + 2 * n
        out[f"{N}x{K}"] = {
            "quantize_us": round(tq * 1e6, 1), "quantize_GBs": round(bq / tq / 1e9, 1), "quantize_frac_of_hbm_peak": round(bq / tq / 1e9 / HBM_PEAK_GBS, 3),
            "dequantize_us": round(td * 1e6, 1), "dequantize_GBs": round(bd / td / 1e9, 1), "dequantize_frac_of_hbm_peak": round(bd / td / 1e9 / HBM_PEAK_GBS, 3),
        }
        del ws, packed
    return out


def llama_decode(torch, ta, n_new: int) -> dict:
    """BASELINE config 4, outside the timed region of the GEMV metric: the full Llama-3-8B
    architecture with random-init weights, every nn.Linear NF4-quantized through the transform,
    greedy decode from random prompts of length 512 at batch 1 and 8 (and 32), decode step replayed from a
    HIP graph, Q/K/V and gate/up as one linear each."""
    D = importlib.import_module("lightning-thunder_amd.decode")
    dev = torch.device("cuda:0")
    cfg = D.LlamaConfig.llama3_8b(fused_projections=True, gate_up_interleaved=True)
    model = D.build_llama(cfg, device=dev, seed=4000)
    jm = ta.jit(model, transforms=[ta.BitsAndBytesLinearQuant4bit()])
    nweights = sum(m.weight.numel() for m in model.modules() if isinstance(m, torch.nn.Linear))
    out = {
        "model": "Llama-3-8B architecture (32 layers, d 4096, 32q/8kv heads, FFN 14336, vocab 128256), random init, "
                 "all 161 linears NF4 (QKV and gate/up fused, gate and up rows interleaved), prompt 512, greedy, HIP-graph decode step; "
                 "decode_tok_per_s: residual add + RMSNorm + SiLU*up in the epilogues of the NF4 decode kernels (up to sixteen rows of x), "
                 "rotary + cache + attention and sampling as HIP glue kernels; _separate_glue: all of that work as HIP glue kernels "
                 "between the linears; _torch_glue: as PyTorch ops",
        "new_tokens": n_new,
        "linear_weight_bytes_per_token": int(nweights * 0.5625),
        "hbm_bound_tok_per_s_batch1": round(HBM_PEAK_GBS * 1e9 / (nweights * 0.5625), 1),
    }
    for B in (1, 8, 32):  # 32 is not a BASELINE case: the linears of its step run through nf4hip_gemm (M = 32)
        g = torch.Generator(device=dev).manual_seed(4000 + B)
        prompt = torch.randint(0, cfg.vocab, (B, 512), generator=g, device=dev)
        D.greedy_decode(jm, cfg, prompt, n_new=1, use_graph=False)  # untimed: library start-up, GEMM heuristics
        res, toks = {}, {}
        # the single-token step with residual add / RMSNorm / SiLU * up done by the epilogues of the NF4 decode kernels
        # where those take them (up to sixteen rows of x; rotary + cache + attention and sampling as HIP glue kernels), with
        # all of that work as HIP glue kernels of its own, and with plain PyTorch ops in its place
        for key, glue, epi in (("", True, True), ("_separate_glue", True, False), ("_torch_glue", False, False)):
            if (B > 8 and not glue) or (B > 16 and glue and not epi):
                continue  # beyond sixteen rows of x the linears run as GEMMs, without epilogues: the first variant is the second
            cfg.hip_glue, cfg.linear_epilogues = glue, epi
            toks[key], st = D.greedy_decode(jm, cfg, prompt, n_new=n_new, use_graph=True)
            res[f"decode_tok_per_s{key}"] = round(st["decode_tok_per_s"], 1)
            res[f"ms_per_step{key}"] = round(st["decode_s"] / st["decode_steps"] * 1e3, 3)
            res["prefill_ms"] = round(st["prefill_s"] * 1e3, 1)
        # outside the timed loops: do the variants of the step emit the same tokens?  Per variant, the number of leading
        # tokens (of the first 16) that every sequence shares with the first variant; random-init logits have close
        # runners-up, so a late parting is a tie broken differently, an early one would be a bug (the tests assert it)
        head = min(16, n_new)
        for key, t in toks.items():
            if key:
                same = (t[:, :head] == toks[""][:, :head]).all(dim=0).int().cumprod(0).sum()
                res[f"leading_tokens_equal_of_{head}{key}"] = int(same)
        out[f"batch{B}"] = res
    return out


def _cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(torch, budget_s: float) -> dict:
    """The reference's CPU route (torch-eager NF4 dequantize, then F.linear) on a bounded sample:
    BASELINE config 1, one Linear(4096 -> 4096), x [1, 4096], on this box's host cores.  ``value`` is the whole
    route; the split (dequantize | matmul) and the weights-already-dequantized variant are reported beside it."""
    from oracle import nf4_oracle as O

    N, K, M = 4096, 4096, 1
    w = _cpu_seeded(torch, (N, K), 1000, 0.02)
    x = _cpu_seeded(torch, (M, K), 100000, 1.0)
    qw, absmax = O.C().quantize(w, BLOCKSIZE)
    lut = O.nf4_lut()
    threads = torch.get_num_threads()

    def median_time(fn, budget, most=200):
        fn()  # warm-up
        times, t_end = [], time.perf_counter() + budget
        while len(times) < 3 or (time.perf_counter() < t_end and len(times) < most):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        times.sort()
        return times[len(times) // 2], len(times)

    whole, n_whole = median_time(lambda: O.matmul_4bit_eager(x, qw, None, absmax, lut, BLOCKSIZE, torch.bfloat16, (N, K)), budget_s * 0.5)
    deq_t, _ = median_time(lambda: O.dequantize_4bit_eager(qw, absmax, lut, BLOCKSIZE, torch.bfloat16, (N, K)), budget_s * 0.3)
    wd = O.dequantize_4bit_eager(qw, absmax, lut, BLOCKSIZE, torch.bfloat16, (N, K))
    mm_t, _ = median_time(lambda: torch.nn.functional.linear(x, wd), budget_s * 0.2)
    return {
        "value": round(algorithmic_bytes(M, N, K) / whole / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{n_whole} calls of torch-eager dequantize_4bit + F.linear, NF4 Linear(4096->4096), x [1,4096] bf16 "
                  f"(BASELINE config 1); median {whole * 1e3:.1f} ms per call",
        "ms_whole_route": round(whole * 1e3, 2),
        "ms_dequantize_only": round(deq_t * 1e3, 2),
        "ms_matmul_on_dequantized_weight": round(mm_t * 1e3, 3),
        "torch_num_threads": threads,
        "os_cpu_count": os.cpu_count(),
        "cpu_model": _cpu_model(),
    }


if __name__ == "__main__":
    sys.exit(main())
