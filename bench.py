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
              8 TB/s HBM peak; config.kernels lists all three
  config.prefill = BASELINE config 3 (M in {512, 2048, 8192}) run after the timed region: TFLOP/s of the
              default route (HIP dequantize + dense GEMM) and of the fused GEMM kernel, vs the bf16 MFMA peak
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
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="bound on the CPU baseline sample (0 disables)")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill-regime section (BASELINE config 3) and the quantize/dequantize bandwidth section")
    ap.add_argument("--decode-tokens", type=int, default=128,
                    help="tokens of the Llama-3-8B greedy decode that follows the GEMV pass (0 disables)")
    args = ap.parse_args()
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
    weights = {}
    for si, (N, K) in enumerate(SHAPES):
        n = N * K
        per_copy = n // 2 + 4 * (n // BLOCKSIZE)
        ncopy = max(2, -(-RING_BYTES // per_copy))
        ring = []
        for c in range(ncopy):
            g = torch.Generator(device=dev).manual_seed(2000 + 100 * si + c)
            w = (torch.randn(N, K, generator=g, device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16)
            qw, absmax, _ = ta.quantize_nf4(w, BLOCKSIZE)
            ring.append((qw, absmax))
            del w
        weights[(N, K)] = ring
    xs, outs = {}, {}
    for mi, M in enumerate(MS):
        for si, (N, K) in enumerate(SHAPES):
            g = torch.Generator(device=dev).manual_seed(200000 + 100 * si + mi)
            xs[(M, N, K)] = torch.randn(M, K, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
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

    # the three decode kernels, each timed as a group with HIP events on the launch stream
    groups = [
        ("gemv_rows_kernel", "M = 1, row-streaming", [(M, N, K) for M in MS if M == 1 for (N, K) in SHAPES]),
        ("gemv_quad_kernel", "M = 4, four rows per lane quad", [(M, N, K) for M in MS if 2 <= M <= 4 for (N, K) in SHAPES]),
        ("gemv_tiles_kernel", "M = 16, MFMA tiles", [(M, N, K) for M in MS if M > 4 for (N, K) in SHAPES]),
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
    kernels = []
    for gi, (name, what, calls) in enumerate(groups):
        G = len(groups)
        ms = sum(events[st * G + gi].elapsed_time(events[st * G + gi + 1]) for st in range(args.steps)) / args.steps
        kernels.append({
            "kernel": name, "calls": what, "launches_per_step": len(calls),
            "algorithmic_bytes_per_launch": group_bytes[gi] // len(calls),
            "avg_launch_us": round(ms * 1e3 / len(calls), 3),
            "achieved_GBs": round(group_bytes[gi] / (ms * 1e-3) / 1e9, 1),
            "share_of_step_time": round(ms / ms_per_step, 3),
        })
    dom = max(kernels, key=lambda k: k["share_of_step_time"])

    traffic = None
    tpath = os.path.join(ROOT, "profiles", "gemv_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic = json.load(f).get(dom["kernel"], {}).get("hbm_bytes_per_launch")

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
        "data": "synthetic (seeded bf16 N(0,0.02) weights quantized to NF4 on the GPU, x bf16 N(0,1))",
        "config": {
            "workload": "BASELINE config 2: Llama-3-8B projection shapes [4096,4096],[1024,4096],[14336,4096],"
                        "[4096,14336],[128256,4096] as NF4 linears (blocksize 64, fp32 absmax), M in {1,4,16}; "
                        "15 nf4hip_gemv calls per step, weights rotated through >= 640 MB rings",
            "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
            "algorithmic_bytes_per_step": bytes_step,
            "kernels": kernels,
        },
        "roofline": {
            "kernel": f"{dom['kernel']} ({dom['calls']}: the {dom['launches_per_step']} calls per step that take the most time)",
            "bound": "hbm",
            "achieved": dom["achieved_GBs"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(dom["achieved_GBs"] / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "algorithmic_bytes_per_launch": dom["algorithmic_bytes_per_launch"],
            "avg_launch_us": dom["avg_launch_us"],
        },
    }

    del weights, xs, outs, ws
    torch.cuda.empty_cache()
    if not args.no_prefill:
        result["config"]["prefill"] = prefill_section(torch, ta)
        result["config"]["codec"] = codec_section(torch, ta)
    if args.decode_tokens > 1:
        result["config"]["decode"] = llama_decode(torch, ta, args.decode_tokens)
    if args.cpu_seconds > 0:
        result["cpu_baseline"] = cpu_baseline(torch, args.cpu_seconds)
    print(json.dumps(result))
    return 0


MFMA_BF16_PEAK_TFLOPS = 2516.6  # 256 CUs x 2.4 GHz x 4096 flop/clk/CU


def prefill_section(torch, ta) -> dict:
    """BASELINE config 3, outside the timed region of the GEMV metric: the Llama-3-8B projection
    shapes (and the fused gate/up weight [28672, 4096]) with M in {512, 2048, 8192} rows of x through
    ``matmul_nf4`` -- which routes them to nf4hip_dequantize + the dense library GEMM, or to the fused
    NF4 GEMM kernel (nf4hip_gemm) for the tall weight at M = 512 -- and the fused kernel forced at
    M = 2048 for comparison.  TFLOP/s = 2 M N K / time, HIP events bracket 10 calls (3 for the forced
    fused kernel) after 3 warm-up calls.  ``rows64``: the same weights with 64 rows of x, the router's
    route (the fused kernel, K split over workgroups) next to the dense route forced."""
    dev = torch.device("cuda:0")
    F = ta.functional
    code = ta.nf4_code(dev)

    def timed(fn, reps):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / reps

    rows, mid = [], []
    routes = {"dequant+gemm": "nf4hip_dequantize + dense GEMM", "gemm": "nf4hip_gemm (fused)"}
    for si, (N, K) in enumerate([(4096, 4096), (14336, 4096), (4096, 14336), (28672, 4096)]):
        g = torch.Generator(device=dev).manual_seed(3000 + si)
        w = (torch.randn(N, K, generator=g, device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16)
        qw, absmax, _ = ta.quantize_nf4(w, BLOCKSIZE)
        del w
        for M in (512, 2048, 8192):
            x = torch.randn(M, K, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
            route = routes[F.fused_route(x, None, BLOCKSIZE, torch.bfloat16, (N, K))]
            t = timed(lambda: ta.matmul_nf4(x, qw, None, absmax, code, BLOCKSIZE, torch.bfloat16, (N, K)), 10)
            row = {"N": N, "K": K, "M": M, "route": route, "us": round(t * 1e6, 1),
                   "tflops": round(2.0 * M * N * K / t / 1e12, 1),
                   "frac_of_mfma_peak": round(2.0 * M * N * K / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}
            rows.append(row)
            if M == 2048:
                saved, F.DENSE_ROUTE_MIN_M = F.DENSE_ROUTE_MIN_M, 1 << 30
                try:
                    assert F.fused_route(x, None, BLOCKSIZE, torch.bfloat16, (N, K)) == "gemm"
                    t = timed(lambda: ta.matmul_nf4(x, qw, None, absmax, code, BLOCKSIZE, torch.bfloat16, (N, K)), 3)
                finally:
                    F.DENSE_ROUTE_MIN_M = saved
                rows.append({"N": N, "K": K, "M": M, "route": "nf4hip_gemm (fused, forced)", "us": round(t * 1e6, 1),
                             "tflops": round(2.0 * M * N * K / t / 1e12, 1),
                             "frac_of_mfma_peak": round(2.0 * M * N * K / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)})
        # 64 rows of x (between the decode and the prefill regime): the router's choice, which is the fused
        # kernel with K split over workgroups, next to the dense route (dequantize + library GEMM) forced
        x = torch.randn(64, K, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        route = F.fused_route(x, None, BLOCKSIZE, torch.bfloat16, (N, K))
        t = timed(lambda: ta.matmul_nf4(x, qw, None, absmax, code, BLOCKSIZE, torch.bfloat16, (N, K)), 20)
        td = timed(lambda: torch.nn.functional.linear(x, F.dequantize_nf4(qw, absmax, code, BLOCKSIZE, torch.bfloat16, (N, K))), 20)
        mid.append({"N": N, "K": K, "M": 64, "route": route, "us": round(t * 1e6, 1), "dense_route_us": round(td * 1e6, 1)})
    return {"peak_tflops": MFMA_BF16_PEAK_TFLOPS, "cases": rows, "rows64": mid}


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
            for i in range(ncopy):
                fn(i)
            torch.cuda.synchronize()
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
    cfg = D.LlamaConfig.llama3_8b(fused_projections=True)
    model = D.build_llama(cfg, device=dev, seed=4000)
    jm = ta.jit(model, transforms=[ta.BitsAndBytesLinearQuant4bit()])
    nweights = sum(m.weight.numel() for m in model.modules() if isinstance(m, torch.nn.Linear))
    out = {
        "model": "Llama-3-8B architecture (32 layers, d 4096, 32q/8kv heads, FFN 14336, vocab 128256), random init, "
                 "all 161 linears NF4 (QKV and gate/up fused), prompt 512, greedy, HIP-graph decode step; norms / rotary + attention / SiLU*up between the linears as 3 HIP kernels "
                 "(decode_tok_per_s) or as PyTorch ops (decode_tok_per_s_torch_glue)",
        "new_tokens": n_new,
        "linear_weight_bytes_per_token": int(nweights * 0.5625),
        "hbm_bound_tok_per_s_batch1": round(HBM_PEAK_GBS * 1e9 / (nweights * 0.5625), 1),
    }
    for B in (1, 8, 32):  # 32 is not a BASELINE case: the linears of its step run through nf4hip_gemm (M = 32)
        g = torch.Generator(device=dev).manual_seed(4000 + B)
        prompt = torch.randint(0, cfg.vocab, (B, 512), generator=g, device=dev)
        D.greedy_decode(jm, cfg, prompt, n_new=1, use_graph=False)  # untimed: library start-up, GEMM heuristics
        res = {}
        # the single-token step with the HIP glue kernels (norm, rotary + cache + attention, SiLU * up)
        # around the NF4 linears, and with plain PyTorch ops in their place
        for key, glue in (("", True), ("_torch_glue", False)):
            if B > 8 and not glue:
                continue
            cfg.hip_glue = glue
            _, st = D.greedy_decode(jm, cfg, prompt, n_new=n_new, use_graph=True)
            res[f"decode_tok_per_s{key}"] = round(st["decode_tok_per_s"], 1)
            res[f"ms_per_step{key}"] = round(st["decode_s"] / st["decode_steps"] * 1e3, 3)
            res["prefill_ms"] = round(st["prefill_s"] * 1e3, 1)
        out[f"batch{B}"] = res
    return out


def cpu_baseline(torch, budget_s: float) -> dict:
    """The reference's CPU route (torch-eager NF4 dequantize, then F.linear) on a bounded sample:
    BASELINE config 1, one Linear(4096 -> 4096), x [1, 4096]."""
    from oracle import nf4_oracle as O

    N, K, M = 4096, 4096, 1
    g = torch.Generator().manual_seed(1000)
    w = (torch.randn(N, K, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(100000), dtype=torch.float32).to(torch.bfloat16)
    qw, absmax = O.C().quantize(w, BLOCKSIZE)
    lut = O.nf4_lut()
    threads = torch.get_num_threads()
    O.matmul_4bit_eager(x, qw, None, absmax, lut, BLOCKSIZE, torch.bfloat16, (N, K))  # warm-up
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 200):
        t0 = time.perf_counter()
        O.matmul_4bit_eager(x, qw, None, absmax, lut, BLOCKSIZE, torch.bfloat16, (N, K))
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": round(algorithmic_bytes(M, N, K) / med / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{len(times)} calls of torch-eager dequantize_4bit + F.linear, NF4 Linear(4096->4096), x [1,4096] bf16 "
                  f"(BASELINE config 1); median {med * 1e3:.1f} ms per call, {os.cpu_count()} host cpus visible",
    }


if __name__ == "__main__":
    sys.exit(main())
