#!/usr/bin/env python3
"""Benchmark of the quantized-GEMM hot path on one MI355X.

A step is one ``mxfp8_scaled_mm`` of M=N=K=8192 (BASELINE config 2, the shape the metric is quoted
on): e4m3 operands with e8m0 per-32 scales in the 128x4 layout, bf16 output, inputs resident in HBM.
``value`` is its throughput in TFLOP/s (2*M*N*K per step).  The same JSON line carries
  roofline      the MXFP8 GEMM kernel against the dense fp8 MFMA peak (5.0 PFLOP/s),
  cpu_baseline  the PyTorch-CPU dequantize + fp32 matmul reference on a bounded sample,
  extra         the other workloads of the metric: NVFP4 block quantize GB/s at the config-5
                activation size (with its own HBM roofline), NVFP4 GEMM 8192^3, the dense-LLM
                shapes of config 3, and the grouped GEMMs of configs 4 and 5.
Synthetic data: seeded N(0,1) / N(0,0.02) bf16 tensors quantized by the library's own quantizers.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0   # MI355X dense fp8 MFMA
PEAK_FP4_TFLOPS = 10100.0  # dense fp6 / fp4 MFMA
PEAK_F16_TFLOPS = 2500.0   # dense bf16 / fp16 MFMA
PEAK_HBM_GBS = 8000.0      # HBM3E


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--preheat-ms", type=float, default=300.0,
                    help="before the warm-up steps of every measurement the same call is repeated for this long: the "
                         "clocks of an idle GPU take some 100 ms of load to settle (0.43 ms per step right after idle, "
                         "0.37 ms from then on)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg (profiling runs)")
    ap.add_argument("--no-extra", action="store_true", help="only the headline MXFP8 workload")
    ap.add_argument("--calib", action="store_true", help="profiling aid: also run a plain 1 GiB device copy a few times, "
                    "so that a counter run shows what FETCH_SIZE / WRITE_SIZE read for a kernel of known traffic")
    ap.add_argument("--no-graph", action="store_true", help="profiling aid: skip the HIP-graph timings of the decode-sized GEMMs "
                    "(counter runs attribute a replayed graph's kernels poorly)")
    ap.add_argument("--only", default="", help="profiling aid: run just this extra workload "
                    "(quant | fused | nvfp4 | llm | grouped | gnvfp4) and print its line")
    ap.add_argument("--shapes", default="", help="profiling aid: time dense GEMMs of these shapes only and print their "
                    "launches, e.g. mxfp8:128x14336x4096,nvfp4:160x28672x14336 (bf16 result, N(0,1) activations)")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; every kernel of the path is single-device "
              "(run with --gpus 1).", file=sys.stderr)
        sys.exit(2)

    import torch

    from fuser_amd import capi, nvf_cutlass, ops

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    torch.cuda.set_device(0)
    one = torch.tensor(1.0, device=dev)

    def timed(fn, steps, warmup):
        """Average milliseconds per call: HIP events on the launch stream around `steps` calls."""
        t_end = time.perf_counter() + args.preheat_ms * 1e-3
        while time.perf_counter() < t_end:  # steady clocks first; untimed, like the warm-up steps
            for _ in range(8):
                fn()
            torch.cuda.synchronize()
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / steps
        return e0.elapsed_time(e1) / steps, wall

    if args.shapes:
        res = {}
        gen = torch.Generator(device=dev).manual_seed(0)
        for spec in args.shapes.split(","):
            op, dims = spec.split(":")
            m, n, k = (int(v) for v in dims.split("x"))
            x = torch.randn(m, k, device=dev, generator=gen).bfloat16()
            w = (torch.randn(n, k, device=dev, generator=gen) * 0.02).bfloat16()
            if op == "mxfp8":
                (qx, sx), (qw, sw) = (ops.nv_block_quantize(t, None, True, 32, torch.float8_e4m3fn) for t in (x, w))
                fn, name = (lambda: nvf_cutlass.mxfp8_scaled_mm(qx, qw, sx, sw, one, torch.bfloat16)), "mxfp8_scaled_mm"
            else:
                (qx, sx), (qw, sw) = (ops.nv_block_quantize(t, None, True, 16) for t in (x, w))
                fn, name = (lambda: nvf_cutlass.nvfp4_scaled_mm(qx, qw, sx, sw, one, torch.bfloat16)), "nvfp4_scaled_mm"
            ms, _ = timed(fn, args.steps, args.warmup)
            res[spec] = {"us": round(ms * 1e3, 2), "TFLOP/s": round(2.0 * m * n * k / ms / 1e9, 1),
                         "launches": capi.describe_dispatch(name, m, n, k)}
        print(json.dumps({"shapes": res}))
        return

    def timed_graph(calls, replays=20):
        if args.no_graph:
            return float("nan")
        return _timed_graph(calls, replays)

    def _timed_graph(calls, replays):
        """Average milliseconds per call of the list `calls`, captured once as a HIP graph (one node sequence per call) and
        replayed: the launches cost no host time, so a call of a few microseconds is timed by what the GPU does."""
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            for fn in calls[:2]:
                fn()  # one-time set-up of the kernels outside the capture
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for fn in calls:
                    fn()
            t_end = time.perf_counter() + min(args.preheat_ms, 100.0) * 1e-3
            while time.perf_counter() < t_end:
                graph.replay()
                torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(replays):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (replays * len(calls))

    def ru(x, y):
        return (x + y - 1) // y * y

    def moe_top2(tokens, experts, seed):
        gen = torch.Generator().manual_seed(seed)
        logits = torch.randn(tokens, experts, generator=gen) + torch.linspace(-1.5, 1.5, experts)
        return torch.bincount(logits.topk(2, dim=1).indices.flatten(), minlength=experts)

    def moe_zipf(tokens, topk, experts, s, seed):
        gen = torch.Generator().manual_seed(seed)
        p = 1.0 / torch.arange(1, experts + 1).float() ** s
        p = p[torch.randperm(experts, generator=gen)]
        idx = torch.multinomial(p.expand(tokens, experts), topk, replacement=False, generator=gen).flatten()
        return torch.bincount(idx, minlength=experts)

    extra = {}
    gen = torch.Generator(device=dev).manual_seed(0)

    # CPU baselines ("port": the oracle's recipes, i.e. its scalar C restatement for the quantizer and torch-CPU
    # dequantize + fp32 matmul for the GEMMs), timed on this box's host cores on a bounded sample of each workload.
    cpu_threads = os.cpu_count() or 1
    if not args.no_cpu:
        torch.set_num_threads(cpu_threads)
        from oracle import nvf_oracle as O

    def cpu_timed(fn, budget_s=6.0, max_runs=3):
        """Median seconds of up to max_runs runs of fn (stops early once budget_s is spent)."""
        runs, spent = [], 0.0
        while len(runs) < max_runs and (not runs or spent < budget_s):
            t0 = time.perf_counter()
            fn()
            runs.append(time.perf_counter() - t0)
            spent += runs[-1]
        runs.sort()
        return runs[len(runs) // 2], len(runs)
    measured_traffic = {}
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        measured_traffic = json.load(open(tpath))

    # ------------------------------------------------------------------ extras
    def run_quant():
        m, k = 65536, 7168
        x = torch.randn(m, k, device=dev, generator=gen).bfloat16()
        gs = (2688.0 / x.float().abs().max()).float()
        ms, _ = timed(lambda: ops.nv_block_quantize(x, gs, True, 16), 30, 5)
        gbs = m * k * 2.5625 / ms / 1e6
        extra["nvfp4_quantize"] = {"workload": "bf16 [65536,7168] -> NVFP4, 128x4 swizzled scales (config 5 activations)",
                                   "ms": round(ms, 4), "GB/s": round(gbs, 1),
                                   "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                                "frac": round(gbs / PEAK_HBM_GBS, 4),
                                                "traffic": measured_traffic.get("nvfp4_quantize_65536x7168_bytes_per_launch"),
                                                "kernel": "nvfp4_quantize_kernel",
                                                "bytes_per_launch": m * k * 2.5625}}
        if not args.no_cpu:
            rows = 4096
            hx, hgs = x[:rows].cpu(), float(gs)
            sec, n_runs = cpu_timed(lambda: O.block_quantize_nvfp4(hx, hgs, True))
            extra["nvfp4_quantize"]["cpu_baseline"] = {
                "value": round(rows * k * 2.5625 / sec / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"the first {rows} of the 65536 rows, median of {n_runs} runs of the oracle's scalar C quantizer"}
        sizes = moe_zipf(8192, 8, 256, 1.1, 0).int()
        padded = (sizes + 127) // 128 * 128
        eo = (torch.cumsum(sizes, 0) - sizes).int().to(dev)
        so = (torch.cumsum(padded, 0) - padded).int().to(dev)
        ms, _ = timed(lambda: ops.nv_grouped_block_quantize(x, eo, so, None, 16), 30, 5)
        extra["nvfp4_grouped_quantize"] = {"workload": "same tensor, 256 Zipf(1.1) groups", "ms": round(ms, 4),
                                           "GB/s": round(m * k * 2.5625 / ms / 1e6, 1)}
        for (mm, kk) in ((256, 1024), (2048, 4096)):
            xs = torch.randn(mm, kk, device=dev, generator=gen).bfloat16()
            ms, _ = timed(lambda: ops.nv_block_quantize(xs, gs, True, 16), 50, 5)
            extra[f"nvfp4_quantize_{mm}x{kk}"] = {"us": round(ms * 1e3, 2), "GB/s": round(mm * kk * 2.5625 / ms / 1e6, 1)}

    def run_fused():
        # the steps either side of the quantizer in the NVFP4 MoE layer at config 5's intermediate size
        m, k = 65536, 2048
        gate = torch.randn(m, k, device=dev, generator=gen).bfloat16()
        up = torch.randn(m, k, device=dev, generator=gen).bfloat16()
        sizes = moe_zipf(8192, 8, 256, 1.1, 0).int()
        padded = (sizes + 127) // 128 * 128
        eo = (torch.cumsum(sizes, 0) - sizes).int().to(dev)
        so = (torch.cumsum(padded, 0) - padded).int().to(dev)
        ms_f, _ = timed(lambda: ops.silu_mul_nv_grouped_block_quantize(gate, up, eo, so, None), 30, 5)
        ms_c, _ = timed(lambda: ops.nv_grouped_block_quantize(torch.nn.functional.silu(gate) * up, eo, so, None, 16), 30, 5)
        extra["silu_mul_grouped_quantize"] = {
            "workload": "silu(gate) * up -> NVFP4, gate/up bf16 [65536,2048], 256 Zipf(1.1) groups",
            "fused_ms": round(ms_f, 4), "fused_GB/s": round(m * k * 4.5625 / ms_f / 1e6, 1),
            "unfused_chain_ms": round(ms_c, 4), "note": "fused bytes/element: 4 read + 0.5625 written; the chain moves 12.56"}
        x = torch.randn(65536, 7168, device=dev, generator=gen).bfloat16()
        ms_g, _ = timed(lambda: ops.compute_nvfp4_global_scale(x), 30, 5)
        ms_t, _ = timed(lambda: (2688.0 / x.abs().max().float()), 10, 2)
        extra["nvfp4_global_scale"] = {"workload": "bf16 [65536,7168] -> fp32 scalar on the device",
                                       "ms": round(ms_g, 4), "GB/s": round(x.numel() * 2 / ms_g / 1e6, 1),
                                       "torch_abs_max_ms": round(ms_t, 4)}

    def quantized_nvfp4(rows, k, std):
        x = (torch.randn(rows, k, device=dev, generator=gen) * std).bfloat16()
        gs = (2688.0 / x.float().abs().max()).float()
        q, s = ops.nv_block_quantize(x, gs, True, 16)
        return q, s, gs

    def run_nvfp4():
        m = n = k = 8192
        a, sa, ga = quantized_nvfp4(m, k, 1.0)
        b, sb, gb = quantized_nvfp4(n, k, 1.0)
        alpha = (1.0 / (ga * gb)).float()
        ms, _ = timed(lambda: nvf_cutlass.nvfp4_scaled_mm(a, b, sa, sb, alpha, torch.bfloat16), 20, 3)
        tf = 2.0 * m * n * k / ms / 1e9
        extra["nvfp4_gemm_8192"] = {"ms": round(ms, 4), "TFLOP/s": round(tf, 1),
                                    "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
                                                 "frac": round(tf / PEAK_F16_TFLOPS, 4),
                                                 "frac_of_fp8_peak": round(tf / PEAK_FP8_TFLOPS, 4),
                                                 "frac_of_fp4_peak": round(tf / PEAK_FP4_TFLOPS, 4),
                                                 "traffic": measured_traffic.get("nvfp4_gemm_8192_bytes_per_launch"),
                                                 "kernel": "nvfp4_gemm_256_kernel",
                                                 "note": "priced against the fp16 MFMA peak, the instruction issued (e2m1 x e4m3 is "
                                                         "dequantised exactly to fp16: the block-16 e4m3 scale has no scaled-MFMA form); "
                                                         "the fractions of the fp8 and fp4 peaks are what the same rate is worth there"}}
        if not args.no_cpu:
            ha, hsa, hb, hsb = (t.view(torch.uint8).cpu() for t in (a, sa, b, sb))
            al = float(alpha)
            sec, n_runs = cpu_timed(lambda: O.ref_nvfp4_scaled_mm(ha, hb, hsa, hsb, al), budget_s=4.0)
            extra["nvfp4_gemm_8192"]["cpu_baseline"] = {
                "value": round(2.0 * m * n * k / sec / 1e12, 4), "unit": "TFLOP/s", "cores": cpu_threads, "kind": "port",
                "sample": f"the whole 8192^3 workload, median of {n_runs} runs: torch-CPU dequantize + fp32 matmul"}
            del ha, hsa, hb, hsb
        # a prefill of a token count that is no multiple of 128: rows up to the cut on the persistent kernel, the rest streamed
        mr = 8100
        ar, sar = a[:mr].contiguous(), sa[: 8192].contiguous()
        ms_r, _ = timed(lambda: nvf_cutlass.nvfp4_scaled_mm(ar, b, sar, sb, alpha, torch.bfloat16), 20, 3)
        extra["nvfp4_gemm_8100x8192x8192"] = {"ms": round(ms_r, 4), "TFLOP/s": round(2.0 * mr * n * k / ms_r / 1e9, 1),
                                              "launches": capi.describe_dispatch("nvfp4_scaled_mm", mr, n, k)}
        gn = torch.ones((), device=dev)
        ms_b, _ = timed(lambda: nvf_cutlass.nvfp4_scaled_mm_blockscale(a, b, sa, sb, alpha, gn), 20, 3)
        extra["nvfp4_gemm_blockscale_8192"] = {"ms": round(ms_b, 4), "TFLOP/s": round(2.0 * m * n * k / ms_b / 1e9, 1),
                                               "vs_plain_gemm": round(ms_b / ms, 4),
                                               "note": "one launch: the product is re-quantized to NVFP4 in the GEMM's epilogue"}

    def run_llm():
        # BASELINE config 3.  The decode-sized shapes (M = 16, 128) are bound by streaming the weights once, and one
        # weight tensor of 9-33 MB lives in the 256 MB last-level cache: they are therefore timed three ways - eager calls
        # on one weight tensor (`gemm_us`, as a Python serving loop would issue them: the host's launch cost is in it),
        # the same calls replayed from a HIP graph (`gemm_us_graph_warm`), and a graph that rotates over enough weight
        # tensors to exceed the cache (`gemm_us_graph_rotated`: every call streams its weights from HBM).  The roofline
        # fractions are those of the rotated figure.
        res = {}
        for (n, k) in ((4096, 4096), (14336, 4096), (4096, 14336)):
            copies = int(320e6 // (n * k * 0.5625)) + 1
            ws = [quantized_nvfp4(n, k, 0.02) for _ in range(copies)]
            w, sw, gw = ws[0]
            for m in (16, 128, 2048):
                x = torch.randn(m, k, device=dev, generator=gen).bfloat16()
                gx = (2688.0 / x.float().abs().max()).float()
                alpha = (1.0 / (gx * gw)).float()
                qx, sx = ops.nv_block_quantize(x, gx, True, 16)
                ms_q, _ = timed(lambda: ops.nv_block_quantize(x, gx, True, 16), 50, 5)
                ms_g, _ = timed(lambda: nvf_cutlass.nvfp4_scaled_mm(qx, w, sx, sw, alpha, torch.bfloat16), 50, 5)

                def seq(wi=w, swi=sw):
                    q, s = ops.nv_block_quantize(x, gx, True, 16)
                    return nvf_cutlass.nvfp4_scaled_mm(q, wi, s, swi, alpha, torch.bfloat16)

                ms_s, _ = timed(seq, 50, 5)
                reps = copies if m < 2048 else 4
                ms_gw = timed_graph([lambda: nvf_cutlass.nvfp4_scaled_mm(qx, w, sx, sw, alpha, torch.bfloat16)] * reps)
                ms_gr = timed_graph([(lambda wi=wi, swi=swi: nvf_cutlass.nvfp4_scaled_mm(qx, wi, sx, swi, alpha, torch.bfloat16))
                                     for (wi, swi, _) in ws[:reps]])
                ms_sr = timed_graph([(lambda wi=wi, swi=swi: seq(wi, swi)) for (wi, swi, _) in ws[:reps]])
                byts = n * k * 0.5625 + m * k * 0.5625 + 2 * m * n
                res[f"M{m}_N{n}_K{k}"] = {"quant_us": round(ms_q * 1e3, 2), "gemm_us": round(ms_g * 1e3, 2), "seq_us": round(ms_s * 1e3, 2),
                                          "gemm_us_graph_warm": round(ms_gw * 1e3, 2), "gemm_us_graph_rotated": round(ms_gr * 1e3, 2),
                                          "seq_us_graph_rotated": round(ms_sr * 1e3, 2), "weight_tensors_in_rotation": reps,
                                          "gemm_TFLOP/s": round(2.0 * m * n * k / ms_gr / 1e9, 1), "gemm_GB/s": round(byts / ms_gr / 1e6, 1),
                                          "frac_of_f16_peak": round(2.0 * m * n * k / ms_gr / 1e9 / PEAK_F16_TFLOPS, 4),
                                          "frac_of_hbm_peak": round(byts / ms_gr / 1e6 / PEAK_HBM_GBS, 4)}
                if not args.no_cpu:
                    hq, hs, hw, hsw = (t.view(torch.uint8).cpu() for t in (qx, sx, w, sw))
                    al = float(alpha)
                    sec, _ = cpu_timed(lambda: O.ref_nvfp4_scaled_mm(hq, hw, hs, hsw, al), max_runs=1)
                    res[f"M{m}_N{n}_K{k}"]["cpu_us"] = round(sec * 1e6, 0)
            del ws
        res["timing"] = ("gemm_us / quant_us / seq_us: eager calls on one weight tensor, HIP events (host launch cost included); "
                         "*_graph_warm: the same call replayed from a HIP graph; *_graph_rotated: a graph over enough weight tensors "
                         "to exceed the 256 MB last-level cache (> 320 MB), so that the weights stream from HBM; TFLOP/s, GB/s and "
                         "the fractions are those of gemm_us_graph_rotated")
        if not args.no_cpu:
            res["cpu_baseline"] = {"unit": "us per call (cpu_us of every shape)", "cores": cpu_threads, "kind": "port",
                                   "sample": "each of the nine shapes once, whole: torch-CPU dequantize of both operands + fp32 matmul"}
        extra["nvfp4_gemm_llm_shapes"] = res
        # the same shapes through mxfp8_scaled_mm (not a BASELINE config: the decode / prefill use of the headline op)
        one = torch.ones((), device=dev)
        res8 = {}
        for (n, k) in ((4096, 4096), (14336, 4096), (4096, 14336)):
            w8, sw8 = ops.nv_block_quantize((torch.randn(n, k, device=dev, generator=gen) * 0.02).bfloat16(), None, True, 32,
                                            torch.float8_e4m3fn)
            for m in (16, 128, 2048):
                x8, sx8 = ops.nv_block_quantize(torch.randn(m, k, device=dev, generator=gen).bfloat16(), None, True, 32,
                                                torch.float8_e4m3fn)
                ms_g, _ = timed(lambda: nvf_cutlass.mxfp8_scaled_mm(x8, w8, sx8, sw8, one, torch.bfloat16), 50, 5)
                byts = n * k * 1.03125 + m * k * 1.03125 + 2 * m * n
                res8[f"M{m}_N{n}_K{k}"] = {"gemm_us": round(ms_g * 1e3, 2), "gemm_TFLOP/s": round(2.0 * m * n * k / ms_g / 1e9, 1),
                                           "gemm_GB/s": round(byts / ms_g / 1e6, 1)}
        extra["mxfp8_gemm_llm_shapes"] = res8

    def run_grouped():
        g, k, n = 8, 4096, 14336
        sizes = moe_top2(4096, g, 0).int()
        rows = int(sizes.sum())
        a = torch.randn(rows, k, device=dev, generator=gen).bfloat16()
        b = (torch.randn(g, n, k, device=dev, generator=gen) * 0.02).bfloat16()
        ps = torch.stack([sizes, torch.full_like(sizes, n), torch.full_like(sizes, k)], 1).int().to(dev)
        eo = (torch.cumsum(sizes, 0) - sizes).int().to(dev)
        st = torch.full((g,), k, dtype=torch.int64, device=dev)
        ct = torch.full((g,), n, dtype=torch.int64, device=dev)
        ms, _ = timed(lambda: nvf_cutlass.grouped_mm(a, b, st, ct, ps, eo), 15, 3)
        tf = 2.0 * rows * n * k / ms / 1e9
        # the vendor library's plain GEMM, one launch per expert on the same slices (a comparison figure)
        offs = eo.tolist()
        slices = [(a[o : o + int(t)], b[e].t()) for e, (o, t) in enumerate(zip(offs, sizes.tolist())) if t]
        ms_v, _ = timed(lambda: [torch.matmul(x, w) for x, w in slices], 15, 3)
        extra["grouped_mm_bf16"] = {"workload": f"config 4: 8 experts, sizes {sizes.tolist()}, K=4096, N=14336", "ms": round(ms, 4),
                                    "TFLOP/s": round(tf, 1), "frac_of_bf16_peak": round(tf / PEAK_F16_TFLOPS, 4),
                                    "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
                                                 "frac": round(tf / PEAK_F16_TFLOPS, 4),
                                                 "traffic": measured_traffic.get("grouped_mm_config4_bytes_per_launch"),
                                                 "kernel": "grouped16_gemm_256_kernel"},
                                    "hipblaslt_one_matmul_per_expert_ms": round(ms_v, 4)}
        if not args.no_cpu:
            ha, hb = a.cpu(), b.cpu()
            hps, heo = ps.cpu(), eo.cpu()
            sec, n_runs = cpu_timed(lambda: O.ref_grouped_mm(ha, hb, hps, heo), budget_s=3.0)
            extra["grouped_mm_bf16"]["cpu_baseline"] = {
                "value": round(2.0 * rows * n * k / sec / 1e12, 4), "unit": "TFLOP/s", "cores": cpu_threads, "kind": "port",
                "sample": f"the whole config-4 workload, median of {n_runs} runs: torch-CPU fp32 matmul per expert"}
            del ha, hb

    def run_gnvfp4():
        g, rows = 256, 65536
        sizes = moe_zipf(8192, 8, g, 1.1, 0).int()
        padded = (sizes + 127) // 128 * 128
        eo = (torch.cumsum(sizes, 0) - sizes).int().to(dev)
        so = (torch.cumsum(padded, 0) - padded).int().to(dev)
        res = {"group_sizes_min_median_max": [int(sizes.min()), int(sizes.median()), int(sizes.max())]}
        for (k, n) in ((7168, 2048), (2048, 7168)):
            x = torch.randn(rows, k, device=dev, generator=gen).bfloat16()
            aq, asf = ops.nv_grouped_block_quantize(x, eo, so, None, 16)
            bq = torch.empty(g, n, k // 2, dtype=torch.uint8, device=dev)
            bsf = torch.empty(g, n, k // 16, dtype=torch.uint8, device=dev)
            alphas = torch.empty(g, device=dev)
            for e in range(g):
                w = (torch.randn(n, k, device=dev, generator=gen) * 0.02).bfloat16()
                gs = (2688.0 / w.float().abs().max()).float()
                q, s = ops.nv_block_quantize(w, gs, True, 16)
                bq[e], bsf[e], alphas[e] = q.view(torch.uint8), s.view(torch.uint8), 1.0 / gs
            bq4, bsf8 = bq.view(torch.float4_e2m1fn_x2), bsf.view(torch.float8_e4m3fn)
            ps = torch.stack([sizes, torch.full_like(sizes, n), torch.full_like(sizes, k)], 1).int().to(dev)
            st = torch.full((g,), k, dtype=torch.int64, device=dev)
            ct = torch.full((g,), n, dtype=torch.int64, device=dev)
            ms, _ = timed(lambda: nvf_cutlass.nvfp4_scaled_grouped_mm(aq, bq4, asf, bsf8, alphas, st, ct, ps, eo, so, torch.bfloat16), 10, 2)
            tf = 2.0 * rows * n * k / ms / 1e9
            res[f"K{k}_N{n}"] = {"ms": round(ms, 4), "useful_TFLOP/s": round(tf, 1), "frac_of_f16_peak": round(tf / PEAK_F16_TFLOPS, 4),
                                 "frac_of_fp8_peak": round(tf / PEAK_FP8_TFLOPS, 4), "frac_of_fp4_peak": round(tf / PEAK_FP4_TFLOPS, 4),
                                 "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
                                              "frac": round(tf / PEAK_F16_TFLOPS, 4),
                                              "traffic": measured_traffic.get(f"nvfp4_grouped_mm_config5_K{k}_N{n}_bytes_per_call"),
                                              "kernel": "nvfp4_gemm_256_kernel (+ nvfp4_group_panel_kernel, nvfp4_skinny_ring_kernel: the call's launches)",
                                              "algorithmic_bytes": int(g * n * k * 0.5625 + rows * k * 0.5625 + 2 * rows * n)}}
            if not args.no_cpu:
                ne = 16  # the first 16 experts and their rows
                r_end, s_end = int(eo[ne]), int(so[ne])
                h = [t.view(torch.uint8).cpu() for t in (aq[:r_end], bq[:ne], asf[:s_end], bsf[:ne])]
                hal, hps, heo, hso = alphas[:ne].cpu(), ps[:ne].cpu(), eo[:ne].cpu(), so[:ne].cpu()
                sec, _ = cpu_timed(lambda: O.ref_nvfp4_scaled_grouped_mm(h[0], h[1], h[2], h[3], hal, hps, heo, hso), max_runs=1)
                res[f"K{k}_N{n}"]["cpu_baseline"] = {
                    "value": round(2.0 * r_end * n * k / sec / 1e12, 4), "unit": "TFLOP/s", "cores": cpu_threads, "kind": "port",
                    "sample": f"the first {ne} of the 256 experts ({r_end} of the 65536 rows), once: torch-CPU dequantize + fp32 matmul per expert"}
                del h
            # the same experts at decode size: 64 tokens x top-8 = 512 rows spread uniformly (bound by streaming the
            # weights of the active experts once)
            d_sizes = torch.bincount(torch.randint(0, g, (512,), generator=torch.Generator().manual_seed(0)), minlength=g).int()
            d_pad = (d_sizes + 127) // 128 * 128
            d_eo = (torch.cumsum(d_sizes, 0) - d_sizes).int().to(dev)
            d_so = (torch.cumsum(d_pad, 0) - d_pad).int().to(dev)
            d_q, d_sf = ops.nv_grouped_block_quantize(x[:512].contiguous(), d_eo, d_so, None, 16)
            d_ps = torch.stack([d_sizes, torch.full_like(d_sizes, n), torch.full_like(d_sizes, k)], 1).int().to(dev)
            ms_d, _ = timed(lambda: nvf_cutlass.nvfp4_scaled_grouped_mm(d_q, bq4, d_sf, bsf8, alphas, st, ct, d_ps, d_eo, d_so,
                                                                        torch.bfloat16), 10, 2)
            wbytes = int((d_sizes > 0).sum()) * n * k * 0.5625
            res[f"decode_512rows_K{k}_N{n}"] = {"us": round(ms_d * 1e3, 1), "active_experts": int((d_sizes > 0).sum()),
                                                "weight_GB/s": round(wbytes / ms_d / 1e6, 1)}
            # and with the prefill's skew of the routing (64 tokens x top-8 over Zipf(1.1) loads: a few experts get 33
            # rows or more)
            z_sizes = moe_zipf(64, 8, g, 1.1, 0).int()
            z_pad = (z_sizes + 127) // 128 * 128
            z_eo = (torch.cumsum(z_sizes, 0) - z_sizes).int().to(dev)
            z_so = (torch.cumsum(z_pad, 0) - z_pad).int().to(dev)
            z_q, z_sf = ops.nv_grouped_block_quantize(x[:512].contiguous(), z_eo, z_so, None, 16)
            z_ps = torch.stack([z_sizes, torch.full_like(z_sizes, n), torch.full_like(z_sizes, k)], 1).int().to(dev)
            ms_z, _ = timed(lambda: nvf_cutlass.nvfp4_scaled_grouped_mm(z_q, bq4, z_sf, bsf8, alphas, st, ct, z_ps, z_eo, z_so,
                                                                        torch.bfloat16), 10, 2)
            zbytes = int((z_sizes > 0).sum()) * n * k * 0.5625
            res[f"decode_512rows_zipf_K{k}_N{n}"] = {"us": round(ms_z * 1e3, 1), "active_experts": int((z_sizes > 0).sum()),
                                                     "largest_group": int(z_sizes.max()), "weight_GB/s": round(zbytes / ms_z / 1e6, 1)}
            del bq, bsf, bq4, bsf8, x, aq, asf
        extra["nvfp4_grouped_mm"] = res

    if args.calib:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 256)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    runners = {"quant": run_quant, "fused": run_fused, "nvfp4": run_nvfp4, "llm": run_llm, "grouped": run_grouped,
               "gnvfp4": run_gnvfp4}
    if args.only:
        runners[args.only]()
        print(json.dumps({"only": args.only, "extra": extra}))
        return

    # ------------------------------------------------------------------ headline: MXFP8 8192^3
    m = n = k = 8192
    a = torch.randn(m, k, device=dev, generator=gen).bfloat16()
    b = torch.randn(n, k, device=dev, generator=gen).bfloat16()
    qa, sa = ops.nv_block_quantize(a, None, True, 32, torch.float8_e4m3fn)
    qb, sb = ops.nv_block_quantize(b, None, True, 32, torch.float8_e4m3fn)
    del a, b
    flops = 2.0 * m * n * k
    # cold figure: a few calls right after idle, no warm-up (the clock governor's ramp is part of it; the library's
    # one-time set-up of the kernel is not: one call goes first)
    nvf_cutlass.mxfp8_scaled_mm(qa, qb, sa, sb, one, torch.bfloat16)
    torch.cuda.synchronize()
    time.sleep(1.0)
    c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    c0.record()
    for _ in range(5):
        nvf_cutlass.mxfp8_scaled_mm(qa, qb, sa, sb, one, torch.bfloat16)
    c1.record()
    torch.cuda.synchronize()
    cold_ms = c0.elapsed_time(c1) / 5
    ms, wall_ms = timed(lambda: nvf_cutlass.mxfp8_scaled_mm(qa, qb, sa, sb, one, torch.bfloat16), args.steps, args.warmup)
    tflops = flops / ms / 1e9

    traffic = measured_traffic.get("mxfp8_gemm_8192_bytes_per_launch")

    # ------------------------------------------------------------------ CPU baseline (bounded sample)
    cpu = None
    if not args.no_cpu:
        threads = cpu_threads
        ha, hsa = qa.view(torch.uint8).cpu(), sa.view(torch.uint8).cpu()
        hb, hsb = qb.view(torch.uint8).cpu(), sb.view(torch.uint8).cpu()
        runs = []
        for _ in range(5):
            t0 = time.perf_counter()
            da = O.dequantize_mxfp8_fast(ha, hsa)
            db = O.dequantize_mxfp8_fast(hb, hsb)
            t1 = time.perf_counter()
            ref = torch.matmul(da, db.t())
            t2 = time.perf_counter()
            runs.append((t2 - t0, t1 - t0, t2 - t1))
            if sum(r[0] for r in runs) > 25.0:
                break
        runs.sort()
        tot, tdq, tmm = runs[len(runs) // 2]
        got = nvf_cutlass.mxfp8_scaled_mm(qa, qb, sa, sb, one, torch.bfloat16)
        rows = torch.arange(0, m, 61)
        err = ((got[rows.to(dev)].float().cpu() - ref[rows]).abs().max() / ref[rows].abs().max()).item()
        cpu = {"value": round(flops / tot / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
               "sample": f"the whole 8192^3 workload, median of {len(runs)} runs: torch-CPU dequantize ({tdq:.2f} s) + fp32 matmul "
                         f"({tmm:.2f} s)",
               "gpu_vs_cpu_max_abs_err_over_max_abs_ref": round(err, 6)}
        del da, db, ref, got

    # ------------------------------------------------------------------ the vendor library on the same payloads
    # hipBLASLt through torch._scaled_mm: its MXFP8 kernel (unit e8m0 scales in its own layout: timing only) and its
    # plain fp8 kernel with one scale per tensor.  A comparison figure for what the chip sustains on this data.
    if not args.no_extra:
        vendor = {}
        try:
            bt = qb.t()
            u8 = torch.full((m, k // 32), 127, dtype=torch.uint8, device=dev).view(torch.float8_e8m0fnu)
            v_ms, _ = timed(lambda: torch._scaled_mm(qa, bt, u8, u8, out_dtype=torch.bfloat16), args.steps, args.warmup)
            vendor["hipblaslt_mxfp8_TFLOP/s"] = round(flops / v_ms / 1e9, 1)
        except Exception as exc:  # not every build of the library has the block-scaled kernel
            vendor["hipblaslt_mxfp8_TFLOP/s"] = None
            vendor["hipblaslt_mxfp8_error"] = str(exc)[:120]
        try:
            v_ms, _ = timed(lambda: torch._scaled_mm(qa, qb.t(), one, one, out_dtype=torch.bfloat16), args.steps, args.warmup)
            vendor["hipblaslt_fp8_per_tensor_scale_TFLOP/s"] = round(flops / v_ms / 1e9, 1)
        except Exception as exc:
            vendor["hipblaslt_fp8_per_tensor_scale_TFLOP/s"] = None
            vendor["hipblaslt_fp8_error"] = str(exc)[:120]
        extra["vendor_library_8192"] = vendor
        # a prefill of a token count that is no multiple of 128: one launch of 256x256 tiles, the last row tile with 164 rows
        mr = 8100
        qar = qa[:mr].contiguous()
        r_ms, _ = timed(lambda: nvf_cutlass.mxfp8_scaled_mm(qar, qb, sa, sb, one, torch.bfloat16), args.steps, args.warmup)
        extra["mxfp8_gemm_8100x8192x8192"] = {"ms": round(r_ms, 4), "TFLOP/s": round(2.0 * mr * n * k / r_ms / 1e9, 1),
                                              "launches": capi.describe_dispatch("mxfp8_scaled_mm", mr, n, k)}

    if not args.no_extra:
        for name in ("quant", "fused", "nvfp4", "llm", "grouped", "gnvfp4"):
            runners[name]()

    line = {
        "metric": "mxfp8_scaled_mm TFLOP/s, M=N=K=8192, bf16 out (+ NVFP4 quantize GB/s and NVFP4 GEMM TFLOP/s in extra)",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "preheat_ms": args.preheat_ms,
        "untimed_before_the_timed_region": f"{args.preheat_ms:.0f} ms of the same call back to back (clock settling), then the {args.warmup} warm-up steps",
        "cold": {"ms_per_step": round(cold_ms, 5), "TFLOP/s": round(flops / cold_ms / 1e9, 1), "frac": round(flops / cold_ms / 1e9 / PEAK_FP8_TFLOPS, 4),
                 "what": "5 calls right after 1 s of idle, no warm-up"},
        "ms_per_step": round(ms, 5),
        "wall_ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3 x fp8_e4m3 -> f32 accumulate -> bf16",
        "data": "synthetic: seeded N(0,1) bf16 quantized to MXFP8 on the GPU",
        "config": {"workload": "BASELINE config 2: MXFP8 scaled GEMM M=N=K=8192, e8m0 per-32 scales in 128x4 layout, A row-major, B K-major"},
        "roofline": {"bound": "mfma", "achieved": round(tflops, 2), "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_FP8_TFLOPS, 4), "traffic": traffic,
                     "kernel": "mxfp8_gemm_256_kernel", "flops_per_launch": flops},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
