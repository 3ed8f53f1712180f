#!/usr/bin/env python3
"""Benchmark of the 4-bit GPTQ hot path on one MI355X.

Workload (config.workload): one batch-1 decode token through the quantised linears of a
LLaMA-7B-shape decoder - 32 layers x [fused QKV + rotary (4096 -> 12288), o_proj
(4096 -> 4096), fused gate/up + SiLU*mul (4096 -> 2 x 11008), down_proj (11008 -> 4096)],
4-bit, groupsize 128, every layer with its own synthetic weights (3.2 GB, so each
launch streams its weights from HBM, not from the 256 MB Infinity Cache).  The 128
launches of a step are captured once in a HIP graph and replayed; a "step" is one
replay.  value = tokens/s = 1 / step time.  The attention core, norms and lm_head are
not part of this path and are not in the step.

Also reported on the same line:
  roofline      the dominant kernel (small-M gate/up GEMV, 46.9 MB per launch): its
                average duration over back-to-back launches on distinct weights
                (HIP events on the launch stream), as algorithmic bytes / time against
                the 8 TB/s HBM peak
  cpu_baseline  the PyTorch CPU dequantise-then-fp32-matmul path (oracle/torch_cpu.py)
                on the host cores for 1 of the 32 layers, extrapolated to a token
  extra         per-operator decode timings and prefill TFLOP/s (M = 128 / 512 / 2048)

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_FP16_PEAK_TFLOPS = 2500.0

HIDDEN, INTER, HEADS, LAYERS, GROUPSIZE = 4096, 11008, 32, 32, 128


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def weight_bytes(k, n, g):
    groups = k // g
    return k * n // 2 + groups * n // 2 + groups * n * 2


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the per-operator / prefill extras")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="for rocprofv3 --pmc runs: a 256 MiB device copy (calibration) followed by plain launches of "
                         "each decode operator on distinct weights; prints no JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures the single-GPU hot path: run with --gpus 1 (nothing here uses a second GPU)",
              file=sys.stderr)
        sys.exit(2)

    import torch

    import gptq_triton_amd as G
    from gptq_triton_amd import _lib

    lib = _lib.load()  # fails loudly if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)

    def make(k, n):
        groups = k // GROUPSIZE
        qw = torch.randint(-2**31, 2**31 - 1, (k // 8, n), dtype=torch.int32, device=dev, generator=gen)
        qz = torch.randint(-2**31, 2**31 - 1, (groups, n // 8), dtype=torch.int32, device=dev, generator=gen)
        sc = (0.002 + 0.018 * torch.rand((groups, n), device=dev, generator=gen)).half()
        return qw, qz, sc

    log("building 32 layers of synthetic 4-bit weights ...")
    layers = [dict(qkv=make(HIDDEN, 3 * HIDDEN), o=make(HIDDEN, HIDDEN), gate=make(HIDDEN, INTER),
                   up=make(HIDDEN, INTER), down=make(INTER, HIDDEN)) for _ in range(LAYERS)]
    cos, sin = G.RotaryTable(128, 2048).get(dev, 2048)

    def qkv_op(x, L, pos):
        qw, qz, sc = L["qkv"]
        return G.qkv_rotary(GROUPSIZE, x, qw, sc, qz, pos, cos, sin, HEADS)

    def o_op(x, L):
        qw, qz, sc = L["o"]
        return G.matmul4(GROUPSIZE, x, qw, sc, qz)

    def gateup_op(x, L):
        (gq, gz, gs_), (uq, uz, us_) = L["gate"], L["up"]
        return G.llama_mlp_4(GROUPSIZE, x, gq, gs_, gz, uq, us_, uz)

    def down_op(h, L):
        qw, qz, sc = L["down"]
        return G.matmul4(GROUPSIZE, h, qw, sc, qz)

    def capture(fn):
        """Run fn once on a side stream (allocates the per-stream workspace outside the
        graph), then capture it into a HIP graph on that stream."""
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            fn()
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            out = fn()
        g.replay()
        torch.cuda.synchronize()
        return g, out

    def time_graph(g, reps, warm=3):
        for _ in range(warm):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ts = []
        for _ in range(reps):
            e0.record()
            g.replay()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1))  # ms
        return ts

    # ------------------------------------------------------------------ the decode step
    x1 = torch.randn((1, 1, HIDDEN), device=dev, generator=gen).half()
    pos1 = torch.tensor([[2047]], device=dev, dtype=torch.int32)

    if args.traffic_probe:
        # counters are read per dispatch, so no graph here; the copy kernel moves a known
        # 256 MiB in and 256 MiB out and calibrates FETCH_SIZE / WRITE_SIZE
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(generator=gen)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        for L in layers:
            qkv_op(x1, L, pos1)
        for L in layers:
            o_op(x1, L)
        hs = [gateup_op(x1, L) for L in layers]
        for h, L in zip(hs, layers):
            down_op(h, L)
        torch.cuda.synchronize()
        log("traffic probe done")
        return

    def decode_step():
        outs = []
        for L in layers:
            q, k, v = qkv_op(x1, L, pos1)
            o = o_op(x1, L)
            h = gateup_op(x1, L)
            y = down_op(h, L)
            outs.append((q, k, v, o, y))
        return outs

    step_graph, _ = capture(decode_step)
    for _ in range(args.warmup):
        step_graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(args.steps):
        step_graph.replay()
    e1.record()
    torch.cuda.synchronize()
    ms_per_step = e0.elapsed_time(e1) / args.steps
    tok_s = 1000.0 / ms_per_step
    layer_bytes = (weight_bytes(HIDDEN, 3 * HIDDEN, GROUPSIZE) + weight_bytes(HIDDEN, HIDDEN, GROUPSIZE)
                   + 2 * weight_bytes(HIDDEN, INTER, GROUPSIZE) + weight_bytes(INTER, HIDDEN, GROUPSIZE))
    log(f"decode step: {ms_per_step * 1e3:.1f} us -> {tok_s:.1f} tok/s "
        f"({LAYERS * layer_bytes / ms_per_step / 1e6:.0f} GB/s of weights over the whole step)")

    # ----------------------------------------------- roofline of the dominant kernel
    def gateup_all():
        return [gateup_op(x1, L) for L in layers]

    gu_graph, _ = capture(gateup_all)
    gu_ms = time_graph(gu_graph, reps=max(10, args.steps // 2))
    gu_us = statistics.median(gu_ms) * 1e3 / LAYERS
    gu_bytes = 2 * weight_bytes(HIDDEN, INTER, GROUPSIZE) + HIDDEN * 2 + INTER * 2
    gu_gbs = gu_bytes / gu_us / 1e3
    roofline = {"bound": "hbm", "achieved": round(gu_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(gu_gbs / HBM_PEAK_GBS, 4),
                # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
                # `bench.py --traffic-probe`, scaled by a 256 MiB copy (x2.000 / x1.000)
                "traffic": 50_651_000 + 1_286_000,
                "kernel": "gptq4_gemv_kernel<SILU_MUL> (gate/up GEMV, M=1, K=4096, I=11008, g=128)",
                "bytes_per_launch": gu_bytes, "avg_launch_us": round(gu_us, 2)}
    log(f"gate/up GEMV: {gu_us:.2f} us/launch, {gu_gbs:.0f} GB/s = {100 * gu_gbs / HBM_PEAK_GBS:.1f}% of HBM peak")

    # --------------------------------------------------------------------------- extras
    extra = {}
    if not args.no_extra:
        def per_op(name, fn, nbytes, flops, nsets=LAYERS, reps=10):
            g, _ = capture(lambda: [fn(L) for L in layers[:nsets]])
            us = statistics.median(time_graph(g, reps)) * 1e3 / nsets
            extra[name] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
                           "TFLOPs": round(flops / us / 1e6, 2)}
            log(f"  {name:34s} {us:9.2f} us  {nbytes / us / 1e3:8.0f} GB/s  {flops / us / 1e6:8.1f} TFLOP/s")
            del g

        wq, wo, wg, wd = (weight_bytes(HIDDEN, 3 * HIDDEN, GROUPSIZE), weight_bytes(HIDDEN, HIDDEN, GROUPSIZE),
                          weight_bytes(HIDDEN, INTER, GROUPSIZE), weight_bytes(INTER, HIDDEN, GROUPSIZE))
        h1 = torch.randn((1, INTER), device=dev, generator=gen).half()
        per_op("decode M=1 qkv+rotary", lambda L: qkv_op(x1, L, pos1), wq + 2 * HIDDEN + 6 * HIDDEN, 2 * HIDDEN * 3 * HIDDEN)
        per_op("decode M=1 o_proj", lambda L: o_op(x1, L), wo + 4 * HIDDEN, 2 * HIDDEN * HIDDEN)
        per_op("decode M=1 gate/up+silu*mul", lambda L: gateup_op(x1, L), gu_bytes, 4 * HIDDEN * INTER)
        per_op("decode M=1 down_proj", lambda L: down_op(h1, L), wd + 2 * INTER + 2 * HIDDEN, 2 * HIDDEN * INTER)
        for m in (16, 128, 512, 2048):
            xm = torch.randn((1, m, HIDDEN), device=dev, generator=gen).half()
            hm = torch.randn((m, INTER), device=dev, generator=gen).half()
            posm = torch.arange(m, device=dev, dtype=torch.int32).unsqueeze(0)
            ns = 8 if m <= 128 else 4
            per_op(f"M={m} qkv+rotary", lambda L: qkv_op(xm, L, posm), wq + 2 * m * HIDDEN + 6 * m * HIDDEN,
                   2 * m * HIDDEN * 3 * HIDDEN, nsets=ns, reps=5)
            per_op(f"M={m} gate/up+silu*mul", lambda L: gateup_op(xm, L), 2 * wg + 2 * m * HIDDEN + 2 * m * INTER,
                   4 * m * HIDDEN * INTER, nsets=ns, reps=5)
            per_op(f"M={m} down_proj", lambda L: down_op(hm, L), wd + 2 * m * INTER + 2 * m * HIDDEN,
                   2 * m * HIDDEN * INTER, nsets=ns, reps=5)
            per_op(f"M={m} o_proj (4096x4096)", lambda L: o_op(xm, L), wo + 4 * m * HIDDEN, 2 * m * HIDDEN * HIDDEN,
                   nsets=ns, reps=5)
        best_prefill = max(v["TFLOPs"] for k, v in extra.items() if k.startswith("M=2048"))
        extra["prefill_best_TFLOPs"] = best_prefill
        extra["prefill_frac_of_fp16_mfma_peak"] = round(best_prefill / MFMA_FP16_PEAK_TFLOPS, 4)

    # --------------------------------------------------------------------- CPU baseline
    cpu_baseline = None
    if not args.no_cpu:
        from oracle import torch_cpu as T
        L0 = {k: tuple(t.cpu() for t in v) for k, v in layers[0].items()}
        xc = x1.cpu().view(1, HIDDEN)
        torch.set_grad_enabled(False)

        def cpu_layer():
            T.quant_matmul(xc, *L0["qkv"], GROUPSIZE)
            T.quant_matmul(xc, *L0["o"], GROUPSIZE)
            T.mlp(xc, L0["gate"], L0["up"], L0["down"], GROUPSIZE)

        cpu_layer()
        ts = []
        for _ in range(3):
            t0 = time.perf_counter()
            cpu_layer()
            ts.append(time.perf_counter() - t0)
        t_layer = statistics.median(ts)
        cpu_baseline = {"value": round(1.0 / (t_layer * LAYERS), 4), "unit": "tok/s", "cores": torch.get_num_threads(),
                        "kind": "port",
                        "sample": f"1 of {LAYERS} layers (qkv, o_proj, gate/up+silu*mul, down at M=1; dequantise + fp32 "
                                  f"matmul per call), median of 3 runs = {t_layer:.3f} s, extrapolated x{LAYERS}; "
                                  f"host has {os.cpu_count()} logical CPUs"}
        log(f"cpu baseline: {t_layer:.3f} s per layer on {torch.get_num_threads()} threads")

    result = {
        "metric": "LLaMA-7B-shape 4-bit decode tok/s", "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "fp16", "data": "synthetic",
        "config": {"workload": "llama7b-shape decode, batch 1, position 2047: 32 layers x [fused qkv+rotary, o_proj, "
                               "fused gate/up+silu*mul, down_proj], 4-bit, groupsize 128, distinct weights per layer, "
                               "one HIP-graph replay per token (quantised-linear hot path only)",
                   "hidden": HIDDEN, "intermediate": INTER, "layers": LAYERS, "groupsize": GROUPSIZE,
                   "weight_bytes_per_token": LAYERS * layer_bytes},
        "roofline": roofline, "cpu_baseline": cpu_baseline, "extra": extra,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
