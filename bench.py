#!/usr/bin/env python3
"""Benchmark of the 4-bit GPTQ hot path on one MI355X.

Workload (config.workload): greedy decode of a random-init LLaMA-7B-shape decoder at batch 1
behind a 2048-token prompt - 32 layers x [RMSNorm + fused QKV + rotary into the KV cache
(4096 -> 12288), one-token attention over the cache, o_proj (4096 -> 4096), RMSNorm + fused
gate/up + SiLU*mul (4096 -> 2 x 11008), down_proj (11008 -> 4096)], final norm, fp16 lm_head,
argmax; 4-bit, groupsize 128, every layer with its own synthetic weights (3.2 GB, so each launch
streams its weights from HBM, not from the 256 MB Infinity Cache), packed weights in streaming
order (what the decode kernel reads).  The launches of a step are captured once in a HIP graph
and replayed; a "step" is one replay = one token.  value = tokens/s = 1 / step time.

`linears_only` (top level): the same step with nothing but its 128 quantised-linear launches - the
hot path by itself, what `value` was in earlier builds.

Also reported on the same line:
  roofline      the dominant kernel (gate/up GEMV on streaming-order weights, 46.9 MB per
                launch): its average duration over back-to-back launches on distinct weights
                (HIP events on the launch stream), as algorithmic bytes / time against
                the 8 TB/s HBM peak; floor_us / frac_of_floor: the same bytes read by a plain
                16-byte-per-lane kernel, launch included (the stand-alone floor probe, when it
                is built); attention: the one-token attention kernel's own fraction
  cpu_baseline  the PyTorch CPU dequantise-then-fp32-matmul path (oracle/torch_cpu.py)
                on the host cores for 1 of the 32 layers, extrapolated to a token
                (+ step_frac: the weights of the whole 128-launch step over the step time;
                traffic: HBM bytes per launch from rocprofv3 counters, a constant taken from
                profiles/decode_stream_llama7b_m1.md, see traffic_source)
  extra         baseline_configs: one row per configuration of BASELINE.json that fits this
                path - C1 QuantLinear 4096 x 4096 (one group) at M = 1 and 128, C2 the fused
                MLP (gate/up + SiLU*mul, then down; groupsize 128) at M = 1, 16 and 512, C3
                fused QKV + rotary (one group) at M = 1 (position 2047) and M = 2048 - each
                with its time, algorithmic bytes and flops, and the fraction of the HBM or
                fp16 MFMA peak that bounds it;
                decoders: the whole-decoder workloads below (7B, 13B act-order, 30B at batch
                1 and 8), unless --no-decoders;
                per-operator decode timings ("hot" = one layer's weights over and over, served by
                the Infinity Cache; everything else streams from HBM), batched and prefill
                TFLOP/s (M = 16 ... 8192) and the vendor library's dense fp16 GEMM on the
                M = 2048 shapes
  --chain-probe / --chain-timeline: the chained decode launch (gptq4_decode_chain) against the
                separate launches it would replace
  --attention-probe: the causal prompt-attention kernel beside torch's fused attention + transpose
  --floor-probe what a launch costs before it computes anything: empty launches and plain reads of
                the four decode operators' bytes (csrc/probe/floor_probe, a stand-alone program),
                then each decode operator's own access pattern with the arithmetic left out
                (gptq4_stream_probe) beside the operator itself; prints text and one JSON line

Other workloads (--workload llama7b | llama13b | llama30b): a full random-init decoder of
that shape (embedding, RMSNorm, fused QKV + rotary into a preallocated KV cache, the
library's prompt and decode attention, o_proj, fused MLP, fp16 lm_head + greedy argmax) - one
timed prefill of --prompt
tokens, then --new-tokens greedy tokens with one HIP-graph replay per token; value =
decode tokens/s over the batch, prefill TFLOP/s and the eager (kernel-by-kernel) decode
rate in `extra`.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]
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


DECODERS = {
    # layers, hidden, intermediate, heads, groupsize, act-order
    "llama7b": (32, 4096, 11008, 32, 128, False),
    "llama13b": (40, 5120, 13824, 40, 128, True),
    "llama30b": (60, 6656, 17920, 52, 512, False),
}


def decoder_figures(workload, bsz, prompt, new, steps=None, warmup=None):
    """Full-decoder workload: prefill + graph-replayed greedy decode on a random-init model.  Returns the result
    record (the JSON line of `--workload llamaNNb`).  steps / warmup: exactly that many timed / untimed graph replays
    (new is then derived from them)."""
    eager_steps = 8 if steps is None else 4
    if steps is not None:
        warmup = 0 if warmup is None else warmup
        new = 1 + eager_steps + 2 + warmup + steps
    import gc

    import torch

    torch.set_grad_enabled(False)

    import gptq_triton_amd as G
    from gptq_triton_amd import _lib
    from gptq_triton_amd.fused_attention import LlamaConfigLite
    from gptq_triton_amd.llama import GreedyDecoder, LlamaForCausalLM, LlamaRMSNorm

    _lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    layers, hidden, inter, heads, groupsize, act_order = DECODERS[workload]
    cfg = LlamaConfigLite()
    cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads, cfg.num_hidden_layers = hidden, inter, heads, layers
    cfg.vocab_size, cfg.max_position_embeddings = 32000, max(2048, prompt + new)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)

    log(f"building a random-init {workload} decoder ({layers} layers, groupsize {groupsize}, act-order {act_order}) ...")
    dtype0 = torch.get_default_dtype()
    torch.set_default_dtype(torch.half)
    try:
        with torch.device("meta"):
            model = LlamaForCausalLM(cfg)
    finally:
        torch.set_default_dtype(dtype0)
    with torch.device("meta"):
        G.make_quant(model, 4, groupsize, act_order=act_order)
    model = model.to_empty(device=dev)
    qbytes = 0
    for layer in model.model.layers:
        # projections that share an input share its act-order permutation
        perms = {}
        for group, names in (("attn_in", ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj")),
                             ("attn_out", ("self_attn.o_proj",)), ("mlp_in", ("mlp.gate_proj", "mlp.up_proj")),
                             ("mlp_out", ("mlp.down_proj",))):
            for name in names:
                q = layer.get_submodule(name)
                q.qweight.copy_(torch.randint(-2**31, 2**31 - 1, q.qweight.shape, dtype=torch.int32, device=dev, generator=gen))
                q.qzeros.copy_(torch.randint(-2**31, 2**31 - 1, q.qzeros.shape, dtype=torch.int32, device=dev, generator=gen))
                # scales sized so that activations stay O(1) through the depth of the stack
                q.scales.copy_(((0.2 + 0.3 * torch.rand(q.scales.shape, device=dev, generator=gen)) / (4.6 * q.infeatures ** 0.5)).half())
                qbytes += q.qweight.numel() * 4 + q.qzeros.numel() * 4 + q.scales.numel() * 2
                if act_order:
                    if group not in perms:
                        g = q.infeatures // (q.infeatures if groupsize == -1 else groupsize)
                        base = torch.arange(q.infeatures, device=dev) // (q.infeatures // g)
                        perms[group] = base[torch.randperm(q.infeatures, device=dev, generator=gen)].int()
                    q.g_idx.copy_(perms[group])
    for m in model.modules():
        if isinstance(m, LlamaRMSNorm):
            m.weight.fill_(1.0)
    model.model.embed_tokens.weight.copy_(torch.randn(model.model.embed_tokens.weight.shape, device=dev, generator=gen) * 0.5)
    model.lm_head.weight.copy_(torch.randn(model.lm_head.weight.shape, device=dev, generator=gen) * 0.02)
    G.make_quant_attn(model)
    G.make_fused_mlp(model)
    if act_order:
        G.quant_linear.compact_act_order(model)  # one copy of every packed weight, in the layout the kernels read

    ids = torch.randint(0, cfg.vocab_size, (bsz, prompt), device=dev, generator=gen)
    dec = GreedyDecoder(model, bsz, prompt + new)
    log("warm-up prefill ...")
    dec.prefill(ids)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    first = dec.prefill(ids)
    enqueue_s = time.perf_counter() - t0  # the host's share: every launch of the prompt pass is issued from Python
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    per_token_kn = layers * (hidden * 3 * hidden + hidden * hidden + 2 * hidden * inter + inter * hidden)
    prefill_tf = 2.0 * bsz * prompt * per_token_kn / prefill_s / 1e12
    log(f"prefill: {prefill_s * 1e3:.1f} ms for {bsz} x {prompt} tokens = {prefill_tf:.0f} TFLOP/s in the quantised linears "
        f"(the host needed {enqueue_s * 1e3:.1f} ms to issue its launches)")

    eager_steps = min(eager_steps, new - 1)
    # kernel-by-kernel steps: the first two untimed (they load the decode kernels and make the workspaces)
    cold = min(2, max(eager_steps - 1, 0))
    generated = [first, dec.decode(cold)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    generated.append(dec.decode(eager_steps - cold))
    torch.cuda.synchronize()
    eager_s = (time.perf_counter() - t0) / max(eager_steps - cold, 1)
    generated.append(dec.decode(2, use_graph=True))  # captures the step
    if steps is None:
        steps = new - 1 - eager_steps - 2
    elif warmup:
        generated.append(dec.decode(warmup, use_graph=True))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    toks = dec.decode(steps, use_graph=True)
    torch.cuda.synchronize()
    step_s = (time.perf_counter() - t0) / steps
    kv_bytes = 2 * layers * bsz * heads * (prompt + new) * 128 * 2
    step_bytes = qbytes + model.lm_head.weight.numel() * 2 + kv_bytes
    gbs = step_bytes / step_s / 1e9
    # Check beyond "tokens came out": the prompt + the first j generated tokens through the prefill path (tiled GEMM, torch's
    # attention over the whole sequence) must choose generated token j, which the decode path (GEMV kernels, one-token
    # attention over the cache, graph replay) chose.  Random-init logits have near-ties, so the count is reported, not asserted.
    generated = torch.cat(generated + [toks], dim=1)
    probes = sorted({1, eager_steps + 3, generated.shape[1] // 2, generated.shape[1] - 1})
    agree = 0
    for j in probes:
        nxt = dec.prefill(torch.cat([ids, generated[:, :j]], dim=1))
        agree += int((nxt[:, 0] == generated[:, j]).sum())
    agreement = f"{agree}/{len(probes) * bsz}"
    log(f"prefill path re-run on prompt + generated tokens agrees with the decode path on {agreement} next tokens (probes {probes})")
    log(f"decode: {step_s * 1e3:.3f} ms/step graph-replayed ({bsz / step_s:.1f} tok/s), {eager_s * 1e3:.3f} ms/step eager; "
        f"{step_bytes / 1e9:.2f} GB per step -> {gbs:.0f} GB/s")
    result = {
        "metric": f"{workload}-shape 4-bit greedy decode tok/s (full decoder)", "value": round(bsz / step_s, 2),
        "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": eager_steps + 2 + (warmup or 0), "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp16", "data": "synthetic",
        "config": {"workload": f"random-init {workload}-shape decoder, batch {bsz}, {prompt}-token prompt prefill then "
                               f"{new} greedy tokens, 4-bit groupsize {groupsize}{' act-order' if act_order else ''}, "
                               f"fp16 lm_head, one HIP-graph replay per token, packed weights in "
                               "streaming order",
                   "layers": layers, "hidden": hidden, "intermediate": inter, "heads": heads, "batch": bsz,
                   "prompt": prompt, "new_tokens": new},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "whole decode step: packed weights + fp16 lm_head + the full-capacity KV cache, read once",
                     "bytes_per_launch": step_bytes, "avg_launch_us": round(step_s * 1e6, 1)},
        "cpu_baseline": None,
        "extra": {"prefill_ms": round(prefill_s * 1e3, 2), "prefill_host_issue_ms": round(enqueue_s * 1e3, 2),
                  "prefill_linear_TFLOPs": round(prefill_tf, 1),
                  "prefill_frac_of_fp16_mfma_peak": round(prefill_tf / MFMA_FP16_PEAK_TFLOPS, 4),
                  "eager_decode_ms_per_step": round(eager_s * 1e3, 3), "last_tokens": toks[0, -4:].tolist(),
                  "prefill_path_agrees_with_decode_path_on_next_tokens": agreement},
    }
    del dec, model, toks, ids
    gc.collect()
    torch.cuda.empty_cache()
    return result


def run_decoder(args):
    print(json.dumps(decoder_figures(args.workload, args.batch, args.prompt, args.new_tokens)), flush=True)


# HBM bytes one launch of the dominant kernel moves, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (see roofline.traffic_source)
TRAFFIC_GATEUP_STREAM = 48316000  # 48.17 MB fetched + 0.14 MB written

FLOOR_BINARY = os.path.join(ROOT, "gptq-triton_amd", "csrc", "probe", "floor_probe")


def run_floor_binary():
    """Figures of the stand-alone floor probe (csrc/probe/floor_probe.hip) as {name: value}, or None when it is not built.
    Runs as a child process, before this process has many launches in flight; about ten seconds."""
    import subprocess
    if not os.path.exists(FLOOR_BINARY):
        log("floor probe not built (python gptq-triton_amd/build.py builds it): no floor figures")
        return None
    try:
        out = subprocess.run([FLOOR_BINARY], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120).stdout
    except Exception as e:
        log(f"floor probe failed: {e!r}")
        return None
    figures = {}
    for line in out.splitlines():
        parts = line.split()
        if len(parts) == 3:
            try:
                figures[parts[0]] = float(parts[1])
            except ValueError:
                pass
    if not figures:
        log("floor probe printed no figures (it does not run under a profiler): no floor figures")
    return figures or None


def floor_probe(args, layers, x1, dev, capture, time_graph, s_o_op, s_gateup_op, s_down_op, s_qkv_op, pos1):
    """`--floor-probe`: per decode operator of the 7B shape, at one row and with the weights coming from HBM - the launch
    floor, a plain read of the operator's bytes, the operator's own access pattern with the arithmetic left out, the
    operator.  Text on stderr, one JSON line on stdout."""
    import torch

    import gptq_triton_amd as G
    from gptq_triton_amd import _lib

    lib = _lib.load()
    figures = run_floor_binary() or {}
    for k, v in figures.items():
        log(f"  {k:44s} {v:10.3f}")
    ws = _lib.workspace(dev, _lib.WS_HEAD_BYTES)
    h1 = torch.randn((1, INTER), device=dev).half()
    x = x1.view(1, HIDDEN)
    y = torch.empty((1, max(INTER, 3 * HIDDEN)), device=dev).half()

    def pattern(op, xin, k, n, a, b=None):
        def run():
            st = _lib.current_stream(dev)
            for L in layers:
                (sw, mt), up = L[a], (L[b] if b else (None, None))
                rc = lib.gptq4_stream_probe(op, xin.data_ptr(), sw.data_ptr(), mt.data_ptr(), _lib.ptr(up[0]), _lib.ptr(up[1]), y.data_ptr(),
                                            1, k, n, GROUPSIZE, ws.data_ptr(), ws.numel(), st)
                _lib.check(rc, "gptq4_stream_probe")
        return run

    rows = {}
    plain = {"o_proj": "plain_read_8.7MB", "down_proj": "plain_read_23.4MB", "qkv+rotary": "plain_read_26.1MB", "gate/up+silu*mul": "plain_read_46.9MB"}
    ops = {"o_proj": (lambda: [s_o_op(x, L) for L in layers], pattern(0, x, HIDDEN, HIDDEN, "s_o")),
           "down_proj": (lambda: [s_down_op(h1, L) for L in layers], pattern(0, h1, INTER, HIDDEN, "s_down")),
           # (the rotary epilogue has no variant without arithmetic: the plain projection's pattern on the same bytes stands in)
           "qkv+rotary": (lambda: [s_qkv_op(x1, L, pos1) for L in layers], pattern(0, x, HIDDEN, 3 * HIDDEN, "s_qkv")),
           "gate/up+silu*mul": (lambda: [s_gateup_op(x, L) for L in layers], pattern(1, x, HIDDEN, INTER, "s_gate", "s_up"))}
    log(f"  {'operator (M = 1, 7B shape, weights from HBM)':46s} {'launch floor':>12s} {'plain read':>11s} {'pattern only':>13s} {'operator':>9s}   us")
    for name, (full, loads_only) in ops.items():
        g1, _ = capture(full)
        g2, _ = capture(loads_only)
        t_full = statistics.median(time_graph(g1, 10)) * 1e3 / LAYERS
        t_loads = statistics.median(time_graph(g2, 10)) * 1e3 / LAYERS
        del g1, g2
        rows[name] = {"operator_us": round(t_full, 2), "access_pattern_without_arithmetic_us": round(t_loads, 2),
                      "plain_read_us": figures.get(plain[name]), "launch_floor_us": figures.get("launch_floor_1wg_per_cu_512t_81k")}
        log(f"  {name:46s} {rows[name]['launch_floor_us'] or float('nan'):12.2f} {rows[name]['plain_read_us'] or float('nan'):11.2f} {t_loads:13.2f} {t_full:9.2f}")
    print(json.dumps({"floor_probe": rows, "device_figures": figures}), flush=True)


def chain_probe(args):
    """Chained decode launch (gptq4_decode_chain) against the separate launches on LLaMA-7B shapes, us per layer
    under graph replay; with a timing build of the library (python gptq-triton_amd/build.py -DGPTQ4_CHAIN_TIMERS)
    also the in-kernel timeline of one o_proj -> add+RMSNorm -> gate/up -> down_proj launch.  Prints text, no JSON."""
    import numpy as np
    import torch

    import gptq_triton_amd as G
    from gptq_triton_amd import _lib
    from gptq_triton_amd import chain as C
    from gptq_triton_amd.decoder_ops import add_rms_norm

    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    m, gs = args.batch, GROUPSIZE

    def make(k, n):
        g = k // gs
        return (torch.randint(-2**31, 2**31 - 1, (k // 8, n), dtype=torch.int32, device=dev, generator=gen),
                torch.randint(-2**31, 2**31 - 1, (g, n // 8), dtype=torch.int32, device=dev, generator=gen),
                ((0.002 + 0.018 * torch.rand((g, n), device=dev, generator=gen)) * (6.0 / k ** 0.5)).half())

    layers = [dict(qkv=make(HIDDEN, 3 * HIDDEN), o=make(HIDDEN, HIDDEN), gate=make(HIDDEN, INTER), up=make(HIDDEN, INTER),
                   down=make(INTER, HIDDEN)) for _ in range(LAYERS)]
    cos, sin = G.RotaryTable(128, 2048).get(dev, 2048)
    x = torch.randn((m, HIDDEN), device=dev, generator=gen).half()
    h = torch.randn((m, HIDDEN), device=dev, generator=gen).half()
    w = torch.ones(HIDDEN, device=dev).half()
    pos = torch.full((m,), 2047, dtype=torch.int32, device=dev)
    q = torch.empty((m, HEADS, 1, 128), device=dev).half()
    kk, vv = torch.empty_like(q), torch.empty_like(q)
    s, y = torch.empty((m, HIDDEN), device=dev).half(), torch.empty((m, HIDDEN), device=dev).half()

    def graph_us(fn, reps=20):
        st = torch.cuda.Stream()
        st.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(st):
            fn()
        torch.cuda.current_stream().wait_stream(st)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            fn()
        for _ in range(3):
            g.replay()
        torch.cuda.synchronize()
        ts = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1))
        return statistics.median(ts) * 1e3 / LAYERS

    p_o = lambda L: C.projection(*L["o"], gs, x=x)
    p_gu = lambda L: C.projection(*L["gate"], gs, up=L["up"], input=C.IN_NORM_PREV, x=h, norm_weight=w, eps=1e-6, sum_out=s)
    p_dn = lambda L: C.projection(*L["down"], gs, input=C.IN_PREV, output=C.OUT_ROWS, y=y)
    rope = dict(position_ids=pos, cos=cos, sin=sin, q=q, k=kk, v=vv, heads=HEADS)
    p_qkv = lambda L: C.projection(*L["qkv"], gs, x=x, output=C.OUT_ROPE, rope=rope)

    def separate(with_qkv):
        def run():
            for L in layers:
                if with_qkv:
                    G.qkv_rotary(gs, x.view(m, 1, HIDDEN), L["qkv"][0], L["qkv"][2], L["qkv"][1], pos.view(m, 1), cos, sin, HEADS)
                o = G.matmul4(gs, x, L["o"][0], L["o"][2], L["o"][1])
                _, xn = add_rms_norm(h, o, w, 1e-6)
                a = G.llama_mlp_4(gs, xn, L["gate"][0], L["gate"][2], L["gate"][1], L["up"][0], L["up"][2], L["up"][1])
                G.matmul4(gs, a, L["down"][0], L["down"][2], L["down"][1])
        return run

    def chained(phases_of):
        def run():
            for L in layers:
                C.decode_chain(phases_of(L), m, dev)
        return run

    print(f"LLaMA-7B shapes, M = {m}, groupsize {gs}, {LAYERS} layers of distinct weights, us per layer (graph replay)")
    print(f"  separate launches, with QKV + rotary (5 launches)     {graph_us(separate(True)):7.2f}")
    print(f"  separate launches, o_proj .. down_proj (4 launches)   {graph_us(separate(False)):7.2f}")
    print(f"  chain o_proj -> norm -> gate/up -> down (1 launch)    {graph_us(chained(lambda L: [p_o(L), p_gu(L), p_dn(L)])):7.2f}")
    print(f"  chain with QKV + rotary in front (1 launch)           {graph_us(chained(lambda L: [p_qkv(L), p_o(L), p_gu(L), p_dn(L)])):7.2f}")
    if not args.chain_timeline:
        return
    # the in-kernel timeline: needs the library built with the stamps (its workspace is then 1 MiB larger)
    ph = [p_o(layers[0]), p_gu(layers[0]), p_dn(layers[0])]
    arr = (_lib.Phase * 3)(*ph)
    need = lib.gptq4_chain_workspace_bytes(arr, 3, m)
    ws = torch.zeros(need, dtype=torch.uint8, device=dev)
    for L in layers[:4]:
        C.decode_chain([p_o(L), p_gu(L), p_dn(L)], m, dev, ws=ws)
    torch.cuda.synchronize()
    stamps = ws[need - (1 << 20):need - (1 << 20) + 256 * 64 * 8].view(torch.int64).cpu().numpy().reshape(256, 64).astype(np.float64) / 100.0
    t0 = stamps[:, 0].min()
    print("  timeline of one chained launch, us from the first stamp: min / median / max over the workgroups")
    for p, name in enumerate(("o_proj", "gate/up", "down_proj")):
        for j, what in ((3, "rows staged in LDS"), (5, "all streaming waves through"), (6, "partial tiles stored"), (1, "slice of finished values stored")):
            col = stamps[:, 2 + 7 * p + j] - t0
            print(f"    {name:10s} {what:34s} {col.min():7.2f} {np.median(col):7.2f} {col.max():7.2f}")


def attention_probe():
    """`--attention-probe`: gptq4_prefill_attention against torch.nn.functional.scaled_dot_product_attention(is_causal=True)
    followed by the transpose into o_proj's input layout, HIP events around single launches, median of 20."""
    import torch

    from gptq_triton_amd import _lib, decoder_ops

    _lib.load()
    dev = torch.device("cuda:0")
    rows = {}
    for (b, h, s) in ((1, 32, 2048), (1, 40, 2048), (8, 52, 2048), (1, 32, 512)):
        q = torch.randn((b, h, s, 128), device=dev).half()
        k, v = torch.randn_like(q), torch.randn_like(q)

        def timed(fn, reps=20):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            ts = []
            for _ in range(reps):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                fn()
                e1.record()
                torch.cuda.synchronize()
                ts.append(e0.elapsed_time(e1) * 1e3)
            return statistics.median(ts)

        mine = timed(lambda: decoder_ops.prefill_attention(q, k, v))
        ref = timed(lambda: torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(b, s, h * 128))
        flops = 4 * b * h * s * s * 128 / 2
        rows[f"B={b} H={h} S={s}"] = {"us": round(mine, 1), "causal_TFLOPs": round(flops / mine / 1e6, 1), "torch_sdpa_plus_transpose_us": round(ref, 1)}
        log(f"  B={b} H={h} S={s}: {mine:8.1f} us ({flops / mine / 1e6:.0f} TFLOP/s causal)   torch: {ref:8.1f} us")
    print(json.dumps({"attention_probe": rows}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the per-operator / prefill extras")
    ap.add_argument("--no-decoders", action="store_true", help="skip the full-decoder workloads (C4 / C5) in the extras")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="for rocprofv3 --pmc runs: a 256 MiB device copy (calibration) followed by plain launches of "
                         "each decode operator on distinct weights; prints no JSON")
    ap.add_argument("--attention-probe", action="store_true",
                    help="the causal prompt-attention kernel against torch's fused attention + transpose at LLaMA shapes")
    ap.add_argument("--floor-probe", action="store_true",
                    help="launch floor, plain reads and each decode operator's access pattern without its arithmetic beside the "
                         "operator itself (7B shapes, one row); prints text and one JSON line")
    ap.add_argument("--chain-probe", action="store_true",
                    help="time gptq4_decode_chain against the separate launches (7B shapes, --batch rows); prints text, no JSON")
    ap.add_argument("--chain-timeline", action="store_true",
                    help="with --chain-probe: also print the in-kernel timeline (needs the library built with -DGPTQ4_CHAIN_TIMERS)")
    ap.add_argument("--workload", default="linears7b", choices=["linears7b"] + sorted(DECODERS),
                    help="linears7b (default): the quantised-linear hot path of one 7B decode token; llamaNNb: a full "
                         "random-init decoder of that shape, prefill + greedy decode")
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--new-tokens", type=int, default=128)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures the single-GPU hot path: run with --gpus 1 (nothing here uses a second GPU)",
              file=sys.stderr)
        sys.exit(2)

    if args.chain_probe:
        return chain_probe(args)
    if args.attention_probe:
        return attention_probe()
    if args.workload != "linears7b":
        return run_decoder(args)

    import torch

    import gptq_triton_amd as G
    from gptq_triton_amd import _lib

    lib = _lib.load()  # fails loudly if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)

    def make(k, n, g=GROUPSIZE):
        groups = 1 if g == -1 else k // g
        qw = torch.randint(-2**31, 2**31 - 1, (k // 8, n), dtype=torch.int32, device=dev, generator=gen)
        qz = torch.randint(-2**31, 2**31 - 1, (groups, n // 8), dtype=torch.int32, device=dev, generator=gen)
        sc = (0.002 + 0.018 * torch.rand((groups, n), device=dev, generator=gen)).half()
        return qw, qz, sc

    log("building 32 layers of synthetic 4-bit weights ...")
    layers = [dict(qkv=make(HIDDEN, 3 * HIDDEN), o=make(HIDDEN, HIDDEN), gate=make(HIDDEN, INTER),
                   up=make(HIDDEN, INTER), down=make(INTER, HIDDEN)) for _ in range(LAYERS)]
    # the same weights in streaming order, the resident layout of a model that decodes up to sixteen sequences
    for L in layers:
        for name in ("qkv", "o", "gate", "up", "down"):
            qw, qz, sc = L[name]
            L["s_" + name] = G.stream_pack(qw, qz, sc, GROUPSIZE)
    cos, sin = G.RotaryTable(128, 2048).get(dev, 2048)

    def s_qkv_op(x, L, pos):
        return G.qkv_rotary_stream(GROUPSIZE, x, *L["s_qkv"], pos, cos, sin, HEADS)

    def s_o_op(x, L):
        return G.matmul4_stream(GROUPSIZE, x, *L["s_o"])

    def s_gateup_op(x, L):
        return G.llama_mlp_4_stream(GROUPSIZE, x, *L["s_gate"], *L["s_up"])

    def s_down_op(h, L):
        return G.matmul4_stream(GROUPSIZE, h, *L["s_down"])

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
        for L in layers:
            s_qkv_op(x1, L, pos1)
        for L in layers:
            s_o_op(x1, L)
        hs = [s_gateup_op(x1, L) for L in layers]
        for h, L in zip(hs, layers):
            s_down_op(h, L)
        torch.cuda.synchronize()
        log("traffic probe done")
        return

    if args.floor_probe:
        return floor_probe(args, layers, x1, dev, capture, time_graph, s_o_op, s_gateup_op, s_down_op, s_qkv_op, pos1)

    def decode_step():
        outs = []
        for L in layers:
            q, k, v = s_qkv_op(x1, L, pos1)
            o = s_o_op(x1.view(1, HIDDEN), L)
            h = s_gateup_op(x1.view(1, HIDDEN), L)
            y = s_down_op(h, L)
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
    log(f"decode step, quantised linears only: {ms_per_step * 1e3:.1f} us -> {tok_s:.1f} tok/s "
        f"({LAYERS * layer_bytes / ms_per_step / 1e6:.0f} GB/s of weights over the whole step)")

    # ----------------------------------------------- roofline of the dominant kernel
    def gateup_all():
        return [s_gateup_op(x1.view(1, HIDDEN), L) for L in layers]

    gu_graph, _ = capture(gateup_all)
    gu_ms = time_graph(gu_graph, reps=max(10, args.steps // 2))
    gu_us = statistics.median(gu_ms) * 1e3 / LAYERS
    # algorithmic bytes of one launch = one unit of work: the two projections' packed words, zeros and scales as the
    # checkpoint holds them, the input row and the output row
    gu_bytes = 2 * weight_bytes(HIDDEN, INTER, GROUPSIZE) + HIDDEN * 2 + INTER * 2
    gu_gbs = gu_bytes / gu_us / 1e3
    floor = run_floor_binary()
    roofline = {"bound": "hbm", "achieved": round(gu_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(gu_gbs / HBM_PEAK_GBS, 4),
                # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
                # `bench.py --traffic-probe`, scaled by a 256 MiB copy
                "traffic": TRAFFIC_GATEUP_STREAM,
                "traffic_source": "constant: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this kernel, profiles/decode_stream_llama7b_m1.md",
                "step_frac": round(LAYERS * layer_bytes / ms_per_step / 1e6 / HBM_PEAK_GBS, 4),
                "step_GBps": round(LAYERS * layer_bytes / ms_per_step / 1e6, 1),
                "kernel": "gptq4_stream_kernel<SILU_MUL> (gate/up GEMV on streaming-order weights, M=1, K=4096, I=11008, g=128)",
                "bytes_per_launch": gu_bytes, "avg_launch_us": round(gu_us, 2)}
    if floor and "plain_read_46.9MB" in floor:
        # what ANY launch pays to read these bytes: the launch floor plus a plain 16-byte-per-lane read of 46.9 MB from HBM
        roofline["floor_us"] = floor["plain_read_46.9MB"]
        roofline["frac_of_floor"] = round(floor["plain_read_46.9MB"] / gu_us, 4)
        roofline["launch_floor_us"] = floor.get("launch_floor_1wg_per_cu_512t_81k")
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
        x1f = x1.view(1, HIDDEN)
        per_op("decode M=1 qkv+rotary", lambda L: s_qkv_op(x1, L, pos1), wq + 2 * HIDDEN + 6 * HIDDEN, 2 * HIDDEN * 3 * HIDDEN)
        per_op("decode M=1 o_proj", lambda L: s_o_op(x1f, L), wo + 4 * HIDDEN, 2 * HIDDEN * HIDDEN)
        per_op("decode M=1 gate/up+silu*mul", lambda L: s_gateup_op(x1f, L), gu_bytes, 4 * HIDDEN * INTER)
        per_op("decode M=1 down_proj", lambda L: s_down_op(h1, L), wd + 2 * INTER + 2 * HIDDEN, 2 * HIDDEN * INTER)
        for mm in (2, 4, 8, 16):  # (from five rows on: the variant that fetches the rows with every unit)
            xm = torch.randn((mm, 1, HIDDEN), device=dev, generator=gen).half()
            hm = torch.randn((mm, INTER), device=dev, generator=gen).half()
            posm = torch.full((mm, 1), 2047, device=dev, dtype=torch.int32)
            per_op(f"decode M={mm} qkv+rotary", lambda L: s_qkv_op(xm, L, posm), wq + 8 * mm * HIDDEN, 2 * mm * HIDDEN * 3 * HIDDEN)
            per_op(f"decode M={mm} o_proj", lambda L: s_o_op(xm.view(mm, HIDDEN), L), wo + 4 * mm * HIDDEN, 2 * mm * HIDDEN * HIDDEN)
            per_op(f"decode M={mm} gate/up+silu*mul", lambda L: s_gateup_op(xm.view(mm, HIDDEN), L), 2 * wg + 2 * mm * (HIDDEN + INTER), 4 * mm * HIDDEN * INTER)
            per_op(f"decode M={mm} down_proj", lambda L: s_down_op(hm, L), wd + 2 * mm * (INTER + HIDDEN), 2 * mm * HIDDEN * INTER)
        # the kernels for the checkpoint layout on the same shapes (what a model kept in that layout runs at one row)
        per_op("checkpoint layout M=1 qkv+rotary", lambda L: qkv_op(x1, L, pos1), wq + 2 * HIDDEN + 6 * HIDDEN, 2 * HIDDEN * 3 * HIDDEN)
        per_op("checkpoint layout M=1 o_proj", lambda L: o_op(x1, L), wo + 4 * HIDDEN, 2 * HIDDEN * HIDDEN)
        per_op("checkpoint layout M=1 gate/up+silu*mul", lambda L: gateup_op(x1, L), gu_bytes, 4 * HIDDEN * INTER)
        per_op("checkpoint layout M=1 down_proj", lambda L: down_op(h1, L), wd + 2 * INTER + 2 * HIDDEN, 2 * HIDDEN * INTER)
        # one-token attention over a 2048-row cache: 32 caches of 33.5 MB, one per layer, so that every launch reads HBM
        from gptq_triton_amd.decoder_ops import decode_attention
        caches = [(torch.randn((1, HEADS, 2048, 128), device=dev, generator=gen).half(), torch.randn((1, HEADS, 2048, 128), device=dev, generator=gen).half())
                  for _ in range(LAYERS)]
        qa = torch.randn((1, HEADS, 1, 128), device=dev, generator=gen).half()
        pa = torch.tensor([2047], device=dev, dtype=torch.int32)
        att_bytes = 2 * HEADS * 2048 * 128 * 2 + 4 * HEADS * 128
        ga, _ = capture(lambda: [decode_attention(qa, kc, vc, pa) for kc, vc in caches])
        att_us = statistics.median(time_graph(ga, 10)) * 1e3 / LAYERS
        del ga, caches
        extra["decode attention, 2048 cached tokens"] = {"us": round(att_us, 2), "GBps": round(att_bytes / att_us / 1e3, 1)}
        roofline["attention"] = {"kernel": "gptq4_decode_attention (32 heads x 128, 2048 cached tokens, one query token)",
                                 "bytes_per_launch": att_bytes, "avg_launch_us": round(att_us, 2),
                                 "frac": round(att_bytes / att_us / 1e3 / HBM_PEAK_GBS, 4)}
        log(f"  {'decode attention, 2048 tokens':34s} {att_us:9.2f} us  {att_bytes / att_us / 1e3:8.0f} GB/s")
        # "hot": the same launches on ONE layer's weights over and over, so that they come out of the
        # 256 MB Infinity Cache instead of HBM.  Not an HBM figure; it shows what the memory side costs.
        def per_op_hot(name, fn, nbytes, flops, reps=10):
            g, _ = capture(lambda: [fn(layers[0]) for _ in range(LAYERS)])
            us = statistics.median(time_graph(g, reps)) * 1e3 / LAYERS
            extra[name] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1), "TFLOPs": round(flops / us / 1e6, 2)}
            log(f"  {name:34s} {us:9.2f} us  {nbytes / us / 1e3:8.0f} GB/s  {flops / us / 1e6:8.1f} TFLOP/s")
            del g
        per_op_hot("hot M=1 qkv+rotary", lambda L: s_qkv_op(x1, L, pos1), wq + 2 * HIDDEN + 6 * HIDDEN, 2 * HIDDEN * 3 * HIDDEN)
        per_op_hot("hot M=1 o_proj", lambda L: s_o_op(x1f, L), wo + 4 * HIDDEN, 2 * HIDDEN * HIDDEN)
        per_op_hot("hot M=1 gate/up+silu*mul", lambda L: s_gateup_op(x1f, L), gu_bytes, 4 * HIDDEN * INTER)
        per_op_hot("hot M=1 down_proj", lambda L: s_down_op(h1, L), wd + 2 * INTER + 2 * HIDDEN, 2 * HIDDEN * INTER)
        for m in (16, 64, 128, 256, 512, 2048, 8192):
            xm = torch.randn((1, m, HIDDEN), device=dev, generator=gen).half()
            hm = torch.randn((m, INTER), device=dev, generator=gen).half()
            posm = torch.arange(m, device=dev, dtype=torch.int32).unsqueeze(0)
            ns = 8 if m <= 128 else (4 if m <= 2048 else 2)
            per_op(f"M={m} qkv+rotary", lambda L: qkv_op(xm, L, posm), wq + 2 * m * HIDDEN + 6 * m * HIDDEN,
                   2 * m * HIDDEN * 3 * HIDDEN, nsets=ns, reps=5)
            per_op(f"M={m} gate/up+silu*mul", lambda L: gateup_op(xm, L), 2 * wg + 2 * m * HIDDEN + 2 * m * INTER,
                   4 * m * HIDDEN * INTER, nsets=ns, reps=5)
            per_op(f"M={m} down_proj", lambda L: down_op(hm, L), wd + 2 * m * INTER + 2 * m * HIDDEN,
                   2 * m * HIDDEN * INTER, nsets=ns, reps=5)
            per_op(f"M={m} o_proj (4096x4096)", lambda L: o_op(xm, L), wo + 4 * m * HIDDEN, 2 * m * HIDDEN * HIDDEN,
                   nsets=ns, reps=5)
        # ---- the BASELINE.json configurations exactly as stated, each with its own roofline fraction
        rows = []

        def config_row(cfg, op, m, fn, sets, nbytes, flops, reps=10):
            g, _ = capture(lambda: [fn(w) for w in sets])
            us = statistics.median(time_graph(g, reps)) * 1e3 / len(sets)
            del g
            gbs, tf = nbytes / us / 1e3, flops / us / 1e6
            hbm, mfma = gbs / HBM_PEAK_GBS, tf / MFMA_FP16_PEAK_TFLOPS
            # what binds: memory up to 16 rows, the matrix cores beyond (ridge: 312 flop per byte)
            bound = "hbm" if flops / nbytes < MFMA_FP16_PEAK_TFLOPS * 1e3 / HBM_PEAK_GBS else "mfma"
            rows.append({"config": cfg, "op": op, "M": m, "us": round(us, 2), "bytes": nbytes, "flops": flops, "GBps": round(gbs, 1),
                         "TFLOPs": round(tf, 2), "bound": bound, "frac": round(hbm if bound == "hbm" else mfma, 4),
                         "frac_hbm": round(hbm, 4), "frac_mfma": round(mfma, 4)})
            log(f"  {cfg} {op:28s} M={m:<5d} {us:9.2f} us  {gbs:8.0f} GB/s  {tf:8.1f} TFLOP/s  {bound} {rows[-1]['frac']:.3f}")

        # C1: one QuantLinear 4096 -> 4096, one group (groupsize -1), M in {1, 128}; 40 weight sets = 336 MB
        c1 = [make(HIDDEN, HIDDEN, -1) for _ in range(40)]
        w1 = weight_bytes(HIDDEN, HIDDEN, HIDDEN)
        for m in (1, 128):
            xm = torch.randn((m, HIDDEN), device=dev, generator=gen).half()
            config_row("C1", "QuantLinear 4096x4096 g=-1", m, lambda w: G.matmul4(HIDDEN, xm, w[0], w[2], w[1]), c1,
                       w1 + 4 * m * HIDDEN, 2 * m * HIDDEN * HIDDEN)
        c1s = [G.stream_pack(w[0], w[1], w[2], HIDDEN) for w in c1]
        xm = torch.randn((1, HIDDEN), device=dev, generator=gen).half()
        config_row("C1", "QuantLinear 4096x4096 g=-1, streaming order", 1, lambda w: G.matmul4_stream(HIDDEN, xm, w[0], w[1]), c1s,
                   w1 + 4 * HIDDEN, 2 * HIDDEN * HIDDEN)
        del c1, c1s
        # C2: the fused MLP module, gate/up + SiLU*mul then down, groupsize 128, M in {1, 16, 512}
        for m in (1, 16, 512):
            xm = torch.randn((m, HIDDEN), device=dev, generator=gen).half()
            config_row("C2", "MLP gate/up+silu*mul, down g=128", m, lambda L: down_op(gateup_op(xm, L), L), layers,
                       2 * wg + wd + 4 * m * HIDDEN + 4 * m * INTER, 6 * m * HIDDEN * INTER, reps=5)
        for m in (1, 16):
            xm = torch.randn((m, HIDDEN), device=dev, generator=gen).half()
            config_row("C2", "MLP gate/up+silu*mul, down g=128, streaming order", m, lambda L: s_down_op(s_gateup_op(xm, L), L), layers,
                       2 * wg + wd + 4 * m * HIDDEN + 4 * m * INTER, 6 * m * HIDDEN * INTER, reps=5)
        # C3: fused QKV + rotary 4096 -> 12288, one group, M = 1 at position 2047 and a 2048-token prefill
        c3 = [make(HIDDEN, 3 * HIDDEN, -1) for _ in range(12)]
        w3 = weight_bytes(HIDDEN, 3 * HIDDEN, HIDDEN)
        pos2047 = torch.tensor([[2047]], device=dev, dtype=torch.int32)
        x1r = torch.randn((1, 1, HIDDEN), device=dev, generator=gen).half()
        config_row("C3", "QKV+rotary 4096x12288 g=-1", 1, lambda w: G.qkv_rotary(HIDDEN, x1r, w[0], w[2], w[1], pos2047, cos, sin, HEADS), c3,
                   w3 + 2 * HIDDEN + 6 * HIDDEN, 2 * HIDDEN * 3 * HIDDEN)
        c3s = [G.stream_pack(w[0], w[1], w[2], HIDDEN) for w in c3]
        config_row("C3", "QKV+rotary 4096x12288 g=-1, streaming order", 1, lambda w: G.qkv_rotary_stream(HIDDEN, x1r, w[0], w[1], pos2047, cos, sin, HEADS), c3s,
                   w3 + 2 * HIDDEN + 6 * HIDDEN, 2 * HIDDEN * 3 * HIDDEN)
        del c3s
        xp = torch.randn((1, 2048, HIDDEN), device=dev, generator=gen).half()
        posp = torch.arange(2048, device=dev, dtype=torch.int32).unsqueeze(0)
        config_row("C3", "QKV+rotary 4096x12288 g=-1", 2048, lambda w: G.qkv_rotary(HIDDEN, xp, w[0], w[2], w[1], posp, cos, sin, HEADS), c3[:4],
                   w3 + 2 * 2048 * HIDDEN + 6 * 2048 * HIDDEN, 2 * 2048 * HIDDEN * 3 * HIDDEN, reps=5)
        del c3, xp
        extra["baseline_configs"] = rows

        # Yardstick: the vendor library's DENSE fp16 GEMM (torch) on the same shapes at 128, 512 and 2048 rows,
        # weights already dequantised, in the faster of its two weight layouts ([K, N] and [N, K]), 20 calls
        # replayed from one graph.  It does no 4-bit decode, no fused epilogue and reads 4x the weight bytes; it
        # shows what a tuned kernel sustains on this chip at these shapes.
        def dense(shape, k, n, m, reps=20):
            a = torch.randn((m, k), device=dev, generator=gen).half()
            w = (torch.randn((k, n), device=dev, generator=gen) * 0.02).half()
            wt = w.t().contiguous()
            best = None
            for fn in (lambda: torch.matmul(a, w), lambda: torch.nn.functional.linear(a, wt)):
                for _ in range(3):
                    fn()
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    for _ in range(reps):
                        fn()
                g.replay()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(3):
                    g.replay()
                e1.record()
                torch.cuda.synchronize()
                us = e0.elapsed_time(e1) * 1e3 / (3 * reps)
                best = us if best is None else min(best, us)
                del g
            name = f"dense fp16 library M={m} {shape} shape"
            extra[name] = {"us": round(best, 2), "TFLOPs": round(2.0 * m * k * n / best / 1e6, 2)}
            log(f"  {name:34s} {best:9.2f} us  {'':8s}       {2.0 * m * k * n / best / 1e6:8.1f} TFLOP/s")
        for m in (128, 512, 2048):
            dense("qkv", HIDDEN, 3 * HIDDEN, m)
            dense("gate+up", HIDDEN, 2 * INTER, m)
            dense("down", INTER, HIDDEN, m)
            dense("o_proj", HIDDEN, HIDDEN, m)
        best_prefill = max(v["TFLOPs"] for k, v in extra.items() if k.startswith("M=2048"))
        extra["prefill_best_TFLOPs"] = best_prefill
        extra["prefill_frac_of_fp16_mfma_peak"] = round(best_prefill / MFMA_FP16_PEAK_TFLOPS, 4)

    L0 = None if args.no_cpu else {k: tuple(t.cpu() for t in v) for k, v in layers[0].items() if not k.startswith("s_")}
    # ------------------------------------------------- the headline: the whole 7B decoder, then C4 / C5 (prefill + greedy decode)
    del layers, step_graph, gu_graph
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    head = decoder_figures("llama7b", 1, 2048, None, steps=args.steps, warmup=args.warmup)
    extra["llama7b_b1"] = {"prefill_ms": head["extra"]["prefill_ms"], "prefill_linear_TFLOPs": head["extra"]["prefill_linear_TFLOPs"],
                           "eager_decode_ms_per_step": head["extra"]["eager_decode_ms_per_step"],
                           "step_GBps": head["roofline"]["achieved"], "step_frac_hbm": head["roofline"]["frac"],
                           "prefill_path_agrees_with_decode_path_on_next_tokens":
                               head["extra"]["prefill_path_agrees_with_decode_path_on_next_tokens"]}
    if not args.no_extra and not args.no_decoders:
        decs = {}
        for name, bsz in (("llama13b", 1), ("llama30b", 1), ("llama30b", 8)):
            try:
                r = decoder_figures(name, bsz, 2048, 128 if name != "llama30b" else 256)
            except Exception as e:  # report, do not lose the line
                decs[f"{name}_b{bsz}"] = {"error": repr(e)}
                continue
            decs[f"{name}_b{bsz}"] = {"tok_s": r["value"], "ms_per_step": r["ms_per_step"], "prefill_ms": r["extra"]["prefill_ms"],
                                      "prefill_linear_TFLOPs": r["extra"]["prefill_linear_TFLOPs"],
                                      "step_GBps": r["roofline"]["achieved"], "step_frac_hbm": r["roofline"]["frac"],
                                      "prefill_path_agrees_with_decode_path_on_next_tokens":
                                          r["extra"]["prefill_path_agrees_with_decode_path_on_next_tokens"],
                                      "workload": r["config"]["workload"]}
        extra["decoders"] = decs

    # --------------------------------------------------------------------- CPU baseline
    cpu_baseline = None
    if not args.no_cpu:
        from oracle import torch_cpu as T
        xc = x1.cpu().view(1, HIDDEN)
        torch.set_grad_enabled(False)
        REPS = 5

        def median_s(fn):
            fn()
            ts = []
            for _ in range(REPS):
                t0 = time.perf_counter()
                fn()
                ts.append(time.perf_counter() - t0)
            return statistics.median(ts)

        # (a) what the reference-style path costs per call: dequantise, then a float32 matmul
        def cpu_layer():
            T.quant_matmul(xc, *L0["qkv"], GROUPSIZE)
            T.quant_matmul(xc, *L0["o"], GROUPSIZE)
            T.mlp(xc, L0["gate"], L0["up"], L0["down"], GROUPSIZE)

        t_layer = median_s(cpu_layer)
        # (b) the matmuls alone, on weights dequantised beforehand
        W = {k: T.dequant_fp16(*v, GROUPSIZE).float() for k, v in L0.items()}
        xf = xc.float()

        def cpu_layer_matmul_only():
            xf @ W["qkv"]
            xf @ W["o"]
            h = (torch.nn.functional.silu(xf @ W["gate"]) * (xf @ W["up"])).half().float()
            h @ W["down"]

        t_mm = median_s(cpu_layer_matmul_only)
        # C1 as stated: one 4096 x 4096 layer, M = 1 and 128 (the o_proj tensors have that shape)
        c1 = {}
        for m in (1, 128):
            xm = torch.randn((m, HIDDEN)).half()
            c1[f"M={m}"] = {"dequant+matmul_ms": round(median_s(lambda: T.quant_matmul(xm, *L0["o"], GROUPSIZE)) * 1e3, 2),
                            "matmul_only_ms": round(median_s(lambda: xm.float() @ W["o"]) * 1e3, 3)}
        del W
        cpu_baseline = {"value": round(1.0 / (t_layer * LAYERS), 4), "unit": "tok/s", "cores": torch.get_num_threads(),
                        "kind": "port",
                        "sample": f"1 of {LAYERS} layers (qkv, o_proj, gate/up+silu*mul, down at M=1; dequantise + fp32 "
                                  f"matmul per call), median of {REPS} runs = {t_layer:.3f} s, extrapolated x{LAYERS}; "
                                  f"torch threads {torch.get_num_threads()}, host has {os.cpu_count()} logical CPUs",
                        "matmul_only_value": round(1.0 / (t_mm * LAYERS), 3), "matmul_only_layer_s": round(t_mm, 4),
                        "quantlinear_4096x4096": c1}
        log(f"cpu baseline: {t_layer:.3f} s per layer dequantise + matmul, {t_mm:.4f} s matmul alone, on {torch.get_num_threads()} threads")

    roofline["decoder_step_frac"] = head["roofline"]["frac"]
    roofline["decoder_step_GBps"] = head["roofline"]["achieved"]
    result = {
        "metric": "LLaMA-7B-shape 4-bit decode tok/s", "value": head["value"], "unit": "tok/s", "n_gpus": 1,
        "steps": head["steps"], "warmup": head["warmup"], "ms_per_step": head["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "fp16", "data": "synthetic",
        "config": {"workload": head["config"]["workload"], "hidden": HIDDEN, "intermediate": INTER, "layers": LAYERS,
                   "groupsize": GROUPSIZE, "weight_bytes_per_token": LAYERS * layer_bytes,
                   "bytes_per_token": head["roofline"]["bytes_per_launch"]},
        # the step with nothing but its 128 quantised-linear launches (no attention, norms, lm_head): the hot path alone
        "linears_only": {"tok_s": round(tok_s, 2), "ms_per_step": round(ms_per_step, 5), "steps": args.steps, "warmup": args.warmup,
                         "workload": "32 layers x [fused qkv+rotary, o_proj, fused gate/up+silu*mul, down_proj] at batch 1, position 2047, "
                                     "streaming-order weights, one HIP-graph replay per token"},
        "roofline": roofline, "cpu_baseline": cpu_baseline, "extra": extra,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
