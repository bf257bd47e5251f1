#!/usr/bin/env python3
"""Benchmark of the quantized attention path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input, inputs resident in HBM:
  prefill (the headline `value`): the 1.5B-style configuration, the largest prefill shape of the five -- batch 8,
      seq 4096, 16 heads, head_dim 128, e4m3 Q/K/V with per-row fp32 scales, layers alternating (window 256, slope 0.5)
      and (full causal window, slope 0) -- one step = one pair of such layers (two launches, 616.19 GFLOP), each layer
      on its own Q/K/V buffers.
  "prefill_125M_style": batch 16, seq 1024, 12 heads x 64, e4m3, 12 layers alternating window 64 / full -- one pass
      of 12 launches.
  "decode": batch 64, one bf16 query per sequence, int8 KV cache of 4096 rows, 16 heads x 128, per-row scales; one
      step = one decode launch, rotating over 4 caches so that no launch finds its cache in the Infinity Cache.
  "generation_1p5B_style": the attention calls of the random-init 1.5B-style generation run at their shapes (24 layers
      on the InitAlibi schedule, int8, batch 32, 2048-token prompt, 256 generated tokens).
  "cpu_reference_config": batch 1, seq 1024, 12 heads x 64, int8, full causal window, fp32 output: the shape the
      reference's CPU path is quoted on; the CPU leg of it runs on int8, as that configuration says.
  "prefill_long_span": the two prefill kernels side by side on full-window layers of 32768 tokens at S = 4096, 8192, 16384.
  "token_step_24_layers", "prompt_pass_24_layers": the whole 24-layer stack of the host mirror around those attention
      calls (int8 projections, producer, attention, feed-forward), one generated token and one prompt pass.
  "prompt_then_generate_256": the last configuration end to end in one timed region (embedding, 24 int8 layers, final
      layer, greedy choice): 32 prompts of 2048 tokens, then 256 generated tokens each.
Algorithmic work: FLOPs = 4*d*sum_rows min(row, W) per (sequence, head) (masked tiles count zero,
the zero vector adds none); decode bytes = K + V planes + both scale planes + q + out.

Prints ONE JSON line.  `--gpus N` with N > 1 is refused: this build uses one GPU.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0  # MI355X dense fp8 MFMA
PEAK_I8_TOPS = 5000.0
PEAK_HBM_GBPS = 8000.0



def profile_facts():
    """HBM bytes per launch and matrix-pipe utilisation as rocprofv3 measured them (profiles/*.md: FETCH_SIZE and
    WRITE_SIZE in KiB per dispatch scaled by what the same counters read for a copy of known size; MfmaUtil).  Each
    summary carries its figures once more as a `<!-- facts {...} -->` line together with the first 16 hex digits of the
    sha256 of the kernel source they were measured on; figures of a source that has changed since are not reported."""
    import glob
    import hashlib
    import re
    out = {}
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.md"))):
        for m in re.finditer(r"<!-- facts (.*?) -->", open(path).read()):
            try:
                f = json.loads(m.group(1))
                src = os.path.join(ROOT, "tscale_amd", "csrc", f["source"])
                if hashlib.sha256(open(src, "rb").read()).hexdigest()[:16] != f["source_sha16"]:
                    continue
                for k, v in f["launches"].items():
                    out[k] = dict(v, profile=os.path.basename(path))
            except (KeyError, ValueError, OSError):
                continue
    return out


def roofline(kernel, bound, achieved, flops_or_bytes, launch_ms, fact):
    peak, unit = (PEAK_FP8_TFLOPS, "TFLOP/s") if bound == "mfma" else (PEAK_HBM_GBPS, "GB/s")
    r = {"kernel": kernel, "bound": bound, "achieved": round(achieved, 3), "peak": peak, "unit": unit,
         "frac": round(achieved / peak, 5), "traffic": None, "launch_ms": round(launch_ms, 5)}
    if bound == "mfma":
        # half of the algorithmic FLOPs (P.V) run as f16 matrix instructions at half the fp8 rate: the matrix pipes are
        # full at 2/3 of `peak`
        r["frac_of_executed_mfma_peak"] = round(achieved / (peak * 2.0 / 3.0), 5)
    r["flops_per_launch" if bound == "mfma" else "bytes_per_launch"] = flops_or_bytes
    if fact:
        r["traffic"] = fact.get("traffic_bytes")
        if "mfma_util" in fact:
            r["mfma_util"] = fact["mfma_util"]
        r["traffic_from"] = fact["profile"]
    return r


def pairs(S, W):
    """sum over rows of min(row, W): (query, key) pairs of one sequence and head."""
    W = min(W, S)
    return W * (W - 1) // 2 + (S - W) * W


def prefill_flops(B, S, H, d, W):
    return 4.0 * d * pairs(S, W) * B * H


def layer_schedule(n_layers, wide, short):
    return [(short, 0.5) if i % 2 == 0 else (wide, 0.0) for i in range(n_layers)]


def gpu_time_ms(fn, steps, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def graph_time_ms(fn, calls, replays):
    """Average GPU time of one call of fn, from a HIP graph of `calls` calls replayed `replays` times: for launches short
    enough that the host's call overhead would otherwise be what is timed."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(calls):
            fn()
    torch.cuda.synchronize()
    return gpu_time_ms(graph.replay, replays, 1) / calls


class PrefillWorkload:
    def __init__(self, ctx, dtype, B, S, H, d, n_layers, seed, short=64):
        import torch
        self.ctx, self.dtype, self.B, self.S, self.H, self.d = ctx, dtype, B, S, H, d
        self.layers = layer_schedule(n_layers, S, short)
        n = B * S
        g = torch.Generator(device="cuda").manual_seed(seed)
        self.inputs = []
        for _ in range(n_layers):
            qkv = []
            for _ in range(3):
                x = torch.randn((n, H * d), device="cuda", generator=g)
                qkv.append(ctx.quantize_rows(x, H, dtype))
                del x
            self.inputs.append(qkv)
        off = torch.arange(0, n + 1, S, dtype=torch.int32, device="cuda")
        self.spans = {W: ctx.build_spans(off, n, W) for W in {w for w, _ in self.layers}}
        self.span_tiles = {W: ctx.build_span_tiles(*sp) for W, sp in self.spans.items()}   # once per batch and mask
        self.out = torch.empty((n, H * d), dtype=torch.float16, device="cuda")
        self.flops_layer = [prefill_flops(B, S, H, d, W) for W, _ in self.layers]
        self.flops = sum(self.flops_layer)
        self.mean_qs = [float(inp[0][1].mean()) for inp in self.inputs]
        self.mean_vs = [float(inp[2][1].mean()) for inp in self.inputs]
        torch.cuda.synchronize()

    def run_layer(self, i, span_len_hint=None, const_q_scale=False, const_v_scale=False):
        (q, qs), (k, ks), (v, vs) = self.inputs[i]
        if const_q_scale:   # one number as the query scale, as TScale's own model passes (gpt_att_fp8.cuh:137); of the planes' size
            qs = self.mean_qs[i]
        if const_v_scale:   # ... and as the value scale (cpu_infer.cpp:454)
            vs = self.mean_vs[i]
        W, slope = self.layers[i]
        st, fi = self.spans[W]
        # equal-length sequences: tell the library the causal period of the wide layers (a launch-order hint)
        # (and the layer's attention width: with long spans the library takes its workspace kernel)
        self.ctx.compute_val_lookup(self.dtype, self.H, q, k, v, qs, ks, vs, st, fi, slope, out=self.out,
                                    causal_period=self.S if W >= self.S else 0, span_tiles=self.span_tiles[W],
                                    span_len_hint=min(W, self.S) if span_len_hint is None else span_len_hint)

    def step(self):
        for i in range(len(self.layers)):
            self.run_layer(i)


class DecodeWorkload:
    def __init__(self, ctx, B, L, H, d, n_caches, seed):
        import torch
        from tscale_amd import KVCache, capi
        self.ctx, self.B, self.L, self.H, self.d = ctx, B, L, H, d
        g = torch.Generator(device="cuda").manual_seed(seed)
        self.caches = []
        for _ in range(n_caches):
            c = KVCache(ctx, capi.I8, B, H, L, d)
            for plane, scale in ((c.k, c.k_scale), (c.v, c.v_scale)):
                for b0 in range(0, B, 8):  # bounded temporaries
                    x = torch.randn((8 * H * L, d), device="cuda", generator=g)
                    q8, s = ctx.quantize_rows(x, 1, capi.I8)
                    plane[b0:b0 + 8].copy_(q8.view(8, H, L, d))
                    scale[b0:b0 + 8].copy_(s.view(8, H, L))
                    del x, q8, s
            c.cache_len.fill_(L)
            self.caches.append(c)
        self.q = torch.randn((B, H * d), device="cuda", generator=g).to(torch.bfloat16)
        self.out = torch.empty((B, H * d), dtype=torch.float32, device="cuda")
        self.i = 0
        # K + V planes, two scale planes, bf16 q, f32 out
        self.bytes = 2 * B * H * L * d + 2 * B * H * L * 4 + B * H * d * 2 + B * H * d * 4
        torch.cuda.synchronize()

    def step(self):
        c = self.caches[self.i % len(self.caches)]
        self.i += 1
        self.ctx.compute_val_lookup_decode(c, self.q, None, 10 ** 6, 0.0, out=self.out)


class GenerationWorkload:
    """Attention share of the 1.5B-style greedy-decode configuration: 24 layers (InitAlibi's schedule: 4 of
    width 1, 10 of width 64 with slope 0.5, 10 full), 16 heads x 128, int8 Q/K/V with per-row scales, batch 32,
    a 2048-token prompt, then 256 generated tokens.  Per layer: prefill over the prompt, the prompt's K/V rows
    moved into that layer's KV cache, and per generated token one append + one decode launch pair.  The
    projections, FFN and sampling of the model are not part of this path; the new tokens' Q/K/V are synthetic."""

    def __init__(self, ctx, B=32, prompt=2048, n_new=256, H=16, d=128, depth=24, seed=1313 + 5):
        import torch
        from tscale_amd import KVCache, capi
        from tscale_amd.attention import alibi_layer_schedule
        self.ctx, self.B, self.prompt, self.n_new, self.H, self.d = ctx, B, prompt, n_new, H, d
        self.L = prompt + n_new
        self.i8 = capi.I8
        self.sched = alibi_layer_schedule(depth, self.L)
        n = B * prompt
        g = torch.Generator(device="cuda").manual_seed(seed)
        self.qkv = [ctx.quantize_rows(torch.randn((n, H * d), device="cuda", generator=g), H, capi.I8) for _ in range(3)]
        self.off = torch.arange(0, n + 1, prompt, dtype=torch.int32, device="cuda")
        self.spans = {W: ctx.build_spans(self.off, n, W) for W in {w for w, _ in self.sched}}
        self.span_tiles = {W: ctx.build_span_tiles(*sp) for W, sp in self.spans.items()}
        self.out = torch.empty((n, H * d), dtype=torch.float16, device="cuda")
        self.caches = [KVCache(ctx, capi.I8, B, H, self.L, d) for _ in range(depth)]
        new = [ctx.quantize_rows(torch.randn((B, H * d), device="cuda", generator=g), H, capi.I8) for _ in range(3)]
        self.new = [(x, s.t().contiguous()) for x, s in new]     # scales as [B, H]
        self.dout = torch.empty((B, H * d), dtype=torch.float32, device="cuda")
        self.kinds = sorted({w for w, _ in self.sched})
        self.mean_qs = float(self.qkv[0][1].mean())
        self.mean_vs = float(self.qkv[2][1].mean())
        torch.cuda.synchronize()

    def prefill_layer(self, i, const_q_scale=False):
        (q, qs), (k, ks), (v, vs) = self.qkv
        if const_q_scale:   # one number as the query scale and one as the value scale, as the reference's own layer passes (cpu_infer.cpp:448,454)
            qs, vs = self.mean_qs, self.mean_vs
        W, slope = self.sched[i]
        st, fi = self.spans[W]
        self.ctx.compute_val_lookup(self.i8, self.H, q, k, v, qs, ks, vs, st, fi, slope, out=self.out,
                                    causal_period=self.prompt if W >= self.prompt else 0, span_tiles=self.span_tiles[W],
                                    span_len_hint=min(W, self.prompt))

    def fill_caches(self):
        (_, _), (k, ks), (v, vs) = self.qkv
        for c in self.caches:
            c.cache_len.zero_()
            c.fill_from_prefill(self.off, k, ks, v, vs)

    def decode_step(self):
        (q, qs), (k, ks), (v, vs) = self.new
        for c, (W, slope) in zip(self.caches, self.sched):
            # append fused into the decode launches (two kernels per layer and token instead of four)
            self.ctx.compute_val_lookup_decode(c, q, qs, W, slope, out=self.dout, append=(k, ks, v, vs))

    def prefill_flops(self, i):
        return prefill_flops(self.B, self.prompt, self.H, self.d, self.sched[i][0])

    def decode_bytes(self):
        """Cache rows each generated token reads (K + V rows and their two scales), its q and its output."""
        total = 0
        for t in range(self.n_new):
            n = self.prompt + t + 1
            for W, _ in self.sched:
                rows = min(n - 1, W)
                total += self.B * self.H * (rows * (2 * self.d + 8) + self.d + 4 + 4 * self.d)
        return total


def bench_generation(ctx, steps, facts=None):
    import torch
    facts = facts or {}
    gw = GenerationWorkload(ctx)
    res = {"config": "24 layers (4 x W=1, 10 x W=64 slope 0.5, 10 x full), B32, prompt 2048 + 256 generated tokens, "
                     "H16 d128 int8 Q/K/V + per-row f32 scales; attention launches only"}
    first = {W: [i for i, (w, _) in enumerate(gw.sched) if w == W][0] for W in gw.kinds}
    pre_ms = {W: gpu_time_ms(lambda i=i: gw.prefill_layer(i), max(50 if W == max(gw.kinds) else 10, steps // 5), 1) for W, i in first.items()}
    total_ms = sum(pre_ms[w] for w, _ in gw.sched)
    total_flops = sum(gw.prefill_flops(i) for i in range(len(gw.sched)))
    wide = max(gw.kinds)
    res["prefill"] = {"layer_ms": {f"W={w}": round(t, 5) for w, t in pre_ms.items()},
                      "pass_ms": round(total_ms, 4), "TOP/s": round(total_flops / total_ms / 1e9, 2),
                      "full_layer_TOP/s": round(gw.prefill_flops(first[wide]) / pre_ms[wide] / 1e9, 2),
                      "full_layer_frac_of_int8_peak": round(gw.prefill_flops(first[wide]) / pre_ms[wide] / 1e9 / PEAK_I8_TOPS, 5),
                      "roofline": {"kernel": "prefill_kernel<int8, d128>, full causal window over the prompt", "bound": "mfma",
                                   "achieved": round(gw.prefill_flops(first[wide]) / pre_ms[wide] / 1e9, 2), "peak": PEAK_I8_TOPS,
                                   "unit": "TOP/s", "frac": round(gw.prefill_flops(first[wide]) / pre_ms[wide] / 1e9 / PEAK_I8_TOPS, 5),
                                   "traffic": None, "launch_ms": round(pre_ms[wide], 5), "flops_per_launch": gw.prefill_flops(first[wide])}}
    cq_ms = gpu_time_ms(lambda: gw.prefill_layer(first[wide], const_q_scale=True), max(50, steps // 5), 1)
    res["prefill"]["full_layer_ms_with_constant_query_and_value_scales"] = round(cq_ms, 5)
    fact = facts.get("prefill_prompt_int8_full")
    if fact:
        res["prefill"]["roofline"].update({"traffic": fact.get("traffic_bytes"), "traffic_from": fact["profile"]})
        if "mfma_util" in fact:
            res["prefill"]["roofline"]["mfma_util"] = fact["mfma_util"]
    fill_ms = gpu_time_ms(gw.fill_caches, 2, 1)
    n = gw.B * gw.prompt
    fill_bytes = len(gw.caches) * 2 * (n * gw.H * gw.d * 2 + n * gw.H * 4 * 2)   # read + write of K, V and both scales
    res["cache_fill"] = {"ms_24_layers": round(fill_ms, 4), "GB/s": round(fill_bytes / fill_ms / 1e6, 1)}
    # generation: one captured step (24 x (append + decode pair)) replayed once per generated token
    gw.fill_caches()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        gw.decode_step()                       # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    gw.fill_caches()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gw.decode_step()
    gw.fill_caches()                           # capture does not run the step
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(gw.n_new):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    gen_ms = e0.elapsed_time(e1)
    lens = {int(c.cache_len[0]) for c in gw.caches}
    assert lens == {gw.L}, lens
    nbytes = gw.decode_bytes()
    res["generate"] = {"ms_256_tokens": round(gen_ms, 3), "ms_per_token": round(gen_ms / gw.n_new, 4),
                       "us_per_layer_step": round(gen_ms / gw.n_new / len(gw.sched) * 1e3, 2),
                       "GB/s": round(nbytes / gen_ms / 1e6, 1), "frac_of_hbm_peak": round(nbytes / gen_ms / 1e6 / PEAK_HBM_GBPS, 4),
                       "bytes": nbytes, "launch": "HIP graph of one step (24 x decode with fused append), replayed per token",
                       "roofline": {"kernel": "decode_split_kernel<int8, d128> with fused append, 24 launches per token (one split each: no merge)",
                                    "bound": "hbm", "achieved": round(nbytes / gen_ms / 1e6, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                                    "frac": round(nbytes / gen_ms / 1e6 / PEAK_HBM_GBPS, 4), "traffic": None,
                                    "bytes_per_token": nbytes // gw.n_new}}
    fact = facts.get("decode_fused_append_token")
    if fact:   # (measured over the 24 launches of the token whose caches hold 2048 + 128 rows: the middle of the run)
        res["generate"]["roofline"].update({"traffic": fact.get("traffic_bytes"), "traffic_from": fact["profile"]})
    return res


def bench_long_span(ctx, steps, facts=None):
    """The launch-time choice between the two prefill kernels (span_len_hint in the arguments): a full-window e4m3 layer of
    32768 tokens, 16 heads x 128, at three sequence lengths, once with no hint (the standard kernel, which stages K and V
    through its waves) and once with a hint of at least TSATTN_PREFILL_LONG_SPAN (the long-span kernel: K and V'^T by DMA
    into LDS, its time includes the kernel that writes V'^T into the workspace)."""
    import torch
    from tscale_amd import capi
    res = {"config": "32768 tokens, H16 d128 e4m3 + per-row f32 scales, full causal window, f16 out; ms per launch and TFLOP/s",
           "threshold": capi.PREFILL_LONG_SPAN}
    for B, S in ((8, 4096), (4, 8192), (2, 16384)):
        wl = PrefillWorkload(ctx, capi.E4M3, B, S, 16, 128, 2, seed=1313 + 6, short=256)
        n = max(50, steps)
        std, lng = [], []
        for _ in range(2):   # alternating, so that both see the same state of the clocks; the better of two
            std.append(gpu_time_ms(lambda: wl.run_layer(1, span_len_hint=0), n, 5))
            lng.append(gpu_time_ms(lambda: wl.run_layer(1, span_len_hint=max(S, capi.PREFILL_LONG_SPAN)), n, 5))
        std, lng = min(std), min(lng)
        res[f"B{B}_S{S}"] = {"standard_ms": round(std, 5), "long_span_ms": round(lng, 5),
                             "standard_TFLOP/s": round(wl.flops_layer[1] / std / 1e9, 1), "long_span_TFLOP/s": round(wl.flops_layer[1] / lng / 1e9, 1),
                             "library_picks": "long-span" if S >= capi.PREFILL_LONG_SPAN else "standard"}
        if S == 8192:
            res[f"B{B}_S{S}"]["roofline"] = roofline("prefill_long_kernel<e4m3, d128> + widen_v_kernel, full causal window", "mfma",
                                                     wl.flops_layer[1] / lng / 1e9, wl.flops_layer[1], lng, (facts or {}).get("prefill_long_s8192"))
        del wl
        torch.cuda.empty_cache()
    return res


def bench_producer(ctx, steps):
    """RoPE + per-head RMS normalisation + int8 conversion of one projection result of the 1.5B-style prompt
    (B32 x 2048 rows, 16 heads x 128, f32 in): bytes = 4 in + 1 out per element, the rope row, the scales."""
    import torch
    from tscale_amd import capi
    n, H, d = 32 * 2048, 16, 128
    x = torch.randn((n, H * d), device="cuda", generator=torch.Generator(device="cuda").manual_seed(1313 + 6))
    pos = (torch.arange(n, device="cuda", dtype=torch.int32) % 2048).contiguous()
    rope = ctx.fill_rope_table(d, 2048)
    ms = graph_time_ms(lambda: ctx.rope_normalize_rows(x, H, capi.I8, pos=pos, rope=rope), 10, max(3, steps // 10))
    nbytes = n * H * d * 5 + n * H * 4 + n * 4 + n * d * 4
    return {"config": "rope_normalize_rows: 65536 rows x 16 heads x 128, f32 -> int8 + f32 scale per (row, head), with RoPE",
            "ms": round(ms, 4), "GB/s": round(nbytes / ms / 1e6, 1), "frac_of_hbm_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBPS, 4),
            "bytes": nbytes}


def bench_kv_product(ctx, steps):
    """KVProduct on the decode output of the 1.5B-style prompt batch: int8 k + f32 attention output -> 4 x int8."""
    import torch
    n, H, d = 32 * 2048, 16, 128
    g = torch.Generator(device="cuda").manual_seed(1313 + 7)
    k = torch.randint(0, 256, (n, H * d), dtype=torch.uint8, device="cuda", generator=g)
    val = torch.randn((n, H * d), device="cuda", generator=g) * 0.3
    ms = graph_time_ms(lambda: ctx.kv_product(k, val, H), 10, max(3, steps // 10))
    nbytes = n * H * d * (1 + 4 + 4)
    return {"config": "kv_product: 65536 rows x 16 heads x 128, int8 k x f32 value -> 4 x int8", "ms": round(ms, 4),
            "GB/s": round(nbytes / ms / 1e6, 1), "frac_of_hbm_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBPS, 4), "bytes": nbytes}


def bench_matmul(ctx, steps):
    """The combiner product of the 1.5B-style configuration (kv [rows][16 heads x 128 x 4] int8 times the combiner
    matrix [2048][8192] int8, added to the f32 state): once for the prompt batch (32 x 2048 rows: matrix cores),
    once for one generated token per sequence (32 rows: each layer's matrix is read from HBM once per token; 24
    layers' matrices in turn, launched as one HIP graph like the generation loop)."""
    import torch
    from tscale_amd import capi
    k, n, depth = 16 * 128 * 4, 2048, 24
    g = torch.Generator(device="cuda").manual_seed(1313 + 8)
    ws = [torch.randint(0, 256, (n, k), dtype=torch.uint8, device="cuda", generator=g) for _ in range(depth)]
    res = {"config": "combiner: int8 [rows][8192] x int8 [2048][8192]^T, f32 state += sums * scale"}
    m = 32 * 2048
    a = torch.randint(0, 256, (m, k), dtype=torch.uint8, device="cuda", generator=g)
    state = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    ms = gpu_time_ms(lambda: ctx.matmul_i8(a, ws[0], mode=capi.MM_ADD_SCALED, scale=1e-6, out=state), max(3, steps // 10), 2)
    ops = 2.0 * m * n * k
    res["prompt"] = {"rows": m, "ms": round(ms, 4), "TOP/s": round(ops / ms / 1e9, 2), "frac_of_int8_peak": round(ops / ms / 1e9 / PEAK_I8_TOPS, 4)}
    del a, state
    # a square product with an int32 result: the kernel without the state update
    m2 = 8192
    a = torch.randint(0, 256, (m2, k), dtype=torch.uint8, device="cuda", generator=g)
    w2 = torch.randint(0, 256, (m2, k), dtype=torch.uint8, device="cuda", generator=g)
    out = torch.empty((m2, m2), dtype=torch.int32, device="cuda")
    ms = gpu_time_ms(lambda: ctx.matmul_i8(a, w2, out=out), max(3, steps // 10), 2)
    res["square_8192"] = {"ms": round(ms, 4), "TOP/s": round(2.0 * m2 * m2 * k / ms / 1e9, 2),
                          "frac_of_int8_peak": round(2.0 * m2 * m2 * k / ms / 1e9 / PEAK_I8_TOPS, 4)}
    del a, w2, out
    # the four projections of the prompt batch as one product with the producer as its epilogue: RoPE on the qk and
    # qv heads, per-head normalisation, int8 rows and the key scales; the int32 sums are never stored
    m, kp, npj, H = 32 * 2048, 2048, 4 * 16 * 128, 16
    a = torch.randint(0, 256, (m, kp), dtype=torch.uint8, device="cuda", generator=g)
    wp = torch.randint(0, 256, (npj, kp), dtype=torch.uint8, device="cuda", generator=g)
    rope = ctx.fill_rope_table(128, 2048)
    pos = torch.arange(2048, dtype=torch.int32, device="cuda").repeat(32)
    scratch = torch.empty(m * npj, dtype=torch.int32, device="cuda")
    ms = gpu_time_ms(lambda: ctx.matmul_normalize(a, wp, 4 * H, capi.I8, scratch, pos=pos, rope=rope, scale_mult=0.01, rope_heads=2 * H,
                                                  scale_heads=(H, H)), max(3, steps // 10), 2)
    res["prompt_projections_with_producer"] = {"rows": m, "k": kp, "n": npj, "ms": round(ms, 4), "TOP/s": round(2.0 * m * npj * kp / ms / 1e9, 2),
                                               "frac_of_int8_peak": round(2.0 * m * npj * kp / ms / 1e9 / PEAK_I8_TOPS, 4)}
    del a, wp, scratch
    m = 32
    a = torch.randint(0, 256, (m, k), dtype=torch.uint8, device="cuda", generator=g)
    state = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    room = torch.empty(16 * 4 * m * n, dtype=torch.uint8, device="cuda")   # split-K partial sums
    def step():
        for w in ws:
            ctx.matmul_i8(a, w, mode=capi.MM_ADD_SCALED, scale=1e-6, out=state, workspace=room)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    ms = gpu_time_ms(graph.replay, steps, 2) / depth
    nbytes = m * k + n * k + 2 * m * n * 4
    res["token"] = {"rows": m, "us_per_layer": round(ms * 1e3, 2), "GB/s": round(nbytes / ms / 1e6, 1),
                    "frac_of_hbm_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBPS, 4), "bytes": nbytes,
                    "launch": "HIP graph of 24 layers' products, K split with a workspace"}
    return res


class Int8Layers:
    """24 layers of the int8 inference path (AddLookupProduct, gpt/train/cpu_infer.cpp:465-527) at the 1.5B-style
    attention shape: model width 2048, 16 heads x 128, feed-forward width 2048, per-layer attention width and slope
    from InitAlibi's schedule (tscale_amd/host/model_init.cpp), weights as the reference's random model has them:
    InitMatrixNormal's table-of-normals values times 0.5 for every matrix -- combiner and contract included
    (COMBINER_INIT_RANDOM: with the zero start of create_model() the attention output would never reach the result,
    gpt/train/main_gpt.cpp:274) -- converted by ConvertMatrix (int8 of rms 32, scale = rms / 32), the matrix scales what
    that conversion returned; one KV cache per layer for B = 32 sequences.  Embedding, final layer and sampling are not
    part of it."""

    def __init__(self, ctx, cache_len, seed, n_new=64):
        import torch
        from tscale_amd import KVCache, capi
        from tscale_amd.attention import alibi_layer_schedule, VEC_SCALE
        self.ctx = ctx
        self.B, self.H, self.d, self.dim, self.depth, self.prompt, self.n_new = 32, 16, 128, 2048, 24, 2048, n_new
        self.L = self.prompt + self.n_new
        qsum = self.H * self.d
        g = torch.Generator(device="cuda").manual_seed(seed)
        self.g = g
        from tscale_amd import model_init
        self.seed = seed
        def matrices(count, n, k, salt):
            q, sc = model_init.random_int8_matrices(seed * 1000 + salt, count, n, k)
            return torch.from_numpy(q.view(np.uint8).reshape(count * n, k)).cuda(), sc
        self.sched = model_init.init_alibi(self.depth, self.L)
        assert self.sched == [(w, float(np.float32(sl))) for w, sl in alibi_layer_schedule(self.depth, self.L)]
        self.layers, self.caches = [], []
        for li, (w, slope) in enumerate(self.sched):
            proj, psc = matrices(4, qsum, self.dim, 10 * li)             # QK, QV, K, V one after the other
            comb, csc = matrices(1, self.dim, qsum * 4, 10 * li + 1)
            expand, _ = matrices(1, qsum, self.dim, 10 * li + 2)
            contract, tsc = matrices(1, self.dim, qsum, 10 * li + 3)
            self.layers.append({"proj": proj, "combiner": comb, "expand": expand, "contract": contract,
                                "qv_scale": float(psc[1]), "combiner_scale": float(csc[0]), "contract_scale": float(tsc[0]),
                                "width": w, "slope": slope})
            c = KVCache(ctx, capi.I8, self.B, self.H, self.L, self.d)
            if cache_len > 0:   # a cache that already holds a prompt: random rows
                c.k.copy_((torch.randn(c.k.shape, device="cuda", generator=g) * 24).round().clamp(-127, 127).to(torch.int8).view(torch.uint8))
                c.v.copy_((torch.randn(c.v.shape, device="cuda", generator=g) * 24).round().clamp(-127, 127).to(torch.int8).view(torch.uint8))
                c.k_scale.copy_((torch.rand(c.k_scale.shape, device="cuda", generator=g) + 0.5) * 1e-4)
            c.v_scale.fill_(VEC_SCALE)
            c.cache_len.fill_(cache_len)
            self.caches.append(c)
        self.rope = ctx.fill_rope_table(self.d, self.L)
        self.weight_bytes = sum(sum(v.numel() for v in layer.values() if isinstance(v, torch.Tensor)) for layer in self.layers)
        self.matmul_ops_per_token = 2.0 * sum(sum(v.numel() for v in layer.values() if isinstance(v, torch.Tensor)) for layer in self.layers)


def model_ends(m, vocab, dim):
    """Embedding and final layer of the random model (InitEmbedMatrix: table values as they are, the first 32 labels' rows
    zero; InitMatrixNormal with sko 1 for the final layer; gpt/model_params/model_params.cpp:47-66, 135-143), converted."""
    import torch
    from tscale_amd import model_init
    e = model_init.init_matrix_normal(m.seed * 1000 + 900, 2.0, vocab, dim)
    e[:32] = 0
    eq, es = model_init.convert_matrix(e)
    fq, fs = model_init.random_int8_matrices(m.seed * 1000 + 901, 1, vocab, dim)
    return torch.from_numpy(eq.view(np.uint8)).cuda(), es, torch.from_numpy(fq[0].view(np.uint8)).cuda(), float(fs[0])


def bench_token_step(ctx, steps):
    """One generated token per sequence through all 24 layers (per layer: state normalisation, four projections,
    RoPE + per-head normalisation, cache append + attention over the cache with KVProduct, combiner, feed-forward; 9-10
    library calls), B32 at cache length 2048+."""
    import torch
    from tscale_amd.attention import add_lookup_product, flush_state
    m = Int8Layers(ctx, cache_len=2048, seed=1313 + 9)
    B, H, d, dim, qsum = m.B, m.H, m.d, m.dim, m.H * m.d
    state = torch.randn((B, dim), device="cuda", generator=m.g)
    t = torch.full((B,), m.prompt, dtype=torch.int32, device="cuda")
    room = torch.empty(16 * 4 * B * max(dim, qsum), dtype=torch.uint8, device="cuda")
    keep = {}
    def step():
        pending = None
        for layer, c in zip(m.layers, m.caches):
            _, pending = add_lookup_product(ctx, layer, c, t, m.rope, state, workspace=room, scratch=keep, pending=pending, defer=True)
        flush_state(ctx, pending, state)
        t.add_(1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    torch.cuda.synchronize()
    reps = min(m.n_new - 2, max(10, steps))
    ms = gpu_time_ms(graph.replay, reps, 0)
    assert bool(torch.isfinite(state).all())
    n = m.prompt + 1 + reps // 2
    cache_bytes = sum(B * H * min(n - 1, w) * (2 * d + 8) for w, _ in m.sched)
    return {"config": "24 layers, B32, cache length ~2048+, model width 2048, 16 heads x 128, int8 weights and KV cache; "
                      "9-10 library calls per layer in one HIP graph per token",
            "ms_per_token_step": round(ms, 4), "tokens_per_s": round(B / ms * 1e3, 1),
            "weight_bytes": m.weight_bytes, "cache_bytes_per_step": cache_bytes,
            "GB/s": round((m.weight_bytes + cache_bytes) / ms / 1e6, 1),
            "frac_of_hbm_peak": round((m.weight_bytes + cache_bytes) / ms / 1e6 / PEAK_HBM_GBPS, 4)}


def bench_generate_model(ctx, steps):
    """Greedy generation with the whole int8 model on the device (ComputePrediction, gpt/train/cpu_infer.cpp:552-582):
    embedding of the previous choice -> 24 layers -> final normalisation, final-layer product (50257 x 2048), softmax
    and greedy choice, which is the next step's label; one HIP graph per token, B32 at cache length 2048+."""
    import numpy as np
    import torch
    from tscale_amd import capi
    from tscale_amd.attention import add_lookup_product, flush_state, VEC_SCALE
    m = Int8Layers(ctx, cache_len=2048, seed=1313 + 11)
    B, H, d, dim, qsum = m.B, m.H, m.d, m.dim, m.H * m.d
    vocab = 50257
    embed, embed_scale, final, final_layer_scale = model_ends(m, vocab, dim)
    bias = torch.randn(vocab, device="cuda", generator=m.g) * 0.1
    f32 = np.float32
    final_scale = float(f32(np.sqrt(f32(1.0) / f32(dim))) * (f32(1.0) / f32(0.693147)) * f32(final_layer_scale) * f32(VEC_SCALE))
    labels = torch.randint(0, vocab, (B,), dtype=torch.int32, device="cuda", generator=m.g)
    state = torch.empty((B, dim), dtype=torch.float32, device="cuda")
    t = torch.full((B,), m.prompt, dtype=torch.int32, device="cuda")
    room = torch.empty(16 * 4 * B * max(dim, qsum), dtype=torch.uint8, device="cuda")
    planes = torch.empty(16 * B * vocab, dtype=torch.int32, device="cuda")
    keep = {}
    def step():
        ctx.embed_rows(labels, embed, embed_scale, out=state)
        pending = None
        for layer, c in zip(m.layers, m.caches):
            _, pending = add_lookup_product(ctx, layer, c, t, m.rope, state, workspace=room, scratch=keep, pending=pending, defer=True)
        norm = flush_state(ctx, pending, state)
        logits = ctx.matmul_i8(norm, final, mode=capi.MM_I32_PLANES, out=planes)
        ctx.softmax_rows(logits, final_scale, bias, want_prob=False, argmax=labels)
        t.add_(1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    torch.cuda.synchronize()
    reps = min(m.n_new - 2, max(10, steps))
    first = labels.clone()
    ms = gpu_time_ms(graph.replay, reps, 0)
    assert bool(torch.isfinite(state).all()) and int(labels.min()) >= 0 and int(labels.max()) < vocab
    head_bytes = final.numel() + B * dim
    return {"config": "greedy generation, whole int8 model on the device: embedding, 24 layers, final layer 50257 x 2048, softmax, "
                      "argmax fed back; B32, cache length ~2048+; one HIP graph per token",
            "ms_per_token_step": round(ms, 4), "tokens_per_s": round(B / ms * 1e3, 1),
            "weight_bytes": m.weight_bytes + head_bytes, "choices_changed": bool((labels != first).any())}


def bench_prompt_then_generate(ctx, n_new=256):
    """The whole of the last configuration in one timed region: 32 prompts of 2048 random token ids (uniform over the
    vocabulary) through the embedding and the 24 layers in batch form, the final layer on each prompt's last token,
    then greedy generation of n_new tokens, one HIP graph replay per token (recorded beforehand, outside the timed
    region).  Nothing is reused between the phases but the KV caches the prompt pass filled."""
    import numpy as np
    import torch
    from tscale_amd import capi
    from tscale_amd.attention import add_lookup_product, add_lookup_product_prompt, flush_state, VEC_SCALE
    m = Int8Layers(ctx, cache_len=0, seed=1313 + 12, n_new=n_new)
    B, H, d, dim, qsum = m.B, m.H, m.d, m.dim, m.H * m.d
    vocab = 50257
    embed, embed_scale, final, final_layer_scale = model_ends(m, vocab, dim)
    bias = torch.randn(vocab, device="cuda", generator=m.g) * 0.1
    f32 = np.float32
    final_scale = float(f32(np.sqrt(f32(1.0) / f32(dim))) * (f32(1.0) / f32(0.693147)) * f32(final_layer_scale) * f32(VEC_SCALE))
    n = B * m.prompt
    ids = torch.randint(0, vocab, (n,), dtype=torch.int32, device="cuda", generator=m.g)
    off = torch.arange(0, n + 1, m.prompt, dtype=torch.int32, device="cuda")
    pos = torch.arange(m.prompt, dtype=torch.int32, device="cuda").repeat(B)
    last = (off[1:] - 1).long()
    spans = {w: ctx.build_spans(off, n, w) for w in {w for w, _ in m.sched}}
    tiles = {w: ctx.build_span_tiles(*sp) for w, sp in spans.items()}
    prompt_state = torch.empty((n, dim), dtype=torch.float32, device="cuda")
    labels = torch.zeros((B,), dtype=torch.int32, device="cuda")
    state = torch.empty((B, dim), dtype=torch.float32, device="cuda")
    t = torch.full((B,), m.prompt, dtype=torch.int32, device="cuda")
    room = torch.empty(16 * 4 * B * max(dim, qsum), dtype=torch.uint8, device="cuda")
    planes = torch.empty(16 * B * vocab, dtype=torch.int32, device="cuda")
    keep = {}
    def choose(norm):
        logits = ctx.matmul_i8(norm, final, mode=capi.MM_I32_PLANES, out=planes)
        ctx.softmax_rows(logits, final_scale, bias, want_prob=False, argmax=labels)
    def prompt_phase():
        ctx.embed_rows(ids, embed, embed_scale, out=prompt_state)
        norm = None
        for layer, c in zip(m.layers, m.caches):
            w = layer["width"]
            _, norm = add_lookup_product_prompt(ctx, layer, c, off, pos, m.rope, prompt_state, *spans[w], span_tiles=tiles[w],
                                                causal_period=m.prompt if w >= m.prompt else 0, norm=norm, want_norm=True,
                                                want_val=False)
        choose(norm[last].contiguous())   # NormalizeState of each prompt's last token, made by the last product
    def step():
        ctx.embed_rows(labels, embed, embed_scale, out=state)
        pending = None
        for layer, c in zip(m.layers, m.caches):
            _, pending = add_lookup_product(ctx, layer, c, t, m.rope, state, workspace=room, scratch=keep, pending=pending, defer=True)
        choose(flush_state(ctx, pending, state))
        t.add_(1)
    def rewind():
        for c in m.caches:
            c.cache_len.zero_()
        t.fill_(m.prompt)
    # once untimed: the prompt (so that a step sees caches of the right length), a step eagerly, the graph of a step
    prompt_phase()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    torch.cuda.synchronize()
    rewind()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    torch.cuda.synchronize()
    ev[0].record()
    prompt_phase()
    ev[1].record()
    chosen = [labels.clone()]
    for _ in range(n_new - 1):
        graph.replay()
        chosen.append(labels.clone())
    ev[2].record()
    torch.cuda.synchronize()
    ms_prompt, ms_gen = ev[0].elapsed_time(ev[1]), ev[1].elapsed_time(ev[2])
    chosen = torch.stack(chosen)
    assert int(m.caches[0].cache_len[0]) == m.prompt + n_new - 1 and int(chosen.min()) >= 0 and int(chosen.max()) < vocab
    assert bool(torch.isfinite(state).all())
    return {"config": "B32: 2048-token prompts (random ids over 50257) through embedding + 24 int8 layers + final layer, then greedy "
                      "generation of %d tokens (the first from the prompt pass, the others one HIP graph replay each); int8 KV cache" % n_new,
            "ms_total": round(ms_prompt + ms_gen, 2), "ms_prompt_to_first_token": round(ms_prompt, 2),
            "ms_per_generated_token": round(ms_gen / (n_new - 1), 4),
            "generated_tokens_per_s": round(B * n_new / (ms_prompt + ms_gen) * 1e3, 1),
            "distinct_tokens_chosen": int(torch.unique(chosen).numel())}


def bench_prompt_pass(ctx, steps):
    """The prompt of the same configuration through the same 24 layers in batch form (add_lookup_product_prompt):
    32 x 2048 tokens, per layer one prefill attention launch, one cache fill, seven matrix products in four calls, each
    with the normalisation that follows it as its epilogue."""
    import torch
    from tscale_amd.attention import add_lookup_product_prompt
    m = Int8Layers(ctx, cache_len=0, seed=1313 + 10)
    B, H, d, dim = m.B, m.H, m.d, m.dim
    n = B * m.prompt
    off = torch.arange(0, n + 1, m.prompt, dtype=torch.int32, device="cuda")
    pos = torch.arange(m.prompt, dtype=torch.int32, device="cuda").repeat(B)
    spans = {w: ctx.build_spans(off, n, w) for w in {w for w, _ in m.sched}}
    tiles = {w: ctx.build_span_tiles(*sp) for w, sp in spans.items()}
    state0 = torch.randn((n, dim), device="cuda", generator=m.g)
    state = torch.empty_like(state0)
    def run():
        state.copy_(state0)
        norm = None
        for layer, c in zip(m.layers, m.caches):
            c.cache_len.zero_()
            w = layer["width"]
            _, norm = add_lookup_product_prompt(ctx, layer, c, off, pos, m.rope, state, *spans[w], span_tiles=tiles[w],
                                                causal_period=m.prompt if w >= m.prompt else 0, norm=norm, want_norm=True,
                                                want_val=False)
    ms = gpu_time_ms(run, 2, 1)
    assert bool(torch.isfinite(state).all()) and int(m.caches[0].cache_len[0]) == m.prompt
    att_flops = sum(prefill_flops(B, m.prompt, H, d, w) for w, _ in m.sched)
    mm_ops = m.matmul_ops_per_token * n
    return {"config": "24 layers, B32 x 2048 prompt tokens, model width 2048, 16 heads x 128, int8; batch form of the layer",
            "ms": round(ms, 3), "tokens_per_s": round(n / ms * 1e3, 1),
            "matmul_TOP": round(mm_ops / 1e12, 2), "attention_TOP": round(att_flops / 1e12, 2),
            "TOP/s": round((mm_ops + att_flops) / ms / 1e9, 1), "frac_of_int8_peak": round((mm_ops + att_flops) / ms / 1e9 / PEAK_I8_TOPS, 4)}


def cpu_baseline_prefill(wl, n_seq_sample, layers=None, repeat=1):
    """The oracle (a port of the reference's CPU attention) on the same quantised inputs: the first
    `n_seq_sample` sequences of every layer of the pass, all host threads; plus one sequence of one
    full-window layer on a single thread (the reference's CPU path has no threading)."""
    import numpy as np
    from oracle import pyoracle as orc
    S, H, d = wl.S, wl.H, wl.d
    n = n_seq_sample * S
    threads = orc.max_threads()
    flops = 0.0
    t_total = 0.0
    layers_done = 0
    for li in (layers if layers is not None else range(len(wl.layers))):
        (q, qs), (k, ks), (v, vs) = wl.inputs[li]
        W, slope = wl.layers[li]
        hq, hk, hv = (x[:n].cpu().numpy() for x in (q, k, v))
        hqs, hks, hvs = (np.ascontiguousarray(x[:, :n].cpu().numpy()) for x in (qs, ks, vs))
        st, fi = orc.make_spans([S] * n_seq_sample, W)
        t0 = time.perf_counter()
        for _ in range(repeat):
            orc.prefill_q8(wl.dtype, hq, hk, hv, H, hqs, hks, hvs, st, fi, slope, n_threads=threads)
        t_total += time.perf_counter() - t0
        flops += repeat * prefill_flops(n_seq_sample, S, H, d, W)
        layers_done += 1
        if t_total > 20.0 and layers_done % 2 == 0:
            break
    (q, qs), (k, ks), (v, vs) = wl.inputs[1]
    hq, hk, hv = (x[:S].cpu().numpy() for x in (q, k, v))
    hqs, hks, hvs = (np.ascontiguousarray(x[:, :S].cpu().numpy()) for x in (qs, ks, vs))
    st, fi = orc.make_spans([S], S)
    t0 = time.perf_counter()
    orc.prefill_q8(wl.dtype, hq, hk, hv, H, hqs, hks, hvs, st, fi, 0.0, n_threads=1)
    t1 = time.perf_counter() - t0
    return {
        "value": flops / t_total / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": f"{n_seq_sample} of {wl.B} sequences, {layers_done} of {len(wl.layers)} layers"
                  + (f" x {repeat} repetitions" if repeat > 1 else "") + f", {threads} OpenMP threads, {t_total:.2f} s",
        "single_thread_value": prefill_flops(1, S, H, d, S) / t1 / 1e12,
        "single_thread_sample": f"1 sequence, one full-window layer, 1 thread, {t1:.2f} s",
    }


def cpu_baseline_decode(wl, n_seq_sample, reps):
    import numpy as np
    from oracle import pyoracle as orc
    c = wl.caches[0]
    k = c.k[:n_seq_sample].cpu().numpy(); v = c.v[:n_seq_sample].cpu().numpy()
    ks = c.k_scale[:n_seq_sample].cpu().numpy(); vs = c.v_scale[:n_seq_sample].cpu().numpy()
    import torch
    bits = wl.q[:n_seq_sample].cpu().view(torch.int16).numpy().view(np.uint16)
    q8, qs = orc.quantize_rows(orc.I8, bits, wl.H)
    qs = np.ascontiguousarray(qs.T)
    lens = np.full(n_seq_sample, wl.L, np.int32)
    threads = orc.max_threads()
    t0 = time.perf_counter()
    for _ in range(reps):
        orc.decode(orc.I8, q8, qs, k, v, ks, vs, lens, 10 ** 6, 0.0, exp2_mode=1, use_simd=True, n_threads=threads)
    t = (time.perf_counter() - t0) / reps
    nbytes = wl.bytes * n_seq_sample / wl.B
    return {"value": nbytes / t / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{n_seq_sample} of {wl.B} sequences, {reps} repetitions, vpdpbusd level {orc.simd_level()}, "
                      f"{threads} OpenMP threads, {t * reps:.2f} s"}


def run_only(ctx, args):
    """Profiling aid: one kind of launch, repeated; used for the rocprofv3 runs recorded in profiles/."""
    from tscale_amd import capi
    name = args.only
    if args.calibrate:
        # a plain copy of known size in the same profile: 256 MiB read + 256 MiB written
        import torch
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
    if name == "generate-model":
        print(json.dumps({"only": name, **bench_generate_model(ctx, args.steps)}))
        return
    if name == "prompt-pass":
        print(json.dumps({"only": name, **bench_prompt_pass(ctx, args.steps)}))
        return
    if name == "prompt-then-generate":
        print(json.dumps({"only": name, **bench_prompt_then_generate(ctx)}))
        return
    if name == "token-step":
        print(json.dumps({"only": name, **bench_token_step(ctx, args.steps)}))
        return
    if name == "matmul":
        print(json.dumps({"only": name, **bench_matmul(ctx, args.steps)}))
        return
    if name == "producer":
        print(json.dumps({"only": name, **bench_producer(ctx, args.steps * 5)}))
        return
    if name == "decode":
        dw = DecodeWorkload(ctx, 64, 4096, 16, 128, n_caches=4, seed=1313 + 3)
        ms = gpu_time_ms(dw.step, args.steps, args.warmup)
        print(json.dumps({"only": name, "ms": ms, "GB/s": dw.bytes / ms / 1e6}))
        return
    if name in ("prompt-int8-full", "decode-append-token"):
        import torch
        gw = GenerationWorkload(ctx)
        if name == "prompt-int8-full":   # the full-window prefill launch over the 1.5B-style prompt (B32 x 2048, int8, d128)
            i = [j for j, (w, _) in enumerate(gw.sched) if w == max(gw.kinds)][0]
            ms = gpu_time_ms(lambda: gw.prefill_layer(i), args.steps, args.warmup)
            print(json.dumps({"only": name, "ms": ms, "TOP/s": gw.prefill_flops(i) / ms / 1e9}))
            return
        # one generated token in the middle of the run: 24 decode launches with the append fused, caches at 2048 + 128 rows
        gw.fill_caches()
        for c in gw.caches:
            c.cache_len.fill_(gw.prompt + gw.n_new // 2)
        lens = torch.full((gw.B,), gw.prompt + gw.n_new // 2, dtype=torch.int32, device="cuda")
        def token():
            for c in gw.caches:
                c.cache_len.copy_(lens)
            gw.decode_step()
        ms = gpu_time_ms(token, args.steps, args.warmup)
        n = gw.prompt + gw.n_new // 2 + 1
        nbytes = sum(gw.B * gw.H * (min(n - 1, W) * (2 * gw.d + 8) + gw.d + 4 + 4 * gw.d) for W, _ in gw.sched)
        print(json.dumps({"only": name, "ms_per_token": ms, "bytes_per_token": nbytes, "GB/s": nbytes / ms / 1e6}))
        return
    if name == "long-s8192":   # the long-span kernel's own shape: B4 S8192, full window
        wl = PrefillWorkload(ctx, capi.E4M3, 4, 8192, 16, 128, 2, seed=1313 + 6, short=256)
        li = 1
    elif name == "c1-int8":
        wl = PrefillWorkload(ctx, capi.I8, 1, 1024, 12, 64, 2, seed=1313 + 1)
        li = 1
    elif name.startswith("c2"):
        wl = PrefillWorkload(ctx, capi.E4M3, 16, 1024, 12, 64, 2, seed=1313 + 2)
        li = 0 if name.endswith("short") else 1
    else:
        wl = PrefillWorkload(ctx, capi.E4M3, 8, 4096, 16, 128, 2, seed=1313 + 4, short=256)
        li = 0 if name.endswith("short") else 1
    ms = gpu_time_ms(lambda: wl.run_layer(li), args.steps, args.warmup)
    print(json.dumps({"only": name, "ms": ms, "TFLOP/s": wl.flops_layer[li] / ms / 1e9}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--extra", action="store_true",
                    help="also time the producer, KVProduct, the int8 matrix products and generation with the whole int8 model")
    ap.add_argument("--only", default=None,
                    choices=["c2-short", "c2-full", "c4-short", "c4-full", "c1-int8", "decode", "prompt-int8-full", "decode-append-token", "long-s8192", "producer", "matmul", "token-step", "prompt-pass", "generate-model", "prompt-then-generate"],
                    help="profiling aid: run just this launch --steps times and print its timing")
    ap.add_argument("--calibrate", action="store_true",
                    help="with --only: first run three 256 MiB device copies (counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)

    import torch
    from tscale_amd import AttentionContext, capi
    if not torch.cuda.is_available():
        print("bench.py: no HIP device", file=sys.stderr)
        sys.exit(1)
    ctx = AttentionContext(0, max_seqs=64, max_heads=16, max_head_dim=128, max_splits=32)
    if args.only:
        run_only(ctx, args)
        return

    facts = profile_facts()
    # ---- prefill, 1.5B-style: the headline -----------------------------------------------------
    B, S, H, d = 8, 4096, 16, 128
    wl = PrefillWorkload(ctx, capi.E4M3, B, S, H, d, 2, seed=1313 + 4, short=256)
    ms = gpu_time_ms(wl.step, args.steps, args.warmup)
    tflops = wl.flops / (ms * 1e-3) / 1e12
    lsteps = max(50, args.steps)   # the launch durations behind `roofline`: at least 50 launches each
    ms_short = gpu_time_ms(lambda: wl.run_layer(0), lsteps, 2)
    ms_wide = gpu_time_ms(lambda: wl.run_layer(1), lsteps, 2)
    ms_wide_cq = gpu_time_ms(lambda: wl.run_layer(1, const_q_scale=True), lsteps, 2)
    ms_wide_cqv = gpu_time_ms(lambda: wl.run_layer(1, const_q_scale=True, const_v_scale=True), lsteps, 2)
    ach = wl.flops_layer[1] / (ms_wide * 1e-3) / 1e12
    result = {
        "metric": "prefill attn TFLOP/s + decode attn HBM GB/s (% of MI355X peak), 1 GPU",
        "value": round(tflops, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "e4m3 (fp32 accumulate; f16 P.V)", "data": "synthetic",
        "config": {"workload": "prefill-1.5B-style: B8 S4096 H16 d128 e4m3 + per-row f32 scales, one pair of layers "
                               "(W=256, slope 0.5) + (W=4096, slope 0), f16 out; 616.19 GFLOP per step",
                   "frac_of_fp8_peak": round(tflops / PEAK_FP8_TFLOPS, 5),
                   "layer_ms": {"window256": round(ms_short, 5), "full": round(ms_wide, 5),
                                # (not part of `value`: the same launch with one number as the query scale, and as the value scale
                                # too, which is what TScale's own model passes)
                                "full_with_constant_query_scale": round(ms_wide_cq, 5),
                                "full_with_constant_query_and_value_scales": round(ms_wide_cqv, 5)},
                   "layer_tflops": {"window256": round(wl.flops_layer[0] / ms_short / 1e9, 2),
                                    "full": round(wl.flops_layer[1] / ms_wide / 1e9, 2)}},
        # the dominant kernel: the full-window launch (549.62 of the step's 616.19 GFLOP), timed back to back on its own
        "roofline": roofline("prefill_kernel<e4m3, d128>, full causal window", "mfma", ach, wl.flops_layer[1], ms_wide,
                             facts.get("prefill_c4_full")),
        "roofline_window256": roofline("prefill_kernel<e4m3, d128, slope>, window 256", "mfma",
                                       wl.flops_layer[0] / (ms_short * 1e-3) / 1e12, wl.flops_layer[0], ms_short,
                                       facts.get("prefill_c4_short")),
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline_prefill(wl, 2)
    del wl
    torch.cuda.empty_cache()

    # ---- prefill, 125M-style -----------------------------------------------------------------
    B, S, H, d, NL = 16, 1024, 12, 64, 12
    wl = PrefillWorkload(ctx, capi.E4M3, B, S, H, d, NL, seed=1313 + 2)
    ms = gpu_time_ms(wl.step, args.steps, args.warmup)
    ms_short = graph_time_ms(lambda: wl.run_layer(0), 20, max(3, args.steps // 5))
    ms_wide = graph_time_ms(lambda: wl.run_layer(1), 20, max(3, args.steps // 5))
    c2 = {"value": round(wl.flops / (ms * 1e-3) / 1e12, 3), "unit": "TFLOP/s", "ms_per_step": round(ms, 5), "steps": args.steps,
          "config": {"workload": "prefill-125M-style: B16 S1024 H12 d64 e4m3 + per-row f32 scales, 12 layers alternating "
                                 "(W=64, slope 0.5)/(W=1024, slope 0), f16 out; 173.18 GFLOP per step",
                     "layer_ms": {"window64": round(ms_short, 5), "full": round(ms_wide, 5)}},
          "roofline": roofline("prefill_kernel<e4m3, d64>, full causal window", "mfma", wl.flops_layer[1] / (ms_wide * 1e-3) / 1e12,
                               wl.flops_layer[1], ms_wide, facts.get("prefill_c2_full")),
          "roofline_window64": roofline("prefill_kernel<e4m3, d64, slope>, window 64", "mfma",
                                        wl.flops_layer[0] / (ms_short * 1e-3) / 1e12, wl.flops_layer[0], ms_short,
                                        facts.get("prefill_c2_short"))}
    c2["roofline_window64"]["hbm_GB/s"] = round(65.3e6 / (ms_short * 1e-3) / 1e9, 1)   # 65.3 MB of inputs and output per launch
    if not args.no_cpu:
        c2["cpu_baseline"] = cpu_baseline_prefill(wl, 16)
    result["prefill_125M_style"] = c2
    del wl
    torch.cuda.empty_cache()

    # ---- the CPU-reference configuration (int8, B1) ------------------------------------------------
    wl = PrefillWorkload(ctx, capi.I8, 1, 1024, 12, 64, 2, seed=1313 + 1)
    ms1 = graph_time_ms(lambda: wl.run_layer(1), 20, max(3, args.steps // 5))
    c1 = {"config": {"workload": "B1 S1024 H12 d64 int8 + per-row f32 scales, full causal window; 1.609 GFLOP"},
          "gpu_ms": round(ms1, 5), "gpu_TOP/s": round(wl.flops_layer[1] / ms1 / 1e9, 3)}
    if not args.no_cpu:
        c1["cpu_baseline"] = cpu_baseline_prefill(wl, 1, layers=[1], repeat=8)
    result["cpu_reference_config"] = c1
    del wl
    torch.cuda.empty_cache()

    # ---- decode, int8 KV ----------------------------------------------------------------------
    if not args.no_decode:
        dw = DecodeWorkload(ctx, 64, 4096, 16, 128, n_caches=4, seed=1313 + 3)
        dsteps = max(args.steps, 20)
        dms = gpu_time_ms(dw.step, dsteps, max(args.warmup, 4))
        gbps = dw.bytes / (dms * 1e-3) / 1e9
        dec = {"value": round(gbps, 2), "unit": "GB/s", "ms_per_step": round(dms, 5), "steps": dsteps, "dtype": "int8",
               "config": {"workload": "decode: B64, 1 bf16 query/seq, int8 KV cache L=4096, H16 d128, per-row f32 scales; "
                                      "1108.08 MB per step; 4 caches in rotation"},
               "roofline": roofline("decode_split_kernel<int8, d128>", "hbm", gbps, dw.bytes, dms, facts.get("decode_c3"))}
        if not args.no_cpu:
            dec["cpu_baseline"] = cpu_baseline_decode(dw, 64, 200)
        result["decode"] = dec
        del dw
        torch.cuda.empty_cache()
        # ---- the attention calls of the 1.5B-style generation run ---------------------------------
        result["generation_1p5B_style"] = bench_generation(ctx, args.steps, facts)
        torch.cuda.empty_cache()
        result["prefill_long_span"] = bench_long_span(ctx, args.steps, facts)
        # ---- the whole layer stack around the attention calls (a few seconds) ------------------------
        result["token_step_24_layers"] = bench_token_step(ctx, args.steps)
        result["prompt_pass_24_layers"] = bench_prompt_pass(ctx, args.steps)
        torch.cuda.empty_cache()
        # ---- the last configuration end to end: 32 prompts through the whole int8 model, then 256 greedy tokens each ----
        result["prompt_then_generate_256"] = bench_prompt_then_generate(ctx)
        torch.cuda.empty_cache()

    # ---- optional: 1.5B-style prefill shapes ---------------------------------------------------------
    if args.extra:
        result["producer"] = bench_producer(ctx, args.steps)
        torch.cuda.empty_cache()
        result["kv_product"] = bench_kv_product(ctx, args.steps)
        result["combiner_matmul"] = bench_matmul(ctx, args.steps)
        result["generate_whole_model"] = bench_generate_model(ctx, args.steps)
        torch.cuda.empty_cache()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
