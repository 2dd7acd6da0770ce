#!/usr/bin/env python3
"""Benchmark of the KV-cache compression hot path on one MI355X.

Headline workload (configuration 3 of the benchmark set, the "@32k ctx" decode the metric is
quoted on): Qwen3-8B shape, 36 layers, 32 query / 8 kv heads, D=128, batch 16,
32768 tokens of context per sequence stored as 4-bit packed KIVI codes (keys per
channel, values per token, group 64) plus an fp16 tail.  One step = one decode
token for every sequence through all 36 layers: append K/V to the fp16 tail,
flush a 64-token block into the packed store when one is due, attend -- in the
reference's layer-batched form (one attention launch over a leading layer axis,
veloxquant_mlx/metal/_scalar_attend.py:496-647); ``per_layer_launches`` holds the same
step issued as one launch per layer.

Prints ONE JSON line.  ``value`` is algorithmic HBM bytes per step divided by
the step time, inputs resident in HBM.  ``roofline`` prices the attention
launch alone (HIP events on the launch stream); ``cpu_baseline`` times the reference's
CPU path (its operations restated on torch CPU, all host threads torch is given) on a
bounded sample of the same workload; ``extras.cpu_baselines`` holds the same for the
other workloads and the one-thread scalar C port.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0


def _parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=20)
    p.add_argument("--warmup", type=int, default=3)
    p.add_argument("--layers", type=int, default=36)
    p.add_argument("--batch", type=int, default=16)
    p.add_argument("--ctx", type=int, default=32768)
    p.add_argument("--bits", type=int, default=4)
    p.add_argument("--group", type=int, default=64)
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    p.add_argument("--no-extras", action="store_true", help="skip the per-kernel side measurements")
    p.add_argument("--only-kernel", action="store_true",
                   help="time the attention launch only (profiling): the layer-batched launch, or with --per-layer "
                        "the loop of one launch per layer")
    p.add_argument("--per-layer", action="store_true", help="with --only-kernel: one launch per layer")
    p.add_argument("--only", default=None, metavar="NAME",
                   help="run one side workload in a loop and print its timing (for rocprofv3): "
                        "decode_2bit_B16, decode_2bit_B1, decode_d256_2bit_32k_B16, decode_d256_4bit_32k_B16, decode_3bit_32k_B16, decode_3bit_tight_32k_B16, decode_1bit_32k_B16, decode_d64_4bit_32k_B16, decode_d64_unpaired_4bit_32k_B16, vq_assign, flash_prefill_<S>, prefill, quant_pack, quant_dequant, zipcache, skvq")
    p.add_argument("--copy-calib", action="store_true",
                   help="run a plain 1 GiB device copy a few times and exit (calibrates HBM byte counters)")
    return p.parse_args()


def _side_ms(fn, iters, torch, rounds=3):
    """Side measurements: median over ``rounds`` of the average milliseconds per call
    (the reference's own rule is medians, tests/metal/test_kivi_quant.py:297-347)."""
    return sorted(_event_ms(fn, iters, torch) for _ in range(rounds))[rounds // 2]


def _event_ms(fn, iters, torch):
    """Average milliseconds per call, HIP events on the current stream."""
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters


def _graph_ms(fn, torch, calls=20, replays=5):
    """Milliseconds per call with the calls replayed from a HIP graph: what the GPU needs when the
    host's per-call cost (argument marshalling in Python, ~20 us) is out of the way."""
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _ in range(3):
            fn()
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(calls):
                fn()
    graph.replay()
    torch.cuda.synchronize()
    best = None
    for _ in range(replays):
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        graph.replay()
        e.record()
        torch.cuda.synchronize()
        ms = s.elapsed_time(e) / calls
        best = ms if best is None else min(best, ms)
    return best


def _algorithmic_bytes_per_layer(B, Hkv, ctx, D, bits, g):
    codes = 2 * B * Hkv * ctx * D * bits // 8
    meta = B * Hkv * (ctx // g) * D * 2 * 2 + B * Hkv * ctx * (D // g) * 2 * 2  # fp16 scale+zero, K and V
    return codes + meta


def _synthetic_layer(torch, B, Hkv, S, D, seed, dev):
    g = torch.Generator(device=dev).manual_seed(seed)
    f = torch.exp(torch.randn(D, generator=g, device=dev))
    k = (torch.randn((B, Hkv, S, D), generator=g, device=dev) * f).to(torch.float16)
    v = torch.randn((B, Hkv, S, D), generator=g, device=dev).to(torch.float16)
    return k, v


def main() -> int:
    a = _parse()
    if a.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (every kernel is independent per (sequence, kv head); "
              f"--gpus {a.gpus} is not supported)", file=sys.stderr)
        return 2
    import numpy as np
    import torch

    from veloxquant_mlx_amd import kernels as K
    from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory

    if not K.hip_available():
        print("bench.py: no ROCm device / kernel library", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if a.copy_calib:
        src = torch.arange(1 << 29, device=dev, dtype=torch.int32).view(torch.float16)  # 2 GiB, read half
        dst = torch.empty(1 << 29, device=dev, dtype=torch.float16)                     # 1 GiB written
        ms = _event_ms(lambda: dst.copy_(src[: 1 << 29]), 5, torch)
        print(json.dumps({"copy_bytes_read": 1 << 30, "copy_bytes_written": 1 << 30, "ms": ms,
                          "GBps": (2 << 30) / ms / 1e6}))
        return 0
    if a.only:
        return _only(a, torch, K, dev)
    NL, B, Hq, Hkv, D, ctx, bits, g = a.layers, a.batch, 32, 8, 128, a.ctx, a.bits, a.group
    R = 128
    scale = 1.0 / math.sqrt(D)

    # ---- build the resident caches: prefill ctx + R tokens per layer in chunks
    cfg = KVCacheConfig(method="kivi", head_dim=D, bit_width_inlier=bits, kivi_group_size=g, residual_length=R,
                        fused_sdpa=True, fused_sdpa_memory_bound=True, fused_sdpa_max_ctx=ctx + 4096)
    caches = []
    chunk = 4096
    # stop short of the next 64-token flush so that it falls inside the timed steps of the headline form
    # (the per-layer form before it appends 2 + n_pl tokens, the warm-up a.warmup)
    n_pl = max(3, a.steps // 4)
    short = 2 + n_pl + a.warmup + max(1, a.steps // 2)
    prefill = ctx + R + g - (short if short < g else 10)
    for l in range(NL):
        c = KVCacheFactory.create(cfg)
        for s0 in range(0, prefill, chunk):
            n = min(chunk, prefill - s0)
            k, v = _synthetic_layer(torch, B, Hkv, n, D, 1000 * l + s0, dev)
            c.update_and_fetch(k, v)
        caches.append(c)
    del k, v
    torch.cuda.synchronize()
    assert caches[0]._n_quantized == ctx, caches[0]._n_quantized

    gen = torch.Generator(device=dev).manual_seed(7)
    q = torch.randn((NL, B, Hq, 1, D), generator=gen, device=dev).to(torch.float16)
    k_new = torch.randn((NL, B, Hkv, 1, D), generator=gen, device=dev).to(torch.float16)
    v_new = torch.randn((NL, B, Hkv, 1, D), generator=gen, device=dev).to(torch.float16)

    # Two forms of the same step.  The headline is the reference's layer-batched form (the kernel with a leading
    # NL axis, metal/_scalar_attend.py:496-647, which the 36-layer configuration is quoted on): every layer's
    # cache takes its token through the ordinary cache API (nothing is launched: the token is pending), then ONE
    # launch stores the 36 x 16 new tokens and attends for all layers.  The per-layer form (one launch per layer,
    # what a model's forward pass issues) is timed beside it.
    def step_per_layer():
        for l, c in enumerate(caches):
            c.update_and_fetch(k_new[l], v_new[l])
            c.fused_sdpa(q[l], scale)

    def attend_per_layer():
        for l, c in enumerate(caches):
            c.fused_sdpa(q[l], scale)

    layer_bytes = _algorithmic_bytes_per_layer(B, Hkv, ctx, D, bits, g)
    step_bytes = layer_bytes * NL
    per_layer = None
    if not a.only_kernel or a.per_layer:
        n = n_pl if not a.only_kernel else a.steps
        for _ in range(2 if not a.only_kernel else a.warmup):
            (attend_per_layer if a.only_kernel else step_per_layer)()
        if a.only_kernel:
            ms = _event_ms(attend_per_layer, n, torch) / NL
            print(json.dumps({"form": "one launch per layer", "attend_ms_per_layer": ms, "GBps": layer_bytes / ms / 1e6}))
            return 0
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            step_per_layer()
        torch.cuda.synchronize()
        dt_pl = (time.perf_counter() - t0) / n
        kern_pl = _event_ms(attend_per_layer, n, torch) / NL
        per_layer = {
            "ms_per_step": round(dt_pl * 1e3, 4), "GBps": round(step_bytes / dt_pl / 1e9, 1),
            "frac_hbm": round(step_bytes / dt_pl / 1e9 / HBM_PEAK_GBS, 4), "steps": n,
            "attend_ms_per_launch": round(kern_pl, 5), "attend_GBps": round(layer_bytes / kern_pl / 1e6, 1),
            "attend_frac_hbm": round(layer_bytes / kern_pl / 1e6 / HBM_PEAK_GBS, 4), "bytes_per_launch": layer_bytes,
            "note": "the same step as one append + one attention launch per layer (what a model's forward pass issues)"}

    # the layers' caches adopted by a layer-stacked cache: their buffers become slices of [NL*B, ...] stacks
    # (copied once, here), every layer's cache object keeps working on its slice
    from veloxquant_mlx_amd.cache import LayerStackedKIVICache
    stack = LayerStackedKIVICache.from_layers(caches)

    def step():
        for l, c in enumerate(caches):
            c.update_and_fetch(k_new[l], v_new[l])
        stack.fused_sdpa_all(q, scale)

    def attend_only():
        stack.fused_sdpa_all(q, scale)

    if a.only_kernel:
        for _ in range(a.warmup):
            attend_only()
        ms = _event_ms(attend_only, a.steps, torch)
        print(json.dumps({"form": f"one launch for {NL} layers", "attend_ms_per_launch": ms, "attend_ms_per_layer": ms / NL,
                          "GBps": step_bytes / ms / 1e6}))
        return 0

    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / a.steps
    value = step_bytes / dt / 1e9

    # ---- roofline of the dominant kernel (the attention launch), events on the launch stream
    kern_ms = _event_ms(attend_only, max(3, a.steps // 2), torch)
    achieved = step_bytes / (kern_ms * 1e-3) / 1e9
    # HBM bytes one attention launch moved under rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (calibrated
    # against a 1 GiB device copy): read from profiles/hbm_traffic.json, which records the hash of the
    # attention sources it was measured on -- a kernel changed since then reports null
    default_workload = (NL, B, ctx, bits, g) == (36, 16, 32768, 4, 64)
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": _recorded_traffic("decode_cfg3_4bit_g64_B16_36_layers") if default_workload else None,
                "kernel": f"attend_mfma_packed_kernel<4, f16, 2, 4>: one launch stores the new token of {NL} layers x {B} "
                          "sequences, runs their fp16 tails and packed prefixes and merges the splits "
                          "(vq_kivi_attend with k_new / v_new and sync counters, the layer axis folded into the batch axis)",
                "bytes_per_launch": step_bytes, "ms_per_launch": round(kern_ms, 5)}

    out = {
        "metric": "dequant-SDPA decode HBM GB/s @32k ctx", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(dt * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8/f16 (f32 accumulate)",
        "data": "synthetic",
        "config": {"workload": f"configs[3]: batched decode, {NL} layers, 32q/8kv heads, D=128, batch {B}, "
                               f"context {ctx}, {bits}-bit packed KV group {g}; per step every layer's cache appends its "
                               "token (flushing a 64-token block when one is due), then one layer-batched launch attends",
                   "layers": NL, "batch": B, "context": ctx, "bits": bits, "group": g,
                   "algorithmic_bytes_per_step": step_bytes},
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "roofline": roofline,
    }
    if per_layer is not None:
        out["per_layer_launches"] = per_layer

    if not a.no_extras:
        out["extras"] = _extras(torch, K, dev)
    if not a.no_cpu:
        head, others = _cpu_baselines(np, torch, caches[0], q[0], ctx, Hkv, D, bits, g, scale)
        out["cpu_baseline"] = head
        out.setdefault("extras", {})["cpu_baselines"] = others
    print(json.dumps(out))
    return 0


_ROWS_CASES = {"decode_d256_2bit_32k_B16": (12, 4, 256, 2, 32), "decode_d256_4bit_32k_B16": (12, 4, 256, 4, 64),
               "decode_3bit_32k_B16": (32, 8, 128, 3, 32), "decode_3bit_tight_32k_B16": (32, 8, 128, 3, 32),
               "decode_1bit_32k_B16": (32, 8, 128, 1, 32), "decode_d64_4bit_32k_B16": (32, 8, 64, 4, 32),
               "decode_d64_unpaired_4bit_32k_B16": (32, 8, 64, 4, 32)}
_ROWS_NOTES = {"decode_d256_2bit_32k_B16": "matrix-unit decode kernel, head of 256 channels (two launches: the fp16 tail comes from the vector kernel, four runs)",
               "decode_d256_4bit_32k_B16": "matrix-unit decode kernel, head of 256 channels, four waves per CU",
               "decode_3bit_32k_B16": "3-bit codes in 4-bit fields (the cache's default): matrix-unit decode kernel",
               "decode_3bit_tight_32k_B16": "3-bit codes ten to a word (kivi_code_field='tight'): vector-unit kernel (attend_rows_kernel), four query rows of a kv head per block",
               "decode_1bit_32k_B16": "1-bit codes in 2-bit fields (the cache's default): matrix-unit decode kernel",
               "decode_d64_4bit_32k_B16": "heads of 64 channels (Llama-3.2-1B: 32 query / 8 kv heads), kv heads kept in pairs as heads of 128 channels (the cache's default): matrix-unit decode kernel, queries zero-padded into their half",
               "decode_d64_unpaired_4bit_32k_B16": "heads of 64 channels, kivi_pair_heads=False: vector-unit kernel (attend_rows_kernel)"}


def _decode_rows_case(torch, dev, name):
    """Decode outside the headline's head shape: the head size of config 2's model (Falcon3-7B: 12 query / 4 kv heads,
    D = 256) at 2 and 4 bits, on the matrix-unit kernel's 256-channel form, and 3-bit / 1-bit codes at the headline's
    head shape: in 4-bit / 2-bit fields on the matrix-unit kernel (the cache's default) and ten 3-bit codes to a word on
    the vector kernel; heads of 64 channels kept in pairs (the default) and singly; batch 16, 32768 packed tokens plus
    the fp16 residual."""
    from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory
    hq, hkv, d, bits, g = _ROWS_CASES[name]
    cfg = KVCacheConfig(method="kivi", head_dim=d, bit_width_inlier=bits, kivi_group_size=g, residual_length=128,
                        fused_sdpa=True, fused_sdpa_memory_bound=True, kivi_code_field="tight" if "tight" in name else "auto",
                        kivi_pair_heads="unpaired" not in name)
    c = KVCacheFactory.create(cfg)
    for s0 in range(0, 32768 + 128, 8192):
        n = min(8192, 32768 + 128 - s0)
        k, v = _synthetic_layer(torch, 16, hkv, n, d, 5 + s0, dev)
        c.update_and_fetch(k, v)
    q = torch.randn((16, hq, 1, d), device=dev).to(torch.float16)
    words = -(-d // (32 // c._field))     # 32-bit words a token row of codes takes
    nbytes = 2 * 16 * hkv * 32768 * words * 4 + 2 * 16 * hkv * (32768 // g) * d * 2 * 2
    return c, (lambda: c.fused_sdpa(q, 1 / math.sqrt(d))), nbytes


def _decode_2bit_case(torch, dev, B):
    """2-bit group-32 packed cache of 32768 tokens plus the fp16 residual, one query token (the "@32k" target)."""
    from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory
    D, Hq, Hkv = 128, 32, 8
    cfg = KVCacheConfig(method="kivi", head_dim=D, bit_width_inlier=2, kivi_group_size=32, residual_length=128,
                        fused_sdpa=True, fused_sdpa_memory_bound=True)
    c = KVCacheFactory.create(cfg)
    for s0 in range(0, 32768 + 128, 8192):
        n = min(8192, 32768 + 128 - s0)
        k, v = _synthetic_layer(torch, B, Hkv, n, D, 5 + s0, dev)
        c.update_and_fetch(k, v)
    q = torch.randn((B, Hq, 1, D), device=dev).to(torch.float16)
    return c, (lambda: c.fused_sdpa(q, 1 / math.sqrt(D))), _algorithmic_bytes_per_layer(B, Hkv, 32768, D, 2, 32)


def _decode_cfg1_case(torch, dev):
    """Config 1: 32 query / 8 kv heads, D=128, B=1, 8192 tokens as 2-bit group-32 packed codes plus the
    most recent 128 tokens in fp16, one fp16 query token.  Bytes: codes 2 x 2,097,152 + fp16 scale / zero
    2 x 1,048,576 + tail 524,288 + query and output 16,384 = 6,832,128."""
    from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory
    D, Hq, Hkv, S, R = 128, 32, 8, 8192, 128
    cfg = KVCacheConfig(method="kivi", head_dim=D, bit_width_inlier=2, kivi_group_size=32, residual_length=R,
                        fused_sdpa=True, fused_sdpa_memory_bound=True)
    c = KVCacheFactory.create(cfg)
    k, v = _synthetic_layer(torch, 1, Hkv, S + R, D, 3, dev)
    c.update_and_fetch(k, v)
    assert c._n_quantized == S, c._n_quantized
    q = torch.randn((1, Hq, 1, D), device=dev).to(torch.float16)
    nbytes = _algorithmic_bytes_per_layer(1, Hkv, S, D, 2, 32) + 2 * Hkv * R * D * 2 + 2 * Hq * D * 2
    assert nbytes == 6832128, nbytes
    return c, (lambda: c.fused_sdpa(q, 1 / math.sqrt(D))), nbytes


def _prefill_case(torch, dev, Hq=32, Hkv=8, D=128):
    """Config 4: 8 chunks of 512 bf16 queries over a 4-bit packed prefix of 4096 tokens plus their own,
    quantise-on-write (group 32, residual 128).  Returns a function that runs one whole pass and
    gives its milliseconds."""
    from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory

    def prefill_pass():
        cfg = KVCacheConfig(method="kivi", head_dim=D, bit_width_inlier=4, kivi_group_size=32, residual_length=128,
                            fused_sdpa=True, fused_sdpa_memory_bound=True, fused_sdpa_max_ctx=8192)
        c = KVCacheFactory.create(cfg)
        k, v = _synthetic_layer(torch, 1, Hkv, 4096, D, 77, dev)
        c.update_and_fetch(k.to(torch.bfloat16), v.to(torch.bfloat16))
        chunks = []
        for ci in range(8):
            k, v = _synthetic_layer(torch, 1, Hkv, 512, D, 78 + ci, dev)
            chunks.append((k.to(torch.bfloat16), v.to(torch.bfloat16),
                           torch.randn((1, Hq, 512, D), device=dev).to(torch.bfloat16)))
        torch.cuda.synchronize()
        s_, e_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s_.record()
        for k, v, q in chunks:
            c.update_and_fetch(k, v)
            c.fused_sdpa(q, 1 / math.sqrt(D), causal=True)
        e_.record()
        torch.cuda.synchronize()
        return s_.elapsed_time(e_)
    return prefill_pass


def _flash_prefill_case(torch, K, dev, S, H=32, D=128):
    """Causal self-attention over plain fp16 K/V, one sequence, H heads (no GQA), S_q = S_kv = S: the
    shape the reference quotes its flash-prefill kernel on.  Returns (call, flops)."""
    q = torch.randn((1, H, S, D), device=dev).to(torch.float16)
    k = torch.randn((1, H, S, D), device=dev).to(torch.float16)
    v = torch.randn((1, H, S, D), device=dev).to(torch.float16)
    out = torch.empty_like(q)
    fn = lambda: K.kivi_packed_attend(q, k_tail=k, v_tail=v, n_tail=S, scale=D ** -0.5, causal=True, out=out)
    return fn, 4 * D * H * (S * (S + 1) // 2)


def _vq_assign_case(torch, K, dev):
    """Config 2: keys [4, 4096, 256] fp16 with channel outliers, 256 centroids of 8 dims, uint8 indices."""
    x = (torch.randn((4, 4096, 256), device=dev) * torch.exp(torch.randn(256, device=dev))).to(torch.float16)
    cb = torch.randn((256, 8), device=dev).to(torch.float16)
    return x, cb, (lambda: K.vecinfer_quantize_metal(x, cb, 8, index_dtype=torch.uint8))


def _vq_census(torch, x, cb, idx):
    """Brute force on the device in the reference's arithmetic (float32 differences, squares rounded separately,
    dimensions added left to right, allocators/vecinfer.py:301-315): whether every index is the lowest-index
    argmin, and how many sub-vectors have their two nearest centroids within 4 ulp of the best distance -- the
    cases where a different (unpinned) summation order in the reference's own backend could pick the other one."""
    sub = cb.shape[1]
    xs = x.reshape(-1, sub).float()
    c = cb.float()
    got = idx.reshape(-1).long()
    near = 0
    equal = True
    for lo in range(0, xs.shape[0], 32768):
        xv = xs[lo: lo + 32768]
        d = torch.zeros((xv.shape[0], c.shape[0]), dtype=torch.float32, device=xs.device)
        for i in range(sub):
            diff = xv[:, i: i + 1] - c[None, :, i]
            d = d + diff * diff
        best2 = torch.topk(d, 2, dim=1, largest=False).values
        # lowest index among the exact minima
        first_min = (d == best2[:, :1]).float().argmax(dim=1)
        equal = equal and bool((got[lo: lo + 32768] == first_min).all())
        ulp = torch.nextafter(best2[:, 0], torch.full_like(best2[:, 0], float("inf"))) - best2[:, 0]
        near += int(((best2[:, 1] - best2[:, 0]) <= 4 * ulp).sum())
    return {"indices_match_bruteforce": equal, "near_ties_le_4ulp": near, "sub_vectors_checked": int(xs.shape[0])}


def _only(a, torch, K, dev):
    """One side workload in a loop, for profilers: prints its average milliseconds."""
    name = a.only
    if name in ("decode_2bit_B16", "decode_2bit_B1"):
        c, fn, nbytes = _decode_2bit_case(torch, dev, 16 if name.endswith("16") else 1)
    elif name in _ROWS_CASES:
        c, fn, nbytes = _decode_rows_case(torch, dev, name)
    elif name == "vq_assign":
        x, cb, fn = _vq_assign_case(torch, K, dev)
        nbytes = None
    elif name.startswith("flash_prefill"):
        fn, flops = _flash_prefill_case(torch, K, dev, int(name.rsplit("_", 1)[1]) if name[-1].isdigit() else 8192)
        for _ in range(a.warmup):
            fn()
        ms = _event_ms(fn, max(1, a.steps), torch)
        print(json.dumps({"only": name, "ms": ms, "TFLOPs": flops / ms / 1e9}))
        return 0
    elif name == "prefill":
        run = _prefill_case(torch, dev)
        run()
        ms = min(run() for _ in range(max(1, a.steps)))
        print(json.dumps({"only": name, "ms": ms}))
        return 0
    elif name == "zipcache":
        from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory
        kk = (torch.randn((16, 8, 8192, 128), device=dev) * torch.exp(torch.randn(128, device=dev))).to(torch.float16)
        zc = KVCacheFactory.create(KVCacheConfig(method="zipcache", head_dim=128))
        fn = lambda: zc._compress(kk, True)
        nbytes = 2 * kk.numel() * 2
    elif name == "skvq":
        from veloxquant_mlx_amd.quantizers.skvq import DEFAULT_ALPHA_GRID
        kk = (torch.randn((16, 8, 8192, 128), device=dev) * torch.exp(torch.randn(128, device=dev))).to(torch.float16)
        perm = torch.stack([torch.randperm(128, device=dev) for _ in range(8)]).to(torch.int32)
        inv = torch.argsort(perm.long(), dim=-1).to(torch.int32)
        out = torch.empty_like(kk)
        fn = lambda: K.skvq_clipped_round_trip(kk, 4, 32, DEFAULT_ALPHA_GRID, perm=perm, inv=inv, out=out)
        nbytes = 2 * kk.numel() * 2
    elif name in ("quant_pack", "quant_pack_2calls", "quant_dequant"):
        k, v = _synthetic_layer(torch, 16, 8, 8192, 128, 11, dev)
        if name == "quant_pack":
            fn = lambda: K.kivi_quant_pack_kv(k, v, 32, 4, v_layout="token")
            nbytes = 2 * (k.numel() * 2 + k.numel() // 2 + (k.numel() // 32) * 4)
        elif name == "quant_pack_2calls":
            def fn():
                K.kivi_quant_pack(k, -2, 32, 4)
                K.kivi_quant_pack(v, -1, 32, 4, v_layout="token")
            nbytes = 2 * (k.numel() * 2 + k.numel() // 2 + (k.numel() // 32) * 4)
        else:
            def fn():
                K.kivi_group_quant_dequant(k, -2, 32, 15)
                K.kivi_group_quant_dequant(v, -1, 32, 15)
            nbytes = 2 * (k.numel() * 2 + k.numel() * 2)
    else:
        print(f"bench.py: unknown --only {name!r}", file=sys.stderr)
        return 2
    for _ in range(a.warmup):
        fn()
    ms = _event_ms(fn, max(1, a.steps), torch)
    out = {"only": name, "ms": ms}
    if nbytes:
        out["GBps"] = nbytes / ms / 1e6
    print(json.dumps(out))
    return 0


def _extras(torch, K, dev):
    """Side measurements the metric string also names: 2-bit 32k decode, quantise GB/s,
    VQ assignment MFMA utilisation.  Each is an event-timed loop of one kernel."""
    from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory
    ex = {}
    D, Hq, Hkv = 128, 32, 8
    # ceilings measured in this run, beside the published peaks: a 1 GiB device copy (read + write),
    # a 2 GiB read (library reduction) and a large fp16 matrix product (library GEMM)
    src = torch.empty(1 << 29, dtype=torch.float16, device=dev).normal_()
    dst = torch.empty_like(src)
    big = torch.empty(1 << 30, dtype=torch.float16, device=dev).fill_(0.25)
    ga = torch.randn((8192, 8192), device=dev).to(torch.float16)
    gb = torch.randn((8192, 8192), device=dev).to(torch.float16)
    for f in (lambda: dst.copy_(src), lambda: big.view(torch.int32).max(), lambda: ga @ gb):
        for _ in range(3):
            f()
    ms_c, ms_r, ms_g = (_side_ms(lambda: dst.copy_(src), 20, torch), _side_ms(lambda: big.view(torch.int32).max(), 20, torch),
                        _side_ms(lambda: ga @ gb, 10, torch))
    ex["measured_ceilings"] = {"copy_GBps": round((2 << 30) / ms_c / 1e6, 1), "read_GBps_library_reduction": round((2 << 30) / ms_r / 1e6, 1),
                               "gemm_f16_TFLOPs": round(2 * 8192 ** 3 / ms_g / 1e9, 1)}
    del src, dst, big, ga, gb
    for B in (1, 16):
        c, fn, nbytes = _decode_2bit_case(torch, dev, B)
        for _ in range(3):
            fn()
        ms = _side_ms(fn, 30, torch)
        ms_g = _graph_ms(fn, torch)
        ex[f"decode_2bit_32k_B{B}"] = {"ms": round(ms, 5), "GBps": round(nbytes / ms / 1e6, 1),
                                        "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4), "bytes": nbytes,
                                        "ms_graph": round(ms_g, 5), "frac_hbm_graph": round(nbytes / ms_g / 1e6 / HBM_PEAK_GBS, 4),
                                        "note": "ms: one Python call per launch; ms_graph: the same launches replayed from a HIP graph"}
        del c
    # the same 2-bit cache for eight layers in the layer-batched form: the launch ramp and the uneven finish of
    # the compute units are paid once for eight layers' bytes
    from veloxquant_mlx_amd.cache import LayerStackedKIVICache
    NL2 = 8
    layers2 = [_decode_2bit_case(torch, dev, 16)[0] for _ in range(NL2)]
    stack2 = LayerStackedKIVICache.from_layers(layers2)
    q2 = torch.randn((NL2, 16, Hq, 1, D), device=dev).to(torch.float16)
    fn2 = lambda: stack2.fused_sdpa_all(q2, 1 / math.sqrt(D))
    for _ in range(3):
        fn2()
    ms2 = _side_ms(fn2, 10, torch)
    nbytes2 = NL2 * _algorithmic_bytes_per_layer(16, Hkv, 32768, D, 2, 32)
    ex["decode_2bit_32k_B16_8_layers_one_launch"] = {
        "ms": round(ms2, 5), "ms_per_layer": round(ms2 / NL2, 5), "GBps": round(nbytes2 / ms2 / 1e6, 1),
        "frac_hbm": round(nbytes2 / ms2 / 1e6 / HBM_PEAK_GBS, 4), "bytes": nbytes2}
    del layers2, stack2, q2
    # decode outside the headline's head shape: heads of 256 channels, 3-bit codes
    for name in _ROWS_CASES:
        cv, fnv, nb = _decode_rows_case(torch, dev, name)
        for _ in range(2):
            fnv()
        msv = _side_ms(fnv, 5, torch)
        ex[name] = {"ms": round(msv, 4), "GBps": round(nb / msv / 1e6, 1), "frac_hbm": round(nb / msv / 1e6 / HBM_PEAK_GBS, 4),
                    "bytes": nb, "note": _ROWS_NOTES[name]}
        del cv, fnv
    # config 1: Llama-3-8B layer, one sequence, 8192 tokens as 2-bit group-32 codes plus a 128-token fp16 tail
    c1, fn1, nbytes1 = _decode_cfg1_case(torch, dev)
    for _ in range(3):
        fn1()
    ms1, ms1_g = _side_ms(fn1, 30, torch), _graph_ms(fn1, torch)
    ex["decode_cfg1"] = {"ms": round(ms1, 5), "GBps": round(nbytes1 / ms1 / 1e6, 1), "bytes": nbytes1,
                         "frac_hbm": round(nbytes1 / ms1 / 1e6 / HBM_PEAK_GBS, 4),
                         "ms_graph": round(ms1_g, 5), "frac_hbm_graph": round(nbytes1 / ms1_g / 1e6 / HBM_PEAK_GBS, 4),
                         "note": "32 query / 8 kv heads, B=1, 8192 packed tokens + 128 fp16 tail tokens, one launch; "
                                 "ms: one Python call per launch, ms_graph: replayed from a HIP graph"}
    del c1
    # config 0: quantise + pack of one layer's K and V [1,8,2048,128], 4-bit, group 32; and a large flush
    for name, shape in (("cfg0_[1,8,2048,128]", (1, 8, 2048, 128)), ("large_[16,8,8192,128]", (16, 8, 8192, 128))):
        k, v = _synthetic_layer(torch, shape[0], shape[1], shape[2], shape[3], 11, dev)
        qp = lambda: K.kivi_quant_pack_kv(k, v, 32, 4, v_layout="token")   # keys and values of a flush: one launch
        def rt():
            K.kivi_group_quant_dequant(k, -2, 32, 15)
            K.kivi_group_quant_dequant(v, -1, 32, 15)
        for _ in range(3):
            qp(); rt()
        n = k.numel()
        b_qp = 2 * (n * 2 + n // 2 + (n // 32) * 4)
        b_rt = 2 * (n * 2 + n * 2)
        ms_qp, ms_rt = _side_ms(qp, 30, torch), _side_ms(rt, 30, torch)
        ex[f"quant_pack_{name}"] = {"ms": round(ms_qp, 5), "GBps": round(b_qp / ms_qp / 1e6, 1), "bytes": b_qp,
                                    "note": "keys and values of the layer in one launch (kivi_quant_pack_kv)"}
        def qp2():
            K.kivi_quant_pack(k, -2, 32, 4)
            K.kivi_quant_pack(v, -1, 32, 4, v_layout="token")
        qp2()
        ms_qp2 = _side_ms(qp2, 30, torch)
        ex[f"quant_pack_two_calls_{name}"] = {"ms": round(ms_qp2, 5), "GBps": round(b_qp / ms_qp2 / 1e6, 1), "bytes": b_qp}
        ex[f"quant_dequant_{name}"] = {"ms": round(ms_rt, 5), "GBps": round(b_rt / ms_rt / 1e6, 1), "bytes": b_rt}
        if shape[0] == 1:
            # config 0's second half: the standalone dequantise of the packed layer back to fp16
            # (scalar_decode_once, metal/_scalar_attend.py:650-699): packed codes + fp16 scale / zero in,
            # fp16 K and V out -- the quantise+pack traffic in reverse
            S_, D_ = shape[2], shape[3]
            kp, ks, kz = K.kivi_quant_pack(k, -2, 32, 4)
            vp, vs, vz = K.kivi_quant_pack(v, -1, 32, 4, v_layout="token")
            def dq():
                K.kivi_dequant(kp, ks, kz, -2, 32, 4, S_, D_)
                K.kivi_dequant(vp, vs, vz, -1, 32, 4, S_, D_, v_layout="token")
            for _ in range(3):
                dq()
            ms_dq, ms_dq_g = _side_ms(dq, 30, torch), _graph_ms(dq, torch)
            ex["dequant_cfg0"] = {"ms": round(ms_dq, 5), "GBps": round(b_qp / ms_dq / 1e6, 1), "bytes": b_qp,
                                  "ms_graph": round(ms_dq_g, 5), "GBps_graph": round(b_qp / ms_dq_g / 1e6, 1),
                                  "note": "K.kivi_dequant of K and V (two launches); ms: Python call per launch, "
                                          "ms_graph: replayed from a HIP graph"}
            ms_qp_g = _graph_ms(qp, torch)
            ex[f"quant_pack_{name}"].update({"ms_graph": round(ms_qp_g, 5), "GBps_graph": round(b_qp / ms_qp_g / 1e6, 1)})
    # config 4: causal prefill of 4096 bf16 queries in chunks of 512 over a 4-bit packed prefix of 4096
    # tokens plus their own tokens, quantise-on-write (group 32, residual 128)
    prefill_pass = _prefill_case(torch, dev)
    prefill_pass()
    ms = min(prefill_pass() for _ in range(3))
    flops = 412350414848
    ex["prefill_cfg4"] = {"ms": round(ms, 4), "TFLOPs": round(flops / ms / 1e9, 1),
                          "frac_mfma_f16_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4), "flops": flops,
                          "note": "8 chunks of 512 queries: quantise-on-write append + attention per chunk; "
                                  "the packed store is sized once by fused_sdpa_max_ctx=8192"}
    # config 4's pass at the head counts of other models of the reference's scripts: GQA groups the matrix-unit kernels do
    # not tile run filled up to the next size that they do, 64-channel heads in pairs, 256-channel heads in 128-row blocks
    for tag, hq, hkv, d, note in (
            ("24q_8kv", 24, 8, 128, "Llama-3.2-3B: groups of 3 heads, 85 positions a block"),
            ("28q_4kv", 28, 4, 128, "Qwen2.5-7B: groups of 7 heads, 36 positions a block"),
            ("32q_8kv_d64", 32, 8, 64, "Llama-3.2-1B: kv heads of 64 channels in pairs, groups of 8"),
            ("12q_4kv_d256", 12, 4, 256, "Falcon3-7B: heads of 256 channels, 128-row blocks, one launch per half of the output's channels; groups of 3 heads, 42 positions a block")):
        run_ = _prefill_case(torch, dev, hq, hkv, d)
        run_()
        ms_ = min(run_() for _ in range(3))
        fl_ = flops * hq * d // (32 * 128)
        ex[f"prefill_cfg4_{tag}"] = {"ms": round(ms_, 4), "TFLOPs": round(fl_ / ms_ / 1e9, 1), "flops": fl_, "note": note}
    # causal attention over plain fp16 K/V (the reference's flash-prefill shape: 32 heads, D 128, S_q = S_kv)
    for S in (2048, 8192):
        fn, flops = _flash_prefill_case(torch, K, dev, S)
        for _ in range(3):
            fn()
        ms = _side_ms(fn, 10, torch)
        ex[f"flash_prefill_S{S}_H32"] = {"ms": round(ms, 4), "TFLOPs": round(flops / ms / 1e9, 1),
                                         "frac_mfma_f16_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4), "flops": flops,
                                         "note": "flops count the causal half only"}
    # config 2: VQ assignment, keys [4,4096,256], 256 centroids x 8 dims
    x, cb, fn = _vq_assign_case(torch, K, dev)
    for _ in range(3):
        fn()
    ms = _side_ms(fn, 20, torch)
    flops = 2 * 524288 * 256 * 8
    ex["vq_assign_cfg2"] = {"ms": round(ms, 5), "TFLOPs_gemm_form": round(flops / ms / 1e9, 2),
                            "frac_mfma_f16_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 5)}
    ex["vq_assign_cfg2"].update(_vq_census(torch, x, cb, fn()))
    # the reference's default key codebook: 4096 centroids of 4 dims (key_codebook_bits 12, key_sub_dim 4,
    # cache/options.py:36-43), Llama-shaped keys [4, 4096, 128] -> 524 288 sub-vectors, int32 indices
    x4d = (torch.randn((4, 4096, 128), device=dev) * torch.exp(torch.randn(128, device=dev))).to(torch.float16)
    cb4 = torch.randn((4096, 4), device=dev).to(torch.float16)
    fn4 = lambda: K.vecinfer_quantize_metal(x4d, cb4, 4)
    for _ in range(3):
        fn4()
    ms4 = _side_ms(fn4, 10, torch)
    flops4 = 2 * 524288 * 4096 * 4
    ex["vq_assign_4096_centroids_sub4"] = {"ms": round(ms4, 5), "TFLOPs_gemm_form": round(flops4 / ms4 / 1e9, 2),
                                           "frac_mfma_f16_peak": round(flops4 / ms4 / 1e9 / MFMA_F16_PEAK_TFLOPS, 5),
                                           "note": "codebook tiles streamed from LDS, 16 chunks of 256 centroids"}
    ex["vq_assign_4096_centroids_sub4"].update(_vq_census(torch, x4d[:1, :1024], cb4, fn4()[:1, :1024]))
    del x4d, cb4
    # Kitty keys (mixed 4/2-bit by channel variance): two launches of the key-axis round trip plus the ranking
    kc = KVCacheFactory.create(KVCacheConfig(method="kitty", head_dim=D))
    kk = (torch.randn((16, Hkv, 8192, D), device=dev) * torch.exp(torch.randn(D, device=dev))).to(torch.float16)
    fn = lambda: kc._quantize_keys(kk)
    for _ in range(3):
        fn()
    ms = _side_ms(fn, 10, torch)
    nb = 2 * kk.numel() * 2
    ex["kitty_keys_[16,8,8192,128]"] = {"ms": round(ms, 5), "GBps": round(nb / ms / 1e6, 1), "bytes": nb,
                                        "note": "fp16 keys in, fp16 mixed-precision reconstruction out"}
    # AgeTieredKV: 8192 tokens re-derived at 8 / 4 / 2 bits by age (one launch per stretch of groups of one tier)
    from veloxquant_mlx_amd.quantizers.age_tiered import age_tier_quantize_batched, assign_age_tiers, default_age_tiers
    tiers = assign_age_tiers([8192 - (i + 1) for i in range(8192)], 128, 1024)
    group_tier = [tiers[gi * 32] for gi in range(256)]
    raw = kk.reshape(16 * Hkv, 8192, D)
    fn = lambda: age_tier_quantize_batched(raw, group_tier, default_age_tiers(8, 4, 2), 32)
    for _ in range(3):
        fn()
    ms = _side_ms(fn, 10, torch)
    ex["age_tiered_keys_[16,8,8192,128]"] = {"ms": round(ms, 5), "GBps": round(nb / ms / 1e6, 1), "bytes": nb,
                                             "note": "fp16 tokens in, fp16 reconstruction out, three tiers"}
    del raw
    # SKVQ flush arithmetic: clipped group round trip with the five-factor clip search and a per-head channel order
    from veloxquant_mlx_amd.quantizers.skvq import DEFAULT_ALPHA_GRID
    perm = torch.stack([torch.randperm(D, device=dev) for _ in range(Hkv)]).to(torch.int32)
    sk_inv = torch.argsort(perm.long(), dim=-1).to(torch.int32)
    sk_out = torch.empty_like(kk)
    fn = lambda: K.skvq_clipped_round_trip(kk, 4, 32, DEFAULT_ALPHA_GRID, perm=perm, inv=sk_inv, out=sk_out)
    for _ in range(3):
        fn()
    ms = _side_ms(fn, 10, torch)
    ex["skvq_round_trip_[16,8,8192,128]"] = {"ms": round(ms, 5), "GBps": round(nb / ms / 1e6, 1), "bytes": nb,
                                             "note": "fp16 rows in, fp16 reconstruction out, 4-bit, group 32, "
                                                     "five clip factors searched per group, permuted channels"}
    del sk_out, perm, sk_inv
    # ZipCache-adapted keys: norms, stable ranks, gather, two token-axis round trips (4 / 2 bits), scatter
    zc = KVCacheFactory.create(KVCacheConfig(method="zipcache", head_dim=D))
    fn = lambda: zc._compress(kk, True)
    for _ in range(2):
        fn()
    ms = _side_ms(fn, 5, torch)
    ex["zipcache_keys_[16,8,8192,128]"] = {"ms": round(ms, 5), "GBps": round(nb / ms / 1e6, 1), "bytes": nb,
                                           "note": "fp16 keys in, fp16 mixed-precision reconstruction out: four launches "
                                                   "(row norms, routing order, one routed round trip per bit width)"}
    del zc
    del kk, kc
    # config 2 with the key transform in front: (keys / smooth) @ Hadamard -> indices, one launch,
    # and with the reconstruction written as well
    from veloxquant_mlx_amd.allocators.vecinfer import walsh_hadamard_matrix
    x4 = x.reshape(1, 4, 4096, 256)
    Hm = walsh_hadamard_matrix(256).to(dev)
    sm = torch.exp(torch.randn((4, 256), device=dev) * 0.3)
    for name, hat in (("indices", False), ("indices+k_hat", True)):
        fn = lambda: K.vecinfer_encode_decode_metal(x4, cb, 8, Hm, sm, index_dtype=torch.uint8, want_k_hat=hat)
        for _ in range(3):
            fn()
        ms = _side_ms(fn, 20, torch)
        nbytes = x4.numel() * 2 + x4.numel() // 8 + (x4.numel() * 2 if hat else 0)
        ex[f"vq_encode_keys_cfg2_{name}"] = {"ms": round(ms, 5), "GBps": round(nbytes / ms / 1e6, 1), "bytes": nbytes}
    # attention straight from VecInfer indices: 32768 tokens, 8 kv heads x 4 query heads, D 128 in 16
    # sub-vectors of 256 centroids (uint8 indices, 32 B per token and kv head); LDS-bound by design
    for B in (1, 16):
        ki = torch.randint(0, 256, (B, Hkv, 32768, 16), device=dev).to(torch.uint8)
        vi = torch.randint(0, 256, (B, Hkv, 32768, 16), device=dev).to(torch.uint8)
        kcb, vcb = cb, torch.randn((256, 8), device=dev).to(torch.float16)
        q = torch.randn((B, Hq, 1, D), device=dev).to(torch.float16)
        fn = lambda: K.metal_fused_sdpa(q, ki, kcb, vi, vcb, 1 / math.sqrt(D))
        for _ in range(3):
            fn()
        ms = _side_ms(fn, 30, torch)
        nbytes = 2 * ki.numel()
        lds_ops = B * Hq * 32768 * 16 * 2 / 64    # one look-up and one histogram addition per row, token and sub-vector, 64 lanes an instruction
        ex[f"index_attend_32k_B{B}"] = {"ms": round(ms, 5), "GBps": round(nbytes / ms / 1e6, 1), "bytes": nbytes,
                                        "lds_cycles_per_wave_op_per_cu": round(ms * 1e-3 * 2.1e9 * 256 / lds_ops, 2)}
    # the same at the head shape of config 2's model (12 query / 4 kv heads, D 256 in 32 sub-vectors): one query row a block
    ki = torch.randint(0, 256, (16, 4, 32768, 32), device=dev).to(torch.uint8)
    vi = torch.randint(0, 256, (16, 4, 32768, 32), device=dev).to(torch.uint8)
    q = torch.randn((16, 12, 1, 256), device=dev).to(torch.float16)
    fn = lambda: K.metal_fused_sdpa(q, ki, kcb, vi, vcb, 1 / math.sqrt(256))
    for _ in range(3):
        fn()
    ms = _side_ms(fn, 30, torch)
    ex["index_attend_d256_32k_B16"] = {"ms": round(ms, 5), "GBps": round(2 * ki.numel() / ms / 1e6, 1), "bytes": 2 * ki.numel()}
    return ex


def _unpacked_sequences(np, torch, cache, n_seq, ctx, D, bits, g):
    """Codes (uint8) and float32 scale / zero of the first ``n_seq`` sequences of a resident packed
    cache, in the reference's layout: keys ``[B,H,S,D]`` + ``[B,H,S/g,D]``, values ``[B,H,S,D]`` +
    ``[B,H,S,D/g]``."""
    from oracle import kivi as ok
    per = 32 // bits
    kp = cache._kp[:n_seq, :, :ctx].cpu().numpy().view(np.uint32)
    codes_k = ok.unpack_indices(kp, bits, D)
    ks = cache._ks[:n_seq, :, : ctx // g].float().cpu().numpy()
    kz = cache._kz[:n_seq, :, : ctx // g].float().cpu().numpy()
    vp = cache._vp[:n_seq, :, : ctx // per].cpu().numpy().view(np.uint32)       # [n,H,ctx/per,D]
    codes_v = np.ascontiguousarray(ok.unpack_indices(np.ascontiguousarray(vp.swapaxes(-1, -2)), bits, ctx).swapaxes(-1, -2))
    vs = np.ascontiguousarray(cache._vs[:n_seq, :, :, :ctx].float().cpu().numpy().swapaxes(-1, -2))
    vz = np.ascontiguousarray(cache._vz[:n_seq, :, :, :ctx].float().cpu().numpy().swapaxes(-1, -2))
    return codes_k, ks, kz, codes_v, vs, vz


def _timed(fn, min_seconds, max_reps=50):
    fn()                                  # warm-up (allocator, thread pool)
    t0 = time.perf_counter()
    reps = 0
    while reps < max_reps and (reps == 0 or time.perf_counter() - t0 < min_seconds):
        fn()
        reps += 1
    return (time.perf_counter() - t0) / reps, reps


def _cpu_baselines(np, torch, cache, q_layer, ctx, Hkv, D, bits, g, scale):
    """The reference's CPU path (oracle/cpu_path.py: its pure-MLX operations restated one for one on
    torch CPU tensors, same materialised intermediates) timed on this box's host cores on bounded
    samples of the four workloads, and the scalar C oracle (one thread) on the decode sample.
    Returns (headline cpu_baseline = decode, dict of the others)."""
    from oracle import cpu_path as cp, cref
    cores = torch.get_num_threads()
    model = cp.cpu_model()
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))

    # decode (the headline workload): one sequence of one layer, dequantise-then-SDPA
    codes_k, ks, kz, codes_v, vs, vz = _unpacked_sequences(np, torch, cache, 1, ctx, D, bits, g)
    qn = q_layer[:1].cpu()
    args = [t(a) for a in (codes_k, ks, kz, codes_v, vs, vz)]
    dt, reps = _timed(lambda: cp.decode_dequant_then_sdpa(qn, *args, g, scale), 6.0)
    nbytes = _algorithmic_bytes_per_layer(1, Hkv, ctx, D, bits, g)
    head = {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": cores, "kind": "port", "cpu_model": model,
            "sample": f"one sequence of one layer ({Hkv} kv heads x {ctx} tokens, 32 query heads): the reference's "
                      f"dequantise-then-SDPA arm (benchmark_real_model_scalar_attend.py:194-217) restated on torch CPU "
                      f"(oracle/cpu_path.py), {cores} threads, {reps} repetitions of {dt:.3f} s; GB/s of the same "
                      f"algorithmic packed bytes the GPU figure counts"}
    others = {}
    # the scalar C port of the fused decode arithmetic, one thread, same sample
    cref.lib()
    qf = qn.float().numpy()
    cargs = (codes_k, ks, kz, np.ascontiguousarray(codes_v), vs, vz)
    dtc, repsc = _timed(lambda: cref.attend(qf, *cargs, g, scale), 3.0, max_reps=5)
    others["decode_scalar_c_port"] = {"GBps": round(nbytes / dtc / 1e9, 4), "cores": 1, "seconds": round(dtc, 3),
                                      "note": "oracle/c/kv_oracle.c:kvo_attend, one thread, same sample"}
    del codes_k, codes_v, args, cargs

    # config 0: 4-bit group-32 round trip of K (per channel) and V (per token), [1,8,2048,128] fp16
    rng = np.random.default_rng(0)
    f = np.exp(rng.standard_normal(128)).astype(np.float32)
    k0 = t((rng.standard_normal((1, 8, 2048, 128)).astype(np.float32) * f).astype(np.float16))
    v0 = t(rng.standard_normal((1, 8, 2048, 128)).astype(np.float16))
    dt0, reps0 = _timed(lambda: (cp.kivi_round_trip(k0, -2, 32, 15), cp.kivi_round_trip(v0, -1, 32, 15)), 3.0)
    others["cfg0_round_trip"] = {"GBps": round(16777216 / dt0 / 1e9, 3), "ms": round(dt0 * 1e3, 3), "cores": cores, "bytes": 16777216,
                                 "note": "KIVIKVCache._quant_dequant_along (kivi_cache.py:181-201), K and V of config 0, full size"}
    # config 2: VQ assignment at full size, chunked difference tensor
    x2 = t((rng.standard_normal((4, 4096, 256)).astype(np.float32) * np.exp(rng.standard_normal(256)).astype(np.float32)).astype(np.float16))
    cb2 = t(rng.standard_normal((256, 8)).astype(np.float16))
    dt2, reps2 = _timed(lambda: cp.quantize_vq(x2, cb2, 8), 4.0, max_reps=10)
    others["cfg2_vq_assign"] = {"ms": round(dt2 * 1e3, 2), "TFLOPs_gemm_form": round(2 * 524288 * 256 * 8 / dt2 / 1e12, 4), "cores": cores,
                                "note": "quantize_vq (allocators/vecinfer.py:281-318), 524288 sub-vectors x 256 centroids, full size"}
    # config 4: chunked quantise-on-write prefill at full size (float32 arithmetic over the fp16 history)
    kc = [t((rng.standard_normal((1, 8, 512, 128)).astype(np.float32) * f).astype(np.float16)) for _ in range(8)]
    vc = [t(rng.standard_normal((1, 8, 512, 128)).astype(np.float16)) for _ in range(8)]
    qc = [t(rng.standard_normal((1, 32, 512, 128)).astype(np.float16)) for _ in range(8)]
    pk = t((rng.standard_normal((1, 8, 4096, 128)).astype(np.float32) * f).astype(np.float16))
    pv = t(rng.standard_normal((1, 8, 4096, 128)).astype(np.float16))
    dt4, reps4 = _timed(lambda: cp.chunked_prefill(qc, kc, vc, pk, pv, 4, 32, 128, 1 / math.sqrt(128)), 4.0, max_reps=5)
    others["cfg4_prefill"] = {"ms": round(dt4 * 1e3, 1), "TFLOPs": round(412350414848 / dt4 / 1e12, 4), "cores": cores,
                              "note": "KIVIKVCache.update_and_fetch per chunk (kivi_cache.py:206-262) + dense causal SDPA over the "
                                      "whole history, 8 chunks of 512 queries, full size"}
    others["cpu_model"] = model
    return head, others


# ---- HBM traffic of the headline kernel, measured with rocprofv3 --pmc and kept under profiles/
def _kernel_source_sha():
    import hashlib
    h = hashlib.sha256()
    d = os.path.join(ROOT, "veloxquant_mlx_amd", "csrc")
    # the sources of the decode launch the traffic figure belongs to (the prefill and vector kernels may change freely)
    decode_sources = ("attend.hip", "attend.hpp", "attend_mfma.hip", "attend_mfma.hpp", "attend_mfma_packed.hpp")
    for name in sorted(os.listdir(d)):
        if name in decode_sources or (name.startswith("attend_mfma_packed_") and name.endswith(".hip")):
            with open(os.path.join(d, name), "rb") as f:
                h.update(name.encode())
                h.update(f.read())
    return h.hexdigest()


def _recorded_traffic(key):
    """Bytes per launch from profiles/hbm_traffic.json, or None when the attention sources have
    changed since the counters were taken (the figure would be stale)."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            rec = json.load(f).get(key)
    except (OSError, ValueError):
        return None
    if not rec or rec.get("attend_sources_sha256") != _kernel_source_sha():
        return None
    return rec.get("traffic_bytes")


if __name__ == "__main__":
    sys.exit(main())
