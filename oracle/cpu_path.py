"""The reference's CPU path, restated op for op on torch CPU tensors.

TEST / MEASUREMENT INFRASTRUCTURE ONLY (see oracle/__init__.py): ``bench.py`` times these on
the GPU box's host cores as the CPU baseline.  The reference runs its pure-MLX path on the CPU
when no Metal device is present; MLX cannot be installed here, so each function below follows
the cited reference lines operation by operation and materialises the same intermediates
(the moved-axis copy, the padded copy, the group view, codes and reconstruction for KIVI; the
``[chunk, n_centroids, sub_dim]`` difference tensor for VQ; the reconstructed fp16 K/V handed
to a dense SDPA for decode).  They are checked against the numpy oracle in
tests/test_oracle_cpu_path.py.  Threads are whatever torch is configured with; callers report
``torch.get_num_threads()``.
"""

from __future__ import annotations

import math

import torch


def kivi_round_trip(x: torch.Tensor, axis: int, group_size: int, levels: int, eps: float = 1e-8) -> torch.Tensor:
    """``KIVIKVCache._quant_dequant_along`` (veloxquant_mlx/cache/kivi_cache.py:181-201)."""
    gs = group_size
    x32 = x.to(torch.float32)
    L = x32.shape[axis]
    n_groups = (L + gs - 1) // gs
    pad = n_groups * gs - L
    xm = torch.movedim(x32, axis, -1).contiguous()                 # [..., other, L]
    if pad:
        tail = xm[..., -1:]
        xm = torch.cat([xm, tail.expand(xm.shape[:-1] + (pad,))], dim=-1)
    xg = xm.reshape(xm.shape[:-1] + (n_groups, gs))               # [..., other, G, gs]
    gmin = xg.amin(dim=-1, keepdim=True)
    gmax = xg.amax(dim=-1, keepdim=True)
    scale = torch.clamp((gmax - gmin) / levels, min=eps)
    codes = torch.clamp(torch.round((xg - gmin) / scale), 0, levels)
    recon = codes * scale + gmin
    recon = recon.reshape(xm.shape)[..., :L]
    recon = torch.movedim(recon, -1, axis)
    return recon.to(x.dtype)


def quantize_vq(x: torch.Tensor, codebook: torch.Tensor, sub_dim: int) -> torch.Tensor:
    """``quantize_vq`` (veloxquant_mlx/allocators/vecinfer.py:281-318): chunked argmin over a
    materialised difference tensor, ``chunk = 1_000_000 // n_centroids``."""
    *leading, D = x.shape
    n_sub = D // sub_dim
    flat = x.reshape(*leading, n_sub, sub_dim).reshape(-1, sub_dim).to(torch.float32)
    cb = codebook.to(torch.float32)
    n_centroids = cb.shape[0]
    chunk = max(1, 1_000_000 // max(n_centroids, 1))
    chunks = []
    for start in range(0, flat.shape[0], chunk):
        sub = flat[start:start + chunk]
        diff = sub[:, None, :] - cb[None, :, :]
        d2 = (diff * diff).sum(dim=-1)
        chunks.append(torch.argmin(d2, dim=-1).to(torch.int32))
    out = chunks[0] if len(chunks) == 1 else torch.cat(chunks, dim=0)
    return out.reshape(*leading, n_sub)


def dequantized_kv(k_codes, k_scale, k_zero, v_codes, v_scale, v_zero, group_size: int, heads_per_kv: int):
    """``dequantized_kv`` (benchmark_scripts/benchmark_real_model_scalar_attend.py:194-217):
    codes ``[B,H_kv,S,D]`` uint8, key scale/zero ``[B,H_kv,S/g,D]``, value scale/zero
    ``[B,H_kv,S,D/g]`` -> fp16 K_hat, V_hat repeated to the query heads."""
    S_kv, D = k_codes.shape[2], k_codes.shape[3]
    kg = torch.arange(S_kv) // group_size
    k_hat = (k_codes.to(torch.float32) * k_scale.index_select(2, kg) + k_zero.index_select(2, kg)).to(torch.float16)
    vgi = torch.arange(D) // group_size
    v_hat = (v_codes.to(torch.float32) * v_scale.index_select(3, vgi) + v_zero.index_select(3, vgi)).to(torch.float16)
    if heads_per_kv > 1:
        k_hat = k_hat.repeat_interleave(heads_per_kv, dim=1)
        v_hat = v_hat.repeat_interleave(heads_per_kv, dim=1)
    return k_hat, v_hat


def sdpa(q, k, v, scale: float, causal: bool = False) -> torch.Tensor:
    """Dense softmax attention, queries aligned to the end of the keys, float32 arithmetic over the
    fp16 operands (the library routine the reference's unpatched path calls is
    ``mx.fast.scaled_dot_product_attention``)."""
    q32, k32, v32 = q.to(torch.float32), k.to(torch.float32), v.to(torch.float32)
    s = torch.matmul(q32, k32.transpose(-1, -2)) * scale
    if causal:
        Sq, Sk = q.shape[-2], k.shape[-2]
        vis = torch.arange(Sk)[None, :] <= (torch.arange(Sq)[:, None] + (Sk - Sq))
        s = s.masked_fill(~vis, float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.matmul(p, v32).to(q.dtype)


def decode_dequant_then_sdpa(q, k_codes, k_scale, k_zero, v_codes, v_scale, v_zero, group_size: int, scale: float):
    """The unpatched arm of the reference's decode comparison: reconstruct, then dense SDPA."""
    heads_per_kv = q.shape[1] // k_codes.shape[1]
    k_hat, v_hat = dequantized_kv(k_codes, k_scale, k_zero, v_codes, v_scale, v_zero, group_size, heads_per_kv)
    return sdpa(q, k_hat, v_hat, scale)


class KiviCpuCache:
    """``KIVIKVCache.update_and_fetch`` on the CPU (veloxquant_mlx/cache/kivi_cache.py:206-262): an
    fp16 history whose aged-out prefix is round-tripped in place in whole groups."""

    def __init__(self, bits: int, group_size: int, residual_length: int):
        self.levels, self.g, self.R = (1 << bits) - 1, group_size, residual_length
        self.keys = self.values = None
        self.n_quantized = 0

    @property
    def offset(self) -> int:
        return 0 if self.keys is None else self.keys.shape[2]

    def update_and_fetch(self, k: torch.Tensor, v: torch.Tensor):
        self.keys = k if self.keys is None else torch.cat([self.keys, k], dim=2)
        self.values = v if self.values is None else torch.cat([self.values, v], dim=2)
        boundary = (max(0, self.offset - self.R) // self.g) * self.g
        if boundary > self.n_quantized:
            lo, hi = self.n_quantized, boundary
            self.keys[:, :, lo:hi] = kivi_round_trip(self.keys[:, :, lo:hi], -2, self.g, self.levels)
            self.values[:, :, lo:hi] = kivi_round_trip(self.values[:, :, lo:hi], -1, self.g, self.levels)
            self.n_quantized = boundary
        return self.keys, self.values


def chunked_prefill(q_chunks, k_chunks, v_chunks, prefix_k, prefix_v, bits: int, group_size: int, residual_length: int,
                    scale: float):
    """Config 4 on the CPU: the prefix goes through the cache first, then each chunk is appended
    (quantise-on-write of what aged out) and attended causally with a dense SDPA over the whole
    history, GQA by repeat."""
    cache = KiviCpuCache(bits, group_size, residual_length)
    cache.update_and_fetch(prefix_k, prefix_v)
    outs = []
    for q, k, v in zip(q_chunks, k_chunks, v_chunks):
        k_all, v_all = cache.update_and_fetch(k, v)
        rep = q.shape[1] // k_all.shape[1]
        outs.append(sdpa(q, k_all.repeat_interleave(rep, dim=1), v_all.repeat_interleave(rep, dim=1), scale, causal=True))
    return outs


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


__all__ = ["kivi_round_trip", "quantize_vq", "dequantized_kv", "sdpa", "decode_dequant_then_sdpa", "KiviCpuCache",
           "chunked_prefill", "cpu_model"]
