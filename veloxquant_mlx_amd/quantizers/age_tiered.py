"""AgeTieredKV primitives: a token's bit width follows from its age alone.  Mirrors
veloxquant_mlx/quantizers/age_tiered.py:52-203.  The round trip of a run of token groups is the
key-axis group kernel (``vq_kivi_quant_dequant``), for keys and values alike (both are grouped
along tokens here)."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import kernels as K

RECENT, MID, OLD = 0, 1, 2


@dataclass(frozen=True)
class AgeTierConfig:
    tier: int
    bits: int


def default_age_tiers(bits_recent: int, bits_mid: int, bits_old: int) -> tuple[AgeTierConfig, ...]:
    return (AgeTierConfig(RECENT, bits_recent), AgeTierConfig(MID, bits_mid), AgeTierConfig(OLD, bits_old))


def assign_age_tiers(ages, age_recent_boundary: int, age_mid_boundary: int) -> list[int]:
    """age < recent boundary -> RECENT, < mid boundary -> MID, else OLD (age_tiered.py:69-96)."""
    return [RECENT if a < age_recent_boundary else MID if a < age_mid_boundary else OLD for a in ages]


def _round_trip(x: torch.Tensor, bits: int, group_size: int) -> torch.Tensor:
    """``[G, N, D]`` -> round trip along tokens in ``x.dtype``; the reconstruction passes through float16
    (``_group_quant_dequant_batched(...).astype(raw.dtype)``, age_tiered.py:171)."""
    if bits >= 16 or x.shape[1] == 0:
        return x
    levels = (1 << bits) - 1
    if x.dtype == torch.float16:
        return K.kivi_group_quant_dequant(x, -2, group_size, levels)
    return K.kivi_group_quant_dequant(x.float(), -2, group_size, levels).to(torch.float16).to(x.dtype)


def age_tier_quantize(x: torch.Tensor, bits: int, group_size: int = 32) -> torch.Tensor:
    """A same-tier run ``[N, D]`` (age_tiered.py:99-114)."""
    return _round_trip(x[None], bits, group_size)[0]


def age_tier_quantize_batched(raw: torch.Tensor, group_tier, tiers_config, group_size: int = 32) -> torch.Tensor:
    """``raw [G, N, D]`` with one tier per ``group_size`` window (age_tiered.py:117-174).  Windows are
    independent, so every stretch of windows that share a tier is one launch at that tier's bit width."""
    g, n, d = raw.shape
    if n == 0:
        return raw
    bits = {c.tier: c.bits for c in tiers_config}
    if raw.dtype == torch.float16 and d == 128 and group_size in (32, 64) and len(group_tier) * group_size >= n:
        # one launch with a level count per window (0: a tier kept in 16 bits passes through)
        levels = torch.tensor([0.0 if bits[t] >= 16 else float((1 << bits[t]) - 1) for t in group_tier[: -(-n // group_size)]],
                              dtype=torch.float32, device=raw.device)
        return K.kivi_group_quant_dequant_grouplevels(raw, levels, group_size)
    out = torch.empty_like(raw)
    i, n_groups = 0, len(group_tier)
    while i < n_groups:
        j = i
        while j < n_groups and group_tier[j] == group_tier[i]:
            j += 1
        a, b = i * group_size, min(j * group_size, n)
        out[:, a:b] = _round_trip(raw[:, a:b], bits[group_tier[i]], group_size)
        i = j
    return out


def age_tiered_bytes(tier_counts: dict, tiers, head_dim: int) -> int:
    """Stored bytes of keys + values for the given per-tier token counts (age_tiered.py:177-196)."""
    by_tier = {c.tier: c.bits for c in tiers}
    return sum(n * ((head_dim * by_tier[t] + 7) // 8) * 2 for t, n in tier_counts.items() if n > 0)


def full_fp16_bytes(tokens_seen: int, head_dim: int) -> int:
    return tokens_seen * head_dim * 2 * 2


__all__ = ["RECENT", "MID", "OLD", "AgeTierConfig", "default_age_tiers", "assign_age_tiers", "age_tier_quantize",
           "age_tier_quantize_batched", "age_tiered_bytes", "full_fp16_bytes"]
