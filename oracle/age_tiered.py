"""numpy restatement of AgeTieredKV (test infrastructure only): veloxquant_mlx/quantizers/age_tiered.py
and veloxquant_mlx/cache/age_tiered_cache.py.  The model recomputes the whole history from the raw
tokens on every call -- what the reference's incremental splice is tested to equal
(tests/cache/test_age_tiered_incremental_requantize.py:46-56)."""

from __future__ import annotations

import numpy as np

from . import kivi

RECENT, MID, OLD = 0, 1, 2


def assign_age_tiers(ages, recent_boundary: int, mid_boundary: int):
    """age_tiered.py:69-96."""
    return [RECENT if a < recent_boundary else MID if a < mid_boundary else OLD for a in ages]


def age_tiered_bytes(tier_counts: dict, bits_by_tier: dict, head_dim: int) -> int:
    """age_tiered.py:177-196: keys + values, codes only."""
    return sum(n * ((head_dim * bits_by_tier[t] + 7) // 8) * 2 for t, n in tier_counts.items() if n > 0)


class AgeTieredCacheModel:
    """``cast`` turns the float16 reconstruction into the storage dtype (identity for float16)."""

    def __init__(self, head_dim: int, recent_boundary: int = 128, mid_boundary: int = 1024, bits=(8, 4, 2),
                 group_size: int = 32, cast=None):
        self.D, self.rb, self.mb, self.g = head_dim, recent_boundary, mid_boundary, group_size
        self.bits = {RECENT: bits[0], MID: bits[1], OLD: bits[2]}
        self.cast = cast or (lambda a: a)
        self.raw_k = self.raw_v = None
        self.pos = 0
        self.tokens_seen = self.full_seq_bytes = self.age_tiered_bytes = 0

    def _tiers(self, n):
        return assign_age_tiers([self.pos - (i + 1) for i in range(n)], self.rb, self.mb)

    def _requantize(self, raw):
        """Every ``group_size`` window at the bit width of its first token's tier (age_tiered_cache.py:283-287,
        age_tiered.py:117-174); a window is independent of the others."""
        G, n, D = raw.shape
        tiers = self._tiers(n)
        out = np.empty_like(raw)
        for a in range(0, n, self.g):
            b = min(a + self.g, n)
            bits = self.bits[tiers[a]]
            if bits >= 16:
                out[:, a:b] = raw[:, a:b]
            else:
                rt = kivi.quant_dequant_along(raw[:, a:b], -2, self.g, (1 << bits) - 1, cast=lambda r: r.astype(np.float16))
                out[:, a:b] = self.cast(rt)
        return out

    def update_and_fetch(self, keys, values):
        keys, values = np.asarray(keys), np.asarray(values)
        B, H, S, D = keys.shape
        self.full_seq_bytes += B * H * S * D * 2 * 2
        self.tokens_seen += B * H * S
        self.pos += S
        k, v = keys.reshape(B * H, S, D), values.reshape(B * H, S, D)
        self.raw_k = k if self.raw_k is None else np.concatenate([self.raw_k, k], axis=1)
        self.raw_v = v if self.raw_v is None else np.concatenate([self.raw_v, v], axis=1)
        n = self.raw_k.shape[1]
        counts = self.tier_counts()
        self.age_tiered_bytes = age_tiered_bytes(counts, self.bits, self.D)
        return self._requantize(self.raw_k).reshape(B, H, n, D), self._requantize(self.raw_v).reshape(B, H, n, D)

    def tier_counts(self):
        if self.raw_k is None:
            return {RECENT: 0, MID: 0, OLD: 0}
        G, n, _ = self.raw_k.shape
        tiers = self._tiers(n)
        return {t: tiers.count(t) * G for t in (RECENT, MID, OLD)}
