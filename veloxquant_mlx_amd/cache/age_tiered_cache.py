"""AgeTieredKV cache (``method="age_tiered"``): every token is kept, at a bit width set by how long
ago it was written; a group of tokens is re-derived from its never-quantised copy when its oldest
token crosses a tier boundary.  Mirrors ``AgeTieredKVCache``
(veloxquant_mlx/cache/age_tiered_cache.py:38-388): position-aligned groups, a group's tier = the
tier of its first token, a group is recomputed only when its tier changed or it was not yet full.

A sibling of KIVI on the same kernel: every recomputed stretch of groups is a launch of the
key-axis group round trip, for keys and values.  Raw and reconstructed tokens live in buffers
that grow geometrically; the reference concatenates per call, the contents are the same.
"""

from __future__ import annotations

from typing import Any

import torch

from .. import kernels as K
from ..core.exceptions import QuantizerConfigError
from ..quantizers.age_tiered import (MID, OLD, RECENT, age_tier_quantize_batched, age_tiered_bytes, assign_age_tiers,
                                     default_age_tiers, full_fp16_bytes)
from ._fp16_cache import FP16KVCache


class AgeTieredKVCache(FP16KVCache):
    def __init__(self, config: Any) -> None:
        super().__init__()
        if not K._lib.library_present():
            raise RuntimeError("AgeTieredKVCache: the HIP kernel library is not available on this build; there is no fallback path.")
        self._age_recent_boundary = int(getattr(config, "age_recent_boundary", 128))
        self._age_mid_boundary = int(getattr(config, "age_mid_boundary", 1024))
        if self._age_recent_boundary <= 0:
            raise QuantizerConfigError(
                f"AgeTieredKVCache: age_recent_boundary must be > 0, got {self._age_recent_boundary}.")
        if self._age_mid_boundary < self._age_recent_boundary:
            raise QuantizerConfigError(
                f"AgeTieredKVCache: age_mid_boundary ({self._age_mid_boundary}) must be "
                f">= age_recent_boundary ({self._age_recent_boundary}).")
        bits = [int(getattr(config, n, d)) for n, d in (("age_bits_recent", 8), ("age_bits_mid", 4), ("age_bits_old", 2))]
        for name, b in zip(("age_bits_recent", "age_bits_mid", "age_bits_old"), bits):
            if not 1 <= b <= 16:
                raise QuantizerConfigError(f"AgeTieredKVCache: {name} must be in [1, 16], got {b}.")
        self._tiers = default_age_tiers(*bits)
        self._group_size = int(getattr(config, "age_group_size", 32))
        self._head_dim = int(getattr(config, "head_dim", 128))
        self._B = self._H = 0
        self._n = 0                       # tokens per (b, h) row
        self._raw: list[torch.Tensor | None] = [None, None]   # keys, values: [G, cap, D], never quantised
        self._out: list[torch.Tensor | None] = [None, None]   # [G, cap, D], the reconstruction handed out
        self._group_tier: list[int] = []
        self._tokens_seen_total = 0
        self._current_position = 0
        self._age_tiered_bytes = 0
        self._full_seq_bytes = 0
        self._storage_dtype: torch.dtype | None = None

    # ------------------------------------------------------------------ storage
    def _append_raw(self, which: int, step: torch.Tensor) -> None:
        G, S, D = step.shape
        buf = self._raw[which]
        if buf is None or self._n + S > buf.shape[1]:
            cap = max(self._n + S, 2 * (0 if buf is None else buf.shape[1]), 256)
            for store in (self._raw, self._out):
                new = torch.zeros((G, cap, D), dtype=step.dtype, device=step.device)
                if store[which] is not None and self._n:
                    new[:, : self._n] = store[which][:, : self._n]
                store[which] = new
        self._raw[which][:, self._n: self._n + S] = step

    def _requantize(self, which: int, n: int, n_prev: int, new_group_tier: list[int]) -> None:
        """Recompute from the raw copy the groups whose tier changed or that were not full (age_tiered_cache.py:248-331)."""
        gs = self._group_size
        n_groups = len(new_group_tier)
        prev = self._group_tier
        reusable = [g < len(prev) and prev[g] == new_group_tier[g] and (g + 1) * gs <= n_prev for g in range(n_groups)]
        raw, out = self._raw[which], self._out[which]
        g = 0
        while g < n_groups:
            end_g = g
            while end_g < n_groups and reusable[end_g] == reusable[g]:
                end_g += 1
            if not reusable[g]:
                a, b = g * gs, min(end_g * gs, n)
                out[:, a:b] = age_tier_quantize_batched(raw[:, a:b], new_group_tier[g:end_g], self._tiers, gs)
            g = end_g

    # ------------------------------------------------------------------ protocol
    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        B, H, S, D = keys.shape
        if self._raw[0] is None:
            self._B, self._H = B, H
        if self._storage_dtype is None:
            self._storage_dtype = torch.bfloat16 if keys.dtype == values.dtype == torch.bfloat16 else torch.float16
        self._full_seq_bytes += full_fp16_bytes(B * H * S, D)
        self._tokens_seen_total += B * H * S
        self._current_position += S
        G = B * H
        n_prev = self._n
        self._append_raw(0, keys.reshape(G, S, D).to(self._storage_dtype))
        self._append_raw(1, values.reshape(G, S, D).to(self._storage_dtype))
        n = self._n = n_prev + S
        gs = self._group_size
        tiers = self._token_tiers(n)
        new_group_tier = [tiers[g * gs] for g in range((n + gs - 1) // gs)]
        self._requantize(0, n, n_prev, new_group_tier)
        self._requantize(1, n, n_prev, new_group_tier)
        self._group_tier = new_group_tier
        self._age_tiered_bytes = age_tiered_bytes(self._tier_counts_from_tiers(tiers), self._tiers, self._head_dim)
        self.keys = self._out[0].view(B, H, -1, D)
        self.values = self._out[1].view(B, H, -1, D)
        self.offset = n
        return self.keys[:, :, :n], self.values[:, :, :n]

    def _token_tiers(self, n: int) -> list[int]:
        return assign_age_tiers([self._current_position - (i + 1) for i in range(n)], self._age_recent_boundary,
                                self._age_mid_boundary)

    def _tier_counts_from_tiers(self, tiers) -> dict[int, int]:
        counts = {RECENT: 0, MID: 0, OLD: 0}
        if tiers is None or self._out[0] is None:
            return counts
        for t in tiers:
            counts[t] += 1
        n_heads = int(self._out[0].shape[0])
        return {k: v * n_heads for k, v in counts.items()}

    def _accumulate_tier_counts(self) -> dict[int, int]:
        if self._out[0] is None:
            return {RECENT: 0, MID: 0, OLD: 0}
        return self._tier_counts_from_tiers(self._token_tiers(self._n))

    def is_trimmable(self) -> bool:
        """False: the per-token tier state does not roll back (age_tiered_cache.py:335-340)."""
        return False

    # ------------------------------------------------------------------ properties
    @property
    def age_tiered_bytes(self) -> int:
        return self._age_tiered_bytes

    @property
    def full_seq_bytes(self) -> int:
        return self._full_seq_bytes

    @property
    def compression_ratio(self) -> float:
        return 1.0 if self._age_tiered_bytes == 0 else self._full_seq_bytes / self._age_tiered_bytes

    @property
    def tokens_seen(self) -> int:
        return self._tokens_seen_total

    @property
    def tokens_kept(self) -> int:
        return self._n

    @property
    def tokens_recent(self) -> int:
        return self._accumulate_tier_counts()[RECENT]

    @property
    def tokens_mid(self) -> int:
        return self._accumulate_tier_counts()[MID]

    @property
    def tokens_old(self) -> int:
        return self._accumulate_tier_counts()[OLD]


__all__ = ["AgeTieredKVCache"]
