"""KIVI with protected high-key-norm tokens (``method="kivi_sink"``).

What it does is the reference's ``SinkProtectedKVCache`` (veloxquant_mlx/cache/sink_cache.py:44-278):
per sequence of the batch, the ``n_sink_tokens`` positions with the largest key norm (L2 over
channels, mean over kv heads) seen so far stay exact; when such a position ages out of the residual
window its row neither takes part in its group's min/max (the nearest unprotected row of the
block stands in for it, the one before it if there is one) nor is replaced by its reconstruction.
Everything else is KIVI.

How it is done here: the running top-k lives in two small host tensors ``[B, n]`` kept ordered
by (norm descending, position ascending), which is the order the reference's stable sort of its
position->norm mapping yields; a flush turns the protected positions of the block into one
gather index and one row mask per batch element and runs gather -> group round trip -> select
on the device for the whole batch at once.  The packed (``fused_sdpa``) modes of ``KIVIKVCache``
are not offered: a protected row would have to be hidden from the packed prefix inside the
attention kernels.
"""

from __future__ import annotations

from typing import Any

import torch

from ..core.exceptions import QuantizerConfigError
from ._fp16_cache import FP16KVCache
from .kivi_cache import KIVIKVCache

_NO_POS = torch.iinfo(torch.int64).max      # position of an empty candidate slot (orders last)


class _TopNorms:
    """Per-sequence running top-``n`` of (norm, position), on the host."""

    def __init__(self, n: int) -> None:
        self.n = n
        self.norm = torch.empty((0, n), dtype=torch.float32)
        self.pos = torch.empty((0, n), dtype=torch.int64)

    def _grow(self, B: int) -> None:
        have = self.norm.shape[0]
        if have < B:
            self.norm = torch.cat([self.norm, torch.full((B - have, self.n), float("-inf"))])
            self.pos = torch.cat([self.pos, torch.full((B - have, self.n), _NO_POS)])

    def fold(self, norms: torch.Tensor, first_pos: int) -> None:
        """Merge the norms ``[B, S]`` of positions ``first_pos..`` into the first ``B`` sequences."""
        B, S = norms.shape
        self._grow(B)
        if self.n == 0:
            return
        cand_norm = torch.cat([self.norm[:B], norms], dim=1)
        cand_pos = torch.cat([self.pos[:B], torch.arange(first_pos, first_pos + S).expand(B, S)], dim=1)
        # (norm descending, position ascending): order by position, then a stable sort by norm
        by_pos = torch.argsort(cand_pos, dim=1, stable=True)
        cand_norm, cand_pos = cand_norm.gather(1, by_pos), cand_pos.gather(1, by_pos)
        by_norm = torch.argsort(cand_norm, dim=1, descending=True, stable=True)[:, : self.n]
        self.norm[:B], self.pos[:B] = cand_norm.gather(1, by_norm), cand_pos.gather(1, by_norm)

    def drop_from(self, first_dropped: int) -> None:
        """Forget candidates at positions >= ``first_dropped``."""
        gone = (self.pos >= first_dropped) & (self.pos != _NO_POS)
        if bool(gone.any()):
            self.norm[gone], self.pos[gone] = float("-inf"), _NO_POS
            order = torch.argsort(self.norm, dim=1, descending=True, stable=True)
            self.norm, self.pos = self.norm.gather(1, order), self.pos.gather(1, order)

    def positions(self, b: int) -> list[int]:
        if b >= self.pos.shape[0]:
            return []
        return [int(p) for p in self.pos[b].tolist() if p != _NO_POS]

    def inside(self, lo: int, hi: int) -> torch.Tensor:
        """Row mask ``[B, hi - lo]``: which positions of ``[lo, hi)`` are protected."""
        B = self.pos.shape[0]
        mask = torch.zeros((B, hi - lo), dtype=torch.bool)
        live = (self.pos >= lo) & (self.pos < hi)
        rows, cols = live.nonzero(as_tuple=True)
        mask[rows, self.pos[rows, cols] - lo] = True
        return mask


def _stand_in_index(protected: torch.Tensor) -> torch.Tensor:
    """For a row mask ``[B, n]`` the index ``[B, n]`` each row is read from before the group
    parameters are computed: itself when unprotected; for a protected row the nearest unprotected
    row below it, else the nearest above it, else itself (sink_cache.py:152-173)."""
    B, n = protected.shape
    idx = torch.arange(n).expand(B, n)
    below = torch.where(protected, torch.full_like(idx, -1), idx).cummax(dim=1).values
    above = torch.where(protected, torch.full_like(idx, n), idx).flip(1).cummin(dim=1).values.flip(1)
    source = torch.where(below >= 0, below, above)
    return torch.where(source < n, source, idx)


class SinkProtectedKVCache(KIVIKVCache):
    def __init__(self, config: Any) -> None:
        super().__init__(config)
        if self._fused_enabled:
            raise QuantizerConfigError(
                "SinkProtectedKVCache: fused_sdpa / packed storage is not available for method='kivi_sink'; "
                "use method='kivi' for the packed cache.")
        self._n_sink = int(getattr(config, "n_sink_tokens", 5))
        if self._n_sink < 0:
            raise QuantizerConfigError(f"SinkProtectedKVCache: n_sink_tokens={self._n_sink} must be >= 0.")
        self._top = _TopNorms(self._n_sink)
        self._sink_fp16_bytes = 0

    # ------------------------------------------------------------------ protocol
    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        B, H, S, D = keys.shape
        self._shape_bhd = (B, H, D)
        if self._n_sink:
            token_norm = torch.linalg.vector_norm(keys.float(), dim=-1).mean(dim=1)      # [B, S]
            self._top.fold(token_norm.cpu(), self.offset)
        k_all, v_all = FP16KVCache.update_and_fetch(self, keys, values)

        lo, hi = self._n_quantized, self._quantization_boundary()
        n_protected = 0
        if hi > lo:
            k_blk, v_blk = self.keys[:, :, lo:hi], self.values[:, :, lo:hi]
            protected = self._top.inside(lo, hi)[:B] if self._n_sink else None
            if protected is not None and bool(protected.any()):
                n_protected = int(protected.sum(dim=1).max())
                take = _stand_in_index(protected).to(keys.device)[:, None, :, None].expand(B, H, hi - lo, D)
                keep = protected.to(keys.device)[:, None, :, None]
                k_new = torch.where(keep, k_blk, self._quant_dequant_along(k_blk.gather(2, take), axis=-2))
                v_new = torch.where(keep, v_blk, self._quant_dequant_along(v_blk.gather(2, take), axis=-1))
            else:
                k_new = self._quant_dequant_along(k_blk, axis=-2)
                v_new = self._quant_dequant_along(v_blk, axis=-1)
            self.keys[:, :, lo:hi], self.values[:, :, lo:hi] = k_new, v_new
            self._n_quantized = hi
            k_all, v_all = self.keys[:, :, : self.offset], self.values[:, :, : self.offset]

        # accounting (sink_cache.py:227-256): of the rows flushed now, the protected ones (the largest
        # count over the batch) go to the fp16 pool, the rest are priced as plain KIVI rows
        row_bytes = D * 2 * 2 * H * B
        if hi - lo > n_protected:
            k_bytes, v_bytes = self._quantized_bytes(hi - lo - n_protected, B, H, D)
            self._key_bytes_compressed += k_bytes
            self._value_bytes_compressed += v_bytes
        self._sink_fp16_bytes += n_protected * row_bytes
        self._residual_fp16_bytes = (self.offset - self._n_quantized) * row_bytes
        self._key_bytes_fp16 += H * B * S * D * 2
        self._value_bytes_fp16 += H * B * S * D * 2
        self._tokens_seen += S
        return k_all, v_all

    def trim(self, n: int) -> int:
        """Drop the last ``n`` tokens; frontier, candidates and accounting roll back
        (sink_cache.py:200-225).  Candidates that had lost their place earlier do not come back."""
        frontier_before = self._n_quantized
        trimmed = FP16KVCache.trim(self, n)
        if not trimmed:
            return trimmed
        n_rolled = self._rollback_frontier(self.offset)
        # protected rows of the flushed region that is live again, counted as the flush counted them
        back = (self._top.pos >= self._n_quantized) & (self._top.pos < frontier_before)
        n_back = min(int(back.sum(dim=1).max()) if back.numel() else 0, n_rolled)
        self._top.drop_from(self.offset)
        B, H, D = self._shape_bhd
        self._rollback_bytes(trimmed, n_rolled - n_back)
        self._sink_fp16_bytes = max(0, self._sink_fp16_bytes - n_back * D * 2 * 2 * H * B)
        return trimmed

    # ------------------------------------------------------------------ reporting
    @property
    def sink_fp16_bytes(self) -> int:
        """Bytes held in fp16 for protected tokens (keys + values)."""
        return self._sink_fp16_bytes

    @property
    def sink_positions(self) -> list:
        """Protected absolute positions of batch element 0, highest norm first."""
        return self.sink_positions_for(0)

    def sink_positions_for(self, b: int) -> list:
        return self._top.positions(b)


__all__ = ["SinkProtectedKVCache"]
