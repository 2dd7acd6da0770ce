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
on the device for the whole batch at once.

The packed (``fused_sdpa``) modes of ``KIVIKVCache`` work as well, which the reference does not
offer: the block is packed with the stand-ins in place, the value scale / zero of a protected
position are stored as zeros (its stand-in then adds nothing to the attention output), the exact
rows go to a small side store ``[B, H, n, D]`` with their positions, and the attention call takes
the stand-ins' softmax weights out and puts the exact rows in (``sinks`` of
:func:`veloxquant_mlx_amd.kernels.kivi_packed_attend`).
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
    _one_call_append = False     # the rows of a flush pass through _pack_block

    def __init__(self, config: Any) -> None:
        super().__init__(config)
        self._n_sink = int(getattr(config, "n_sink_tokens", 5))
        if self._n_sink < 0:
            raise QuantizerConfigError(f"SinkProtectedKVCache: n_sink_tokens={self._n_sink} must be >= 0.")
        self._top = _TopNorms(self._n_sink)
        self._sink_fp16_bytes = 0
        self._flush_protected = 0        # protected rows of the flush in progress (largest count over the batch)
        self._frontier_before_trim = 0
        # packed modes: exact rows of the protected positions below the frontier
        self._side_k = self._side_v = None     # [B, H, cap, D]
        self._side_pos: list[list[int]] = []   # per sequence, slot order
        self._side_pos_dev = None              # int32 [B, cap], -1 for an unused slot

    # ------------------------------------------------------------------ protocol
    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        B, H, S, D = keys.shape
        self._shape_bhd = (B, H, D)
        if self._n_sink:
            token_norm = torch.linalg.vector_norm(keys.float(), dim=-1).mean(dim=1)      # [B, S]
            self._top.fold(token_norm.cpu(), self.offset)
        if self._memory_bound:
            return self._update_memory_bound(keys, values)
        k_all, v_all = FP16KVCache.update_and_fetch(self, keys, values)

        lo, hi = self._n_quantized, self._quantization_boundary()
        if hi > lo:
            k_blk, v_blk = self.keys[:, :, lo:hi], self.values[:, :, lo:hi]
            if self._fused_enabled:
                self._pack_block(k_blk, v_blk, lo)       # from the still-exact rows
            protected = self._top.inside(lo, hi)[:B] if self._n_sink else None
            if protected is not None and bool(protected.any()):
                self._flush_protected = int(protected.sum(dim=1).max())
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
        self._account_bytes(B, H, S, D, hi - lo if hi > lo else 0)
        return k_all, v_all

    def _account_bytes(self, B: int, H: int, S: int, D: int, n_quant_now: int) -> None:
        """sink_cache.py:227-256: of the rows flushed now, the protected ones (the largest count over
        the batch) go to the fp16 pool, the rest are priced as plain KIVI rows."""
        n_protected, self._flush_protected = min(self._flush_protected, max(n_quant_now, 0)), 0
        row_bytes = D * 2 * 2 * H * B
        if n_quant_now > n_protected:
            k_bytes, v_bytes = self._quantized_bytes(n_quant_now - n_protected, B, H, D)
            self._key_bytes_compressed += k_bytes
            self._value_bytes_compressed += v_bytes
        self._sink_fp16_bytes += n_protected * row_bytes
        self._residual_fp16_bytes = (self.offset - self._n_quantized) * row_bytes
        self._key_bytes_fp16 += H * B * S * D * 2
        self._value_bytes_fp16 += H * B * S * D * 2
        self._tokens_seen += S

    # ------------------------------------------------------------------ packed modes
    def _pack_block(self, k_blk: torch.Tensor, v_blk: torch.Tensor, lo: int) -> None:
        B, H, n, D = k_blk.shape
        protected = self._top.inside(lo, lo + n)[:B] if self._n_sink else None
        if protected is None or not bool(protected.any()):
            return super()._pack_block(k_blk, v_blk, lo)
        self._flush_protected = int(protected.sum(dim=1).max())
        dev = k_blk.device
        take = _stand_in_index(protected).to(dev)[:, None, :, None].expand(B, H, n, D)
        super()._pack_block(k_blk.gather(2, take), v_blk.gather(2, take), lo)
        seqs, rows = protected.nonzero(as_tuple=True)
        seqs_d, rows_d = seqs.to(dev), rows.to(dev)
        # the stand-ins add nothing to the attention output: value scale and zero of their positions are zeros
        if self._v_layout == "token":
            self._vs[seqs_d, :, :, rows_d + lo] = 0
            self._vz[seqs_d, :, :, rows_d + lo] = 0
        else:
            self._vs[seqs_d, :, rows_d + lo] = 0
            self._vz[seqs_d, :, rows_d + lo] = 0
        self._side_add(seqs.tolist(), [lo + r for r in rows.tolist()], k_blk[seqs_d, :, rows_d], v_blk[seqs_d, :, rows_d])

    def _side_add(self, seqs: list, positions: list, k_rows: torch.Tensor, v_rows: torch.Tensor) -> None:
        """Append exact rows ``[n, H, D]`` of (sequence, position) pairs to the side store."""
        B, H, D = self._shape_bhd
        while len(self._side_pos) < B:
            self._side_pos.append([])
        slots = []
        for b, p in zip(seqs, positions):
            slots.append(len(self._side_pos[b]))
            self._side_pos[b].append(p)
        need = max(len(ps) for ps in self._side_pos)
        cap = 0 if self._side_k is None else self._side_k.shape[2]
        if need > cap:
            new_cap = max(8, 2 * cap, need)
            side_k = torch.zeros((B, H, new_cap, D), dtype=k_rows.dtype, device=k_rows.device)
            side_v = torch.zeros_like(side_k)
            if cap:
                side_k[:, :, :cap], side_v[:, :, :cap] = self._side_k, self._side_v
            self._side_k, self._side_v = side_k, side_v
        dev = k_rows.device
        b_idx, s_idx = torch.tensor(seqs, device=dev), torch.tensor(slots, device=dev)
        self._side_k[b_idx, :, s_idx] = k_rows
        self._side_v[b_idx, :, s_idx] = v_rows
        self._side_pos_dev = None

    def _extra_attend_args(self) -> dict:
        if self._side_k is None or not any(self._side_pos):
            return {}
        if self._side_pos_dev is None:
            cap = self._side_k.shape[2]
            table = [ps + [-1] * (cap - len(ps)) for ps in self._side_pos]
            self._side_pos_dev = torch.tensor(table, dtype=torch.int32, device=self._side_k.device)
        return {"sinks": (self._side_k, self._side_v, self._side_pos_dev)}

    def _rollback_bytes(self, n_tokens: int, n_rolled: int) -> None:
        # protected rows of the flushed stretch that is live again, counted as the flush counted them
        back = (self._top.pos >= self._n_quantized) & (self._top.pos < self._frontier_before_trim)
        n_back = min(int(back.sum(dim=1).max()) if back.numel() else 0, n_rolled)
        B, H, D = self._shape_bhd
        super()._rollback_bytes(n_tokens, n_rolled - n_back)
        self._sink_fp16_bytes = max(0, self._sink_fp16_bytes - n_back * D * 2 * 2 * H * B)

    def trim(self, n: int) -> int:
        """Drop the last ``n`` tokens; frontier, candidates, side store and accounting roll back
        (sink_cache.py:200-225).  Candidates that had lost their place earlier do not come back."""
        self._frontier_before_trim = self._n_quantized
        trimmed = KIVIKVCache.trim(self, n)
        if not trimmed:
            return trimmed
        frontier = self._n_quantized
        if self._side_k is not None and any(self._side_pos):
            # rows of the side store at or past the new frontier: back into the fp16 rows they came
            # from (the memory-bound tail was just rebuilt from the packed store, stand-ins and all)
            for b, ps in enumerate(self._side_pos):
                for slot, p in enumerate(ps):
                    if frontier <= p < self.offset and self._memory_bound and self._tail_k is not None:
                        self._tail_k[b, :, p - frontier] = self._side_k[b, :, slot]
                        self._tail_v[b, :, p - frontier] = self._side_v[b, :, slot]
            kept = [[(slot, p) for slot, p in enumerate(ps) if p < frontier] for ps in self._side_pos]
            for b, pairs in enumerate(kept):
                for new_slot, (slot, _) in enumerate(pairs):
                    if new_slot != slot:
                        self._side_k[b, :, new_slot] = self._side_k[b, :, slot]
                        self._side_v[b, :, new_slot] = self._side_v[b, :, slot]
            self._side_pos = [[p for _, p in pairs] for pairs in kept]
            self._side_pos_dev = None
        self._top.drop_from(self.offset)
        return trimmed

    _N_SINK_ARRAYS = 5

    @property
    def state(self):
        """Standard mode: the fp16 history, as KIVI's.  Packed modes: KIVI's arrays followed by
        five more, the exact rows ``[B, H, n, D]`` (keys, values) with their positions ``[B, n]``
        (int32, -1 for an unused slot) and the running candidates (norms float32 ``[B, n_sink]``,
        positions int64 ``[B, n_sink]``), so that a restored cache protects what this one does."""
        base = KIVIKVCache.state.fget(self)
        if not self._fused_enabled or not base:
            return base
        ref = base[0]
        B, H, D = self._shape_bhd
        used = max([len(ps) for ps in self._side_pos], default=0)
        if used:
            side_k, side_v = self._side_k[:, :, :used], self._side_v[:, :, :used]
            table = [ps + [-1] * (used - len(ps)) for ps in self._side_pos]
            side_pos = torch.tensor(table, dtype=torch.int32, device=ref.device)
        else:
            side_k = torch.zeros((B, H, 0, D), dtype=torch.float16, device=ref.device)
            side_v, side_pos = torch.zeros_like(side_k), torch.zeros((B, 0), dtype=torch.int32, device=ref.device)
        self._top._grow(B)
        return (*base, side_k, side_v, side_pos, self._top.norm[:B].to(ref.device), self._top.pos[:B].to(ref.device))

    @state.setter
    def state(self, v) -> None:
        v = tuple(v)
        self._side_k = self._side_v = self._side_pos_dev = None
        self._side_pos = []
        self._top = _TopNorms(self._n_sink)
        if not self._fused_enabled or not v:
            KIVIKVCache.state.fset(self, v)
            return
        if len(v) < self._N_SINK_ARRAYS:
            raise ValueError(f"SinkProtectedKVCache.state: a packed state ends with {self._N_SINK_ARRAYS} arrays for the "
                             f"protected rows, got {len(v)} arrays in all")
        side_k, side_v, side_pos, top_norm, top_pos = v[-self._N_SINK_ARRAYS:]
        KIVIKVCache.state.fset(self, v[: -self._N_SINK_ARRAYS])
        B, H, D = self._shape_bhd
        used = int(side_pos.shape[1]) if side_pos.dim() == 2 else -1
        if (tuple(side_k.shape) != (B, H, used, D) or tuple(side_v.shape) != (B, H, used, D) or int(side_pos.shape[0]) != B
                or tuple(top_norm.shape) != (B, self._n_sink) or tuple(top_pos.shape) != (B, self._n_sink)):
            raise ValueError(f"SinkProtectedKVCache.state: protected rows {tuple(side_k.shape)}/{tuple(side_v.shape)}, positions "
                             f"{tuple(side_pos.shape)}, candidates {tuple(top_norm.shape)}/{tuple(top_pos.shape)} do not fit "
                             f"B={B}, H={H}, head_dim={D}, n_sink_tokens={self._n_sink}")
        table = side_pos.cpu().tolist()
        self._side_pos = [[p for p in row if p >= 0] for row in table]
        for row, ps in zip(table, self._side_pos):
            if row[: len(ps)] != ps or any(not (0 <= p < self._n_quantized) for p in ps):
                raise ValueError("SinkProtectedKVCache.state: positions of the protected rows must fill the slots from the "
                                 "front and lie below the quantised frontier")
        if used:
            cap = max(8, used)
            self._side_k = torch.zeros((B, H, cap, D), dtype=side_k.dtype, device=side_k.device)
            self._side_v = torch.zeros_like(self._side_k)
            self._side_k[:, :, :used], self._side_v[:, :, :used] = side_k, side_v
        self._top.norm = top_norm.detach().to("cpu", torch.float32).clone()
        self._top.pos = top_pos.detach().to("cpu", torch.int64).clone()
        self._rebuild_accounting()

    def _rebuild_accounting(self) -> None:
        """Restored rows priced as the flushes price them: protected ones (the largest count over
        the batch) in fp16, the rest as KIVI rows."""
        super()._rebuild_accounting()
        n_protected = max([len(ps) for ps in self._side_pos], default=0)
        B, H, D = self._shape_bhd
        if n_protected and self._n_quantized:
            k, v = self._quantized_bytes(self._n_quantized - n_protected, B, H, D)
            self._key_bytes_compressed, self._value_bytes_compressed = k, v
        self._sink_fp16_bytes = n_protected * D * 2 * 2 * H * B

    @property
    def nbytes(self) -> int:
        total = KIVIKVCache.nbytes.fget(self)
        for t in (self._side_k, self._side_v):
            if t is not None:
                total += t.numel() * t.element_size()
        return total

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
