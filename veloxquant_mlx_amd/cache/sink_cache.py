"""KIVI with protected high-key-norm tokens (``method="kivi_sink"``): the
``n_sink_tokens`` positions with the largest key norm of every sequence stay in fp16, and
are kept out of the min/max of the token groups they sit in; everything else is KIVI.
Mirrors ``SinkProtectedKVCache`` (veloxquant_mlx/cache/sink_cache.py:44-278): same selection
signal (key L2 norm averaged over kv heads, running top-k per batch element), same
neighbour substitution before the group parameters are computed, same accounting.

The quantise-dequantise round trip runs on the HIP kernel; selection is a handful of host
integers per call, as in the reference.  The packed (``fused_sdpa``) modes of
``KIVIKVCache`` are not offered here: a protected row would have to be masked out of the
packed prefix inside the decode kernel."""

from __future__ import annotations

import math
from typing import Any

import torch

from ..core.exceptions import QuantizerConfigError
from ._fp16_cache import FP16KVCache
from .kivi_cache import KIVIKVCache


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
        self._sink_norms: list[dict[int, float]] = []
        self._sink_fp16_bytes = 0

    # ------------------------------------------------------------------ sink bookkeeping
    def _update_sinks(self, keys: torch.Tensor, start_pos: int) -> list:
        """Fold the block's key norms into every batch element's running top-k (sink_cache.py:87-112)."""
        B = keys.shape[0]
        if len(self._sink_norms) < B:
            self._sink_norms.extend({} for _ in range(B - len(self._sink_norms)))
        if self._n_sink == 0:
            return [set() for _ in range(B)]
        per_tok = torch.linalg.vector_norm(keys.float(), dim=-1).mean(dim=1).tolist()   # [B, S]
        for b in range(B):
            norms_b = self._sink_norms[b]
            for i, v in enumerate(per_tok[b]):
                norms_b[start_pos + i] = float(v)
            if len(norms_b) > self._n_sink:
                self._sink_norms[b] = dict(sorted(norms_b.items(), key=lambda kv: -kv[1])[: self._n_sink])
        return [set(self._sink_norms[b].keys()) for b in range(B)]

    # ------------------------------------------------------------------ protocol
    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        """Quantise aged-out tokens except sinks; keep residual + sinks fp16 (sink_cache.py:117-198)."""
        B, H, S, D = keys.shape
        self._shape_bhd = (B, H, D)
        start = self.offset
        sinks_per_batch = self._update_sinks(keys, start)
        k_all, v_all = FP16KVCache.update_and_fetch(self, keys, values)

        new_boundary = self._quantization_boundary()
        n_quant_now = new_boundary - self._n_quantized
        n_sink_in_block = 0
        if n_quant_now > 0:
            lo, hi = self._n_quantized, new_boundary
            k_region, v_region = self.keys[:, :, lo:hi], self.values[:, :, lo:hi]
            local = [sorted(p - lo for p in sinks_per_batch[b] if lo <= p < hi) for b in range(B)]
            if any(local):
                # a sink must not set its group's min/max: stand-in rows before the parameters are computed
                k_region, v_region = k_region.clone(), v_region.clone()
                for b in range(B):
                    sink_set = set(local[b])
                    for idx in local[b]:
                        src = idx - 1
                        while src in sink_set and src > 0:
                            src -= 1
                        if src < 0 or src in sink_set:
                            src = idx + 1
                            while src in sink_set and src < n_quant_now - 1:
                                src += 1
                        if 0 <= src < n_quant_now and src not in sink_set:
                            k_region[b, :, idx] = self.keys[b, :, lo + src]
                            v_region[b, :, idx] = self.values[b, :, lo + src]
            k_q = self._quant_dequant_along(k_region, axis=-2)
            v_q = self._quant_dequant_along(v_region, axis=-1)
            for b in range(B):
                n_sink_in_block = max(n_sink_in_block, len(local[b]))
                for idx in local[b]:
                    k_q[b, :, idx] = self.keys[b, :, lo + idx]
                    v_q[b, :, idx] = self.values[b, :, lo + idx]
            self.keys[:, :, lo:hi] = k_q
            self.values[:, :, lo:hi] = v_q
            self._n_quantized = new_boundary
            k_all, v_all = self.keys[:, :, : self.offset], self.values[:, :, : self.offset]
        self._account_bytes_with_sinks(B, H, S, D, n_quant_now, n_sink_in_block)
        return k_all, v_all

    def trim(self, n: int) -> int:
        """Drop the last ``n`` tokens; frontier, sink candidates and accounting roll back
        (sink_cache.py:200-225)."""
        old_nq = self._n_quantized
        trimmed = FP16KVCache.trim(self, n)
        if not trimmed:
            return trimmed
        n_rolled = self._rollback_frontier(self.offset)
        n_sink_rolled = 0
        for b, norms_b in enumerate(self._sink_norms):
            n_sink_rolled = max(n_sink_rolled, sum(1 for p in norms_b if self._n_quantized <= p < old_nq))
            self._sink_norms[b] = {p: v for p, v in norms_b.items() if p < self.offset}
        n_sink_rolled = min(n_sink_rolled, n_rolled)
        B, H, D = self._shape_bhd
        self._rollback_bytes(trimmed, n_rolled - n_sink_rolled)
        self._sink_fp16_bytes = max(0, self._sink_fp16_bytes - n_sink_rolled * D * 2 * 2 * H * B)
        return trimmed

    def _account_bytes_with_sinks(self, B: int, H: int, S: int, D: int, n_quant_now: int, n_sink: int) -> None:
        """KIVI accounting with the sinks split out (sink_cache.py:227-256)."""
        n_compressed = n_quant_now - n_sink
        gs = self._group_size
        if n_compressed > 0:
            code = math.ceil(n_compressed * D * self._b / 8) * H * B
            self._key_bytes_compressed += code + math.ceil(n_compressed / gs) * D * 2 * 2 * H * B
            self._value_bytes_compressed += code + n_compressed * math.ceil(D / gs) * 2 * 2 * H * B
        self._sink_fp16_bytes += n_sink * D * 2 * 2 * H * B
        self._residual_fp16_bytes = (self.offset - self._n_quantized) * D * 2 * 2 * H * B
        self._key_bytes_fp16 += H * B * S * D * 2
        self._value_bytes_fp16 += H * B * S * D * 2
        self._tokens_seen += S

    # ------------------------------------------------------------------ reporting
    @property
    def sink_fp16_bytes(self) -> int:
        """Bytes held in fp16 for protected sink tokens (keys + values)."""
        return self._sink_fp16_bytes

    @property
    def sink_positions(self) -> list:
        """Protected absolute positions of batch element 0, highest norm first."""
        return self.sink_positions_for(0)

    def sink_positions_for(self, b: int) -> list:
        if b >= len(self._sink_norms):
            return []
        return [p for p, _ in sorted(self._sink_norms[b].items(), key=lambda kv: -kv[1])]


__all__ = ["SinkProtectedKVCache"]
