"""SKVQ cache (``method="skvq"``): a sliding fp16 window; every ``skvq_window`` tokens that age past
it are round-tripped once through channel reorder -> clipped group quantisation -> inverse reorder
and frozen.  Mirrors ``SKVQKVCache`` (veloxquant_mlx/cache/skvq_cache.py:62-403): the frontier
moves in whole chunks (so one prefill and token-by-token decode leave identical state), the
per-head channel orders come from the first flushed chunk and are kept only on heads where they
lower the round-trip error, the first ``skvq_n_sink`` tokens stay exact, and the byte accounting
follows the same closed forms.

Every flush is one launch of the clipped round-trip kernel per tensor, in place on the chunk's rows
of the cache buffer (sink rows are simply left out of the launch).
"""

from __future__ import annotations

from typing import Any

import torch

from .. import kernels as K
from ..core.exceptions import QuantizerConfigError
from ..quantizers.skvq import DEFAULT_ALPHA_GRID, skvq_compressed_bytes, skvq_fp16_bytes, skvq_round_trip_batched
from ._fp16_cache import FP16KVCache


# (attribute, configuration field, type, default)
_SKVQ_FIELDS = (("_bits_k", "skvq_bits_key", int, 4), ("_bits_v", "skvq_bits_value", int, 4), ("_group_size", "skvq_group_size", int, 32),
                ("_window", "skvq_window", int, 128), ("_n_sink", "skvq_n_sink", int, 5), ("_reorder", "skvq_reorder", bool, True),
                ("_clip_search", "skvq_clip_search", bool, True), ("_clip_alpha", "skvq_clip_alpha", float, 1.0))


class SKVQKVCache(FP16KVCache):
    def __init__(self, config: Any) -> None:
        super().__init__()
        if not K._lib.library_present():
            raise RuntimeError("SKVQKVCache: the HIP kernel library is not available on this build; there is no fallback path.")
        self._D = int(config.head_dim)
        # the skvq_* fields of the configuration with the reference's defaults (skvq_cache.py:88-101)
        for attr, field, kind, default in _SKVQ_FIELDS:
            setattr(self, attr, kind(getattr(config, field, default)))
        cap = getattr(config, "skvq_max_ctx", None)
        self._max_ctx: int | None = int(cap) if cap is not None else None
        # same checks and key phrases as skvq_cache.py:103-127
        for field in ("skvq_bits_key", "skvq_bits_value"):
            width = self._bits_k if field.endswith("key") else self._bits_v
            if width < 1 or width > 8:
                raise QuantizerConfigError(f"SKVQKVCache: {field}={width} must be in [1, 8] (uint8 codes)")
        if self._group_size < 1:
            raise QuantizerConfigError(f"SKVQKVCache: skvq_group_size={self._group_size} must be >= 1")
        if self._window < 2:
            raise QuantizerConfigError(f"SKVQKVCache: skvq_window={self._window} must be >= 2 (the first chunk "
                                       f"supplies the channel statistics)")
        if not 0 <= self._n_sink < self._window:
            raise QuantizerConfigError(f"SKVQKVCache: skvq_n_sink={self._n_sink} must be in [0, skvq_window) so "
                                       f"sinks live entirely inside chunk 0")
        if not 0.0 < self._clip_alpha <= 1.0:
            raise QuantizerConfigError(f"SKVQKVCache: skvq_clip_alpha={self._clip_alpha} must be in (0, 1]")
        self._alphas = DEFAULT_ALPHA_GRID if self._clip_search else (self._clip_alpha,)
        self._perm_k: torch.Tensor | None = None   # [H, D] int32, frozen at the first flush
        self._inv_k: torch.Tensor | None = None
        self._perm_v: torch.Tensor | None = None
        self._inv_v: torch.Tensor | None = None
        self._q_end = 0                            # tokens [0, _q_end) are flushed; a multiple of the window
        self._compressed_key_bytes = self._compressed_value_bytes = 0
        self._fp16_key_bytes = self._fp16_value_bytes = 0
        self._tokens_seen = 0
        self._B = self._H = 1

    # ------------------------------------------------------------------ permutations
    def _round_trip(self, x: torch.Tensor, perm, inv, bits: int, out: torch.Tensor | None = None) -> torch.Tensor:
        """Reorder -> clipped quantise -> dequantise -> inverse reorder (skvq_cache.py:236-251), one launch."""
        return skvq_round_trip_batched(x, perm, bits, self._group_size, self._alphas, out=out, inv=inv)

    def _per_head_perms(self, chunk: torch.Tensor, bits: int):
        """Channels of each head sorted by range over the chunk's non-sink rows, kept only where that lowers the
        head's round-trip error; ties keep the identity (skvq_cache.py:186-224)."""
        B, H, r, D = chunk.shape
        x = chunk[..., self._n_sink:, :].float().contiguous()
        xh = x.transpose(0, 1).reshape(H, -1, D)
        rng = xh.amax(dim=1) - xh.amin(dim=1)
        cand = torch.argsort(rng, dim=-1, stable=True).to(torch.int32)
        cand_inv = torch.argsort(cand, dim=-1, stable=True).to(torch.int32)
        err_id = (self._round_trip(x, None, None, bits) - x).double().square().mean(dim=(0, 2, 3))
        err_cand = (self._round_trip(x, cand, cand_inv, bits) - x).double().square().mean(dim=(0, 2, 3))
        keep = (err_cand < err_id)[:, None]
        identity = torch.arange(D, dtype=torch.int32, device=chunk.device)[None, :].expand(H, D)
        return torch.where(keep, cand, identity).contiguous(), torch.where(keep, cand_inv, identity).contiguous()

    # ------------------------------------------------------------------ protocol
    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        """Append, then flush every completed chunk in place (skvq_cache.py:256-312)."""
        B, H, S, D = keys.shape
        if self._max_ctx is not None and self.offset + S > self._max_ctx:
            raise ValueError(f"SKVQKVCache: context {self.offset + S} exceeds skvq_max_ctx={self._max_ctx}")
        self._B, self._H = B, H
        super().update_and_fetch(keys, values)
        r = self._window
        while self.offset - self._q_end >= r:
            s, e = self._q_end, self._q_end + r
            if s == 0 and self._reorder:
                self._perm_k, self._inv_k = self._per_head_perms(self.keys[:, :, s:e], self._bits_k)
                self._perm_v, self._inv_v = self._per_head_perms(self.values[:, :, s:e], self._bits_v)
            s_q = s + (self._n_sink if s == 0 else 0)   # sink rows keep their exact values
            k_rows, v_rows = self.keys[:, :, s_q:e], self.values[:, :, s_q:e]
            self._round_trip(k_rows, self._perm_k, self._inv_k, self._bits_k, out=k_rows)
            self._round_trip(v_rows, self._perm_v, self._inv_v, self._bits_v, out=v_rows)
            self._account_chunk_bytes(B, H, e - s_q, D)
            self._q_end = e
        self._fp16_key_bytes += B * H * S * D * 2
        self._fp16_value_bytes += B * H * S * D * 2
        self._tokens_seen += S
        return self.keys[:, :, : self.offset], self.values[:, :, : self.offset]

    def _account_chunk_bytes(self, B: int, H: int, n_q: int, D: int) -> None:
        self._compressed_key_bytes += skvq_compressed_bytes(n_q, D, self._bits_k, self._group_size) * B * H
        self._compressed_value_bytes += skvq_compressed_bytes(n_q, D, self._bits_v, self._group_size) * B * H

    def is_trimmable(self) -> bool:
        """False: a flushed chunk cannot be restored and the frontier does not roll back (skvq_cache.py:375-393)."""
        return False

    # ------------------------------------------------------------------ reporting (skvq_cache.py:325-373)
    @property
    def compressed_key_bytes(self) -> int:
        return self._compressed_key_bytes

    @property
    def compressed_value_bytes(self) -> int:
        return self._compressed_value_bytes

    @property
    def fp16_key_bytes(self) -> int:
        return self._fp16_key_bytes

    @property
    def fp16_value_bytes(self) -> int:
        return self._fp16_value_bytes

    @property
    def residual_fp16_bytes(self) -> int:
        n_res = self.offset - self._q_end
        n_sink_kept = min(self._n_sink, self._q_end)
        return skvq_fp16_bytes(n_res + n_sink_kept, self._D) * 2 * self._B * self._H

    @property
    def perm_bytes(self) -> int:
        if self._perm_k is None and self._perm_v is None:
            return 0
        return 2 * self._H * self._D * 4

    @property
    def quantized_tokens(self) -> int:
        return self._q_end

    @property
    def tokens_seen(self) -> int:
        return self._tokens_seen

    @property
    def key_perms(self) -> torch.Tensor | None:
        return self._perm_k

    @property
    def value_perms(self) -> torch.Tensor | None:
        return self._perm_v

    @property
    def assigned_avg_bits(self) -> float:
        n_q = self._q_end - min(self._n_sink, self._q_end)
        if n_q == 0:
            return 16.0
        return 8.0 * self._compressed_key_bytes / (n_q * self._D * self._B * self._H)


__all__ = ["SKVQKVCache"]
