"""Kitty KV cache (``method="kitty"``): keys round-tripped at two bit widths chosen per channel
by running variance, values kept as they come.  Mirrors ``KittyKVCache``
(veloxquant_mlx/cache/kitty_cache.py:50-256): same ranking signal (variance of the first batch
at prefill, running sums of the stored keys afterwards), same accounting, same trim.

A sibling of KIVI on the same kernel: both reconstructions are launches of the key-axis group
round trip (``vq_kivi_quant_dequant``).
"""

from __future__ import annotations

import math
from typing import Any

import torch

from .. import kernels as K
from ..core.exceptions import QuantizerConfigError
from ..quantizers.kitty import (channel_variance_batched, compute_running_variance, hi_mask_from_variance_batched,
                                quantize_mixed_channels_batched)
from ._fp16_cache import FP16KVCache


class KittyKVCache(FP16KVCache):
    def __init__(self, config: Any) -> None:
        super().__init__()
        if not K._lib.library_present():
            raise RuntimeError("KittyKVCache: the HIP kernel library is not available on this build; there is no fallback path.")
        self._D = int(config.head_dim)
        self._hi_fraction = float(getattr(config, "kitty_hi_fraction", 0.25))
        if not 0.0 <= self._hi_fraction <= 1.0:
            raise QuantizerConfigError(f"kitty: kitty_hi_fraction must be in [0, 1], got {self._hi_fraction}")
        self._hi_bit = int(getattr(config, "kitty_hi_bit", 4))
        self._lo_bit = int(getattr(config, "kitty_lo_bit", 2))
        self._group_size = int(getattr(config, "kitty_group_size", 32))
        self._key_sum: torch.Tensor | None = None      # [H, D] float32
        self._key_sq_sum: torch.Tensor | None = None   # [H, D] float32
        self._n_keys = 0
        self._compressed_key_bytes = 0
        self._fp16_key_bytes = 0
        self._value_fp16_bytes = 0

    # ------------------------------------------------------------------ quantisation
    def _quantize_keys(self, keys: torch.Tensor) -> torch.Tensor:
        """``[B,H,S,D]`` -> float16 reconstruction under the current channel ranking (kitty_cache.py:88-117)."""
        B, H, S, D = keys.shape
        flat = keys.reshape(B * H, S, D)
        if self._n_keys == 0:
            variance = channel_variance_batched(flat)
        else:
            var_h = compute_running_variance(self._key_sum, self._key_sq_sum, self._n_keys)
            variance = var_h[None].expand(B, H, D).reshape(B * H, D)
        hi_mask = hi_mask_from_variance_batched(variance, self._hi_fraction)
        out = quantize_mixed_channels_batched(flat, hi_mask, hi_bit=self._hi_bit, lo_bit=self._lo_bit,
                                              group_size=self._group_size)
        return out.reshape(B, H, S, D)

    def _update_accumulators(self, keys: torch.Tensor) -> None:
        """Running sums of the batch-averaged stored keys (kitty_cache.py:119-137)."""
        k_mean_b = keys.float().mean(dim=0)            # [H, S, D]
        new_sum = k_mean_b.sum(dim=1)
        new_sq_sum = (k_mean_b * k_mean_b).sum(dim=1)
        if self._key_sum is None:
            self._key_sum, self._key_sq_sum = new_sum, new_sq_sum
        else:
            self._key_sum = self._key_sum + new_sum
            self._key_sq_sum = self._key_sq_sum + new_sq_sum
        self._n_keys += keys.shape[2]

    # ------------------------------------------------------------------ protocol
    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        B, H, S, D = keys.shape
        k_out = self._quantize_keys(keys)
        self._update_accumulators(k_out)
        self._account_bytes(B, H, S, D)
        return super().update_and_fetch(k_out.to(keys.dtype), values)

    def _channel_bytes(self, n_tokens: int, n_ch: int, b: int, B: int, H: int) -> int:
        code_bytes = math.ceil(n_tokens * n_ch * b / 8)
        param_bytes = math.ceil(n_tokens / self._group_size) * n_ch * 2 * 2
        return (code_bytes + param_bytes) * H * B

    def _key_bytes_for(self, n_tokens: int, B: int, H: int, D: int | None = None) -> int:
        D = self._D if D is None else D
        n_hi = max(1, int(D * self._hi_fraction))
        return self._channel_bytes(n_tokens, n_hi, self._hi_bit, B, H) + \
            self._channel_bytes(n_tokens, D - n_hi, self._lo_bit, B, H)

    def _account_bytes(self, B: int, H: int, S: int, D: int) -> None:
        self._compressed_key_bytes += self._key_bytes_for(S, B, H, D)
        self._fp16_key_bytes += B * H * S * D * 2
        self._value_fp16_bytes += B * H * S * D * 2

    def trim(self, n: int) -> int:
        """Drop the last ``n`` tokens, their share of the running sums and of the accounting
        (kitty_cache.py:176-205)."""
        old_offset = self.offset
        trimmed = min(old_offset, max(int(n), 0))
        if trimmed and self.keys is not None:
            gone = self.keys[..., old_offset - trimmed:old_offset, :]
            B, H = gone.shape[0], gone.shape[1]
            if self._n_keys - trimmed <= 0:
                self._key_sum = self._key_sq_sum = None
                self._n_keys = 0
            else:
                g32 = gone.float().mean(dim=0)
                self._key_sum = self._key_sum - g32.sum(dim=1)
                self._key_sq_sum = self._key_sq_sum - (g32 * g32).sum(dim=1)
                self._n_keys -= trimmed
            self._compressed_key_bytes = max(0, self._compressed_key_bytes - self._key_bytes_for(trimmed, B, H))
            self._fp16_key_bytes = max(0, self._fp16_key_bytes - B * H * trimmed * self._D * 2)
            self._value_fp16_bytes = max(0, self._value_fp16_bytes - B * H * trimmed * self._D * 2)
        return super().trim(n)

    # ------------------------------------------------------------------ properties
    @property
    def compressed_key_bytes(self) -> int:
        return self._compressed_key_bytes

    @property
    def fp16_key_bytes(self) -> int:
        return self._fp16_key_bytes

    @property
    def value_fp16_bytes(self) -> int:
        return self._value_fp16_bytes

    @property
    def assigned_avg_bits(self) -> float:
        n_hi = max(1, int(self._D * self._hi_fraction))
        return (n_hi * self._hi_bit + (self._D - n_hi) * self._lo_bit) / self._D

    @property
    def hi_fraction(self) -> float:
        return self._hi_fraction

    @property
    def hi_bit(self) -> int:
        return self._hi_bit

    @property
    def lo_bit(self) -> int:
        return self._lo_bit

    @property
    def group_size(self) -> int:
        return self._group_size


__all__ = ["KittyKVCache"]
