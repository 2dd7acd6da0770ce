"""numpy restatement of the Kitty mixed-precision key path (test infrastructure only).

Follows veloxquant_mlx/quantizers/kitty.py and veloxquant_mlx/cache/kitty_cache.py; the group
round trip is the one of ``oracle.kivi`` (veloxquant_mlx/quantizers/_quant_utils.py:170-205 is
the same arithmetic as the KIVI key axis: float32 min/max over token groups, the ragged tail
padded with its last row, ``round`` half to even, clip, ``code * scale + min``, float16 result).
"""

from __future__ import annotations

import math

import numpy as np

from . import kivi

F32 = np.float32


def group_round_trip_fp16(x, bits: int, group_size: int) -> np.ndarray:
    """``_group_quant_dequant_batched`` (_quant_utils.py:170-205): ``x [N, S, D]`` -> float16."""
    return kivi.quant_dequant_along(np.asarray(x), -2, group_size, (1 << bits) - 1, cast=lambda r: r.astype(np.float16))


def hi_mask_from_variance(variance, hi_fraction: float) -> np.ndarray:
    """``[N, D]`` -> bool mask of the top ``max(1, int(D * hi_fraction))`` channels per row, ties
    to the lower index (kitty.py:112-135; the stable descending sort of kitty.py:61-64)."""
    variance = np.asarray(variance, dtype=F32)
    d = variance.shape[-1]
    n_hi = max(1, int(d * hi_fraction))
    order = np.argsort(-variance, axis=-1, kind="stable")
    rank = np.argsort(order, axis=-1, kind="stable")
    return rank < n_hi


def rank_channels_by_sensitivity(keys, hi_fraction: float = 0.25):
    """``keys [S, D]`` -> ascending ``(hi_indices, lo_indices)`` (kitty.py:44-67)."""
    variance = np.var(np.asarray(keys).astype(F32), axis=0)
    mask = hi_mask_from_variance(variance[None], hi_fraction)[0]
    return [int(i) for i in np.nonzero(mask)[0]], [int(i) for i in np.nonzero(~mask)[0]]


def quantize_mixed_channels_batched(keys, hi_mask, hi_bit: int = 4, lo_bit: int = 2, group_size: int = 32) -> np.ndarray:
    """``keys [N, S, D]``, ``hi_mask [N, D]`` -> float16 (kitty.py:138-169)."""
    hi = group_round_trip_fp16(keys, hi_bit, group_size)
    lo = group_round_trip_fp16(keys, lo_bit, group_size)
    return np.where(np.asarray(hi_mask)[:, None, :], hi, lo).astype(np.float16)


def compute_running_variance(key_sum, key_sq_sum, n: int) -> np.ndarray:
    """kitty.py:172-190."""
    key_sum = np.asarray(key_sum, dtype=F32)
    if n < 2:
        return np.zeros_like(key_sum)
    mean = key_sum / F32(n)
    return np.maximum(np.asarray(key_sq_sum, dtype=F32) / F32(n) - mean * mean, F32(0))


def key_bytes(n_tokens: int, B: int, H: int, D: int, hi_fraction: float, hi_bit: int, lo_bit: int, group_size: int) -> int:
    """kitty_cache.py:150-174."""
    n_hi = max(1, int(D * hi_fraction))

    def channel_bytes(n_ch: int, b: int) -> int:
        return (math.ceil(n_tokens * n_ch * b / 8) + math.ceil(n_tokens / group_size) * n_ch * 2 * 2) * H * B
    return channel_bytes(n_hi, hi_bit) + channel_bytes(D - n_hi, lo_bit)


class KittyCacheModel:
    """State machine of ``KittyKVCache`` (kitty_cache.py:50-205) on numpy arrays.  ``cast`` turns the
    float16 reconstruction into the dtype the caller's keys have (identity for float16)."""

    def __init__(self, head_dim: int, hi_fraction: float = 0.25, hi_bit: int = 4, lo_bit: int = 2, group_size: int = 32,
                 cast=None):
        self.D, self.hi_fraction, self.hi_bit, self.lo_bit, self.g = head_dim, hi_fraction, hi_bit, lo_bit, group_size
        self.cast = cast or (lambda a: a)
        self.key_sum = self.key_sq_sum = None
        self.n_keys = 0
        self.keys = self.values = None
        self.compressed_key_bytes = self.fp16_key_bytes = self.value_fp16_bytes = 0

    def update_and_fetch(self, keys, values):
        keys = np.asarray(keys)
        B, H, S, D = keys.shape
        flat = keys.reshape(B * H, S, D)
        if self.n_keys == 0:
            variance = np.var(flat.astype(F32), axis=1)
        else:
            var_h = compute_running_variance(self.key_sum, self.key_sq_sum, self.n_keys)
            variance = np.broadcast_to(var_h[None], (B, H, D)).reshape(B * H, D)
        mask = hi_mask_from_variance(variance, self.hi_fraction)
        k_out = quantize_mixed_channels_batched(flat, mask, self.hi_bit, self.lo_bit, self.g).reshape(B, H, S, D)
        k_mean_b = k_out.astype(F32).mean(axis=0, dtype=F32)
        new_sum, new_sq = k_mean_b.sum(axis=1, dtype=F32), (k_mean_b * k_mean_b).sum(axis=1, dtype=F32)
        if self.key_sum is None:
            self.key_sum, self.key_sq_sum = new_sum, new_sq
        else:
            self.key_sum, self.key_sq_sum = self.key_sum + new_sum, self.key_sq_sum + new_sq
        self.n_keys += S
        self.compressed_key_bytes += key_bytes(S, B, H, D, self.hi_fraction, self.hi_bit, self.lo_bit, self.g)
        self.fp16_key_bytes += B * H * S * D * 2
        self.value_fp16_bytes += B * H * S * D * 2
        stored = self.cast(k_out)
        self.keys = stored if self.keys is None else np.concatenate([self.keys, stored], axis=2)
        self.values = np.asarray(values) if self.values is None else np.concatenate([self.values, np.asarray(values)], axis=2)
        self.last_mask = mask
        return self.keys, self.values

    def trim(self, n: int) -> int:
        old = 0 if self.keys is None else self.keys.shape[2]
        trimmed = min(old, max(int(n), 0))
        if trimmed:
            gone = self.keys[:, :, old - trimmed:old]
            B, H = gone.shape[:2]
            if self.n_keys - trimmed <= 0:
                self.key_sum = self.key_sq_sum = None
                self.n_keys = 0
            else:
                g32 = gone.astype(F32).mean(axis=0, dtype=F32)
                self.key_sum = self.key_sum - g32.sum(axis=1, dtype=F32)
                self.key_sq_sum = self.key_sq_sum - (g32 * g32).sum(axis=1, dtype=F32)
                self.n_keys -= trimmed
            kb = key_bytes(trimmed, B, H, self.D, self.hi_fraction, self.hi_bit, self.lo_bit, self.g)
            self.compressed_key_bytes = max(0, self.compressed_key_bytes - kb)
            self.fp16_key_bytes = max(0, self.fp16_key_bytes - B * H * trimmed * self.D * 2)
            self.value_fp16_bytes = max(0, self.value_fp16_bytes - B * H * trimmed * self.D * 2)
            self.keys, self.values = self.keys[:, :, :old - trimmed], self.values[:, :, :old - trimmed]
        return trimmed
