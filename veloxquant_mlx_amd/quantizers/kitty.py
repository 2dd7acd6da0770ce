"""Kitty: channel-wise mixed-precision key quantisation, on the KIVI group kernel.

Mirrors veloxquant_mlx/quantizers/kitty.py:44-190.  At head_dim 128 with groups of 32 or 64 tokens the mixed
reconstruction is one launch of the key-axis group round trip with a level count per channel
(``vq_kivi_quant_dequant_mixed``) and the variance the channels are ranked by one pass over the stored rows
(``vq_channel_moments``); other shapes take two launches of ``vq_kivi_quant_dequant`` and a select, and
``torch.var``.  The ranking itself (two argsorts over ``D`` channels) is host-level torch on the device.
"""

from __future__ import annotations

import torch

from .. import kernels as K


def _group_round_trip_fp16(x: torch.Tensor, bits: int, group_size: int) -> torch.Tensor:
    """``_group_quant_dequant_batched`` (veloxquant_mlx/quantizers/_quant_utils.py:170-205):
    groups along the token axis of ``[..., S, D]``, float32 arithmetic, result as float16."""
    if x.dtype == torch.float16:
        return K.kivi_group_quant_dequant(x, -2, group_size, (1 << bits) - 1)
    return K.kivi_group_quant_dequant(x.float(), -2, group_size, (1 << bits) - 1).to(torch.float16)


def hi_mask_from_variance_batched(variance: torch.Tensor, hi_fraction: float) -> torch.Tensor:
    """``[N, D]`` variances -> bool mask of every row's top ``max(1, int(D * hi_fraction))`` channels,
    ties to the lower channel index (kitty.py:112-135)."""
    d = variance.shape[-1]
    n_hi = max(1, int(d * hi_fraction))
    if variance.is_cuda and variance.ndim == 2 and variance.dtype == torch.float32 and d <= 1024:
        return K.channel_hi_mask(variance, n_hi)
    order = torch.argsort(-variance, dim=-1, stable=True)
    rank = torch.argsort(order, dim=-1, stable=True)
    return rank < n_hi


def rank_channels_by_sensitivity(keys: torch.Tensor, hi_fraction: float = 0.25):
    """``keys [S, D]`` -> ``(hi_indices, lo_indices)``, ascending lists (kitty.py:44-67)."""
    variance = torch.var(keys.float(), dim=0, unbiased=False)
    mask = hi_mask_from_variance_batched(variance[None], hi_fraction)[0].tolist()
    return [i for i, m in enumerate(mask) if m], [i for i, m in enumerate(mask) if not m]


def quantize_mixed_channels_batched(keys: torch.Tensor, hi_mask: torch.Tensor, hi_bit: int = 4, lo_bit: int = 2,
                                    group_size: int = 32) -> torch.Tensor:
    """``keys [N, S, D]``, ``hi_mask [N, D]`` -> float16 reconstruction, hi-bit where the mask is set
    (kitty.py:138-169)."""
    if keys.dtype == torch.float16 and keys.shape[-1] == 128 and group_size in (32, 64):
        # one launch with a level count per channel: the same codes as the two whole-tensor round trips
        # and the select below, which stay for the other shapes
        return K.kivi_group_quant_dequant_mixed(keys, hi_mask, group_size, (1 << lo_bit) - 1, (1 << hi_bit) - 1)
    recon_hi = _group_round_trip_fp16(keys, hi_bit, group_size)
    recon_lo = _group_round_trip_fp16(keys, lo_bit, group_size)
    return torch.where(hi_mask[:, None, :], recon_hi, recon_lo)


def channel_variance_batched(keys: torch.Tensor) -> torch.Tensor:
    """``keys [N, S, D]`` -> float32 ``[N, D]`` population variance over the tokens (kitty_cache.py:96-104):
    one pass over the stored rows where the kernel covers the shape, ``torch.var`` of the float32 copy otherwise."""
    if keys.shape[-1] in (64, 128, 256) and keys.shape[1] > 0 and keys.dtype in (torch.float16, torch.bfloat16, torch.float32):
        return K.channel_variance(keys)
    return torch.var(keys.float(), dim=1, unbiased=False)


def quantize_mixed_channels(keys: torch.Tensor, hi_indices, lo_indices, hi_bit: int = 4, lo_bit: int = 2,
                            group_size: int = 32) -> torch.Tensor:
    """Single ``[S, D]`` form (kitty.py:70-109); channels in neither list pass through as float16."""
    S, D = keys.shape
    out = keys.to(torch.float16).clone()
    if len(hi_indices):
        idx = torch.as_tensor(list(hi_indices), device=keys.device)
        out[:, idx] = _group_round_trip_fp16(keys[None], hi_bit, group_size)[0][:, idx]
    if len(lo_indices):
        idx = torch.as_tensor(list(lo_indices), device=keys.device)
        out[:, idx] = _group_round_trip_fp16(keys[None], lo_bit, group_size)[0][:, idx]
    return out


def compute_running_variance(key_sum: torch.Tensor, key_sq_sum: torch.Tensor, n: int) -> torch.Tensor:
    """Variance from running sums, zeros below two tokens (kitty.py:172-190)."""
    if n < 2:
        return torch.zeros_like(key_sum)
    mean = key_sum / n
    return torch.clamp(key_sq_sum / n - mean * mean, min=0.0)


__all__ = ["rank_channels_by_sensitivity", "quantize_mixed_channels", "compute_running_variance",
           "hi_mask_from_variance_batched", "quantize_mixed_channels_batched", "channel_variance_batched"]
