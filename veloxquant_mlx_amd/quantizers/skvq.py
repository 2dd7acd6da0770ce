"""SKVQ building blocks on torch-ROCm tensors: the clip-factor grid, the clipped group round trip
(one HIP launch) and the analytic byte helpers.  Mirrors the public names of
veloxquant_mlx/quantizers/skvq.py:61-235 that the SKVQ cache uses.
"""

from __future__ import annotations

import math

import torch

from .. import kernels as K

DEFAULT_ALPHA_GRID: tuple = (1.0, 0.97, 0.94, 0.90, 0.85)   # skvq.py:61


def skvq_round_trip_batched(x: torch.Tensor, perm: torch.Tensor | None, bits: int, group_size: int,
                            alphas=DEFAULT_ALPHA_GRID, out: torch.Tensor | None = None,
                            inv: torch.Tensor | None = None) -> torch.Tensor:
    """``[B, H, r, D]`` -> same shape and dtype: channels gathered by ``perm [H, D]``, clipped group
    quantise -> dequantise per token, channels put back (skvq.py:105-207 under
    SKVQKVCache._round_trip, veloxquant_mlx/cache/skvq_cache.py:236-251)."""
    return K.skvq_clipped_round_trip(x, bits, group_size, alphas, perm=perm, out=out, inv=inv)


def skvq_compressed_bytes(n_tokens: int, d: int, bits: int, group_size: int) -> int:
    """Codes plus fp16 (lo, scale) per (token, group) (skvq.py:210-217)."""
    n_groups = (d + group_size - 1) // group_size
    return math.ceil(n_tokens * d * bits / 8) + n_tokens * n_groups * 2 * 2


def skvq_fp16_bytes(n_tokens: int, d: int) -> int:
    """fp16 bytes of one tensor, keys or values (skvq.py:220-222)."""
    return n_tokens * d * 2


__all__ = ["DEFAULT_ALPHA_GRID", "skvq_round_trip_batched", "skvq_compressed_bytes", "skvq_fp16_bytes"]
