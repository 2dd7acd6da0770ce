"""VecInfer building blocks on torch ROCm tensors: smooth calibration,
Walsh-Hadamard transform, product VQ.

Same functions as veloxquant_mlx/allocators/vecinfer.py.  Nearest-centroid
assignment and the centroid gather run in the HIP kernels; the dual transform
is one dense ``[.., D] @ [D, D]`` product, left to the BLAS library.
"""

from __future__ import annotations

import math

import torch

from .. import kernels as K


def calibrate_smooth_factors(keys_calib: torch.Tensor, eps: float = 1e-4) -> torch.Tensor:
    """``lambda_i = sqrt(max_t |K[t, ..., i]|)`` floored at ``eps`` (vecinfer.py:29-54)."""
    if keys_calib.ndim not in (2, 3):
        raise ValueError(f"calibrate_smooth_factors: keys_calib must be 2D or 3D, got shape {tuple(keys_calib.shape)}")
    max_abs = keys_calib.abs().amax(dim=0)
    return torch.sqrt(torch.clamp(max_abs, min=eps))


def walsh_hadamard_matrix(d: int, dtype=torch.float32, device=None) -> torch.Tensor:
    """Orthonormal Sylvester-Hadamard matrix ``[d, d]`` (vecinfer.py:60-87)."""
    if d < 1 or (d & (d - 1)) != 0:
        raise ValueError(f"walsh_hadamard_matrix: d={d} must be a power of 2.")
    H = torch.ones((1, 1), dtype=torch.float32)
    r = 1.0 / math.sqrt(2.0)
    while H.shape[0] < d:
        H = torch.cat([torch.cat([H, H], dim=1), torch.cat([H, -H], dim=1)], dim=0) * r
    return H.to(dtype=dtype, device=device)


def _smooth_for(x: torch.Tensor, smooth: torch.Tensor, repeat_ok: bool) -> torch.Tensor:
    if smooth.ndim == 1:
        return smooth.to(x.dtype)
    if smooth.ndim != 2:
        raise ValueError(f"smooth must be 1D or 2D, got {tuple(smooth.shape)}")
    if x.ndim >= 3 and x.shape[-3] == smooth.shape[0]:
        return smooth[:, None, :].to(x.dtype)
    if repeat_ok and x.ndim >= 3 and smooth.shape[0] > 0 and x.shape[-3] % smooth.shape[0] == 0:
        n_rep = x.shape[-3] // smooth.shape[0]
        return smooth.repeat_interleave(n_rep, dim=0)[:, None, :].to(x.dtype)
    if x.shape[-1] == smooth.shape[-1]:
        return smooth.mean(dim=0).to(x.dtype)
    raise ValueError(f"cannot broadcast smooth {tuple(smooth.shape)} to {tuple(x.shape)}")


def apply_dual_transform_keys(Kt: torch.Tensor, smooth: torch.Tensor, H: torch.Tensor) -> torch.Tensor:
    """``K_tilde = (K / lambda) @ H`` (vecinfer.py:93-134)."""
    return (Kt / _smooth_for(Kt, smooth, repeat_ok=False)) @ H.to(Kt.dtype)


def apply_dual_transform_queries(q: torch.Tensor, smooth: torch.Tensor, H: torch.Tensor) -> torch.Tensor:
    """``q_tilde = (q * lambda) @ H``; per-KV-head factors repeat over the query
    group under GQA so that ``q_tilde @ K_tilde.T == q @ K.T`` (vecinfer.py:137-184)."""
    return (q * _smooth_for(q, smooth, repeat_ok=True)) @ H.to(q.dtype)


def quantize_vq(x: torch.Tensor, codebook: torch.Tensor, sub_dim: int) -> torch.Tensor:
    """Nearest-centroid indices ``[..., D // sub_dim]`` int32 (vecinfer.py:281-318)."""
    D = x.shape[-1]
    if D % sub_dim != 0:
        raise ValueError(f"quantize_vq: D={D} not divisible by sub_dim={sub_dim}")
    return K.vecinfer_quantize_metal(x, codebook, sub_dim)


def dequantize_vq(indices: torch.Tensor, codebook: torch.Tensor) -> torch.Tensor:
    """Centroid gather ``[..., n_sub * sub_dim]`` (vecinfer.py:321-335)."""
    return K.vecinfer_dequant_metal(indices, codebook)


def compute_query_lut(q_tilde: torch.Tensor, codebook: torch.Tensor, sub_dim: int) -> torch.Tensor:
    """``q_sub @ codebook.T`` -> ``[..., n_sub, n_centroids]`` (vecinfer.py:341-359)."""
    D = q_tilde.shape[-1]
    if D % sub_dim != 0:
        raise ValueError(f"compute_query_lut: D={D} not divisible by sub_dim={sub_dim}")
    q_sub = q_tilde.reshape(*q_tilde.shape[:-1], D // sub_dim, sub_dim)
    return q_sub @ codebook.to(q_sub.dtype).T


def train_codebook(x: torch.Tensor, n_centroids: int, max_iter: int = 30, seed: int = 42) -> torch.Tensor:
    """Lloyd's k-means on flat ``[n_samples, sub_dim]`` sub-vectors (vecinfer.py:190-278);
    the assignment step is the HIP nearest-centroid kernel."""
    if x.ndim != 2:
        raise ValueError(f"train_codebook: x must be 2D, got {tuple(x.shape)}")
    x = x.float()
    n, sub = x.shape
    gen = torch.Generator(device="cpu").manual_seed(seed)
    if n <= n_centroids:
        reps = (n_centroids // n) + 2
        x = x.repeat(reps, 1)[: n_centroids * 2]
        n = x.shape[0]
    init = torch.randperm(n, generator=gen)[:n_centroids].to(x.device)
    cent = x[init].clone()
    prev = float("inf")
    for _ in range(max_iter):
        labels = K.vecinfer_quantize_metal(x, cent, sub).reshape(-1).long()
        sums = torch.zeros_like(cent).index_add_(0, labels, x)
        counts = torch.zeros(n_centroids, device=x.device).index_add_(0, labels, torch.ones(n, device=x.device))
        empty = counts == 0
        if bool(empty.any()):
            idx = torch.randperm(n, generator=gen)[: int(empty.sum())].to(x.device)
            sums[empty] = x[idx]
            counts[empty] = 1
        cent = sums / counts[:, None]
        inertia = float(((x - cent[labels]) ** 2).sum())
        if abs(prev - inertia) < 1e-6 * max(prev, 1.0):
            break
        prev = inertia
    return cent


__all__ = ["calibrate_smooth_factors", "walsh_hadamard_matrix", "apply_dual_transform_keys",
           "apply_dual_transform_queries", "train_codebook", "quantize_vq", "dequantize_vq", "compute_query_lut"]
