"""numpy restatement of VecInfer's product-VQ primitives.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Follows ``veloxquant_mlx/allocators/vecinfer.py`` (quantize_vq :281-318,
dequantize_vq :321-335, compute_query_lut :341-359, walsh_hadamard_matrix
:60-87, dual transforms :93-184) and the Metal twin
``veloxquant_mlx/metal/src/vecinfer_quantize.metal:8-28`` for the order of
floating-point operations and the tie rule.

PARITY UNPINNED: the reduction order of ``mx.sum(diff*diff, axis=-1)`` and the
tie order of ``mx.argmin`` cannot be observed without MLX.  The oracle uses
the Metal twin's order (squares rounded separately, left-to-right fp32 sum,
strict ``<`` so the lowest index wins).
"""

from __future__ import annotations

import math

import numpy as np

F32 = np.float32


def _seq_sqdist(sub: np.ndarray, cb: np.ndarray) -> np.ndarray:
    """``[c, n_centroids]`` squared distances, accumulated dimension by
    dimension in float32 (vecinfer_quantize.metal:20-25)."""
    acc = None
    for i in range(sub.shape[1]):
        diff = (sub[:, None, i] - cb[None, :, i]).astype(F32)
        sq = (diff * diff).astype(F32)
        acc = sq if acc is None else (acc + sq).astype(F32)
    return acc


def quantize_vq(x, codebook, sub_dim: int, chunk: int | None = None,
                return_margin: bool = False):
    """Nearest-centroid indices, ``[..., D] -> [..., D // sub_dim]`` int32.

    ``chunk`` defaults to the reference's ``1_000_000 // n_centroids``
    (allocators/vecinfer.py:305-306).  With ``return_margin`` the gap between
    the best and second-best distance is returned as well (used to count
    near-ties)."""
    x = np.asarray(x)
    *lead, D = x.shape
    if D % sub_dim:
        raise ValueError(f"quantize_vq: D={D} not divisible by sub_dim={sub_dim}")
    n_sub = D // sub_dim
    flat = x.reshape(-1, sub_dim).astype(F32)
    cb = np.asarray(codebook).astype(F32)
    nc = cb.shape[0]
    if chunk is None:
        chunk = max(1, 1_000_000 // max(nc, 1))
    out = np.empty(flat.shape[0], np.int32)
    margin = np.empty(flat.shape[0], F32) if return_margin else None
    for s in range(0, flat.shape[0], chunk):
        d2 = _seq_sqdist(flat[s:s + chunk], cb)
        idx = np.argmin(d2, axis=-1)  # first occurrence == lowest index
        out[s:s + chunk] = idx
        if return_margin and nc > 1:
            part = np.partition(d2, 1, axis=-1)
            margin[s:s + chunk] = part[:, 1] - part[:, 0]
    out = out.reshape(*lead, n_sub)
    if return_margin:
        return out, margin.reshape(*lead, n_sub)
    return out


def quantize_vq_loop(x, codebook, sub_dim: int) -> np.ndarray:
    """Pure-Python triple loop of the Metal twin, for tiny inputs only."""
    x = np.asarray(x)
    *lead, D = x.shape
    flat = x.reshape(-1, sub_dim).astype(F32)
    cb = np.asarray(codebook).astype(F32)
    out = np.zeros(flat.shape[0], np.int32)
    for v in range(flat.shape[0]):
        best, bi = F32(np.inf), 0
        for c in range(cb.shape[0]):
            dist = F32(0.0)
            for i in range(sub_dim):
                d = F32(flat[v, i] - cb[c, i])
                dist = F32(dist + F32(d * d))
            if dist < best:
                best, bi = dist, c
        out[v] = bi
    return out.reshape(*lead, D // sub_dim)


def dequantize_vq(indices, codebook) -> np.ndarray:
    """Centroid gather (allocators/vecinfer.py:321-335)."""
    codebook = np.asarray(codebook)
    indices = np.asarray(indices)
    *lead, n_sub = indices.shape
    g = codebook[indices.reshape(-1).astype(np.int64)]
    return g.reshape(*lead, n_sub * codebook.shape[-1])


def compute_query_lut(q_tilde, codebook, sub_dim: int) -> np.ndarray:
    """``q_sub @ codebook.T`` (allocators/vecinfer.py:341-359)."""
    q_tilde = np.asarray(q_tilde)
    *lead, D = q_tilde.shape
    if D % sub_dim:
        raise ValueError(f"compute_query_lut: D={D} not divisible by sub_dim={sub_dim}")
    q_sub = q_tilde.reshape(*lead, D // sub_dim, sub_dim)
    return q_sub @ np.asarray(codebook).astype(q_sub.dtype).T


def walsh_hadamard_matrix(d: int) -> np.ndarray:
    """Orthonormal Sylvester-Hadamard matrix (allocators/vecinfer.py:60-87)."""
    if d < 1 or (d & (d - 1)) != 0:
        raise ValueError(f"walsh_hadamard_matrix: d={d} must be a power of 2.")
    H = np.array([[1.0]], dtype=F32)
    r = F32(1.0 / math.sqrt(2.0))
    while H.shape[0] < d:
        H = (np.block([[H, H], [H, -H]]) * r).astype(F32)
    return H


def _smooth_rows(x: np.ndarray, smooth: np.ndarray) -> np.ndarray:
    if smooth.ndim == 1:
        return smooth
    if x.ndim >= 3 and x.shape[-3] == smooth.shape[0]:
        return smooth[:, None, :]
    if x.ndim >= 3 and smooth.shape[0] > 0 and x.shape[-3] % smooth.shape[0] == 0:
        return np.repeat(smooth, x.shape[-3] // smooth.shape[0], axis=0)[:, None, :]
    return smooth.mean(axis=0)


def apply_dual_transform_keys(K, smooth, H) -> np.ndarray:
    """``(K / lambda) @ H`` (allocators/vecinfer.py:93-134)."""
    K = np.asarray(K).astype(F32)
    smooth = np.asarray(smooth).astype(F32)
    if smooth.ndim == 2 and not (K.ndim >= 3 and K.shape[-3] == smooth.shape[0]):
        sm = smooth.mean(axis=0)
    else:
        sm = _smooth_rows(K, smooth)
    return (K / sm) @ np.asarray(H).astype(F32)


def apply_dual_transform_queries(q, smooth, H) -> np.ndarray:
    """``(q * lambda) @ H`` with per-KV-head factors repeated over the query
    group under GQA (allocators/vecinfer.py:137-184)."""
    q = np.asarray(q).astype(F32)
    smooth = np.asarray(smooth).astype(F32)
    return (q * _smooth_rows(q, smooth)) @ np.asarray(H).astype(F32)


def calibrate_smooth_factors(keys_calib, eps: float = 1e-4) -> np.ndarray:
    """``sqrt(max_t |K|)`` floored at eps (allocators/vecinfer.py:29-54)."""
    k = np.asarray(keys_calib)
    if k.ndim not in (2, 3):
        raise ValueError("calibrate_smooth_factors: keys_calib must be 2D or 3D")
    return np.sqrt(np.maximum(np.abs(k).max(axis=0), eps))


def encode_decode_keys(keys, smooth, H, codebook, sub_dim: int):
    """Key encode+decode of the fused kernel (metal/_vecinfer.py:225-293; the cache's
    composition, cache/vecinfer_cache.py:313-356): ``k_tilde = (K / smooth) @ H`` -> indices ->
    ``k_hat = (codebook[idx] @ H^T) * smooth``.  The two matrix products are accumulated in
    float64 and rounded to float32 once, i.e. the mathematical value rather than one particular
    summation order.  ``smooth``: ``None``, ``[D]`` or ``[H_kv, D]``.  Returns
    ``(k_tilde, idx, k_hat)``, all float32 / int32."""
    K = np.asarray(keys).astype(F32)
    Hm = np.asarray(H).astype(np.float64)
    sm = None
    if smooth is not None:
        sm = np.asarray(smooth).astype(F32)
        sm = sm[:, None, :] if sm.ndim == 2 and sm.shape[0] == K.shape[-3] else (sm.mean(axis=0) if sm.ndim == 2 else sm)
    x = K / sm if sm is not None else K
    k_tilde = (x.astype(np.float64) @ Hm).astype(F32)
    idx = quantize_vq(k_tilde, codebook, sub_dim)
    k_hat = (dequantize_vq(idx, np.asarray(codebook).astype(F32)).astype(np.float64) @ Hm.T).astype(F32)
    if sm is not None:
        k_hat = k_hat * sm
    return k_tilde, idx, k_hat.astype(F32)


def fused_sdpa(q_tilde, k_indices, k_codebook, v_indices, v_codebook, scale: float, causal: bool = True,
               sliding_window: int = 0, acc=np.float64) -> np.ndarray:
    """``softmax((q_tilde @ K_tilde^T) * scale) @ V_hat`` with both operands gathered from
    their codebooks: the reference's own oracle for its table kernel
    (veloxquant_mlx/tests/cache/test_vecinfer_fused_sdpa.py:80-115, for
    veloxquant_mlx/metal/fused_sdpa.py:200-299), queries aligned to the tail."""
    from .attend import sdpa
    k_tilde = dequantize_vq(k_indices, k_codebook)
    v_hat = dequantize_vq(v_indices, v_codebook)
    return sdpa(np.asarray(q_tilde, np.float32), k_tilde, v_hat, scale, causal=causal, acc=acc,
                sliding_window=sliding_window)
