"""numpy restatement of attention over a group-affine quantised KV cache.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

* dense decode attention over reconstructed K/V with GQA repeat-interleave:
  ``veloxquant_mlx/tests/metal/test_scalar_attend.py:85-115`` (the reference's
  own float32 oracle for ``scalar_fused_decode_attend``,
  ``veloxquant_mlx/metal/_scalar_attend.py:370-493``)
* causal, tail-aligned attention (``q_abs = S_kv - S_q + q_pos``):
  ``veloxquant_mlx/tests/metal/test_flash_prefill.py:34-44`` for
  ``flash_prefill_attend`` (``veloxquant_mlx/metal/_flash_prefill.py:171-237``)
* chunked quantise-on-write prefill = ``KIVIKVCache.update_and_fetch`` applied
  per chunk followed by causal attention
  (``veloxquant_mlx/cache/kivi_cache.py:230-262``)
"""

from __future__ import annotations

import numpy as np

from .kivi import KiviCacheModel, group_dequant

F32 = np.float32


def sdpa(q, k, v, scale: float, causal: bool = False, acc=np.float32, sliding_window: int = 0) -> np.ndarray:
    """softmax(q k^T * scale) v with GQA by repeat-interleave.

    q ``[B,H_q,S_q,D]``, k/v ``[B,H_kv,S_kv,D]``.  With ``causal`` the queries
    are aligned to the tail of the keys and slot ``j`` is masked when
    ``j > S_kv - S_q + q_pos``; with ``sliding_window > 0`` slot ``j`` is also
    masked when ``j < q_abs - sliding_window + 1``
    (veloxquant_mlx/tests/cache/test_vecinfer_fused_sdpa.py:105-113)."""
    q = np.asarray(q).astype(acc)
    k = np.asarray(k).astype(acc)
    v = np.asarray(v).astype(acc)
    H, Hkv = q.shape[1], k.shape[1]
    if H != Hkv:
        assert H % Hkv == 0
        k = np.repeat(k, H // Hkv, axis=1)
        v = np.repeat(v, H // Hkv, axis=1)
    S_q, S_kv = q.shape[2], k.shape[2]
    scores = np.einsum("bhqd,bhsd->bhqs", q, k) * acc(scale)
    if causal:
        q_abs = (S_kv - S_q) + np.arange(S_q)
        mask = np.arange(S_kv)[None, :] > q_abs[:, None]
        scores = np.where(mask, -np.inf, scores)
    if sliding_window and sliding_window > 0:
        q_abs = (S_kv - S_q) + np.arange(S_q)
        mask = np.arange(S_kv)[None, :] < (q_abs[:, None] - sliding_window + 1)
        scores = np.where(mask, -np.inf, scores)
    scores = scores - scores.max(axis=-1, keepdims=True)
    w = np.exp(scores)
    w = w / w.sum(axis=-1, keepdims=True)
    return np.einsum("bhqs,bhsd->bhqd", w, v).astype(F32)


def reference_attend(q, kc, ks, kz, vc, vs, vz, g: int, scale: float) -> np.ndarray:
    """Unmasked attention over ``code*scale+zero`` reconstructions
    (test_scalar_attend.py:85-115)."""
    k_hat = group_dequant(kc, ks, kz, -2, g)
    v_hat = group_dequant(vc, vs, vz, -1, g)
    return sdpa(q, k_hat, v_hat, scale, causal=False)


def kivi_attend(q, kc, ks, kz, vc, vs, vz, g: int, k_tail, v_tail, scale: float,
                causal: bool = False, acc=np.float64, recon_dtype=None, sliding_window: int = 0) -> np.ndarray:
    """Attention over a quantised prefix followed by an fp16 tail.

    The tail is what ``KIVIKVCache`` keeps un-quantised (residual window plus
    the partial group); either part may be empty.  ``recon_dtype`` (e.g.
    ``np.float16``) rounds the reconstruction to the dtype the cache stores it in
    before it is attended over (kivi_cache.py:198-201: ``x_hat.astype(x.dtype)``);
    ``None`` keeps the float32 reconstruction of the fused decode kernel
    (metal/src/scalar_affine_attend.metal)."""
    parts_k, parts_v = [], []
    if kc is not None and kc.shape[-2] > 0:
        kh, vh = group_dequant(kc, ks, kz, -2, g), group_dequant(vc, vs, vz, -1, g)
        if recon_dtype is not None:
            kh, vh = kh.astype(recon_dtype).astype(F32), vh.astype(recon_dtype).astype(F32)
        parts_k.append(kh)
        parts_v.append(vh)
    if k_tail is not None and k_tail.shape[-2] > 0:
        parts_k.append(np.asarray(k_tail).astype(F32))
        parts_v.append(np.asarray(v_tail).astype(F32))
    k = np.concatenate(parts_k, axis=2)
    v = np.concatenate(parts_v, axis=2)
    return sdpa(q, k, v, scale, causal=causal, acc=acc, sliding_window=sliding_window)


def chunked_prefill(q, k, v, chunk: int, bits: int, group_size: int,
                    residual_length: int, scale: float,
                    prefix_k=None, prefix_v=None, acc=np.float64) -> np.ndarray:
    """Prefill ``q/k/v`` (fp16 arrays ``[B,H,S,D]``) in chunks through a KIVI
    cache: each chunk is appended, the aged-out group-aligned prefix is round
    tripped in place, then the chunk's queries attend causally over everything
    stored so far.  ``prefix_k/v`` are appended first (without queries)."""
    cache = KiviCacheModel(bits=bits, group_size=group_size, residual_length=residual_length)
    if prefix_k is not None:
        cache.update_and_fetch(np.asarray(prefix_k), np.asarray(prefix_v))
    S = q.shape[2]
    outs = []
    for s0 in range(0, S, chunk):
        s1 = min(S, s0 + chunk)
        k_all, v_all = cache.update_and_fetch(np.asarray(k[:, :, s0:s1]), np.asarray(v[:, :, s0:s1]))
        outs.append(sdpa(q[:, :, s0:s1], k_all, v_all, scale, causal=True, acc=acc))
    return np.concatenate(outs, axis=2)
