"""CPU restatement (numpy) of the ZipCache-adapted cache's per-block compression.  TEST
INFRASTRUCTURE ONLY: imported by tests, never by the product path.

Follows veloxquant_mlx/cache/zipcache_cache.py:106-244 (_batched_saliency_mask, _batched_group_quant,
_batched_group_dequant, _compress) and veloxquant_mlx/quantizers/zipcache.py:412-419 (base_only_bytes).

Pinned by: the group round trip is ``oracle.kivi.quant_dequant_along`` along tokens (itself pinned on
the reference's KIVI tests); hi_fraction = 1 and 0 reduce to that round trip at hi_bits / lo_bits on
the whole block; the routing on a block with hand-picked norms; byte counts by hand; the ordering
properties of the reference's tests (tests/cache/test_zipcache_cache.py:76-100).

Parity unpinned: the float32 reduction order of ``mx.linalg.norm`` -- tokens whose norms agree to the
last bits may be routed differently (tests use rows whose norms differ by clear margins).
"""

from __future__ import annotations

import math

import numpy as np

from . import kivi as ok


def saliency_mask(norms, n_hi):   # zipcache_cache.py:106-116
    BH, S = norms.shape
    if n_hi == 0:
        return np.zeros((BH, S), bool)
    if n_hi >= S:
        return np.ones((BH, S), bool)
    order = np.argsort(norms, axis=-1, kind="stable")
    rank = np.argsort(order, axis=-1, kind="stable")
    return rank >= (S - n_hi)


def base_only_bytes(S, D, bits, group_size=32):   # zipcache.py:412-419
    return math.ceil(S * D * bits / 8) + math.ceil(S / group_size) * D * 2 * 2


def compress(t, is_key, hi_bits, lo_bits, hi_fraction, gs, out_dtype=np.float16):   # zipcache_cache.py:160-244
    """``[B,H,S,D]`` -> (reconstruction, norms [BH,S], (stored, baseline, fp16) bytes)."""
    B, H, S, D = t.shape
    lo_b = lo_bits if is_key else hi_bits
    frac = hi_fraction if is_key else 1.0
    BH = B * H
    x32 = t.reshape(BH, S, D).astype(np.float32)
    norms = np.sqrt(np.sum(x32.astype(np.float64) ** 2, axis=-1)).astype(np.float32)
    n_hi = max(0, min(S, int(math.ceil(S * frac))))
    n_lo = S - n_hi
    mask = saliency_mask(norms, n_hi)
    order = np.argsort(mask.astype(np.int32), axis=-1, kind="stable")
    lo_idx, hi_idx = order[:, :n_lo], order[:, n_lo:]
    out = np.zeros((BH, S, D), np.float32)
    for idx, n, bits in ((lo_idx, n_lo, lo_b), (hi_idx, n_hi, hi_bits)):
        if n == 0:
            continue
        rows = np.take_along_axis(x32, idx[..., None], axis=1)
        recon = ok.quant_dequant_along(rows, -2, gs, (1 << bits) - 1)   # float32 in, float32 out
        np.put_along_axis(out, idx[..., None], recon, axis=1)
    per_slab = (math.ceil(n_hi * D * hi_bits / 8) + math.ceil(n_lo * D * lo_b / 8)
                + (math.ceil(n_hi / gs) if n_hi else 0) * D * 4 + (math.ceil(n_lo / gs) if n_lo else 0) * D * 4 + S)
    bytes_ = (per_slab * BH, base_only_bytes(S, D, lo_bits, gs) * BH, B * H * S * D * 2)
    return out.reshape(B, H, S, D).astype(out_dtype), norms, bytes_
