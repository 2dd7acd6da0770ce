"""CPU restatement (numpy) of SKVQ's clipped group quantisation and of the SKVQ cache's
chunk-flush logic.  TEST INFRASTRUCTURE ONLY: imported by tests, the smoke check and the bench's
CPU-baseline leg, never by the product path.

Follows veloxquant_mlx/quantizers/skvq.py:61-222 (clip-factor grid, clipped_group_quant,
clipped_group_dequant, byte helpers) and veloxquant_mlx/cache/skvq_cache.py:186-312
(_per_head_perms, _round_trip, update_and_fetch).

Pinned by the reference's own tests (tests/quantizers/test_skvq.py, tests/cache/test_skvq_cache.py,
restated in tests/test_oracle_skvq.py on the same seeded generators): alpha = 1 agrees with plain
min/max group quantisation on > 99.9 % of codes and never differs by more than one step; the
searched grid is never worse than alpha = 1 per group; error falls with bits and the 8-bit round
trip is below 1e-4; a single-outlier group is clipped (known answer by hand); the permutation
sorts by range, is stable on ties and is kept per head only when strictly better.

Parity unpinned: the order in which the reference's ``mx.mean`` adds a group's squared errors,
and the per-head error means that decide between the sorted and the identity order, are not
fixed by any test; this restatement adds left to right in float32 (the per-head means in
float64), so a group or head whose two best candidates lie within rounding of each other may
pick differently from MLX.  tests/test_oracle_skvq.py counts how many groups change their
choice between left-to-right and numpy's pairwise summation on the seeded inputs.
"""

from __future__ import annotations

import math

import numpy as np

DEFAULT_ALPHA_GRID = (1.0, 0.97, 0.94, 0.90, 0.85)   # skvq.py:61
_EPS = np.float32(1e-8)                               # skvq.py:63
f32 = np.float32


def _validate(bits, group_size, alphas):   # skvq.py:66-75
    if not 1 <= int(bits) <= 8:
        raise ValueError(f"skvq: bits={bits} must be in [1, 8] (uint8 codes)")
    if int(group_size) < 1:
        raise ValueError(f"skvq: group_size={group_size} must be >= 1")
    if len(alphas) == 0:
        raise ValueError("skvq: alphas must be non-empty")
    for a in alphas:
        if not 0.0 < float(a) <= 1.0:
            raise ValueError(f"skvq: alpha={a} must be in (0, 1]")


def clipped_group_quant(x, bits, group_size, alphas=DEFAULT_ALPHA_GRID, pairwise=False):
    """``[N, D]`` -> ``(codes u8 [N, G*gs], lo f32 [N, G], scale f32 [N, G])`` (skvq.py:105-165).
    ``pairwise=True`` lets numpy choose the order of the error sums (for the near-tie count)."""
    _validate(bits, group_size, alphas)
    x32 = np.asarray(x).astype(f32)
    n, d = x32.shape
    gs = int(group_size)
    G = (d + gs - 1) // gs
    pad = G * gs - d
    if pad:
        x32 = np.concatenate([x32, np.broadcast_to(x32[:, -1:], (n, pad))], axis=1)
    xg = x32.reshape(n, G, gs)
    gmin, gmax = xg.min(axis=-1, keepdims=True), xg.max(axis=-1, keepdims=True)
    mid = (gmax + gmin) * f32(0.5)
    rng = gmax - gmin
    levels = f32((1 << int(bits)) - 1)
    best_err = best_codes = best_lo = best_scale = None
    for a in alphas:
        ar = f32(a) * rng
        lo = mid - ar * f32(0.5)
        scale = np.maximum(ar / levels, _EPS)
        codes = np.clip(np.round((xg - lo) / scale), 0, levels)   # np.round: half to even
        sq = np.square((codes * scale + lo) - xg)
        if pairwise:
            err = sq.mean(axis=-1, dtype=f32)
        else:
            s = np.zeros((n, G), f32)
            for j in range(gs):
                s = s + sq[:, :, j]
            err = s / f32(gs)
        if best_err is None:
            best_err, best_codes, best_lo, best_scale = err, codes, lo[..., 0], scale[..., 0]
        else:   # argmin keeps the first of equal candidates
            better = err < best_err
            best_err = np.where(better, err, best_err)
            best_codes = np.where(better[..., None], codes, best_codes)
            best_lo = np.where(better, lo[..., 0], best_lo)
            best_scale = np.where(better, scale[..., 0], best_scale)
    return best_codes.reshape(n, G * gs).astype(np.uint8), best_lo.astype(f32), best_scale.astype(f32)


def clipped_group_dequant(codes, lo, scale, group_size, d):   # skvq.py:168-183
    n, gs, G = codes.shape[0], int(group_size), lo.shape[1]
    cg = codes.reshape(n, G, gs).astype(f32)
    recon = cg * scale[:, :, None] + lo[:, :, None]
    return recon.reshape(n, G * gs)[:, :d]


def skvq_compressed_bytes(n_tokens, d, bits, group_size):   # skvq.py:210-217
    G = (d + group_size - 1) // group_size
    return math.ceil(n_tokens * d * bits / 8) + n_tokens * G * 2 * 2


def skvq_fp16_bytes(n_tokens, d):   # skvq.py:220-222
    return n_tokens * d * 2


def gather_channels(x, perm):   # skvq_cache.py:226-231
    B, H, r, D = x.shape
    return np.take_along_axis(x, np.broadcast_to(perm[None, :, None, :], (B, H, r, D)), axis=-1)


def round_trip(x, perm, inv, bits, group_size, alphas):   # skvq_cache.py:236-251
    B, H, r, D = x.shape
    x32 = x.astype(f32)
    if perm is not None:
        x32 = gather_channels(x32, perm)
    codes, lo, scale = clipped_group_quant(x32.reshape(B * H * r, D), bits, group_size, alphas)
    recon = clipped_group_dequant(codes, lo, scale, group_size, D).reshape(B, H, r, D)
    if inv is not None:
        recon = gather_channels(recon, inv)
    return recon.astype(x.dtype)


def per_head_perms(chunk, bits, n_sink, group_size, alphas):   # skvq_cache.py:186-224
    B, H, r, D = chunk.shape
    x = chunk[..., n_sink:, :].astype(f32)
    xh = x.transpose(1, 0, 2, 3).reshape(H, -1, D)
    rng = xh.max(axis=1) - xh.min(axis=1)
    cand = np.argsort(rng, axis=-1, kind="stable").astype(np.int32)
    cand_inv = np.argsort(cand, axis=-1, kind="stable").astype(np.int32)
    err_id = np.square(round_trip(x, None, None, bits, group_size, alphas) - x).mean(axis=(0, 2, 3), dtype=np.float64)
    err_cand = np.square(round_trip(x, cand, cand_inv, bits, group_size, alphas) - x).mean(axis=(0, 2, 3),
                                                                                         dtype=np.float64)
    keep = (err_cand < err_id)[:, None]
    identity = np.broadcast_to(np.arange(D, dtype=np.int32)[None, :], (H, D))
    return np.where(keep, cand, identity), np.where(keep, cand_inv, identity), err_id, err_cand


class SKVQCacheModel:
    """update_and_fetch of SKVQKVCache on numpy arrays (skvq_cache.py:256-312)."""

    def __init__(self, bits_k=4, bits_v=4, group_size=32, window=128, n_sink=5, reorder=True, alphas=DEFAULT_ALPHA_GRID):
        self.bits_k, self.bits_v, self.gs, self.window, self.n_sink = bits_k, bits_v, group_size, window, n_sink
        self.reorder, self.alphas = reorder, tuple(alphas)
        self.keys = self.values = None
        self.perm_k = self.inv_k = self.perm_v = self.inv_v = None
        self.q_end = 0
        self.margins = []   # (err_id, err_cand) of every permutation decision taken

    @property
    def offset(self):
        return 0 if self.keys is None else self.keys.shape[2]

    def update_and_fetch(self, keys, values):
        self.keys = keys.copy() if self.keys is None else np.concatenate([self.keys, keys], axis=2)
        self.values = values.copy() if self.values is None else np.concatenate([self.values, values], axis=2)
        r = self.window
        while self.offset - self.q_end >= r:
            s, e = self.q_end, self.q_end + r
            kc, vc = self.keys[:, :, s:e].copy(), self.values[:, :, s:e].copy()
            if s == 0 and self.reorder:
                self.perm_k, self.inv_k, *mk = per_head_perms(kc, self.bits_k, self.n_sink, self.gs, self.alphas)
                self.perm_v, self.inv_v, *mv = per_head_perms(vc, self.bits_v, self.n_sink, self.gs, self.alphas)
                self.margins += [mk, mv]
            kq = round_trip(kc, self.perm_k, self.inv_k, self.bits_k, self.gs, self.alphas)
            vq = round_trip(vc, self.perm_v, self.inv_v, self.bits_v, self.gs, self.alphas)
            if s == 0 and self.n_sink > 0:
                kq[:, :, : self.n_sink] = kc[:, :, : self.n_sink]
                vq[:, :, : self.n_sink] = vc[:, :, : self.n_sink]
            self.keys[:, :, s:e], self.values[:, :, s:e] = kq, vq
            self.q_end = e
        return self.keys, self.values
