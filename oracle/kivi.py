"""numpy restatement of KIVI asymmetric group quantisation and bit packing.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

All arithmetic is IEEE float32 with one rounding per operation, exactly as the
reference's pure-MLX path performs it:

* ``veloxquant_mlx/cache/kivi_cache.py:181-201``  (round trip, edge-replicated
  padding, eps-floored scale, round-half-even, clip, ``code*scale + gmin``)
* ``benchmark_scripts/benchmark_real_model_scalar_attend.py:115-153`` and
  ``veloxquant_mlx/tests/metal/test_scalar_attend.py:51-82`` (split outputs:
  codes / scale / zero)
* ``veloxquant_mlx/quantizers/kivi.py:103-128`` (2-D research API)
* ``veloxquant_mlx/cache/turboquant_rvq_cache.py:82-126`` (uint32 packing)
* ``veloxquant_mlx/metal/src/bit_pack.metal:8-19`` (byte packing)
"""

from __future__ import annotations

import numpy as np

F32 = np.float32


def _grouped(x32: np.ndarray, axis: int, g: int):
    """Move ``axis`` last, pad the ragged tail by repeating the last element
    and reshape to ``[..., n_groups, g]`` (kivi_cache.py:183-193)."""
    xm = np.moveaxis(x32, axis, -1)
    L = xm.shape[-1]
    n_groups = (L + g - 1) // g
    pad = n_groups * g - L
    if pad:
        tail = np.broadcast_to(xm[..., -1:], xm.shape[:-1] + (pad,))
        xm = np.concatenate([xm, tail], axis=-1)
    return xm.reshape(xm.shape[:-1] + (n_groups, g)), L


def group_quant_codes(x, axis: int, group_size: int, levels: int, eps: float = 1e-8):
    """Asymmetric min/max group quantisation along ``axis`` (-2 keys, -1 values).

    Returns ``(codes uint8 like x, scale f32, zero f32)``; for ``axis=-2`` the
    parameter arrays are ``[..., ceil(S/g), D]``, for ``axis=-1`` they are
    ``[..., S, ceil(D/g)]`` (test_scalar_attend.py:51-82).
    """
    if axis not in (-1, -2):
        raise ValueError("axis must be -1 or -2")
    x32 = np.asarray(x).astype(F32)
    xg, L = _grouped(x32, axis, group_size)
    gmin = xg.min(axis=-1, keepdims=True)
    gmax = xg.max(axis=-1, keepdims=True)
    scale = np.maximum((gmax - gmin) / F32(levels), F32(eps)).astype(F32)
    q = np.clip(np.round((xg - gmin) / scale), 0, levels)
    codes = q.reshape(q.shape[:-2] + (-1,))[..., :L].astype(np.uint8)
    codes = np.moveaxis(codes, -1, axis)
    scale = scale[..., 0]
    zero = gmin[..., 0]
    if axis == -2:
        # [..., D, GK] -> [..., GK, D]
        scale = np.swapaxes(scale, -1, -2)
        zero = np.swapaxes(zero, -1, -2)
    return np.ascontiguousarray(codes), np.ascontiguousarray(scale), np.ascontiguousarray(zero)


def group_dequant(codes, scale, zero, axis: int, group_size: int) -> np.ndarray:
    """``code*scale + zero`` with two float32 roundings
    (kivi_group_quant_channel.metal:83-87, scalar_affine_decode_once.metal:44)."""
    codes = np.asarray(codes)
    S, D = codes.shape[-2], codes.shape[-1]
    c32 = codes.astype(F32)
    scale = np.asarray(scale).astype(F32)
    zero = np.asarray(zero).astype(F32)
    if axis == -2:
        gi = np.arange(S) // group_size
        s = scale[..., gi, :]
        z = zero[..., gi, :]
    elif axis == -1:
        gi = np.arange(D) // group_size
        s = scale[..., :, gi]
        z = zero[..., :, gi]
    else:
        raise ValueError("axis must be -1 or -2")
    prod = (c32 * s).astype(F32)
    return (prod + z).astype(F32)


def quant_dequant_along(x, axis: int, group_size: int, levels: int, eps: float = 1e-8,
                        cast=None) -> np.ndarray:
    """The reference cache's in-place round trip (kivi_cache.py:151-201).

    ``cast`` converts the float32 reconstruction to the storage dtype; the
    default casts back to ``x.dtype`` (numpy has no bfloat16, callers pass a
    torch-based cast for that)."""
    x = np.asarray(x)
    codes, scale, zero = group_quant_codes(x, axis, group_size, levels, eps)
    recon = group_dequant(codes, scale, zero, axis, group_size)
    if cast is not None:
        return cast(recon)
    return recon.astype(x.dtype)


# ---------------------------------------------------------------------------
# packing
# ---------------------------------------------------------------------------

def pack_indices(idx, bits: int) -> np.ndarray:
    """Pack the trailing axis into uint32 words, ``32 // bits`` codes per word,
    element ``i`` of a word at bits ``[i*bits, (i+1)*bits)``; a partial last
    word is zero padded (turboquant_rvq_cache.py:82-106)."""
    idx = np.asarray(idx)
    d = idx.shape[-1]
    per = 32 // bits
    pad = (-d) % per
    if pad:
        idx = np.concatenate([idx, np.zeros(idx.shape[:-1] + (pad,), idx.dtype)], axis=-1)
    w = idx.reshape(idx.shape[:-1] + ((d + pad) // per, per)).astype(np.uint64)
    shifts = (np.arange(per, dtype=np.uint64) * np.uint64(bits))
    return (w << shifts).sum(axis=-1).astype(np.uint32)


def unpack_indices(packed, bits: int, d: int) -> np.ndarray:
    """Inverse of :func:`pack_indices` (turboquant_rvq_cache.py:109-126)."""
    packed = np.asarray(packed).astype(np.uint32)
    per = 32 // bits
    shifts = (np.arange(per, dtype=np.uint32) * np.uint32(bits))
    mask = np.uint32((1 << bits) - 1)
    ex = (packed[..., None] >> shifts) & mask
    return ex.reshape(packed.shape[:-1] + (-1,))[..., :d].astype(np.uint8)


def pack_bytes(indices, bits: int) -> np.ndarray:
    """Flat byte packing, ``8 // bits`` codes per byte LSB first
    (bit_pack.metal:8-19, _bit_packing.py:87-118).  ``len(indices)`` must be a
    multiple of ``8 // bits``."""
    flat = np.asarray(indices).reshape(-1).astype(np.uint32)
    per = 8 // bits
    if flat.size % per:
        raise ValueError("length must be a multiple of 8 // bits")
    w = flat.reshape(-1, per) & np.uint32((1 << bits) - 1)
    shifts = np.arange(per, dtype=np.uint32) * np.uint32(bits)
    return (w << shifts).sum(axis=-1).astype(np.uint8)


def unpack_bytes(packed, n: int, bits: int) -> np.ndarray:
    """Inverse of :func:`pack_bytes` (bit_unpack.metal:8-15)."""
    p = np.asarray(packed).reshape(-1).astype(np.uint32)
    per = 8 // bits
    shifts = np.arange(per, dtype=np.uint32) * np.uint32(bits)
    ex = (p[:, None] >> shifts) & np.uint32((1 << bits) - 1)
    return ex.reshape(-1)[:n].astype(np.uint8)


# ---------------------------------------------------------------------------
# cache frontier + byte accounting (pure integer arithmetic)
# ---------------------------------------------------------------------------

def quantization_boundary(offset: int, residual_length: int, group_size: int) -> int:
    """kivi_cache.py:206-225."""
    aged = max(0, offset - residual_length)
    return (aged // group_size) * group_size


def quantized_bytes(n: int, B: int, H: int, D: int, bits: int, group_size: int):
    """kivi_cache.py:301-306 (fp16 scale+zero)."""
    import math
    k = math.ceil(n * D * bits / 8) * H * B + math.ceil(n / group_size) * D * 2 * 2 * H * B
    v = math.ceil(n * D * bits / 8) * H * B + n * math.ceil(D / group_size) * 2 * 2 * H * B
    return k, v


class KiviCacheModel:
    """numpy model of ``KIVIKVCache.update_and_fetch`` / ``trim``
    (kivi_cache.py:230-332): fp16 history, in-place round trip of the
    group-aligned prefix that aged out of the residual window."""

    def __init__(self, bits=2, group_size=32, residual_length=128):
        self.bits, self.g, self.R = bits, group_size, residual_length
        self.levels = (1 << bits) - 1
        self.keys = None
        self.values = None
        self.offset = 0
        self.n_quantized = 0
        self.key_bytes_compressed = 0
        self.value_bytes_compressed = 0
        self.key_bytes_fp16 = 0
        self.value_bytes_fp16 = 0
        self.residual_fp16_bytes = 0
        self.tokens_seen = 0
        self.shape_bhd = (1, 1, 0)

    def update_and_fetch(self, keys, values):
        B, H, S, D = keys.shape
        self.shape_bhd = (B, H, D)
        if self.keys is None:
            self.keys, self.values = keys.copy(), values.copy()
        else:
            self.keys = np.concatenate([self.keys[:, :, : self.offset], keys], axis=2)
            self.values = np.concatenate([self.values[:, :, : self.offset], values], axis=2)
        self.offset += S
        nb = quantization_boundary(self.offset, self.R, self.g)
        n_now = nb - self.n_quantized
        if n_now > 0:
            lo, hi = self.n_quantized, nb
            self.keys[:, :, lo:hi] = quant_dequant_along(self.keys[:, :, lo:hi], -2, self.g, self.levels)
            self.values[:, :, lo:hi] = quant_dequant_along(self.values[:, :, lo:hi], -1, self.g, self.levels)
            self.n_quantized = nb
            k, v = quantized_bytes(n_now, B, H, D, self.bits, self.g)
            self.key_bytes_compressed += k
            self.value_bytes_compressed += v
        self.residual_fp16_bytes = (self.offset - self.n_quantized) * D * 2 * 2 * H * B
        self.key_bytes_fp16 += H * B * S * D * 2
        self.value_bytes_fp16 += H * B * S * D * 2
        self.tokens_seen += S
        return self.keys[:, :, : self.offset], self.values[:, :, : self.offset]

    def trim(self, n: int) -> int:
        n = min(self.offset, n)
        self.offset -= n
        if n:
            B, H, D = self.shape_bhd
            new_nq = min(self.n_quantized, (max(self.offset, 0) // self.g) * self.g)
            rolled = self.n_quantized - new_nq
            self.n_quantized = new_nq
            if rolled > 0:
                k, v = quantized_bytes(rolled, B, H, D, self.bits, self.g)
                self.key_bytes_compressed = max(0, self.key_bytes_compressed - k)
                self.value_bytes_compressed = max(0, self.value_bytes_compressed - v)
            self.key_bytes_fp16 = max(0, self.key_bytes_fp16 - H * B * n * D * 2)
            self.value_bytes_fp16 = max(0, self.value_bytes_fp16 - H * B * n * D * 2)
            self.tokens_seen = max(0, self.tokens_seen - n)
            self.residual_fp16_bytes = (self.offset - self.n_quantized) * D * 2 * 2 * H * B
        return n


class SinkCacheModel(KiviCacheModel):
    """numpy model of ``SinkProtectedKVCache`` (cache/sink_cache.py:62-225): KIVI with the
    ``n_sink`` highest-key-norm token positions of every batch element kept in fp16.  The
    selection signal is the key L2 norm averaged over kv heads (``:97-110``), a running top-k per
    batch element (``:105-110``); inside a block that is being quantised a sink row is replaced
    by its nearest non-sink neighbour of the same batch element before the group parameters are
    computed (``:146-175``) and restored to its fp16 value afterwards (``:178-186``)."""

    def __init__(self, bits=2, group_size=32, residual_length=128, n_sink=5):
        super().__init__(bits, group_size, residual_length)
        self.n_sink = n_sink
        self.sink_norms: list[dict[int, float]] = []
        self.sink_fp16_bytes = 0

    def _update_sinks(self, keys, start):
        B = keys.shape[0]
        while len(self.sink_norms) < B:
            self.sink_norms.append({})
        if self.n_sink == 0:
            return [set() for _ in range(B)]
        per_tok = np.sqrt((keys.astype(F32) ** 2).sum(-1, dtype=F32)).mean(axis=1)   # [B, S]
        for b in range(B):
            d = self.sink_norms[b]
            for i, v in enumerate(per_tok[b].tolist()):
                d[start + i] = float(v)
            if len(d) > self.n_sink:
                self.sink_norms[b] = dict(sorted(d.items(), key=lambda kv: -kv[1])[: self.n_sink])
        return [set(self.sink_norms[b]) for b in range(B)]

    @staticmethod
    def neighbour(idx, sink_set, n):
        """Row that stands in for sink row ``idx`` of an ``n``-row block, or None (:160-171)."""
        src = idx - 1
        while src in sink_set and src > 0:
            src -= 1
        if src < 0 or src in sink_set:
            src = idx + 1
            while src in sink_set and src < n - 1:
                src += 1
        return src if 0 <= src < n and src not in sink_set else None

    def update_and_fetch(self, keys, values):
        B, H, S, D = keys.shape
        self.shape_bhd = (B, H, D)
        start = self.offset
        sinks = self._update_sinks(keys, start)
        if self.keys is None:
            self.keys, self.values = keys.copy(), values.copy()
        else:
            self.keys = np.concatenate([self.keys[:, :, : self.offset], keys], axis=2)
            self.values = np.concatenate([self.values[:, :, : self.offset], values], axis=2)
        self.offset += S
        nb = quantization_boundary(self.offset, self.R, self.g)
        n_now = nb - self.n_quantized
        n_sink_in_block = 0
        if n_now > 0:
            lo, hi = self.n_quantized, nb
            k_reg, v_reg = self.keys[:, :, lo:hi].copy(), self.values[:, :, lo:hi].copy()
            local = [sorted(p - lo for p in sinks[b] if lo <= p < hi) for b in range(B)]
            for b in range(B):
                ss = set(local[b])
                for idx in local[b]:
                    src = self.neighbour(idx, ss, n_now)
                    if src is not None:
                        k_reg[b, :, idx] = self.keys[b, :, lo + src]
                        v_reg[b, :, idx] = self.values[b, :, lo + src]
            k_q = quant_dequant_along(k_reg, -2, self.g, self.levels)
            v_q = quant_dequant_along(v_reg, -1, self.g, self.levels)
            for b in range(B):
                n_sink_in_block = max(n_sink_in_block, len(local[b]))
                for idx in local[b]:
                    k_q[b, :, idx] = self.keys[b, :, lo + idx]
                    v_q[b, :, idx] = self.values[b, :, lo + idx]
            self.keys[:, :, lo:hi] = k_q
            self.values[:, :, lo:hi] = v_q
            self.n_quantized = nb
        n_comp = n_now - n_sink_in_block
        if n_comp > 0:
            k, v = quantized_bytes(n_comp, B, H, D, self.bits, self.g)
            self.key_bytes_compressed += k
            self.value_bytes_compressed += v
        self.sink_fp16_bytes += n_sink_in_block * D * 2 * 2 * H * B
        self.residual_fp16_bytes = (self.offset - self.n_quantized) * D * 2 * 2 * H * B
        self.key_bytes_fp16 += H * B * S * D * 2
        self.value_bytes_fp16 += H * B * S * D * 2
        self.tokens_seen += S
        return self.keys[:, :, : self.offset], self.values[:, :, : self.offset]

    def trim(self, n: int) -> int:
        """sink_cache.py:200-225: the frontier snaps down to a group multiple; protected rows of the
        stretch that is live again (largest count over the batch, as the flush counted them) leave
        the fp16 pool; candidates at dropped positions are forgotten."""
        n = min(self.offset, n)
        if not n:
            return n
        old_nq = self.n_quantized
        self.offset -= n
        B, H, D = self.shape_bhd
        new_nq = min(old_nq, (max(self.offset, 0) // self.g) * self.g)
        rolled = old_nq - new_nq
        self.n_quantized = new_nq
        back = 0
        for b, norms in enumerate(self.sink_norms):
            back = max(back, sum(1 for p in norms if new_nq <= p < old_nq))
            self.sink_norms[b] = {p: x for p, x in norms.items() if p < self.offset}
        back = min(back, rolled)
        if rolled - back > 0:
            k, v = quantized_bytes(rolled - back, B, H, D, self.bits, self.g)
            self.key_bytes_compressed = max(0, self.key_bytes_compressed - k)
            self.value_bytes_compressed = max(0, self.value_bytes_compressed - v)
        self.key_bytes_fp16 = max(0, self.key_bytes_fp16 - H * B * n * D * 2)
        self.value_bytes_fp16 = max(0, self.value_bytes_fp16 - H * B * n * D * 2)
        self.tokens_seen = max(0, self.tokens_seen - n)
        self.residual_fp16_bytes = (self.offset - self.n_quantized) * D * 2 * 2 * H * B
        self.sink_fp16_bytes = max(0, self.sink_fp16_bytes - back * D * 2 * 2 * H * B)
        return n

    def sink_positions_for(self, b):
        if b >= len(self.sink_norms):
            return []
        return [p for p, _ in sorted(self.sink_norms[b].items(), key=lambda kv: -kv[1])]
