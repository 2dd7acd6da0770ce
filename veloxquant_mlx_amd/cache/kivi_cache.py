"""KIVI KV cache on torch ROCm tensors.

Behaviour follows ``KIVIKVCache`` (veloxquant_mlx/cache/kivi_cache.py:83-410):
keys are quantised per channel (groups along tokens), values per token (groups
along channels), the newest ``residual_length`` tokens stay fp16, and tokens are
flushed only in whole ``kivi_group_size`` blocks.

Three storage modes, selected with the same two flags the reference's VecInfer
cache uses (veloxquant_mlx/cache/vecinfer_cache.py:384-411):

* ``fused_sdpa=False`` (default) -- the reference's behaviour: an fp16 history
  whose aged-out prefix is round-tripped in place; ``update_and_fetch`` returns
  fp16 ``[B,H,offset,D]``.
* ``fused_sdpa=True`` -- the same, plus bit-packed codes and scale/zero kept
  beside it so :meth:`fused_sdpa` can attend over the packed prefix.
* ``fused_sdpa=True, fused_sdpa_memory_bound=True`` -- packed prefix and a short
  fp16 tail only; ``update_and_fetch`` returns zero-stride placeholders and
  attention must go through :meth:`fused_sdpa`.
"""

from __future__ import annotations

import math
import os
from typing import Any

import torch

from .. import kernels as K
from ..core.exceptions import QuantizerConfigError
from ._fp16_cache import FP16KVCache

_META = {"float16": torch.float16, "float32": torch.float32}


def pair_heads(x: torch.Tensor) -> torch.Tensor:
    """``[..., H, S, D]`` -> ``[..., ceil(H/2), S, 2D]``: kv heads 2m and 2m+1 side by side in one head of twice the
    channels (an odd count gets a head of zeros for the last one's partner).  Group quantisation along tokens is per
    channel and along channels per group of ``g`` (``g`` divides ``D``), so the codes, scale and zero of the paired head
    are those of the two heads."""
    *lead, H, S, D = x.shape
    if H % 2:
        x = torch.cat([x, x.new_zeros((*lead, 1, S, D))], dim=-3)
        H += 1
    return x.reshape(*lead, H // 2, 2, S, D).transpose(-3, -2).reshape(*lead, H // 2, S, 2 * D)


def pad_queries_for_paired_heads(q: torch.Tensor, n_kv_heads: int, out: torch.Tensor | None = None) -> torch.Tensor:
    """``q [..., H_q, S_q, D]`` -> ``[..., 2 * ceil(H/2) * R, S_q, 2D]`` for a cache of paired kv heads (``H`` kv heads,
    ``R = H_q / H``): a query head's channels in the half of its own kv head, zeros in the other
    (``q . [k_a, k_b] = q . k_a``); with an odd ``H`` the partner of the last kv head brings ``R`` query heads of zeros
    along.  ``out``: a buffer of the result's shape whose other halves are already zero."""
    *lead, Hq, Sq, D = q.shape
    H, R, P = n_kv_heads, Hq // n_kv_heads, (n_kv_heads + 1) // 2
    if out is None:
        out = q.new_zeros((*lead, 2 * P * R, Sq, 2 * D))
    wide = out.view(*lead, P, 2, R, Sq, 2, D).diagonal(dim1=-5, dim2=-2)      # [..., P, R, Sq, D, 2]
    if H % 2 == 0:
        wide.copy_(q.reshape(*lead, P, 2, R, Sq, D).movedim(-4, -1))
    else:
        heads = q.reshape(*lead, H, R, Sq, D)
        wide[..., 0].copy_(heads[..., 0::2, :, :, :])
        if H > 1:
            wide[..., : H // 2, :, :, :, 1].copy_(heads[..., 1::2, :, :, :])
    return out


def own_half_of_paired_output(o: torch.Tensor, n_kv_heads: int) -> torch.Tensor:
    """``o [..., 2 * ceil(H/2) * R, S_q, 2D]`` (attention over paired kv heads) -> ``[..., H * R, S_q, D]``: every
    query head's own half."""
    *lead, Hq2, Sq, D2 = o.shape
    H, P, D = n_kv_heads, (n_kv_heads + 1) // 2, D2 // 2
    R = Hq2 // (2 * P)
    own = o.view(*lead, P, 2, R, Sq, 2, D).diagonal(dim1=-5, dim2=-2)          # [..., P, R, Sq, D, 2]
    if H % 2 == 0:
        return own.movedim(-1, -4).reshape(*lead, H * R, Sq, D)
    res = o.new_empty((*lead, H, R, Sq, D))
    res[..., 0::2, :, :, :] = own[..., 0]
    if H > 1:
        res[..., 1::2, :, :, :] = own[..., : H // 2, :, :, :, 1]
    return res.view(*lead, H * R, Sq, D)


class KIVIKVCache(FP16KVCache):
    """KV cache with KIVI asymmetric group quantisation.

    Never exposes ``.bits`` (a host attention dispatcher would take it for a
    natively quantised cache, kivi_cache.py:93-95); see ``assigned_avg_bits``.
    """

    # append + flush + next tail in one library call; a subclass that works on the rows of a flush
    # before they are packed turns it off and gets them through _pack_block
    _one_call_append = True

    def __init__(self, config: Any) -> None:
        super().__init__()
        self._head_dim = int(config.head_dim)
        b = config.bit_width_inlier
        if isinstance(b, list):
            raise QuantizerConfigError(
                "KIVIKVCache: bit_width_inlier must be a single int; "
                "per-layer lists are dispatched by KVCacheBuilder.for_model().")
        self._b = int(b)
        if not (1 <= self._b <= 8):
            raise QuantizerConfigError(f"KIVIKVCache: bit_width_inlier={self._b} must be in [1, 8].")
        self._group_size = int(getattr(config, "kivi_group_size", 32))
        self._residual_length = int(getattr(config, "residual_length", 128))
        if self._group_size < 1:
            raise QuantizerConfigError(f"KIVIKVCache: kivi_group_size={self._group_size} must be >= 1.")
        self._levels = (1 << self._b) - 1
        self._eps = 1e-8

        # use_metal_kernels keeps its three states (kivi_cache.py:113-130).  The
        # HIP library is the only implementation, so True and None both require
        # it and False selects the same kernels (the reference's two paths are
        # bit-identical by contract).
        requested = getattr(config, "use_metal_kernels", None)
        available = K._lib.library_present()
        if not available:
            raise RuntimeError(
                "KIVIKVCache: the HIP kernel library is not available on this build "
                f"(use_metal_kernels={requested!r}); there is no fallback path.")
        self._use_metal = True

        fused = bool(getattr(config, "fused_sdpa", False))
        self._memory_bound = bool(getattr(config, "fused_sdpa_memory_bound", False))
        if self._memory_bound and not fused:
            raise RuntimeError("KIVIKVCache: fused_sdpa_memory_bound=True requires fused_sdpa=True.")
        self._fused_enabled = fused
        cap = getattr(config, "fused_sdpa_max_ctx", None)
        self._max_ctx = None if cap is None else int(cap)
        meta = getattr(config, "kivi_meta_dtype", "float16")
        if meta not in _META:
            raise QuantizerConfigError(f"KIVIKVCache: kivi_meta_dtype={meta!r} must be 'float16' or 'float32'.")
        self._meta_dtype = _META[meta]
        # bits a code takes in the packed words: the quantiser's own width, or the next width the matrix-unit
        # kernels read (2 for 1-bit codes, 4 for 3-bit codes); the levels, hence every value, are the same
        field = getattr(config, "kivi_code_field", "auto")
        if field not in ("auto", "tight"):
            raise QuantizerConfigError(f"KIVIKVCache: kivi_code_field={field!r} must be 'auto' or 'tight'.")
        self._field = {1: 2, 3: 4}.get(self._b, self._b) if field == "auto" else self._b
        per = 32 // self._field
        layout = getattr(config, "kivi_value_layout", "auto")
        if layout == "auto":
            layout = "token" if self._group_size % per == 0 else "channel"
        if layout not in ("token", "channel"):
            raise QuantizerConfigError(f"KIVIKVCache: kivi_value_layout={layout!r} must be token/channel/auto.")
        if layout == "token" and self._group_size % per != 0:
            raise QuantizerConfigError(
                f"KIVIKVCache: token-packed values need kivi_group_size % {per} == 0 at {self._field} bits a code.")
        self._v_layout = layout
        self._per = per
        # heads of 64 channels, memory-bound mode: kv heads 2m and 2m+1 are kept side by side as one head of 128
        # channels (same codes, scale and zero; queries zero-padded into their own half), the head size the
        # matrix-unit kernels and the one-launch append take; decided at the first tokens (an even head count)
        self._pair_wanted = (bool(getattr(config, "kivi_pair_heads", True)) and self._memory_bound and self._head_dim == 64
                             and type(self) is KIVIKVCache and 64 % self._group_size == 0)
        self._pair = False
        self._kv_heads = 0     # the caller's kv head count while heads are kept in pairs
        self._q_pad = None

        # byte accounting (kivi_cache.py:132-146)
        for counter in ("_key_bytes_compressed", "_key_bytes_fp16", "_value_bytes_compressed", "_value_bytes_fp16",
                        "_residual_fp16_bytes", "_tokens_seen", "_n_quantized"):
            setattr(self, counter, 0)
        self._shape_bhd: tuple[int, int, int] = (1, 1, int(config.head_dim))

        # packed store (fused modes)
        self._kp = self._ks = self._kz = None
        self._vp = self._vs = self._vz = None
        self._packed_cap = 0
        # fp16 tail (memory-bound mode): tokens [_n_quantized, offset)
        self._tail_k = self._tail_v = None
        self._tail_spare = None   # second pair of tail buffers the kept rows move into at a flush
        self._append_args = None  # argument block of the one-call append, refilled from chunk to chunk
        # memory-bound decode: the newest token's (keys, values), counted in ``offset`` but not yet in the
        # tail; the next fused_sdpa stores them in the same launch that attends, anything else stores them first
        self._pending = None
        self._zero_scalar = None
        # memory-bound prefill: the slots once more as ready-made fp16 tiles for prefill-sized attention calls
        # (scratch of the prefill phase, given back at the first decode step); the first _tiles_packed units
        # hold packed slots that cannot change any more
        self.prefill_tiles = os.environ.get("VELOXQUANT_PREFILL_TILES", "1") != "0"
        self.prefill_tiles_max_bytes = 256 << 20   # per cache (layer); a longer prefill goes on without tiles
        self._tiles = None
        self._tiles_packed = 0

    # ------------------------------------------------------------------
    def _quant_dequant_along(self, x: torch.Tensor, axis: int) -> torch.Tensor:
        """Round-trip ``x`` through group quantisation (kivi_cache.py:151-201)."""
        return K.kivi_group_quant_dequant(x, axis=axis, group_size=self._group_size, levels=self._levels,
                                          eps=self._eps)

    def _quantization_boundary(self) -> int:
        """Absolute position up to which tokens may be quantised now (kivi_cache.py:206-225)."""
        aged = max(0, self.offset - self._residual_length)
        return (aged // self._group_size) * self._group_size

    # ------------------------------------------------------------------ packed store
    def _ensure_packed_capacity(self, B: int, H: int, D: int, needed: int, device) -> None:
        if self._max_ctx is not None and needed > self._max_ctx:
            raise RuntimeError(f"KIVIKVCache: context length {needed} exceeded fused_sdpa_max_ctx={self._max_ctx}. "
                               "Raise or unset KVCacheConfig.fused_sdpa_max_ctx.")
        if needed <= self._packed_cap:
            return
        g, per = self._group_size, self._per
        unit = g * per // math.gcd(g, per)
        cap = max(needed, 2 * self._packed_cap, 1024)
        if self._max_ctx is not None:
            # a stated limit sizes the store once, as the reference's index buffers are "allocated at
            # fused_sdpa_max_ctx, not at the live length"
            # (veloxquant_mlx/tests/cache/test_vecinfer_fused_sdpa.py:342-346)
            cap = self._max_ctx
        cap = -(-cap // unit) * unit
        W = -(-D // per)
        GV = -(-D // g)
        z = lambda shape, dt: torch.zeros(shape, dtype=dt, device=device)
        kp = z((B, H, cap, W), torch.int32)
        ks = z((B, H, cap // g, D), self._meta_dtype)
        kz = z((B, H, cap // g, D), self._meta_dtype)
        if self._v_layout == "token":
            vp = z((B, H, cap // per, D), torch.int32)
            vs = z((B, H, GV, cap), self._meta_dtype)
            vz = z((B, H, GV, cap), self._meta_dtype)
        else:
            vp = z((B, H, cap, W), torch.int32)
            vs = z((B, H, cap, GV), self._meta_dtype)
            vz = z((B, H, cap, GV), self._meta_dtype)
        n = self._n_quantized
        if self._kp is not None and n > 0:
            kp[:, :, :n] = self._kp[:, :, :n]
            ks[:, :, : n // g] = self._ks[:, :, : n // g]
            kz[:, :, : n // g] = self._kz[:, :, : n // g]
            if self._v_layout == "token":
                vp[:, :, : n // per] = self._vp[:, :, : n // per]
                vs[..., :n] = self._vs[..., :n]
                vz[..., :n] = self._vz[..., :n]
            else:
                vp[:, :, :n] = self._vp[:, :, :n]
                vs[:, :, :n] = self._vs[:, :, :n]
                vz[:, :, :n] = self._vz[:, :, :n]
        self._kp, self._ks, self._kz, self._vp, self._vs, self._vz = kp, ks, kz, vp, vs, vz
        self._packed_cap = cap

    def _pack_block(self, k_blk: torch.Tensor, v_blk: torch.Tensor, lo: int) -> None:
        """Quantise + pack fp16 tokens (a group-aligned block) at packed position ``lo``."""
        B, H, n, D = k_blk.shape
        self._ensure_packed_capacity(B, H, D, lo + n, k_blk.device)
        K.kivi_quant_pack(k_blk, -2, self._group_size, self._field, levels=self._levels, eps=self._eps,
                          meta_dtype=self._meta_dtype, out=(self._kp, self._ks, self._kz), dst_tok0=lo)
        K.kivi_quant_pack(v_blk, -1, self._group_size, self._field, levels=self._levels, eps=self._eps,
                          meta_dtype=self._meta_dtype, v_layout=self._v_layout, out=(self._vp, self._vs, self._vz), dst_tok0=lo)

    # ------------------------------------------------------------------ protocol
    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        """Append ``[B,H,S,D]`` keys/values and quantise whatever aged out of the
        fp16 residual window, in ``kivi_group_size``-aligned blocks
        (kivi_cache.py:230-262)."""
        B, H, S, D = keys.shape
        if self._memory_bound:
            if self.offset == 0 and self._n_quantized == 0:
                # (an odd head count pairs its last head with a head of zeros: not worth it for a single head)
                self._pair = self._pair_wanted and D == 64 and H >= 2
                self._kv_heads = H
            if self._pair:
                # (a restored state shows the pairs, not whether the last one is whole: the first keys say)
                same = H == self._kv_heads or (self._kv_heads < 0 and (H + 1) // 2 == self._shape_bhd[1])
                if D != 64 or not same:
                    raise ValueError(f"KIVIKVCache.update_and_fetch: this cache pairs {abs(self._kv_heads)} kv heads of 64 channels, "
                                     f"got {tuple(keys.shape)}")
                self._kv_heads = H
                self._shape_bhd = (B, (H + 1) // 2, 2 * D)
                self._update_memory_bound(pair_heads(keys), pair_heads(values))
                z = self._zero_scalar
                return z.expand(B, H, self.offset, D), z.expand(B, H, self.offset, D)
            self._shape_bhd = (B, H, D)
            return self._update_memory_bound(keys, values)
        self._shape_bhd = (B, H, D)
        k_all, v_all = super().update_and_fetch(keys, values)
        new_boundary = self._quantization_boundary()
        n_quant_now = new_boundary - self._n_quantized
        if n_quant_now > 0:
            lo, hi = self._n_quantized, new_boundary
            if self._fused_enabled:
                # pack from the still-exact fp16 rows before they are overwritten
                self._pack_block(self.keys[:, :, lo:hi], self.values[:, :, lo:hi], lo)
            self.keys[:, :, lo:hi] = self._quant_dequant_along(self.keys[:, :, lo:hi], axis=-2)
            self.values[:, :, lo:hi] = self._quant_dequant_along(self.values[:, :, lo:hi], axis=-1)
            self._n_quantized = new_boundary
            k_all, v_all = self.keys[:, :, : self.offset], self.values[:, :, : self.offset]
        self._account_bytes(B, H, S, D, n_quant_now)
        return k_all, v_all

    def _store_pending(self) -> None:
        """Write a deferred newest token into the tail (see ``_pending``)."""
        if self._pending is not None:
            k, v = self._pending
            self._pending = None
            K.kv_tail_append(k, v, self._tail_k, self._tail_v, self.offset - self._n_quantized - 1)

    def _update_memory_bound(self, keys: torch.Tensor, values: torch.Tensor):
        B, H, S, D = keys.shape
        self._store_pending()
        if S == 1:
            self._drop_tiles()   # decoding has begun: the prefill scratch goes back
        n_tail = self.offset - self._n_quantized
        need = n_tail + S
        if (S == 1 and self._n_quantized > 0 and self._tail_k is not None and need <= self._tail_k.shape[2]
                and keys.dtype == self._tail_k.dtype and values.dtype == keys.dtype and D == 128
                and keys.is_contiguous() and values.is_contiguous() and keys.data_ptr() % 16 == 0
                and values.data_ptr() % 16 == 0
                and (max(0, self.offset + 1 - self._residual_length) // self._group_size) * self._group_size
                == self._n_quantized):
            # a plain decode step with no flush due: the attention launch of this step stores the token.
            # Until then the cache holds the caller's tensors, not a copy: a caller that reuses its key /
            # value buffers between update_and_fetch and fused_sdpa must pass clones.
            self._pending = (keys, values)
            self.offset += 1
            self._account_bytes(B, H, S, D, 0)
            z = self._zero_scalar
            if z is None or z.dtype != keys.dtype or z.device != keys.device:
                z = self._zero_scalar = torch.zeros((), dtype=keys.dtype, device=keys.device)
            return z.expand(B, H, self.offset, D), z.expand(B, H, self.offset, D)
        # a flush that would pass fused_sdpa_max_ctx is refused here, before offset or rows change
        new_boundary = (max(0, self.offset + S - self._residual_length) // self._group_size) * self._group_size
        n_quant_now = new_boundary - self._n_quantized
        if n_quant_now > 0:
            self._ensure_packed_capacity(B, H, D, new_boundary, keys.device)
        if self._tail_k is None or need > self._tail_k.shape[2]:
            cap = max(need, self._residual_length + 2 * self._group_size)
            cap = -(-cap // 64) * 64
            tk = torch.zeros((B, H, cap, D), dtype=keys.dtype, device=keys.device)
            tv = torch.zeros((B, H, cap, D), dtype=values.dtype, device=values.device)
            if self._tail_k is not None and n_tail:
                tk[:, :, :n_tail] = self._tail_k[:, :, :n_tail]
                tv[:, :, :n_tail] = self._tail_v[:, :, :n_tail]
            self._tail_k, self._tail_v = tk, tv
        es = keys.element_size()
        one_call = (self._one_call_append and keys.dtype == self._tail_k.dtype and values.dtype == keys.dtype
                    and (D * es) % 16 == 0 and keys.stride(3) == 1 and values.stride(3) == 1)
        if not one_call:
            self._tail_k[:, :, n_tail:need] = keys
            self._tail_v[:, :, n_tail:need] = values
        self.offset += S
        spare = None
        if n_quant_now > 0:
            keep = need - n_quant_now
            # the rows that stay move to the front of a second buffer (one copy each, no
            # temporaries); a very large prefill chunk leaves an oversized buffer behind, which is
            # given back here, while chunked prefill keeps its buffers from chunk to chunk
            floor_cap = -(-(self._residual_length + 2 * self._group_size) // 64) * 64
            cap = self._tail_k.shape[2]
            if cap > max(4 * floor_cap, 16 * keep):
                cap = max(floor_cap, -(-2 * keep // 64) * 64)
            spare = self._tail_spare
            if spare is None or spare[0].shape != (B, H, cap, D) or spare[0].dtype != self._tail_k.dtype:
                spare = (torch.zeros((B, H, cap, D), dtype=self._tail_k.dtype, device=keys.device),
                         torch.zeros((B, H, cap, D), dtype=self._tail_v.dtype, device=keys.device))
        if one_call:
            # append, quantise what aged out and start the next tail in one library call
            if any((st * es) % 16 for st in keys.stride()[:3]) or keys.data_ptr() % 16:
                keys = keys.contiguous()
            if any((st * es) % 16 for st in values.stride()[:3]) or values.data_ptr() % 16:
                values = values.contiguous()
            self._append_args = K.kivi_cache_append(
                keys, values, self._tail_k, self._tail_v, n_tail, max(n_quant_now, 0),
                (self._kp, self._ks, self._kz, self._vp, self._vs, self._vz), self._n_quantized, spare,
                bits=self._field, group_size=self._group_size, levels=self._levels, eps=self._eps,
                v_layout=self._v_layout, args=self._append_args)
        elif n_quant_now > 0:
            self._pack_block(self._tail_k[:, :, :n_quant_now], self._tail_v[:, :, :n_quant_now], self._n_quantized)
            if keep:
                spare[0][:, :, :keep] = self._tail_k[:, :, n_quant_now:need]
                spare[1][:, :, :keep] = self._tail_v[:, :, n_quant_now:need]
        if n_quant_now > 0:
            old = (self._tail_k, self._tail_v)
            self._tail_k, self._tail_v = spare
            self._tail_spare = old if old[0].shape[2] == cap else None
            self._n_quantized = new_boundary
        self._account_bytes(B, H, S, D, n_quant_now)
        z = self._zero_scalar
        if z is None or z.dtype != keys.dtype or z.device != keys.device:
            z = self._zero_scalar = torch.zeros((), dtype=keys.dtype, device=keys.device)
        return z.expand(B, H, self.offset, D), z.expand(B, H, self.offset, D)

    def fused_sdpa(self, q: torch.Tensor, scale: float, *, causal: bool = True, sliding_window: int = 0,
                   fixed_order: bool | None = None, lengths: torch.Tensor | None = None, num_splits: int = 0):
        """Attention of ``q [B,H_q,S_q,D]`` over the packed prefix and the fp16 tail,
        queries aligned to the end of the cache (the contract of
        ``VecInferKVCache.fused_sdpa``, veloxquant_mlx/cache/vecinfer_cache.py:670-731), under an
        optional ``sliding_window`` (a query sees only that many last slots up to its own).
        ``fixed_order=True`` asks for results that are identical from run to run (see
        :func:`veloxquant_mlx_amd.kernels.kivi_packed_attend`).  ``lengths`` (int ``[B]``, on the
        device or the host) gives every sequence of a right-padded batch its own number of live
        tokens: sequence ``b`` attends over its first ``lengths[b]`` slots, its queries aligned to
        the end of those.  ``num_splits`` > 0 fixes into how many runs the context is cut (0: chosen from the
        shapes; two calls that are to agree bit for bit need the same cut as well as ``fixed_order``)."""
        if not self._fused_enabled:
            raise RuntimeError("KIVIKVCache.fused_sdpa called but fused_sdpa was not enabled via "
                               "KVCacheConfig.fused_sdpa=True.")
        if self.offset == 0:
            raise RuntimeError("KIVIKVCache.fused_sdpa called before any tokens were cached via update_and_fetch.")
        if self._pair and q.shape[-1] == 64:
            H = abs(self._kv_heads)
            if self._kv_heads < 0 and q.shape[1] % H and q.shape[1] % (H - 1) == 0:
                H -= 1   # a state restored without its meta_state: the query heads do not divide over an even count
            if q.shape[1] % H:
                raise ValueError(f"KIVIKVCache.fused_sdpa: {q.shape[1]} query heads over {H} kv heads")
            key = (tuple(q.shape), q.dtype, q.device, K._stream_of(q.device))
            if self._q_pad is None or self._q_pad[0] != key:   # the zero halves are written once
                wide_heads = 2 * self._shape_bhd[1] * (q.shape[1] // H)
                self._q_pad = (key, q.new_zeros((q.shape[0], wide_heads, q.shape[2], 128)))
            wide = self.fused_sdpa(pad_queries_for_paired_heads(q, H, self._q_pad[1]), scale, causal=causal,
                                   sliding_window=sliding_window, fixed_order=fixed_order, lengths=lengths, num_splits=num_splits)
            return own_half_of_paired_output(wide, H)
        nq = self._n_quantized
        n_tail = self.offset - nq
        if q.shape[2] == 1:
            self._drop_tiles()   # a decode step, with or without per-sequence lengths
        if self._pending is not None and q.shape[2] != 1:
            self._store_pending()
        if self._memory_bound:
            tk, tv = self._tail_k, self._tail_v
        else:
            tk, tv = self.keys[:, :, nq:], self.values[:, :, nq:]
        kw = dict(k_packed=self._kp, k_scale=self._ks, k_zero=self._kz, v_packed=self._vp, v_scale=self._vs,
                  v_zero=self._vz, n_packed=nq, bits=self._field, group_size=self._group_size, v_layout=self._v_layout,
                  k_tail=tk if n_tail else None, v_tail=tv if n_tail else None, n_tail=n_tail, scale=float(scale),
                  causal=bool(causal) and q.shape[2] > 1, out_dtype=q.dtype, fixed_order=fixed_order,
                  sliding_window=int(sliding_window or 0), num_splits=max(0, int(num_splits)))
        kw.update(self._extra_attend_args())
        plan = None
        if lengths is None and self._offer_tiles(q, kw):
            plan = kw["_plan_out"] = {}
        if lengths is not None:
            self._store_pending()
            n = torch.as_tensor(lengths, device=q.device).to(torch.int64).reshape(-1)
            if n.numel() != q.shape[0]:
                raise ValueError(f"KIVIKVCache.fused_sdpa: lengths has {n.numel()} entries for a batch of {q.shape[0]}")
            kw.update(packed_lens=torch.clamp(n, max=nq), tail_lens=torch.clamp(n - nq, min=0, max=n_tail))
        if self._pending is not None:
            try:   # append and attend in one launch (single-query MFMA decode path)
                out = K.kivi_packed_attend(q, k_new=self._pending[0], v_new=self._pending[1], **kw)
                self._pending = None
                return out
            except ValueError:   # a shape that path does not take: store the token, then attend
                self._store_pending()
        out = K.kivi_packed_attend(q, **kw)
        if plan is not None and plan.get("path") == 2:   # the launch that reads the tiles has rewritten the stale ones
            self._tiles_packed = nq // 32
        return out

    def _offer_tiles(self, q: torch.Tensor, kw: dict) -> bool:
        """Give a prefill-sized call the tiles it reads instead of reconstructing the prefix in every block of the
        launch (same bits either way); the call itself first rewrites what changed since the last one: the units
        that were tail slots then, and the tail."""
        B, Hq, Sq, D = q.shape
        H = self._shape_bhd[1]
        nq, n_tail = kw["n_packed"], kw["n_tail"]
        R = Hq // max(H, 1)
        # the rows a kv head's blocks hold: below 256 the library fills a group up to the next of 1, 2, 4, 8 heads
        rows = (R if R in (1, 2, 4, 8) or (R <= 64 and R * Sq >= 256) else 4 if R == 3 else 8) * Sq
        if not (self.prefill_tiles and self._memory_bound and self._v_layout == "token" and D == 128 and Hq % H == 0
                and rows >= 256 and nq % 32 == 0 and "sinks" not in kw
                and (n_tail == 0 or self._tail_k.dtype in (torch.float16, torch.bfloat16))):
            return False
        units = -(-(nq + n_tail) // 32)
        if B * H * units * K.PREFILL_TILE_BYTES > self.prefill_tiles_max_bytes:
            self._tiles = None
            return False
        t = self._tiles
        if t is None or t.shape[0] != B * H or t.shape[1] < units or t.device != q.device:
            room = self._packed_cap + (self._tail_k.shape[2] if self._tail_k is not None else 0)
            room = min(room, self.prefill_tiles_max_bytes // (B * H * K.PREFILL_TILE_BYTES) * 32)
            t = self._tiles = K.prefill_tiles_empty(B, H, max(room, 32 * units), q.device)
            self._tiles_packed = 0
        kw["tiles"], kw["tiles_stale_from"] = t, min(self._tiles_packed, nq // 32)
        return True

    def _drop_tiles(self) -> None:
        """Give the prefill tile scratch back (it is worth ~1.2x an fp16 copy of K and V while it lives; the
        reference's memory-bound mode never holds more than one transient reconstruction)."""
        self._tiles, self._tiles_packed = None, 0

    def _extra_attend_args(self) -> dict:
        """Further arguments of the attention call (subclasses with rows kept outside the packed store)."""
        return {}

    # ------------------------------------------------------------------ trim / state
    def _rollback_frontier(self, new_offset: int) -> int:
        """kivi_cache.py:264-278: the frontier snaps down to a group multiple."""
        gs = self._group_size
        new_nq = min(self._n_quantized, (max(new_offset, 0) // gs) * gs)
        n_rolled = self._n_quantized - new_nq
        self._n_quantized = new_nq
        self._tiles_packed = 0
        return n_rolled

    def _rollback_bytes(self, n_tokens: int, n_rolled: int) -> None:
        """Take ``n_tokens`` trimmed tokens, ``n_rolled`` of them packed, back out of the counters (none goes below
        zero), kivi_cache.py:280-291."""
        B, H, D = self._shape_bhd
        row16 = B * H * D * 2                                     # one token of keys (or values) in fp16
        packed_k, packed_v = self._quantized_bytes(n_rolled, B, H, D) if n_rolled > 0 else (0, 0)
        for name, less in (("_key_bytes_compressed", packed_k), ("_value_bytes_compressed", packed_v),
                           ("_key_bytes_fp16", row16 * n_tokens), ("_value_bytes_fp16", row16 * n_tokens),
                           ("_tokens_seen", n_tokens)):
            setattr(self, name, max(0, getattr(self, name) - less))
        self._residual_fp16_bytes = 2 * row16 * (self.offset - self._n_quantized)

    def trim(self, n: int) -> int:
        """Drop the last ``n`` tokens and roll frontier and accounting back (kivi_cache.py:293-299)."""
        old_nq = self._n_quantized
        self._store_pending()
        trimmed = super().trim(n)
        if trimmed:
            n_rolled = self._rollback_frontier(self.offset)
            if self._memory_bound and self._tail_k is not None:
                # rows [new frontier, offset) that had been packed come back as their
                # reconstruction, which is what the fp16 history of the other modes holds
                live = self.offset - self._n_quantized
                if n_rolled > 0 and live > 0:
                    B, H, D = self._shape_bhd
                    if live > self._tail_k.shape[2]:
                        self._tail_k = torch.zeros((B, H, -(-live // 64) * 64, D), dtype=self._tail_k.dtype,
                                                   device=self._tail_k.device)
                        self._tail_v = torch.zeros_like(self._tail_k)
                    lo = self._n_quantized
                    self._tail_k[:, :, :live] = K.kivi_dequant(
                        self._kp, self._ks, self._kz, -2, self._group_size, self._field, live, D,
                        out_dtype=self._tail_k.dtype, src_tok0=lo)
                    self._tail_v[:, :, :live] = K.kivi_dequant(
                        self._vp, self._vs, self._vz, -1, self._group_size, self._field, live, D,
                        v_layout=self._v_layout, out_dtype=self._tail_v.dtype, src_tok0=lo)
            self._rollback_bytes(trimmed, n_rolled)
        del old_nq
        return trimmed

    def empty(self) -> bool:
        if self._memory_bound:
            return self.offset == 0
        return super().empty()

    @property
    def state(self):
        """Standard / stash mode: the fp16 history (stash mode appends the live packed
        rows).  Memory-bound mode: live packed rows followed by the live fp16 tail."""
        if not self._fused_enabled:
            return FP16KVCache.state.fget(self)
        self._store_pending()
        packed = self._packed_state()
        if not self._memory_bound:
            return (*FP16KVCache.state.fget(self), *packed)
        n_tail = self.offset - self._n_quantized
        if self._tail_k is None:
            return packed
        return (*packed, self._tail_k[:, :, :n_tail], self._tail_v[:, :, :n_tail])

    def _packed_state(self):
        n, g, per = self._n_quantized, self._group_size, self._per
        if self._kp is None or n == 0:
            return ()
        if self._v_layout == "token":
            v = (self._vp[:, :, : n // per], self._vs[..., :n], self._vz[..., :n])
        else:
            v = (self._vp[:, :, :n], self._vs[:, :, :n], self._vz[:, :, :n])
        return (self._kp[:, :, :n], self._ks[:, :, : n // g], self._kz[:, :, : n // g], *v)

    @state.setter
    def state(self, v) -> None:
        """Inverse of the getter, mode by mode.  The frontier comes from the packed rows' own
        length; byte accounting is rebuilt for the restored token count."""
        v = tuple(v)
        self._pending = None
        if not self._fused_enabled:
            FP16KVCache.state.fset(self, v)
            if v:
                self._shape_bhd = (int(v[0].shape[0]), int(v[0].shape[1]), self._head_dim)
            return
        if self._memory_bound:
            if len(v) not in (0, 2, 6, 8):
                raise ValueError(f"KIVIKVCache.state: a memory-bound packed state has 0, 2, 6 or 8 arrays, got {len(v)}")
            packed, tail = (v[:6] if len(v) >= 6 else ()), (v[-2:] if len(v) in (2, 8) else ())
            self.keys = self.values = None
        else:
            if len(v) not in (0, 2, 8):
                raise ValueError(f"KIVIKVCache.state: a stashed packed state has 0, 2 or 8 arrays, got {len(v)}")
            FP16KVCache.state.fset(self, v[:2])
            packed, tail = v[2:], ()
        ref = packed[0] if packed else (tail[0] if tail else (v[0] if v else None))
        if ref is not None:
            # rows of twice the head size: a state saved with paired heads
            d = int((packed[1] if packed else ref).shape[-1])
            self._pair = self._memory_bound and self._pair_wanted and d == 2 * self._head_dim
            if self._pair:
                self._kv_heads = -2 * int(ref.shape[1])   # negative: taken from the pairs, an odd count is one less
            self._shape_bhd = (int(ref.shape[0]), int(ref.shape[1]), d if self._pair else self._head_dim)
        self._restore_packed(packed)
        if self._memory_bound:
            n_tail = int(tail[0].shape[2]) if tail else 0
            self._tail_k = self._tail_v = None
            if tail:
                tk, tv = tail
                B, H, D = self._shape_bhd
                if tuple(tk.shape) != (B, H, n_tail, D) or tuple(tv.shape) != (B, H, n_tail, D):
                    raise ValueError(f"KIVIKVCache.state: residual rows must be [{B}, {H}, n, {D}], got "
                                     f"{tuple(tk.shape)} and {tuple(tv.shape)}")
                cap = -(-max(n_tail, self._residual_length + 2 * self._group_size) // 64) * 64
                self._tail_k = torch.zeros((B, H, cap, D), dtype=tk.dtype, device=tk.device)
                self._tail_v = torch.zeros((B, H, cap, D), dtype=tv.dtype, device=tv.device)
                self._tail_k[:, :, :n_tail] = tk
                self._tail_v[:, :, :n_tail] = tv
            self.offset = self._n_quantized + n_tail
        self._rebuild_accounting()

    def _restore_packed(self, packed) -> None:
        """Install live packed rows (the six arrays of ``_packed_state``) as the packed store."""
        self._kp = self._ks = self._kz = self._vp = self._vs = self._vz = None
        self._packed_cap = 0
        self._n_quantized = 0
        self._tiles, self._tiles_packed = None, 0
        if not packed:
            return
        kp, ks, kz, vp, vs, vz = packed
        B, H, D = self._shape_bhd
        g, per = self._group_size, self._per
        n = int(kp.shape[2])
        W, GV = -(-D // per), -(-D // g)
        if self._v_layout == "token":
            want_v = ((B, H, n // per, D), (B, H, GV, n), (B, H, GV, n))
        else:
            want_v = ((B, H, n, W), (B, H, n, GV), (B, H, n, GV))
        want = ((B, H, n, W), (B, H, n // g, D), (B, H, n // g, D), *want_v)
        got = tuple(tuple(t.shape) for t in packed)
        if n % g or (self._v_layout == "token" and n % per) or got != want:
            raise ValueError(f"KIVIKVCache.state: packed rows {got} do not fit {self._field} bits a code, group={g}, "
                             f"value layout {self._v_layout!r}, head_dim={D} (expected {want})")
        if any(t.dtype != self._meta_dtype for t in (ks, kz, vs, vz)):
            raise ValueError(f"KIVIKVCache.state: scale/zero must be {self._meta_dtype}")
        self._ensure_packed_capacity(B, H, D, n, kp.device)
        self._kp[:, :, :n] = kp.to(torch.int32) if kp.dtype != torch.int32 else kp
        self._ks[:, :, : n // g] = ks
        self._kz[:, :, : n // g] = kz
        vp32 = vp.to(torch.int32) if vp.dtype != torch.int32 else vp
        if self._v_layout == "token":
            self._vp[:, :, : n // per] = vp32
            self._vs[..., :n] = vs
            self._vz[..., :n] = vz
        else:
            self._vp[:, :, :n] = vp32
            self._vs[:, :, :n] = vs
            self._vz[:, :, :n] = vz
        self._n_quantized = n

    def _rebuild_accounting(self) -> None:
        B, H, D = self._shape_bhd
        k, v = self._quantized_bytes(self._n_quantized, B, H, D) if self._n_quantized else (0, 0)
        self._key_bytes_compressed, self._value_bytes_compressed = k, v
        self._key_bytes_fp16 = self._value_bytes_fp16 = H * B * self.offset * D * 2
        self._residual_fp16_bytes = (self.offset - self._n_quantized) * D * 2 * 2 * H * B
        self._tokens_seen = self.offset

    @property
    def meta_state(self):
        """Strings, as prompt-cache files store them: what a restored cache must agree with
        (offset, frontier, bit width, group, value layout, scale/zero dtype, mode)."""
        mode = "memory_bound" if self._memory_bound else ("stash" if self._fused_enabled else "standard")
        if self._pair and self._kv_heads > 0 and self._kv_heads % 2:
            mode += f"/{self._kv_heads}"   # an odd number of kv heads kept in pairs: the pairs do not show it
        bits = self._b if self._field == self._b else f"{self._b}/{self._field}"   # code width / width of its field
        return tuple(map(str, (self.offset, self._n_quantized, bits, self._group_size, self._v_layout,
                               str(self._meta_dtype).replace("torch.", ""), mode)))

    @meta_state.setter
    def meta_state(self, v) -> None:
        v = tuple(v)
        if len(v) != 7:
            raise ValueError(f"KIVIKVCache.meta_state: expected 7 fields, got {len(v)}")
        mode, _, heads = str(v[6]).partition("/")
        v = (*v[:6], mode)
        if heads and self._pair and (int(heads) + 1) // 2 == self._shape_bhd[1]:
            self._kv_heads = int(heads)
        mine = self.meta_state
        mine = (*mine[:6], mine[6].partition("/")[0])
        if tuple(v[2:]) != mine[2:]:
            raise ValueError(f"KIVIKVCache.meta_state: saved with (bits, group, value layout, meta dtype, mode) = {tuple(v[2:])}, "
                             f"this cache is configured as {mine[2:]}")
        offset, n_q = int(v[0]), int(v[1])
        if self._fused_enabled:
            if (offset, n_q) != (self.offset, self._n_quantized):
                raise ValueError(f"KIVIKVCache.meta_state: offset/frontier {offset}/{n_q} do not match the restored state "
                                 f"({self.offset}/{self._n_quantized}); assign state first")
        else:
            if offset != self.offset:
                raise ValueError(f"KIVIKVCache.meta_state: offset {offset} does not match the restored state ({self.offset})")
            self._n_quantized = n_q   # rows below the frontier of the fp16 history are already reconstructions
            self._rebuild_accounting()

    @classmethod
    def from_state(cls, config: Any, state, meta_state=None) -> "KIVIKVCache":
        c = cls(config)
        c.state = state
        if meta_state is not None:
            c.meta_state = meta_state
        return c

    @property
    def nbytes(self) -> int:
        total = 0 if self._memory_bound else FP16KVCache.nbytes.fget(self)
        for t in (self._kp, self._ks, self._kz, self._vp, self._vs, self._vz, self._tail_k, self._tail_v,
                  *(self._tail_spare or ()), self._tiles):
            if t is not None:
                total += t.numel() * t.element_size()
        return total

    # ------------------------------------------------------------------ accounting
    def _quantized_bytes(self, n: int, B: int, H: int, D: int) -> tuple[int, int]:
        """(key, value) packed-byte cost of ``n`` group-aligned tokens (kivi_cache.py:301-306)."""
        gs = self._group_size
        k = math.ceil(n * D * self._b / 8) * H * B + math.ceil(n / gs) * D * 2 * 2 * H * B
        v = math.ceil(n * D * self._b / 8) * H * B + n * math.ceil(D / gs) * 2 * 2 * H * B
        return k, v

    def _account_bytes(self, B: int, H: int, S: int, D: int, n_quant_now: int) -> None:
        """kivi_cache.py:308-332."""
        if n_quant_now > 0:
            k, v = self._quantized_bytes(n_quant_now, B, H, D)
            self._key_bytes_compressed += k
            self._value_bytes_compressed += v
        n_res = self.offset - self._n_quantized
        self._residual_fp16_bytes = n_res * D * 2 * 2 * H * B
        self._key_bytes_fp16 += H * B * S * D * 2
        self._value_bytes_fp16 += H * B * S * D * 2
        self._tokens_seen += S

    @property
    def compressed_key_bytes(self) -> int:
        """Packed-storage byte cost of quantised key codes + fp16 (scale, zero)."""
        return self._key_bytes_compressed

    @property
    def fp16_key_bytes(self) -> int:
        return self._key_bytes_fp16

    @property
    def compressed_value_bytes(self) -> int:
        return self._value_bytes_compressed

    @property
    def fp16_value_bytes(self) -> int:
        return self._value_bytes_fp16

    @property
    def residual_fp16_bytes(self) -> int:
        """Bytes held in fp16 and not yet quantised (keys + values)."""
        return self._residual_fp16_bytes

    @property
    def assigned_avg_bits(self) -> float:
        return float(self._b)

    @property
    def effective_compression_ratio(self) -> float:
        """End-to-end KV byte ratio vs fp16, residual window included (kivi_cache.py:387-410)."""
        total_fp16 = self._key_bytes_fp16 + self._value_bytes_fp16
        if total_fp16 == 0:
            return 1.0
        total = self._key_bytes_compressed + self._value_bytes_compressed + self._residual_fp16_bytes
        return total_fp16 / total if total else 1.0


__all__ = ["KIVIKVCache"]
