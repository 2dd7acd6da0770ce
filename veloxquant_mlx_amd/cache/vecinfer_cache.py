"""VecInfer KV cache on torch ROCm tensors: smooth + Walsh-Hadamard key transform
and product VQ of keys and values.

Behaviour follows ``VecInferKVCache`` (veloxquant_mlx/cache/vecinfer_cache.py:47-792):
three storage modes (dequantise-only, dequantise + index stash, memory-bound
indices only), geometric growth of the ``[B, H, cap, n_sub]`` index buffers,
``state`` / ``trim`` / ``nbytes`` per mode and :meth:`fused_sdpa` over the stored
indices.  Assignment and gather run in the HIP kernels; the transform is a dense
``D x D`` product (or, with 16-byte aligned keys, part of the fused key-encode kernel).
:meth:`fused_sdpa` attends straight from the stored indices through
``kernels.metal_fused_sdpa`` (the look-up-table attention of
veloxquant_mlx/metal/fused_sdpa.py:200-299).
"""

from __future__ import annotations

import warnings
from typing import Any

import torch

from .. import kernels as K
from ..allocators.vecinfer import (apply_dual_transform_keys, apply_dual_transform_queries,
                                   walsh_hadamard_matrix)
from ..core.exceptions import QuantizerConfigError
from ._fp16_cache import FP16KVCache

_SMOOTH_FLOOR = 1e-12

# KVCacheConfig fields the cache reads, with the defaults of veloxquant_mlx/cache/options.py:36-43
_FIELDS = {"key_sub_dim": 4, "value_sub_dim": 8, "key_codebook_bits": 12, "value_codebook_bits": 8,
           "residual_length": 128, "seed": 42}


class _Tally:
    """Byte and token counters of the cache, kept together so that an append adds to all of them and a trim
    scales all of them (the accounting of vecinfer_cache.py:617-664: tracked per call, so a trim is an
    estimate in proportion to the tokens kept)."""

    NAMES = ("key_compressed", "value_compressed", "key_fp16", "value_fp16", "tokens_seen", "tokens_quantized")

    def __init__(self) -> None:
        self.n = dict.fromkeys(self.NAMES, 0)

    def append(self, rows: int, tokens: int, head_dim: int, key_index_bits: int, value_index_bits: int) -> None:
        """``rows`` = batch x heads x tokens appended; index bits per row of ``head_dim`` channels."""
        self.n["key_compressed"] += -(-key_index_bits // 8) * rows
        self.n["value_compressed"] += -(-value_index_bits // 8) * rows
        self.n["key_fp16"] += rows * head_dim * 2
        self.n["value_fp16"] += rows * head_dim * 2
        self.n["tokens_seen"] += tokens
        self.n["tokens_quantized"] += tokens

    def keep_fraction(self, kept: float) -> None:
        for name in self.NAMES:
            self.n[name] = int(self.n[name] * kept)


class VecInferKVCache(FP16KVCache):
    """KV cache implementing VecInfer's dual-transform product VQ.

    Never exposes ``.bits``; see ``assigned_avg_bits``."""

    def __init__(self, config: Any) -> None:
        super().__init__()
        opt = {name: int(getattr(config, name, default)) for name, default in _FIELDS.items()}
        D = self._head_dim = int(config.head_dim)
        self._key_sub_dim, self._value_sub_dim = opt["key_sub_dim"], opt["value_sub_dim"]
        self._key_bits, self._value_bits = opt["key_codebook_bits"], opt["value_codebook_bits"]
        self._residual_length = opt["residual_length"]
        if D < 1 or (D & (D - 1)) != 0:
            raise QuantizerConfigError(
                f"VecInferKVCache requires a power-of-2 head_dim (the Walsh-Hadamard transform needs it); "
                f"got head_dim={D}. Use another method such as kivi.")
        if D % self._key_sub_dim != 0:
            raise QuantizerConfigError(f"VecInferKVCache: head_dim={D} not divisible by key_sub_dim={self._key_sub_dim}")
        if D % self._value_sub_dim != 0:
            raise QuantizerConfigError(
                f"VecInferKVCache: head_dim={D} not divisible by value_sub_dim={self._value_sub_dim}")

        sm = getattr(config, "smooth_factors", None)
        self._smooth = None if sm is None else torch.as_tensor(sm)
        self._validate_smooth()
        self._H = walsh_hadamard_matrix(D, dtype=torch.float32)

        n_kc, n_vc = 2 ** self._key_bits, 2 ** self._value_bits
        seed = opt["seed"]
        missing = [n for n in ("key_codebook", "value_codebook") if getattr(config, n, None) is None]
        if missing:
            warnings.warn(
                f"VecInferKVCache: no {' / '.join(missing)} given, so random N(0,1) codebooks are used. "
                "They are only meant for shape/wiring tests and distort real keys/values badly. Train codebooks "
                "with veloxquant_mlx_amd.allocators.vecinfer.train_codebook and pass them via "
                "KVCacheConfig(key_codebook=..., value_codebook=...).", UserWarning, stacklevel=2)
        key_cb = getattr(config, "key_codebook", None)
        if key_cb is None:
            key_cb = torch.randn((n_kc, self._key_sub_dim), generator=torch.Generator().manual_seed(seed))
        self._key_codebook = torch.as_tensor(key_cb).float()
        val_cb = getattr(config, "value_codebook", None)
        if val_cb is None:
            val_cb = torch.randn((n_vc, self._value_sub_dim), generator=torch.Generator().manual_seed(seed + 1))
        self._value_codebook = torch.as_tensor(val_cb).float()

        self._tally = _Tally()

        requested = getattr(config, "use_metal_kernels", None)
        if not K._lib.library_present():
            raise RuntimeError(
                f"VecInferKVCache: the HIP kernel library is not available on this build "
                f"(use_metal_kernels={requested!r}); there is no fallback path.")
        self._use_metal = True

        fused_req = getattr(config, "fused_sdpa", False)
        self._fused_enabled = bool(fused_req)
        memory_bound_req = bool(getattr(config, "fused_sdpa_memory_bound", False))
        if memory_bound_req and not self._fused_enabled:
            raise RuntimeError(
                "VecInferKVCache: fused_sdpa_memory_bound=True requires fused_sdpa=True -- the memory-bound "
                "path only exists as a variant of the fused path, it cannot run standalone.")
        self._memory_bound = memory_bound_req
        cap = getattr(config, "fused_sdpa_max_ctx", None)
        self._max_ctx = None if cap is None else int(cap)
        self._n_sub_k = D // self._key_sub_dim
        self._n_sub_v = D // self._value_sub_dim
        # one byte per index when the codebook allows it, int32 otherwise
        self._k_idx_dtype = torch.uint8 if n_kc <= 256 else torch.int32
        self._v_idx_dtype = torch.uint8 if n_vc <= 256 else torch.int32
        self._stored_k_indices: torch.Tensor | None = None
        self._stored_v_indices: torch.Tensor | None = None
        self._stored_S_kv = 0
        self._smooth_kv_heads: int | None = None

    # ------------------------------------------------------------------ smooth factors
    def _validate_smooth(self) -> None:
        """Reject smooth factors that cannot be inverted (vecinfer_cache.py:233-257)."""
        sm = self._smooth
        if sm is None:
            return
        sm32 = sm.float()
        bad = ~(torch.isfinite(sm32) & (sm32 > _SMOOTH_FLOOR))
        n_bad = int(bad.sum())
        if n_bad:
            raise QuantizerConfigError(
                f"VecInferKVCache: smooth_factors must be finite and > {_SMOOTH_FLOOR:g}; {n_bad} of {sm.numel()} "
                "entries are zero, negative, non-finite or too small, which would zero or corrupt those key "
                "channels. Use calibrate_smooth_factors, which floors its output, or clip your factors.")

    def _resolve_smooth_heads(self, n_kv_heads: int) -> None:
        """Make per-head smooth factors consistent between keys and queries (vecinfer_cache.py:259-294)."""
        sm = self._smooth
        if sm is None or sm.ndim != 2 or self._smooth_kv_heads == n_kv_heads:
            return
        rows = int(sm.shape[0])
        if rows not in (1, n_kv_heads):
            if rows > n_kv_heads and rows % n_kv_heads == 0:
                self._smooth = sm.reshape(n_kv_heads, rows // n_kv_heads, sm.shape[-1]).mean(dim=1)
            else:
                raise QuantizerConfigError(
                    f"VecInferKVCache: smooth_factors has {rows} rows but the keys have {n_kv_heads} KV heads. "
                    f"Provide a [1, D], [{n_kv_heads}, D] (per KV head) or a multiple-of-{n_kv_heads}-row "
                    "(per query head, GQA) smooth; any other row count cannot give matching key and query factors.")
        self._smooth_kv_heads = n_kv_heads

    def _to_device(self, ref: torch.Tensor) -> None:
        dev = ref.device
        if self._H.device != dev:
            self._H = self._H.to(dev)
            self._key_codebook = self._key_codebook.to(dev)
            self._value_codebook = self._value_codebook.to(dev)
            if self._smooth is not None:
                self._smooth = self._smooth.to(dev)

    # ------------------------------------------------------------------ encode / decode
    def _transform_keys(self, keys: torch.Tensor) -> torch.Tensor:
        k32 = keys.float()
        if self._smooth is not None:
            return apply_dual_transform_keys(k32, self._smooth.float(), self._H)
        return k32 @ self._H

    def _encode_decode_keys(self, keys: torch.Tensor):
        """smooth -> WHT -> VQ -> gather -> inverse WHT -> un-smooth (vecinfer_cache.py:313-356):
        one launch for 4D keys, the composition below otherwise."""
        if keys.ndim == 4:
            return K.vecinfer_encode_decode_metal(keys, self._key_codebook, self._key_sub_dim, self._H, self._smooth,
                                                  index_dtype=self._k_idx_dtype)
        k_tilde = self._transform_keys(keys)
        k_idx = K.vecinfer_quantize_metal(k_tilde, self._key_codebook, self._key_sub_dim,
                                          index_dtype=self._k_idx_dtype)
        k_hat = K.vecinfer_dequant_metal(k_idx, self._key_codebook) @ self._H.T
        if self._smooth is not None:
            sm = self._smooth.float()
            if sm.ndim == 2 and k_hat.ndim >= 4 and k_hat.shape[-3] == sm.shape[0]:
                sm = sm[:, None, :]
            elif sm.ndim == 2:
                sm = sm.mean(dim=0)
            k_hat = k_hat * sm
        return k_hat.to(keys.dtype), k_idx

    def _encode_decode_values(self, values: torch.Tensor):
        """VQ + gather for values (vecinfer_cache.py:358-379)."""
        v_idx = K.vecinfer_quantize_metal(values, self._value_codebook, self._value_sub_dim,
                                          index_dtype=self._v_idx_dtype)
        v_hat = K.vecinfer_dequant_metal(v_idx, self._value_codebook, out_dtype=values.dtype
                                         if values.dtype in (torch.float16, torch.bfloat16, torch.float32)
                                         else torch.float32)
        return v_hat.to(values.dtype), v_idx

    # ------------------------------------------------------------------ protocol
    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        """Smooth + Hadamard keys, product-VQ K/V, and either return the reconstruction
        for a downstream SDPA or stash indices only (vecinfer_cache.py:384-411)."""
        self._to_device(keys)
        self._resolve_smooth_heads(int(keys.shape[1]))
        if self._fused_enabled:
            if self._memory_bound:
                return self._update_and_fetch_fused(keys, values)
            return self._update_and_fetch_standard_and_stash(keys, values)
        return self._update_and_fetch_standard(keys, values)

    def _ensure_index_capacity(self, B: int, H: int, S: int, device) -> None:
        """Index buffers hold ``_stored_S_kv + S`` tokens, growing geometrically up to
        the optional cap (vecinfer_cache.py:413-443)."""
        needed = self._stored_S_kv + S
        if self._max_ctx is not None and needed > self._max_ctx:
            raise RuntimeError(f"VecInferKVCache: context length {needed} exceeded fused_sdpa_max_ctx={self._max_ctx}. "
                               " Raise or unset KVCacheConfig.fused_sdpa_max_ctx.")
        cur = 0 if self._stored_k_indices is None else self._stored_k_indices.shape[2]
        if needed <= cur:
            return
        cap = max(needed, 256) if cur == 0 else max(needed, 2 * cur)
        if self._max_ctx is not None:
            cap = min(cap, self._max_ctx)
        nk = torch.zeros((B, H, cap, self._n_sub_k), dtype=self._k_idx_dtype, device=device)
        nv = torch.zeros((B, H, cap, self._n_sub_v), dtype=self._v_idx_dtype, device=device)
        if cur:
            nk[:, :, :cur] = self._stored_k_indices
            nv[:, :, :cur] = self._stored_v_indices
        self._stored_k_indices, self._stored_v_indices = nk, nv

    def _stash(self, k_idx: torch.Tensor, v_idx: torch.Tensor) -> None:
        B, H, S, _ = k_idx.shape
        self._ensure_index_capacity(B, H, S, k_idx.device)
        end = self._stored_S_kv + S
        self._stored_k_indices[:, :, self._stored_S_kv:end] = k_idx
        self._stored_v_indices[:, :, self._stored_S_kv:end] = v_idx
        self._stored_S_kv = end

    def _update_and_fetch_standard(self, keys, values):
        B, H, S, D = keys.shape
        k_dequant, _ = self._encode_decode_keys(keys)
        v_hat, _ = self._encode_decode_values(values)
        self._account_bytes(B, H, S, D)
        return super().update_and_fetch(k_dequant, v_hat)

    def _update_and_fetch_standard_and_stash(self, keys, values):
        B, H, S, D = keys.shape
        k_dequant, k_idx = self._encode_decode_keys(keys)
        v_hat, v_idx = self._encode_decode_values(values)
        self._stash(k_idx, v_idx)
        self._account_bytes(B, H, S, D)
        return FP16KVCache.update_and_fetch(self, k_dequant, v_hat)

    def _update_and_fetch_fused(self, keys, values):
        """Indices only; returns zero-stride placeholders (vecinfer_cache.py:491-532)."""
        B, H, S, D = keys.shape
        _, k_idx = K.vecinfer_encode_decode_metal(keys, self._key_codebook, self._key_sub_dim, self._H, self._smooth,
                                                  index_dtype=self._k_idx_dtype, want_k_hat=False)
        v_idx = K.vecinfer_quantize_metal(values, self._value_codebook, self._value_sub_dim,
                                          index_dtype=self._v_idx_dtype)
        self._stash(k_idx, v_idx)
        self.offset += S
        self._account_bytes(B, H, S, D)
        zk = torch.zeros((), dtype=keys.dtype, device=keys.device)
        zv = torch.zeros((), dtype=values.dtype, device=values.device)
        return zk.expand(B, H, self._stored_S_kv, D), zv.expand(B, H, self._stored_S_kv, D)

    # ------------------------------------------------------------------ state / trim
    @property
    def state(self):
        """Standard: fp16 state.  Stash: fp16 state followed by the index buffers.
        Memory-bound: the live index rows only (vecinfer_cache.py:542-571)."""
        if not self._fused_enabled:
            return FP16KVCache.state.fget(self)
        if not self._memory_bound:
            parent = tuple(FP16KVCache.state.fget(self))
            if self._stored_k_indices is None:
                return parent
            return (*parent, self._stored_k_indices, self._stored_v_indices)
        if self._stored_k_indices is None:
            return (torch.zeros((1, 1, 0, self._n_sub_k), dtype=self._k_idx_dtype),
                    torch.zeros((1, 1, 0, self._n_sub_v), dtype=self._v_idx_dtype))
        n = self._stored_S_kv
        return self._stored_k_indices[:, :, :n], self._stored_v_indices[:, :, :n]

    @state.setter
    def state(self, v) -> None:
        """vecinfer_cache.py:573-609."""
        if not self._fused_enabled:
            FP16KVCache.state.fset(self, v)
            return
        v = tuple(v)
        if not self._memory_bound:
            FP16KVCache.state.fset(self, v[:2])
            if len(v) == 4:
                self._stored_k_indices, self._stored_v_indices = v[2], v[3]
                self._stored_S_kv = int(self.offset)
            else:
                self._stored_k_indices = self._stored_v_indices = None
                self._stored_S_kv = 0
            return
        k, val = v
        n = int(k.shape[2])
        if n == 0:
            self._stored_k_indices = self._stored_v_indices = None
        else:
            self._stored_k_indices, self._stored_v_indices = k, val
        self._stored_S_kv = n
        self.offset = n

    def empty(self) -> bool:
        if not self._fused_enabled or not self._memory_bound:
            return super().empty()
        return self._stored_k_indices is None or self._stored_S_kv == 0

    def trim(self, n: int) -> int:
        """Drop the last ``n`` tokens, keeping every parallel buffer in step
        (vecinfer_cache.py:617-639)."""
        old_offset = self.offset
        trimmed = super().trim(n)
        if not trimmed:
            return trimmed
        # the index buffers advance by _stored_S_kv, not by offset: left alone they would keep the dropped tokens
        self._stored_S_kv = min(self._stored_S_kv, self.offset)
        self._tally.keep_fraction(self.offset / old_offset)
        return trimmed

    def size(self) -> int:
        return self.offset

    @property
    def nbytes(self) -> int:
        total = FP16KVCache.nbytes.fget(self)
        if self._fused_enabled and self._stored_k_indices is not None:
            total += (self._stored_k_indices.numel() * self._stored_k_indices.element_size()
                      + self._stored_v_indices.numel() * self._stored_v_indices.element_size())
        return total

    def _account_bytes(self, B: int, H: int, S: int, D: int) -> None:
        """vecinfer_cache.py:654-664."""
        self._tally.append(B * H * S, S, D, (D // self._key_sub_dim) * self._key_bits,
                           (D // self._value_sub_dim) * self._value_bits)

    # ------------------------------------------------------------------ attention
    def fused_sdpa(self, q: torch.Tensor, scale: float, *, causal: bool = True, sliding_window: int = 0):
        """Attention straight from the stored indices; ``q [B,H_q,S_q,D]`` is the plain
        query, the dual transform is applied here (vecinfer_cache.py:670-731)."""
        if not self._fused_enabled:
            raise RuntimeError("VecInferKVCache.fused_sdpa called but fused_sdpa was not enabled via "
                               "KVCacheConfig.fused_sdpa=True.")
        if self._stored_k_indices is None or self._stored_S_kv == 0:
            raise RuntimeError("VecInferKVCache.fused_sdpa called before any tokens were cached via update_and_fetch.")
        self._to_device(q)
        n = self._stored_S_kv
        smooth = self._smooth.float() if self._smooth is not None else torch.ones(
            (self._head_dim,), dtype=torch.float32, device=q.device)
        q_tilde = apply_dual_transform_queries(q.float(), smooth, self._H)
        kcb, vcb = self._key_codebook, self._value_codebook
        n_sub_k, n_sub_v = self._head_dim // kcb.shape[1], self._head_dim // vcb.shape[1]
        table_kernel = (kcb.shape[0] == vcb.shape[0] <= 256 and max(n_sub_k, n_sub_v) <= 32
                        and (n_sub_k + n_sub_v) * kcb.shape[0] * 4 <= 65536
                        and (self._stored_k_indices.dtype != torch.uint8 or (n_sub_k % 4 == 0 and n_sub_v % 4 == 0)))
        # A prefill-sized call (256 query rows or more per kv head at a head size the matrix-unit prefill blocks take)
        # gathers the centroids once into a transient copy in the queries' 16-bit type -- what update_and_fetch hands
        # a host that attends by itself (vecinfer_cache.py:336-379: the reconstruction cast to the input dtype) -- and
        # attends over it with those blocks: the table kernel builds a table per query row, which pays for a few rows
        # per kv head only (512 queries over 4.6k tokens, 32 / 8 heads: 0.64 ms from the tables, 0.09 ms this way).
        H_kv = self._stored_k_indices.shape[1]
        prefill_sized = (self._head_dim in (128, 256) and q.shape[1] % H_kv == 0 and (q.shape[1] // H_kv) * q.shape[2] >= 256
                         and q.dtype in (torch.float16, torch.bfloat16))
        if table_kernel and not prefill_sized:
            # look-up table + centroid histogram straight from the indices
            return K.metal_fused_sdpa(q_tilde, self._stored_k_indices, kcb, self._stored_v_indices, vcb, float(scale),
                                      causal=bool(causal) and q.shape[2] > 1, sliding_window=int(sliding_window or 0),
                                      out_dtype=q.dtype, n_tokens=n)
        rows_dtype = q.dtype if prefill_sized else torch.float32
        k_tilde_hat = K.vecinfer_dequant_metal(self._stored_k_indices[:, :, :n].contiguous(), self._key_codebook,
                                               out_dtype=rows_dtype)
        v_hat = K.vecinfer_dequant_metal(self._stored_v_indices[:, :, :n].contiguous(), self._value_codebook,
                                         out_dtype=rows_dtype)
        return K.kivi_packed_attend(q_tilde, k_tail=k_tilde_hat, v_tail=v_hat, n_tail=n, scale=float(scale),
                                    causal=bool(causal) and q.shape[2] > 1, sliding_window=int(sliding_window or 0),
                                    out_dtype=q.dtype)

    # ------------------------------------------------------------------ reporting
    compressed_key_bytes = property(lambda self: self._tally.n["key_compressed"])
    fp16_key_bytes = property(lambda self: self._tally.n["key_fp16"])
    compressed_value_bytes = property(lambda self: self._tally.n["value_compressed"])
    fp16_value_bytes = property(lambda self: self._tally.n["value_fp16"])
    # (the names the other caches keep their counters under)
    _tokens_seen = property(lambda self: self._tally.n["tokens_seen"])
    _tokens_quantized = property(lambda self: self._tally.n["tokens_quantized"])

    @property
    def codebook_bytes(self) -> int:
        return (2 ** self._key_bits) * self._key_sub_dim * 2 + (2 ** self._value_bits) * self._value_sub_dim * 2

    @property
    def assigned_avg_bits(self) -> float:
        k_bits = (self._head_dim // self._key_sub_dim) * self._key_bits / self._head_dim
        v_bits = (self._head_dim // self._value_sub_dim) * self._value_bits / self._head_dim
        return (k_bits + v_bits) / 2.0

    # a batching host would otherwise merge this cache into a plain one (vecinfer_cache.py:774-789)
    merge = property(lambda self: (_ for _ in ()).throw(
        AttributeError("VecInferKVCache does not support merge()")))


__all__ = ["VecInferKVCache"]
