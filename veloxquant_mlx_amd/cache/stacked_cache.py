"""Layer-stacked packed KIVI cache: the decode attention of every layer in one launch.

The reference's layer-batched decode takes tensors with a leading ``NL`` axis
(``scalar_fused_decode_attend_batched``, veloxquant_mlx/metal/_scalar_attend.py:496-647) and
pays for building them: its per-layer caches own separate arrays, so every call stacks them
first (docs/KV_KERNEL_ROOFLINE_FINDINGS.md:625-665).  Here the stack IS the storage: the
packed store and the fp16 tails of all layers live in ``[NL * B, ...]`` buffers, every layer's
cache object works on its slice of them through the ordinary cache API, and
``fused_sdpa_all`` hands the whole buffers to one attention launch with the layer axis folded
into the batch axis.  Layers whose lengths differ by a step (a forward pass in flight) go
through the per-sequence lengths of the attention entry point.

With ``method="kivi_sink"`` the layers are ``SinkProtectedKVCache`` objects: their exact rows
are gathered into one ``[NL * B, H, cap, D]`` side store (rebuilt only after a flush, a trim
or a restored state changed some layer's rows) and the one launch patches every layer's
protected positions.  ``sliding_window`` is the attention call's.
"""

from __future__ import annotations

from typing import Any

import torch

from .. import kernels as K
from .kivi_cache import KIVIKVCache, own_half_of_paired_output, pad_queries_for_paired_heads
from .sink_cache import SinkProtectedKVCache

_PACKED = ("_kp", "_ks", "_kz", "_vp", "_vs", "_vz")


class LayerStackedKIVICache:
    """``n_layers`` memory-bound packed ``KIVIKVCache`` objects over shared stacked buffers.

    ``cache[l]`` is layer ``l``'s cache (``update_and_fetch`` / ``fused_sdpa`` / ``trim`` /
    ``state`` as usual).  ``fused_sdpa_all(q [NL,B,H_q,S_q,D], scale)`` attends for all layers
    at once.  A layer whose buffers were replaced (capacity growth, a restored state) is
    copied back into the stack on the next ``fused_sdpa_all``; with
    ``KVCacheConfig.fused_sdpa_max_ctx`` set the packed store never moves.
    """

    def __init__(self, config: Any, n_layers: int) -> None:
        if n_layers < 1:
            raise ValueError(f"LayerStackedKIVICache: n_layers={n_layers} must be >= 1")
        if not (getattr(config, "fused_sdpa", False) and getattr(config, "fused_sdpa_memory_bound", False)):
            raise RuntimeError("LayerStackedKIVICache needs KVCacheConfig(fused_sdpa=True, fused_sdpa_memory_bound=True): "
                               "the stack holds packed codes and the fp16 tail, nothing else.")
        kind = SinkProtectedKVCache if getattr(config, "method", "kivi") == "kivi_sink" else KIVIKVCache
        self.layers = [kind(config) for _ in range(n_layers)]
        self._packed: tuple[torch.Tensor, ...] | None = None      # six [NL*B, ...] stacks
        self._tails: list[tuple[torch.Tensor, torch.Tensor]] = []  # two pairs of [NL*B, H, cap, D] stacks
        self._lens = None   # (key, packed_lens, tail_lens) of the last ragged call
        self._sinks = None  # (key, (side_k, side_v, side_pos)) of the last call with protected rows
        self._q_pad = None  # zero-padded queries of a stack of paired 64-channel heads

    @classmethod
    def from_layers(cls, layers) -> "LayerStackedKIVICache":
        """Adopt existing memory-bound packed ``KIVIKVCache`` objects (one per layer, same configuration
        and batch): the first ``fused_sdpa_all`` copies their buffers into the stack once and re-points
        them at their slices."""
        layers = list(layers)
        if not layers or not all(isinstance(c, KIVIKVCache) and c._memory_bound for c in layers):
            raise ValueError("LayerStackedKIVICache.from_layers: needs memory-bound packed KIVIKVCache objects")
        c0 = layers[0]
        if any((c._b, c._field, c._group_size, c._v_layout, c._meta_dtype) != (c0._b, c0._field, c0._group_size, c0._v_layout, c0._meta_dtype)
               for c in layers):
            raise ValueError("LayerStackedKIVICache.from_layers: the layers differ in bit width, group size or layout")
        self = cls.__new__(cls)
        self.layers = layers
        self._packed, self._tails, self._lens, self._sinks = None, [], None, None
        self._q_pad = None
        return self

    def __len__(self) -> int:
        return len(self.layers)

    def __getitem__(self, layer: int) -> KIVIKVCache:
        return self.layers[layer]

    @property
    def nbytes(self) -> int:
        return sum(c.nbytes for c in self.layers)

    # ------------------------------------------------------------------ stacking
    def _which_tail(self, B: int) -> int | None:
        """Index of the tail stack every layer's current tail is a slice of, else ``None``."""
        for i, (tk, tv) in enumerate(self._tails):
            step_k = B * tk.stride(0) * tk.element_size()
            pk, pv = tk.data_ptr(), tv.data_ptr()
            if all(c._tail_k is not None and c._tail_k.data_ptr() == pk + l * step_k
                   and c._tail_v.data_ptr() == pv + l * step_k and c._tail_k.shape[2] == tk.shape[2]
                   for l, c in enumerate(self.layers)):
                return i
        return None

    def _packed_in_place(self, B: int) -> bool:
        if self._packed is None:
            return False
        kp = self._packed[0]
        step = B * kp.stride(0) * kp.element_size()
        return all(c._kp is not None and c._kp.data_ptr() == kp.data_ptr() + l * step and c._packed_cap == kp.shape[2]
                   for l, c in enumerate(self.layers))

    def _restack_packed(self, B: int) -> None:
        NL = len(self.layers)
        c0 = self.layers[0]
        cap = max(c._packed_cap for c in self.layers)
        g, per, token = c0._group_size, c0._per, c0._v_layout == "token"
        stacks = []
        for name in _PACKED:
            first = getattr(c0, name)
            shape = list(first.shape)
            # the axis that counts tokens (or token groups / token words) grows to the common capacity
            if name in ("_ks", "_kz"):
                shape[2] = cap // g
            elif name == "_vp" and token:
                shape[2] = cap // per
            elif name in ("_vs", "_vz") and token:
                shape[3] = cap
            else:
                shape[2] = cap
            st = torch.zeros([NL * B] + shape[1:], dtype=first.dtype, device=first.device)
            for l, c in enumerate(self.layers):
                src, n = getattr(c, name), c._n_quantized
                dst = st[l * B:(l + 1) * B]
                if name in ("_vs", "_vz") and token:
                    dst[..., :n].copy_(src[..., :n])
                else:
                    rows = n // g if name in ("_ks", "_kz") else n // per if (name == "_vp" and token) else n
                    dst[:, :, :rows].copy_(src[:, :, :rows])
                setattr(c, name, dst)
            stacks.append(st)
        for c in self.layers:
            c._packed_cap = cap
        self._packed = tuple(stacks)

    def _restack_tails(self, B: int) -> int:
        NL = len(self.layers)
        cap = max(c._tail_k.shape[2] for c in self.layers)
        t0 = self.layers[0]._tail_k
        shape = (NL * B, t0.shape[1], cap, t0.shape[3])
        self._tails = [(torch.zeros(shape, dtype=t0.dtype, device=t0.device), torch.zeros(shape, dtype=t0.dtype, device=t0.device))
                       for _ in range(2)]
        (tk, tv), (sk, sv) = self._tails
        for l, c in enumerate(self.layers):
            c._store_pending()
            n = c.offset - c._n_quantized
            sl = slice(l * B, (l + 1) * B)
            if n:
                tk[sl, :, :n].copy_(c._tail_k[:, :, :n])
                tv[sl, :, :n].copy_(c._tail_v[:, :, :n])
            c._tail_k, c._tail_v = tk[sl], tv[sl]
            c._tail_spare = (sk[sl], sv[sl])
        return 0

    def _stacked_sinks(self, B: int) -> dict:
        """The exact rows of every layer's protected positions as one side store ``[NL*B, H, cap, D]`` with
        positions ``[NL*B, cap]`` (-1: unused slot).  A layer's rows change only where its ``_side_pos_dev`` is
        dropped (flush, trim, restored state), so the table objects of the layers identify a stack."""
        per_layer = [c._extra_attend_args().get("sinks") if isinstance(c, SinkProtectedKVCache) else None
                     for c in self.layers]
        if not any(s is not None for s in per_layer):
            self._sinks = None
            return {}
        key = tuple(None if s is None else id(s[2]) for s in per_layer)
        if self._sinks is None or self._sinks[0] != key:
            first = next(s for s in per_layer if s is not None)
            H, D = first[0].shape[1], first[0].shape[3]
            cap = max(s[0].shape[2] for s in per_layer if s is not None)
            NL = len(self.layers)
            sk = torch.zeros((NL * B, H, cap, D), dtype=first[0].dtype, device=first[0].device)
            sv = torch.zeros_like(sk)
            sp = torch.full((NL * B, cap), -1, dtype=torch.int32, device=first[0].device)
            for l, s in enumerate(per_layer):
                if s is None:
                    continue
                n = s[0].shape[2]
                sk[l * B:(l + 1) * B, :, :n], sv[l * B:(l + 1) * B, :, :n], sp[l * B:(l + 1) * B, :n] = s
            self._sinks = (key, (sk, sv, sp), [s[2] for s in per_layer if s is not None])   # the tables stay alive: their ids are the key
        return {"sinks": self._sinks[1]}

    # ------------------------------------------------------------------ attention
    def fused_sdpa_all(self, q: torch.Tensor, scale: float, *, causal: bool = True, sliding_window: int = 0,
                       fixed_order: bool | None = None, num_splits: int = 0) -> torch.Tensor:
        """Attention of ``q [NL, B, H_q, S_q, D]`` over every layer's cache in one launch; layer
        ``l``'s queries align to the end of layer ``l``'s tokens.  ``sliding_window``, ``fixed_order`` and
        ``num_splits`` as in ``KIVIKVCache.fused_sdpa``."""
        NL = len(self.layers)
        if q.ndim != 5 or q.shape[0] != NL:
            raise ValueError(f"LayerStackedKIVICache.fused_sdpa_all: q must be [NL={NL},B,H_q,S_q,D], got {tuple(q.shape)}")
        B = q.shape[1]
        if self.layers[0]._pair and q.shape[-1] == 64:   # kv heads of 64 channels kept in pairs: see KIVIKVCache
            H = abs(self.layers[0]._kv_heads)
            if q.shape[2] % H:
                raise ValueError(f"LayerStackedKIVICache.fused_sdpa_all: {q.shape[2]} query heads over {H} kv heads")
            key = (tuple(q.shape), q.dtype, q.device, K._stream_of(q.device))
            if self._q_pad is None or self._q_pad[0] != key:
                wide_heads = 2 * self.layers[0]._shape_bhd[1] * (q.shape[2] // H)
                self._q_pad = (key, q.new_zeros((q.shape[0], q.shape[1], wide_heads, q.shape[3], 128)))
            wide = self.fused_sdpa_all(pad_queries_for_paired_heads(q, H, self._q_pad[1]), scale, causal=causal,
                                       sliding_window=sliding_window, fixed_order=fixed_order, num_splits=num_splits)
            return own_half_of_paired_output(wide, H)
        for l, c in enumerate(self.layers):
            if c.offset == 0 or c._n_quantized == 0:
                raise RuntimeError(f"LayerStackedKIVICache.fused_sdpa_all: layer {l} has no packed tokens yet")
            if c._shape_bhd[0] != B:
                raise ValueError(f"LayerStackedKIVICache.fused_sdpa_all: layer {l} holds batch {c._shape_bhd[0]}, q has {B}")
            c._drop_tiles()   # the stacked launch never reads a layer's prefill tile scratch
        if not self._packed_in_place(B):
            self._restack_packed(B)
        ti = self._which_tail(B)
        if ti is None:
            ti = self._restack_tails(B)
        tk, tv = self._tails[ti]
        c0 = self.layers[0]
        nq = [c._n_quantized for c in self.layers]
        nt = [c.offset - c._n_quantized for c in self.layers]
        ragged = min(nq) != max(nq) or min(nt) != max(nt)
        pending = [c._pending for c in self.layers]
        k_new = v_new = None
        if all(p is not None for p in pending) and q.shape[3] == 1 and not ragged:
            # a decode step of all layers: the launch stores every layer's newest token and attends over it
            k_new = torch.stack([p[0] for p in pending]).reshape(NL * B, tk.shape[1], tk.shape[3])
            v_new = torch.stack([p[1] for p in pending]).reshape(NL * B, tk.shape[1], tk.shape[3])
        else:
            for c in self.layers:
                c._store_pending()
        lens = {}
        if ragged:
            key = (tuple(nq), tuple(nt), B)
            if self._lens is None or self._lens[0] != key:
                rep = lambda xs: torch.tensor([x for x in xs for _ in range(B)], dtype=torch.int32, device=q.device)
                self._lens = (key, rep(nq), rep(nt))
            lens = dict(packed_lens=self._lens[1], tail_lens=self._lens[2])
        kp, ks, kz, vp, vs, vz = self._packed
        kw = dict(k_packed=kp, k_scale=ks, k_zero=kz, v_packed=vp, v_scale=vs, v_zero=vz, n_packed=max(nq), bits=c0._field,
                  group_size=c0._group_size, v_layout=c0._v_layout, k_tail=tk if max(nt) else None,
                  v_tail=tv if max(nt) else None, n_tail=max(nt), scale=float(scale),
                  causal=bool(causal) and q.shape[3] > 1, out_dtype=q.dtype, fixed_order=fixed_order,
                  sliding_window=int(sliding_window or 0), num_splits=max(0, int(num_splits)), **lens,
                  **self._stacked_sinks(B))
        qf = q.reshape((NL * B,) + tuple(q.shape[2:]))
        if k_new is not None:
            try:
                out = K.kivi_packed_attend(qf, k_new=k_new, v_new=v_new, **kw)
                for c in self.layers:
                    c._pending = None
                return out.view((NL, B) + tuple(out.shape[1:]))
            except ValueError:   # a shape the append-and-attend launch does not take
                for c in self.layers:
                    c._store_pending()
        out = K.kivi_packed_attend(qf, **kw)
        return out.view((NL, B) + tuple(out.shape[1:]))
