"""ZipCache-adapted cache (``method="zipcache"``): in every incoming block the key tokens with the
largest L2 norms are round-tripped at ``zipcache_hi_bits``, the rest at ``zipcache_lo_bits``; values
go through at ``zipcache_hi_bits``.  Mirrors ``ZipCacheKVCache``
(veloxquant_mlx/cache/zipcache_cache.py:43-414): the same routing (stable rank of the norms, low
block then high block in original order), the same byte ledger and trim, the same deferred NaN/Inf
report for prefill chunks.

A sibling of KIVI on the same kernel: each of the two blocks is one launch of the token-axis group
round trip (``vq_kivi_quant_dequant``) on the gathered float32 rows; norms, ranks and the gathers
are torch on the device.
"""

from __future__ import annotations

import math
from typing import Any

import torch

from .. import kernels as K
from ..core.exceptions import QuantizerConfigError
from ._fp16_cache import FP16KVCache

_WHO = "zipcache"


def _int_in(value, name, lo, hi=None):
    if isinstance(value, float) and value.is_integer():
        value = int(value)
    if isinstance(value, bool) or not isinstance(value, int) or value < lo or (hi is not None and value > hi):
        rng = f"[{lo}, {hi}]" if hi is not None else f">= {lo}"
        raise QuantizerConfigError(f"{_WHO}: {name}={value!r} must be an integer {rng}.")
    return value


def validate_zipcache_config(config: object) -> dict[str, Any]:
    """Fields and checks of validate_zipcache_config (veloxquant_mlx/quantizers/zipcache.py:87-113)."""
    hi_bits = _int_in(getattr(config, "zipcache_hi_bits", 4), "zipcache_hi_bits", 1, 8)
    lo_bits = _int_in(getattr(config, "zipcache_lo_bits", 2), "zipcache_lo_bits", 1, 8)
    if lo_bits > hi_bits:
        raise QuantizerConfigError(f"{_WHO}: zipcache_lo_bits={lo_bits} must not exceed zipcache_hi_bits={hi_bits}; "
                                   "salient tokens would get fewer bits than the rest.")
    frac = getattr(config, "zipcache_hi_fraction", 0.20)
    if isinstance(frac, bool) or not isinstance(frac, (int, float)) or not math.isfinite(frac) or not 0.0 <= frac <= 1.0:
        raise QuantizerConfigError(f"{_WHO}: zipcache_hi_fraction={frac!r} must be a number in [0, 1].")
    gs = _int_in(getattr(config, "zipcache_group_size", 32), "zipcache_group_size", 1)
    qv = getattr(config, "zipcache_quantize_values", True)
    if not isinstance(qv, bool):
        raise QuantizerConfigError(f"{_WHO}: zipcache_quantize_values={qv!r} must be True or False.")
    return dict(hi_bits=hi_bits, lo_bits=lo_bits, hi_fraction=float(frac), group_size=gs, quantize_values=qv)


def base_only_bytes(S: int, D: int, bits: int, group_size: int = 32) -> int:
    """All tokens at one bit width: codes plus fp16 scale and zero per (group, channel) (zipcache.py:412-419)."""
    return math.ceil(S * D * bits / 8) + math.ceil(S / group_size) * D * 2 * 2


class _Run:
    """Tokens [start, end) of the cache: updates of ``unit`` tokens each, every one at ``cost``."""
    __slots__ = ("start", "end", "unit", "cost")

    def __init__(self, start: int, end: int, unit: int, cost: tuple) -> None:
        self.start, self.end, self.unit, self.cost = start, end, unit, cost


class ZipCacheKVCache(FP16KVCache):
    def __init__(self, config: Any) -> None:
        super().__init__()
        if not K._lib.library_present():
            raise RuntimeError("ZipCacheKVCache: the HIP kernel library is not available on this build; there is no fallback path.")
        cfg = validate_zipcache_config(config)
        self._hi_bits, self._lo_bits = cfg["hi_bits"], cfg["lo_bits"]
        self._hi_fraction, self._gs, self._quant_values = cfg["hi_fraction"], cfg["group_size"], cfg["quantize_values"]
        # what every stretch of tokens cost, in token order: a stretch is one multi-token update, or a run of
        # single-token updates of the same cost (a long generation stays a handful of entries)
        self._runs: list[_Run] = []
        self._pending = None   # (finite flag on the device, tokens, offset after the chunk)

    @staticmethod
    def _batched_saliency_mask(norms: torch.Tensor, n_hi: int, S: int) -> torch.Tensor:
        """``[BH, S]`` bool, the ``n_hi`` largest norms per row, later tokens first on equal norms (zipcache_cache.py:106-116)."""
        BH = norms.shape[0]
        if n_hi == 0:
            return torch.zeros((BH, S), dtype=torch.bool, device=norms.device)
        if n_hi >= S:
            return torch.ones((BH, S), dtype=torch.bool, device=norms.device)
        # the reference ranks by two stable argsorts; the same set without a sort: rank by (norm, position) as one
        # integer key -- the bits of a non-negative float order like the float, the position breaks ties in favour of
        # later rows -- and keep what reaches the n_hi-th largest key
        key = (norms.contiguous().view(torch.int32).to(torch.int64) << 32) | torch.arange(S, device=norms.device)
        kth = torch.kthvalue(key, S - n_hi + 1, dim=-1, keepdim=True).values
        return key >= kth

    @staticmethod
    def _routing_order(mask: torch.Tensor, n_hi: int) -> torch.Tensor:
        """int32 ``[BH, S]``: the rows outside ``mask`` in their own order, then the ``n_hi`` rows inside it in theirs
        (what a stable argsort of the mask gives, zipcache_cache.py:186-190).  Every row of the mask holds exactly
        ``n_hi`` set entries, so a flat selection of the positions falls apart into equal pieces per row."""
        BH, S = mask.shape
        pos = torch.arange(S, dtype=torch.int32, device=mask.device).expand(BH, S)
        return torch.cat([pos[~mask].view(BH, S - n_hi), pos[mask].view(BH, n_hi)], dim=1)

    def _compress(self, t: torch.Tensor, is_key: bool, out_dtype: torch.dtype = torch.float16):
        """``[B,H,S,D]`` -> (reconstruction, row norms ``[BH,S]``, (stored, baseline, fp16) bytes); no state touched
        (zipcache_cache.py:160-244)."""
        if t.ndim != 4:
            raise ValueError(f"zipcache: expected a [B, H, S, D] tensor, got shape {tuple(t.shape)}.")
        B, H, S, D = t.shape
        hi_bits = self._hi_bits
        lo_bits = self._lo_bits if is_key else self._hi_bits
        hi_fraction = self._hi_fraction if is_key else 1.0
        gs, BH = self._gs, B * H
        rows3 = t.reshape(BH, S, D)
        n_hi = max(0, min(S, int(math.ceil(S * hi_fraction))))
        n_lo = S - n_hi
        direct = (out_dtype == t.dtype and t.dtype in (torch.float16, torch.bfloat16, torch.float32) and D in (64, 128, 256)
                  and gs <= 8 * (256 // (D // 8)) and BH <= 65535 and rows3.is_contiguous() and rows3.data_ptr() % 16 == 0)
        if direct:
            # float32 arithmetic on the stored rows themselves: the kernels widen every element on load and round
            # the reconstruction once on store, which is what a float32 copy, round trip and cast give
            norms = K.row_norms(rows3)
            if n_lo == 0 or n_hi == 0:
                out = K.kivi_group_quant_dequant(rows3, -2, gs, (1 << (hi_bits if n_hi else lo_bits)) - 1)
            else:
                order = K.zip_route(norms, n_hi)   # low block, then high block
                out = torch.empty_like(rows3)
                K.kivi_group_quant_dequant_rows(rows3, out, order, 0, n_lo, gs, (1 << lo_bits) - 1)
                K.kivi_group_quant_dequant_rows(rows3, out, order, n_lo, n_hi, gs, (1 << hi_bits) - 1)
            per_slab = (math.ceil(n_hi * D * hi_bits / 8) + math.ceil(n_lo * D * lo_bits / 8)
                        + (math.ceil(n_hi / gs) if n_hi else 0) * D * 4 + (math.ceil(n_lo / gs) if n_lo else 0) * D * 4 + S)
            bytes_ = (per_slab * BH, base_only_bytes(S, D, self._lo_bits, gs) * BH, B * H * S * D * 2)
            return out.reshape(B, H, S, D), norms, bytes_
        x32 = rows3.float()
        norms = torch.linalg.vector_norm(x32, dim=-1)
        if n_lo == 0 or n_hi == 0:   # one block in original order: no gather needed
            out = K.kivi_group_quant_dequant(x32, -2, gs, (1 << (hi_bits if n_hi else lo_bits)) - 1)
        else:
            mask = self._batched_saliency_mask(norms, n_hi, S)
            order = torch.argsort(mask.to(torch.int32), dim=-1, stable=True)   # low block, then high block
            rows = torch.gather(x32, 1, order[..., None].expand(BH, S, D))
            recon = torch.empty_like(rows)
            recon[:, :n_lo] = K.kivi_group_quant_dequant(rows[:, :n_lo].contiguous(), -2, gs, (1 << lo_bits) - 1)
            recon[:, n_lo:] = K.kivi_group_quant_dequant(rows[:, n_lo:].contiguous(), -2, gs, (1 << hi_bits) - 1)
            out = torch.empty_like(rows).scatter_(1, order[..., None].expand(BH, S, D), recon)
        per_slab = (math.ceil(n_hi * D * hi_bits / 8) + math.ceil(n_lo * D * lo_bits / 8)
                    + (math.ceil(n_hi / gs) if n_hi else 0) * D * 4 + (math.ceil(n_lo / gs) if n_lo else 0) * D * 4 + S)
        bytes_ = (per_slab * BH, base_only_bytes(S, D, self._lo_bits, gs) * BH, B * H * S * D * 2)
        return out.reshape(B, H, S, D).to(out_dtype), norms, bytes_

    def _charge(self, tokens: int, cost: tuple) -> None:
        """``tokens`` new tokens at ``cost`` = bytes (key stored, key baseline, key fp16, value stored, baseline, fp16)."""
        runs = self._runs
        at = runs[-1].end if runs else 0
        if tokens == 1 and runs and runs[-1].unit == 1 and runs[-1].cost == cost:
            runs[-1].end += 1
        else:
            runs.append(_Run(at, at + tokens, tokens, cost))

    def trim(self, n: int) -> int:
        """Drop the last ``n`` tokens and what they cost; a multi-token update cut in the middle keeps the share of
        its cost that its remaining tokens are of it (the contract of zipcache_cache.py:263-287)."""
        self._pending = None
        n = super().trim(n)
        runs = self._runs
        end = (runs[-1].end if runs else 0) - n
        while runs and runs[-1].start >= end:
            runs.pop()
        if runs and runs[-1].end > end:
            last = runs[-1]
            if last.unit > 1:
                kept = end - last.start
                last.cost = tuple(round(c * kept / last.unit) for c in last.cost)
                last.unit = kept
            last.end = end
        return n

    def _total(self, i: int) -> int:
        return sum((r.end - r.start) // r.unit * r.cost[i] for r in self._runs)

    def _resolve_pending(self, pending) -> None:
        """Report a previous prefill chunk that held NaN/Inf, after taking it back out (zipcache_cache.py:294-306)."""
        self._pending = None
        ok, tokens, end = pending
        if bool(ok.item()):
            return
        if self.offset == end:
            self.trim(tokens)
        raise QuantizerConfigError("zipcache: the previous prefill chunk held NaN or Inf in its keys/values "
                                   f"(its {tokens} tokens were removed from the cache); the model produced NaN/Inf KV states.")

    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        """Route, round-trip, store (zipcache_cache.py:308-349).  The finiteness flag of a multi-token chunk stays
        on the device and is read by the next call, so no call waits for its own kernels."""
        if self._pending is not None:
            self._resolve_pending(self._pending)
        S = keys.shape[2]
        k_out, k_norms, k_cost = self._compress(keys, True, keys.dtype)
        # values left alone cost their fp16 bytes and nothing else
        v_out, v_norms, v_cost = (self._compress(values, False, values.dtype) if self._quant_values
                                  else (values, None, (0, 0, values.numel() * 2)))
        self._charge(S, (*k_cost, *v_cost))
        out = super().update_and_fetch(k_out, v_out)
        if S > 1:
            ok = torch.isfinite(k_norms).all()
            if v_norms is not None:
                ok = ok & torch.isfinite(v_norms).all()
            self._pending = (ok, S, self.offset)
        return out

    # ------------------------------------------------------------------ reporting (zipcache_cache.py:352-414)
    @property
    def compressed_key_bytes(self) -> int:
        return self._total(0)

    @property
    def baseline_key_bytes(self) -> int:
        return self._total(1)

    @property
    def fp16_key_bytes(self) -> int:
        return self._total(2)

    @property
    def compressed_value_bytes(self) -> int:
        return self._total(3)

    @property
    def baseline_value_bytes(self) -> int:
        return self._total(4)

    @property
    def fp16_value_bytes(self) -> int:
        return self._total(5)

    @property
    def compression_ratio(self) -> float:
        comp = self._total(0)   # key side, as in the reference
        return self._total(2) / comp if comp else 1.0

    @property
    def effective_avg_bits(self) -> float:
        fp16 = self.fp16_key_bytes
        return 16.0 * self._total(0) / fp16 if fp16 else float(self._hi_bits)


__all__ = ["ZipCacheKVCache", "validate_zipcache_config", "base_only_bytes"]
