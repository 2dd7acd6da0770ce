"""Kernel entry points on ``torch`` ROCm tensors.

Same names, argument meaning and error behaviour as the functions the reference
re-exports from ``veloxquant_mlx/metal/kernels.py:111-146`` for the KIVI /
VecInfer hot path; each forwards to the C ABI in ``libveloxquant_hip.so`` on the
current torch stream.  Inputs must live on a ROCm device; nothing here computes
on the CPU.
"""

from __future__ import annotations

import ctypes as C
import math

import torch

from . import _lib
from ._lib import (VQ_AXIS_CHANNEL, VQ_AXIS_TOKEN, VQ_BF16, VQ_F16, VQ_F32, VQ_I32, VQ_U8,
                   VQ_V_CHANNEL_PACKED, VQ_V_TOKEN_PACKED, AttendArgs, LutAttendArgs)

_FLOAT_TAG = {torch.float16: VQ_F16, torch.bfloat16: VQ_BF16, torch.float32: VQ_F32}
_V_LAYOUT = {"channel": VQ_V_CHANNEL_PACKED, "token": VQ_V_TOKEN_PACKED}

# Largest GQA ratio the reference's fused decode accepts (_scalar_attend.py:326).
_MAX_HEADS_PER_KV = 16


def hip_available() -> bool:
    """True when the kernel library loads and a ROCm device is visible (the
    counterpart of ``metal_available``, veloxquant_mlx/metal/__init__.py:26-31)."""
    return _lib.library_present() and torch.cuda.is_available()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """Handle of torch's current stream on the tensor's device (the raw getter skips the Stream object)."""
    if _raw_stream is not None:
        i = t.device.index
        return _raw_stream(torch.cuda.current_device() if i is None else i)
    return torch.cuda.current_stream(t.device).cuda_stream


def _stream_of(device: torch.device) -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device() if device.index is None else device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _need_gpu(name: str, *tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError(f"{name}: tensors must live on a ROCm device (got {t.device}); "
                               "there is no CPU path")


def _ftag(name: str, t: torch.Tensor) -> int:
    if t.dtype not in _FLOAT_TAG:
        raise ValueError(f"{name}: unsupported dtype {t.dtype}; expected one of "
                         f"{sorted(str(d) for d in _FLOAT_TAG)}")
    return _FLOAT_TAG[t.dtype]


def _bytes_as_words(codes: torch.Tensor) -> torch.Tensor:
    """uint8 ``[..., D]`` (D % 4 == 0) reinterpreted as int32 words ``[..., D/4]``."""
    c = codes.to(torch.uint8).contiguous()
    return c.reshape(-1).view(torch.int32).view(c.shape[:-1] + (c.shape[-1] // 4,))


def _axis_tag(name: str, axis: int) -> int:
    if axis not in (-1, -2):
        raise ValueError(f"{name}: axis must be -1 or -2, got {axis}")
    return VQ_AXIS_TOKEN if axis == -2 else VQ_AXIS_CHANNEL


# ---------------------------------------------------------------------------
# KIVI group quantisation
# ---------------------------------------------------------------------------

def kivi_group_quant_dequant(x: torch.Tensor, axis: int, group_size: int, levels: int,
                             eps: float = 1e-8) -> torch.Tensor:
    """Round-trip ``x [..., S, D]`` through KIVI asymmetric group quantisation.

    Drop-in for ``kivi_group_quant_dequant`` (veloxquant_mlx/metal/_kivi_quant.py:138-207):
    ``axis=-2`` per-channel (keys), ``axis=-1`` per-token (values); bit-identical
    to ``KIVIKVCache._quant_dequant_along`` (veloxquant_mlx/cache/kivi_cache.py:151-201).
    """
    name = "kivi_group_quant_dequant"
    ax = _axis_tag(name, axis)
    if x.ndim < 2:
        raise ValueError(f"{name}: x must be at least 2D, got {tuple(x.shape)}")
    if group_size < 1:
        raise ValueError(f"{name}: group_size must be >= 1, got {group_size}")
    if levels < 1:
        raise ValueError(f"{name}: levels must be >= 1, got {levels}")
    tag = _ftag(name, x)
    if x.numel() == 0:
        return x
    _need_gpu(name, x)
    S, D = x.shape[-2], x.shape[-1]
    flat = x.contiguous()
    out = torch.empty_like(flat)
    rc = _lib.load().vq_kivi_quant_dequant(flat.data_ptr(), out.data_ptr(), tag, flat.numel() // (S * D), S, D,
                                           ax, int(group_size), int(levels), float(eps), _stream(x))
    _lib.check(rc)
    return out.view(x.shape)


def skvq_clipped_round_trip(x: torch.Tensor, bits: int, group_size: int, alphas, perm: torch.Tensor | None = None,
                            out: torch.Tensor | None = None, inv: torch.Tensor | None = None) -> torch.Tensor:
    """Round-trip ``x [B, H, r, D]`` through SKVQ's clipped group quantisation.

    ``clipped_group_quant`` then ``clipped_group_dequant`` (veloxquant_mlx/quantizers/skvq.py:105-183)
    on the channels taken in the order ``perm [H, D]`` (int32; ``None`` = as stored), with the result
    put back on the channels it came from, as ``SKVQKVCache._round_trip`` does
    (veloxquant_mlx/cache/skvq_cache.py:236-251).  ``x`` may be a token slice of a larger
    ``[B, H, cap, D]`` buffer; ``out`` (same shape and dtype, may be ``x`` itself) likewise.  ``inv``
    (the inverse of ``perm``, as the cache keeps it) only makes the launch faster.
    """
    name = "skvq_clipped_round_trip"
    if x.ndim != 4:
        raise ValueError(f"{name}: x must be [B, H, r, D], got {tuple(x.shape)}")
    if not 1 <= int(bits) <= 8:
        raise ValueError(f"{name}: bits must be in [1, 8], got {bits}")
    if group_size < 1:
        raise ValueError(f"{name}: group_size must be >= 1, got {group_size}")
    al = [float(a) for a in alphas]
    if not al or len(al) > 8 or any(not 0.0 < a <= 1.0 for a in al):
        raise ValueError(f"{name}: alphas must be 1..8 values in (0, 1], got {al}")
    tag = _ftag(name, x)
    B, H, r, D = x.shape

    def slab(t: torch.Tensor, what: str) -> int:
        """Elements between consecutive (b, h) slabs of a token slice of a contiguous [B, H, cap, D] buffer."""
        st = t.stride()
        step = st[1] if H > 1 else (st[0] if B > 1 else r * D)
        ok = (D == 1 or st[3] == 1) and (r == 1 or st[2] == D) and (B == 1 or H == 1 or st[0] == H * st[1]) \
            and step >= r * D
        if not ok:
            raise ValueError(f"{name}: {what} must be a token slice of a contiguous [B, H, cap, D] buffer, strides {st}")
        return step

    if out is None:
        out = torch.empty((B, H, r, D), dtype=x.dtype, device=x.device)
    elif out.shape != x.shape or out.dtype != x.dtype:
        raise ValueError(f"{name}: out must match x in shape and dtype")
    if x.numel() == 0:
        return out
    _need_gpu(name, x, out)
    xs, os_ = slab(x, "x"), slab(out, "out")
    pp = None
    if perm is not None:
        if perm.shape != (H, D) or perm.dtype != torch.int32:
            raise ValueError(f"{name}: perm must be int32 [H, D] = {(H, D)}, got {perm.dtype} {tuple(perm.shape)}")
        _need_gpu(name, perm)
        perm = perm.contiguous()
        pp = perm.data_ptr()
    ip = None
    if inv is not None:
        if perm is None or inv.shape != (H, D) or inv.dtype != torch.int32:
            raise ValueError(f"{name}: inv goes with perm and must be int32 [H, D]")
        _need_gpu(name, inv)
        inv = inv.contiguous()
        ip = inv.data_ptr()
    arr = (_lib.C.c_float * len(al))(*al)
    rc = _lib.load().vq_skvq_clipped_roundtrip(x.data_ptr(), out.data_ptr(), tag, B, H, r, D, xs, os_, pp, ip, int(bits),
                                               int(group_size), arr, len(al), _stream(x))
    _lib.check(rc)
    return out


def row_norms(x: torch.Tensor) -> torch.Tensor:
    """float32 L2 norms over the last axis of ``x [..., D]`` (D in 64 / 128 / 256), one pass over the stored rows."""
    name = "row_norms"
    tag = _ftag(name, x)
    _need_gpu(name, x)
    x = x.contiguous()
    D = x.shape[-1]
    out = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    _lib.check(_lib.load().vq_row_norms(x.data_ptr(), tag, x.numel() // D, D, out.data_ptr(), _stream(x)))
    return out


def channel_variance(x: torch.Tensor) -> torch.Tensor:
    """Population variance over the tokens of every channel of ``x [N, S, D]`` (D in 64 / 128 / 256), float32
    ``[N, D]``: one pass over the stored rows with double accumulators (``mx.var`` of the float32 copy in the
    reference, veloxquant_mlx/quantizers/kitty.py:44-67)."""
    name = "channel_variance"
    tag = _ftag(name, x)
    _need_gpu(name, x)
    if x.ndim != 3:
        raise ValueError(f"{name}: x must be [N, S, D], got {tuple(x.shape)}")
    x = x.contiguous()
    N, S, D = x.shape
    if S == 0:
        return torch.full((N, D), float("nan"), dtype=torch.float32, device=x.device)
    chunks = max(1, min(64, S // 256))
    partial = torch.empty((N, chunks, 2, D), dtype=torch.float64, device=x.device)
    var = torch.empty((N, D), dtype=torch.float32, device=x.device)
    lib = _lib.load()
    _lib.check(lib.vq_channel_moments(x.data_ptr(), tag, N, S, D, S * D, partial.data_ptr(), chunks, _stream(x)))
    _lib.check(lib.vq_channel_variance(partial.data_ptr(), N, chunks, D, S, var.data_ptr(), _stream(x)))
    return var


def channel_hi_mask(variance: torch.Tensor, n_hi: int) -> torch.Tensor:
    """``[N, D]`` float32 variances -> bool mask of every row's ``n_hi`` channels of largest variance, equal variances
    to the lower channel, a NaN after every number (the double stable argsort of
    veloxquant_mlx/quantizers/kitty.py:112-135), one launch.  D <= 1024."""
    name = "channel_hi_mask"
    _need_gpu(name, variance)
    if variance.ndim != 2 or variance.dtype != torch.float32:
        raise ValueError(f"{name}: variance must be float32 [N, D], got {tuple(variance.shape)} {variance.dtype}")
    variance = variance.contiguous()
    N, D = variance.shape
    mask = torch.empty((N, D), dtype=torch.bool, device=variance.device)
    _lib.check(_lib.load().vq_channel_hi_mask(variance.data_ptr(), N, D, int(n_hi), mask.data_ptr(), _stream(variance)))
    return mask


def kivi_group_quant_dequant_mixed(x: torch.Tensor, hi_mask: torch.Tensor, group_size: int, levels_lo: int, levels_hi: int,
                                   eps: float = 1e-8) -> torch.Tensor:
    """Token-axis round trip of ``x [N, S, 128]`` with ``levels_hi`` levels in the channels where ``hi_mask [N, 128]``
    (bool) is set and ``levels_lo`` in the others, in one launch (``quantize_mixed_channels``,
    veloxquant_mlx/quantizers/kitty.py:138-169).  Groups of 32 or 64 tokens."""
    name = "kivi_group_quant_dequant_mixed"
    tag = _ftag(name, x)
    _need_gpu(name, x)
    if x.ndim != 3 or tuple(hi_mask.shape) != (x.shape[0], x.shape[2]) or hi_mask.dtype != torch.bool:
        raise ValueError(f"{name}: x [N, S, D] and a bool hi_mask [N, D], got {tuple(x.shape)} and {tuple(hi_mask.shape)} {hi_mask.dtype}")
    x = x.contiguous()
    mask = hi_mask.contiguous()
    N, S, D = x.shape
    out = torch.empty_like(x)
    _lib.check(_lib.load().vq_kivi_quant_dequant_mixed(x.data_ptr(), out.data_ptr(), tag, N, S, D, int(group_size), int(levels_lo),
                                                       int(levels_hi), mask.data_ptr(), float(eps), _stream(x)))
    return out


def kivi_group_quant_dequant_grouplevels(x: torch.Tensor, group_levels: torch.Tensor, group_size: int, eps: float = 1e-8) -> torch.Tensor:
    """Token-axis round trip of fp16 / bf16 ``x [N, S, 128]`` with ``group_levels[j]`` levels in token group ``j`` (float32
    on the device, ``ceil(S / group_size)`` entries; 0 = the group passes through), in one launch (``age_tier_quantize``,
    veloxquant_mlx/quantizers/age_tiered.py:117-174).  Groups of 32 or 64 tokens."""
    name = "kivi_group_quant_dequant_grouplevels"
    tag = _ftag(name, x)
    _need_gpu(name, x)
    if x.ndim != 3:
        raise ValueError(f"{name}: x must be [N, S, D], got {tuple(x.shape)}")
    N, S, D = x.shape
    n_groups = -(-S // int(group_size))
    if group_levels.dtype != torch.float32 or group_levels.numel() != n_groups or group_levels.device != x.device:
        raise ValueError(f"{name}: group_levels must be {n_groups} float32 values on {x.device}")
    x = x.contiguous()
    out = torch.empty_like(x)
    _lib.check(_lib.load().vq_kivi_quant_dequant_grouplevels(x.data_ptr(), out.data_ptr(), tag, N, S, D, int(group_size),
                                                             group_levels.contiguous().data_ptr(), float(eps), _stream(x)))
    return out


def zip_route(norms: torch.Tensor, n_hi: int) -> torch.Tensor:
    """int32 ``[BH, S]`` routing order of a salience split of float32 ``norms [BH, S]``: the rows outside the
    ``n_hi`` largest norms in their own order, then the ``n_hi`` largest in theirs, later rows first among equal norms
    at the threshold (``_batched_saliency_mask`` + stable argsort of the mask,
    veloxquant_mlx/cache/zipcache_cache.py:106-116, 186-190)."""
    name = "zip_route"
    if norms.ndim != 2 or norms.dtype != torch.float32:
        raise ValueError(f"{name}: norms must be a float32 [BH, S] tensor")
    _need_gpu(name, norms)
    norms = norms.contiguous()
    BH, S = norms.shape
    order = torch.empty((BH, S), dtype=torch.int32, device=norms.device)
    _lib.check(_lib.load().vq_zip_route(norms.data_ptr(), BH, S, int(n_hi), order.data_ptr(), _stream(norms)))
    return order


def kivi_group_quant_dequant_rows(x: torch.Tensor, out: torch.Tensor, rows: torch.Tensor, start: int, n_rows: int,
                                  group_size: int, levels: int, eps: float = 1e-8) -> torch.Tensor:
    """Token-axis round trip over routed rows, in one launch and without a gathered copy: positions
    ``start .. start + n_rows`` of the routing order ``rows`` (int32 ``[BH, S]``) name rows of ``x [BH, S, D]``;
    consecutive positions form the groups, every reconstruction lands in ``out`` (same shape and dtype as ``x``) at
    its source row.  What gather -> ``_group_quant_dequant_batched`` -> scatter does for one salience block of
    ``ZipCacheKVCache`` (veloxquant_mlx/cache/zipcache_cache.py:118-244)."""
    name = "kivi_group_quant_dequant_rows"
    if x.ndim != 3 or tuple(out.shape) != tuple(x.shape) or out.dtype != x.dtype or not (x.is_contiguous() and out.is_contiguous()):
        raise ValueError(f"{name}: x and out must be contiguous [BH, S, D] tensors of one dtype")
    BH, S, D = x.shape
    if tuple(rows.shape) != (BH, S) or rows.dtype != torch.int32 or not rows.is_contiguous():
        raise ValueError(f"{name}: rows must be a contiguous int32 [{BH}, {S}] tensor")
    if not (0 <= start and start + n_rows <= S):
        raise ValueError(f"{name}: positions [{start}, {start + n_rows}) outside [0, {S})")
    tag = _ftag(name, x)
    _need_gpu(name, x, out, rows)
    rc = _lib.load().vq_kivi_quant_dequant_rows(x.data_ptr(), out.data_ptr(), tag, BH, int(n_rows), D, S * D,
                                                rows.data_ptr() + 4 * int(start), S, int(group_size), int(levels), float(eps),
                                                _stream(x))
    _lib.check(rc)
    return out


def kivi_quant_pack(x: torch.Tensor, axis: int, group_size: int, bits: int, *, levels: int | None = None,
                    eps: float = 1e-8, meta_dtype: torch.dtype = torch.float16, v_layout: str = "channel",
                    out: tuple[torch.Tensor, torch.Tensor, torch.Tensor] | None = None,
                    dst_tok0: int = 0):
    """Quantise ``x [B, H, S, D]`` and bit-pack the codes.

    Codes are those of ``_quant_keys`` / ``_quant_values``
    (benchmark_scripts/benchmark_real_model_scalar_attend.py:115-153); words are
    the ``_pack_indices`` image (veloxquant_mlx/cache/turboquant_rvq_cache.py:82-106).
    Returns ``(packed uint32-as-int32, scale, zero)``:

    * ``axis=-2``: packed ``[B,H,S,W]``, scale/zero ``[B,H,ceil(S/g),D]``
    * ``axis=-1``, ``v_layout="channel"``: packed ``[B,H,S,W]``, scale/zero ``[B,H,S,GV]``
    * ``axis=-1``, ``v_layout="token"``: packed ``[B,H,S/per,D]``, scale/zero ``[B,H,GV,S]``

    With ``out=(packed, scale, zero)`` the results are written at token offset
    ``dst_tok0`` of pre-allocated cache buffers whose token capacity is read
    from ``packed`` (``x`` may then be a slice with a larger head stride).
    """
    name = "kivi_quant_pack"
    ax = _axis_tag(name, axis)
    if x.ndim != 4:
        raise ValueError(f"{name}: x must be 4D [B,H,S,D], got {tuple(x.shape)}")
    if v_layout not in _V_LAYOUT:
        raise ValueError(f"{name}: v_layout must be 'channel' or 'token', got {v_layout!r}")
    if not (1 <= bits <= 8):
        raise ValueError(f"{name}: bits must be in 1..8, got {bits}")
    if meta_dtype not in (torch.float16, torch.float32):
        raise ValueError(f"{name}: meta_dtype must be float16 or float32, got {meta_dtype}")
    tag = _ftag(name, x)
    _need_gpu(name, x)
    B, H, S, D = x.shape
    per = 32 // bits
    levels = (1 << bits) - 1 if levels is None else int(levels)
    tokpacked = ax == VQ_AXIS_CHANNEL and v_layout == "token"
    # accept a [B,H,S,D] view whose rows are dense but whose head stride is larger
    xs = x.stride(1) if H > 1 else (x.stride(0) if B > 1 else S * D)
    if x.stride(-1) != 1 or x.stride(-2) != D or xs < S * D or (B > 1 and H > 1 and x.stride(0) != H * xs):
        x = x.contiguous()
        xs = S * D
    W = -(-D // per)
    GV = -(-D // group_size)
    if out is None:
        cap = S
        if tokpacked:
            packed = torch.empty((B, H, -(-S // per), D), dtype=torch.int32, device=x.device)
            mshape = (B, H, GV, S)
        else:
            packed = torch.empty((B, H, S, W), dtype=torch.int32, device=x.device)
            mshape = (B, H, -(-S // group_size), D) if ax == VQ_AXIS_TOKEN else (B, H, S, GV)
        scale = torch.empty(mshape, dtype=meta_dtype, device=x.device)
        zero = torch.empty(mshape, dtype=meta_dtype, device=x.device)
    else:
        packed, scale, zero = out
        cap = packed.shape[2] * per if tokpacked else packed.shape[2]
        if scale.dtype != meta_dtype or zero.dtype != meta_dtype:
            raise ValueError(f"{name}: out scale/zero dtype must equal meta_dtype")
        for t in (packed, scale, zero):
            if not t.is_contiguous():
                raise ValueError(f"{name}: out buffers must be contiguous")
    rc = _lib.load().vq_kivi_quant_pack(
        x.data_ptr(), tag, B * H, S, D, xs, ax, int(group_size), levels, float(eps), int(bits),
        _V_LAYOUT[v_layout], packed.data_ptr(), scale.data_ptr(), zero.data_ptr(),
        VQ_F16 if meta_dtype == torch.float16 else VQ_F32, cap, int(dst_tok0), _stream(x))
    _lib.check(rc)
    return packed, scale, zero


def kivi_quant_pack_kv(k: torch.Tensor, v: torch.Tensor, group_size: int, bits: int, *, levels: int | None = None,
                       eps: float = 1e-8, meta_dtype: torch.dtype = torch.float16, v_layout: str = "token",
                       out: tuple | None = None, dst_tok0: int = 0):
    """:func:`kivi_quant_pack` of the keys (``axis=-2``) and of the values (``axis=-1``, ``v_layout``) of
    the same tokens in one library call -- one launch at head_dim 128.  ``k`` and ``v`` are
    ``[B, H, S, D]`` of one dtype and one layout.  Returns ``((k_packed, k_scale, k_zero),
    (v_packed, v_scale, v_zero))``; ``out`` takes the same pair of triples (buffers of one token
    capacity) and ``dst_tok0`` the token offset, as there."""
    name = "kivi_quant_pack_kv"
    if k.ndim != 4 or tuple(v.shape) != tuple(k.shape) or v.dtype != k.dtype:
        raise ValueError(f"{name}: k and v must be 4D [B,H,S,D] of one shape and dtype, got {tuple(k.shape)} {k.dtype} "
                         f"and {tuple(v.shape)} {v.dtype}")
    if v_layout not in _V_LAYOUT:
        raise ValueError(f"{name}: v_layout must be 'channel' or 'token', got {v_layout!r}")
    if not (1 <= bits <= 8):
        raise ValueError(f"{name}: bits must be in 1..8, got {bits}")
    if meta_dtype not in (torch.float16, torch.float32):
        raise ValueError(f"{name}: meta_dtype must be float16 or float32, got {meta_dtype}")
    tag = _ftag(name, k)
    _need_gpu(name, k)
    B, H, S, D = k.shape
    per = 32 // bits
    levels = (1 << bits) - 1 if levels is None else int(levels)
    tokpacked = v_layout == "token"
    if not (k.is_contiguous() and v.is_contiguous()):
        k, v = k.contiguous(), v.contiguous()
    W, GV, g = -(-D // per), -(-D // group_size), int(group_size)
    if out is None:
        if tokpacked and S % per:
            raise ValueError(f"{name}: token-packed values need S % {per} == 0, got S={S}")
        new = lambda shape, dt: torch.empty(shape, dtype=dt, device=k.device)
        kd = (new((B, H, S, W), torch.int32), new((B, H, -(-S // g), D), meta_dtype), new((B, H, -(-S // g), D), meta_dtype))
        if tokpacked:
            vd = (new((B, H, S // per, D), torch.int32), new((B, H, GV, S), meta_dtype), new((B, H, GV, S), meta_dtype))
        else:
            vd = (new((B, H, S, W), torch.int32), new((B, H, S, GV), meta_dtype), new((B, H, S, GV), meta_dtype))
        cap = S
    else:
        kd, vd = out
        cap = kd[0].shape[2]
        v_cap = vd[0].shape[2] * per if tokpacked else vd[0].shape[2]
        if v_cap != cap:
            raise ValueError(f"{name}: key and value buffers hold {cap} and {v_cap} tokens")
        for t in (*kd[1:], *vd[1:]):
            if t.dtype != meta_dtype:
                raise ValueError(f"{name}: out scale/zero dtype must equal meta_dtype")
        for t in (*kd, *vd):
            if not t.is_contiguous():
                raise ValueError(f"{name}: out buffers must be contiguous")
    rc = _lib.load().vq_kivi_quant_pack_kv(
        k.data_ptr(), v.data_ptr(), tag, B * H, S, D, S * D, g, levels, float(eps), int(bits), _V_LAYOUT[v_layout],
        kd[0].data_ptr(), kd[1].data_ptr(), kd[2].data_ptr(), vd[0].data_ptr(), vd[1].data_ptr(), vd[2].data_ptr(),
        VQ_F16 if meta_dtype == torch.float16 else VQ_F32, cap, int(dst_tok0), _stream(k))
    _lib.check(rc)
    return kd, vd


def kivi_quant_codes(x: torch.Tensor, axis: int, group_size: int, levels: int, eps: float = 1e-8):
    """``(codes uint8, scale f32, zero f32)`` exactly as the reference's split
    form returns them (test_scalar_attend.py:51-82)."""
    packed, scale, zero = kivi_quant_pack(x, axis, group_size, 8, levels=levels, eps=eps,
                                          meta_dtype=torch.float32)
    B, H, S, D = x.shape
    codes = packed.reshape(-1).view(torch.uint8).view(B, H, S, -1)[..., :D]
    return codes, scale, zero


def kv_tail_append(k_new: torch.Tensor, v_new: torch.Tensor, k_tail: torch.Tensor, v_tail: torch.Tensor,
                   pos: int) -> None:
    """Write ``k_new, v_new [B,H,S,D]`` into rows ``[pos, pos+S)`` of the tails ``[B,H,cap,D]``
    (one launch for both): the concatenation step of ``KIVIKVCache.update_and_fetch``
    (veloxquant_mlx/cache/kivi_cache.py:206-260) into buffers that already have room."""
    name = "kv_tail_append"
    _need_gpu(name, k_new, v_new, k_tail, v_tail)
    if k_new.shape != v_new.shape or k_tail.shape != v_tail.shape or k_new.ndim != 4 or k_tail.ndim != 4:
        raise ValueError(f"{name}: keys/values must be [B,H,S,D] and the tails [B,H,cap,D]")
    B, H, S, D = k_new.shape
    if k_tail.shape[0] != B or k_tail.shape[1] != H or k_tail.shape[3] != D:
        raise ValueError(f"{name}: tail shape {tuple(k_tail.shape)} does not match new tokens {tuple(k_new.shape)}")
    if not (k_new.dtype == v_new.dtype == k_tail.dtype == v_tail.dtype):
        raise ValueError(f"{name}: new tokens and tails must share one dtype")
    if not (k_tail.is_contiguous() and v_tail.is_contiguous()):
        raise ValueError(f"{name}: the tails must be contiguous")
    cap = k_tail.shape[2]
    if pos < 0 or pos + S > cap:
        raise ValueError(f"{name}: tokens [{pos}, {pos + S}) exceed the tail capacity {cap}")

    es = k_new.element_size()

    def strides(t):   # channels contiguous, every other stride a multiple of 16 bytes; else a packed copy
        if B * H * S * D and (t.stride(3) != 1 or any((t.stride(i) * es) % 16 for i in range(3)) or t.data_ptr() % 16):
            t = t.contiguous()
        return t, (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))
    k_new, ks = strides(k_new)
    v_new, vs = strides(v_new)
    _lib.check(_lib.load().vq_kv_tail_append(k_new.data_ptr(), v_new.data_ptr(), ks, vs, k_tail.data_ptr(),
                                             v_tail.data_ptr(), es, B, H, S, D, cap, pos, _stream(k_new)))


def kivi_cache_append(k_new: torch.Tensor, v_new: torch.Tensor, k_tail: torch.Tensor, v_tail: torch.Tensor,
                      n_tail: int, n_flush: int, packed, dst_tok0: int, spare, *, bits: int, group_size: int,
                      levels: int, eps: float, v_layout: str, args=None):
    """One chunk of a packed KIVI cache in one library call (``vq_kivi_cache_append``):
    ``k_new, v_new [B,H,S,D]`` go to rows ``[n_tail, n_tail+S)`` of the tails; with
    ``n_flush > 0`` the first ``n_flush`` tail rows are quantised into ``packed =
    (k_packed, k_scale, k_zero, v_packed, v_scale, v_zero)`` at token ``dst_tok0`` and the
    rest moves to the front of ``spare = (k_spare, v_spare)``.  The steps of
    ``KIVIKVCache.update_and_fetch`` (veloxquant_mlx/cache/kivi_cache.py:206-262) on packed
    buffers.  The caller owns the shapes: all tensors share a device, the new tokens and the
    four tails one dtype, every buffer is contiguous except ``k_new`` / ``v_new``, whose
    channels are.  ``args`` may carry a ``KiviAppendArgs`` from a previous call to refill."""
    name = "kivi_cache_append"
    _need_gpu(name, k_new)
    a = _lib.KiviAppendArgs() if args is None else args
    B, H, S, D = k_new.shape
    if v_new.shape != k_new.shape or k_tail.shape != v_tail.shape or k_tail.ndim != 4:
        raise ValueError(f"{name}: keys/values must be [B,H,S,D] and the tails [B,H,cap,D]")
    if not (k_new.dtype == v_new.dtype == k_tail.dtype == v_tail.dtype):
        raise ValueError(f"{name}: new tokens and tails must share one dtype")
    a.k_new, a.v_new = k_new.data_ptr(), v_new.data_ptr()
    ks, vs = k_new.stride(), v_new.stride()
    if ks[3] != 1 or vs[3] != 1:
        raise ValueError(f"{name}: channels of the new tokens must be contiguous")
    a.k_strides[0], a.k_strides[1], a.k_strides[2] = ks[0], ks[1], ks[2]
    a.v_strides[0], a.v_strides[1], a.v_strides[2] = vs[0], vs[1], vs[2]
    a.dtype = _FLOAT_TAG[k_new.dtype]
    a.B, a.H, a.S, a.D = B, H, S, D
    a.k_tail, a.v_tail, a.tail_cap, a.n_tail = k_tail.data_ptr(), v_tail.data_ptr(), k_tail.shape[2], n_tail
    a.n_flush = n_flush
    if n_flush:
        kp, ksc, kz, vp_, vsc, vz = packed
        per = 32 // bits
        a.k_packed, a.k_scale, a.k_zero = kp.data_ptr(), ksc.data_ptr(), kz.data_ptr()
        a.v_packed, a.v_scale, a.v_zero = vp_.data_ptr(), vsc.data_ptr(), vz.data_ptr()
        a.meta_dtype = VQ_F16 if ksc.dtype == torch.float16 else VQ_F32
        a.cap_tokens, a.dst_tok0 = kp.shape[2], dst_tok0
        if v_layout == "token" and vp_.shape[2] * per != kp.shape[2]:
            raise ValueError(f"{name}: key and value stores differ in capacity")
        a.group, a.levels, a.eps, a.pack_bits, a.v_layout = group_size, levels, eps, bits, _V_LAYOUT[v_layout]
        a.k_spare, a.v_spare, a.spare_cap = spare[0].data_ptr(), spare[1].data_ptr(), spare[0].shape[2]
    _lib.check(_lib.load().vq_kivi_cache_append(C.byref(a), _stream(k_new)))
    return a


def kivi_dequant(packed: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, axis: int, group_size: int,
                 bits: int, S: int, D: int, *, v_layout: str = "channel", out_dtype: torch.dtype = torch.float16,
                 src_tok0: int = 0) -> torch.Tensor:
    """Rebuild ``[B,H,S,D]`` from packed codes (``code*scale+zero``, two roundings)."""
    name = "kivi_dequant"
    ax = _axis_tag(name, axis)
    _need_gpu(name, packed, scale, zero)
    if out_dtype not in _FLOAT_TAG:
        raise ValueError(f"{name}: unsupported out dtype {out_dtype}")
    B, H = packed.shape[0], packed.shape[1]
    per = 32 // bits
    tokpacked = ax == VQ_AXIS_CHANNEL and v_layout == "token"
    cap = packed.shape[2] * per if tokpacked else packed.shape[2]
    out = torch.empty((B, H, S, D), dtype=out_dtype, device=packed.device)
    rc = _lib.load().vq_kivi_dequant(
        packed.data_ptr(), scale.data_ptr(), zero.data_ptr(),
        VQ_F16 if scale.dtype == torch.float16 else VQ_F32, B * H, S, D, ax, int(group_size), int(bits),
        _V_LAYOUT[v_layout], cap, int(src_tok0), out.data_ptr(), _FLOAT_TAG[out_dtype], _stream(packed))
    _lib.check(rc)
    return out


def scalar_decode_once(codes: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, group_size: int,
                       mode: str) -> torch.Tensor:
    """uint8 codes + fp32 scale/zero -> fp16 (veloxquant_mlx/metal/_scalar_attend.py:650-699)."""
    if mode not in ("K", "V"):
        raise ValueError(f"scalar_decode_once: mode must be 'K' or 'V', got {mode!r}")
    if codes.ndim != 4:
        raise ValueError(f"scalar_decode_once: codes must be 4D, got {tuple(codes.shape)}")
    B, H, S, D = codes.shape
    if D % 4:
        raise ValueError("scalar_decode_once: D must be a multiple of 4")
    words = _bytes_as_words(codes)
    return kivi_dequant(words, scale.float().contiguous(), zero.float().contiguous(),
                        -2 if mode == "K" else -1, group_size, 8, S, D, out_dtype=torch.float16)


# ---------------------------------------------------------------------------
# bit packing
# ---------------------------------------------------------------------------

def pack_indices(idx: torch.Tensor, bits: int) -> torch.Tensor:
    """``_pack_indices`` (veloxquant_mlx/cache/turboquant_rvq_cache.py:82-106): trailing
    axis -> uint32 words (returned as int32 storage), LSB first, zero padded."""
    if not (1 <= bits <= 8):
        raise ValueError(f"pack_indices: bits must be in 1..8, got {bits}")
    _need_gpu("pack_indices", idx)
    d = idx.shape[-1]
    per = 32 // bits
    flat = idx.to(torch.uint8).contiguous()
    out = torch.empty(idx.shape[:-1] + (-(-d // per),), dtype=torch.int32, device=idx.device)
    rows = flat.numel() // d if d else 0
    _lib.check(_lib.load().vq_pack_words(flat.data_ptr(), rows, d, bits, out.data_ptr(), _stream(idx)))
    return out


def unpack_indices(packed: torch.Tensor, bits: int, d: int) -> torch.Tensor:
    """``_unpack_indices`` (turboquant_rvq_cache.py:109-126)."""
    if not (1 <= bits <= 8):
        raise ValueError(f"unpack_indices: bits must be in 1..8, got {bits}")
    _need_gpu("unpack_indices", packed)
    per = 32 // bits
    if packed.shape[-1] != -(-d // per):
        raise ValueError(f"unpack_indices: {packed.shape[-1]} words cannot hold d={d} at bits={bits}")
    flat = packed.contiguous()
    out = torch.empty(packed.shape[:-1] + (d,), dtype=torch.uint8, device=packed.device)
    rows = out.numel() // d if d else 0
    _lib.check(_lib.load().vq_unpack_words(flat.data_ptr(), rows, d, bits, out.data_ptr(), _stream(packed)))
    return out


def turboquant_bit_pack(indices: torch.Tensor, b: int) -> torch.Tensor:
    """``turboquant_bit_pack`` (veloxquant_mlx/metal/_bit_packing.py:87-118)."""
    if b not in (1, 2, 4):
        raise ValueError(f"turboquant_bit_pack: b must be 1, 2, or 4, got {b}")
    N = indices.numel()
    if N % (8 // b) != 0:
        raise ValueError(f"turboquant_bit_pack: N={N} not divisible by {8 // b} (= 8/b)")
    _need_gpu("turboquant_bit_pack", indices)
    flat = indices.reshape(-1).to(torch.uint8).contiguous()
    out = torch.empty(N * b // 8, dtype=torch.uint8, device=indices.device)
    _lib.check(_lib.load().vq_bit_pack(flat.data_ptr(), N, b, out.data_ptr(), _stream(indices)))
    return out


def turboquant_bit_unpack(packed: torch.Tensor, N: int, b: int) -> torch.Tensor:
    """``turboquant_bit_unpack`` (veloxquant_mlx/metal/_bit_packing.py:121-148)."""
    if b not in (1, 2, 4):
        raise ValueError(f"turboquant_bit_unpack: b must be 1, 2, or 4, got {b}")
    if N < 0:
        raise ValueError(f"turboquant_bit_unpack: N must be >= 0, got {N}")
    need = -(-N * b // 8)
    if packed.numel() < need:
        raise ValueError(f"turboquant_bit_unpack: packed has {packed.numel()} byte(s) but N={N} "
                         f"at b={b} needs {need}")
    _need_gpu("turboquant_bit_unpack", packed)
    flat = packed.reshape(-1).to(torch.uint8).contiguous()
    out = torch.empty(N, dtype=torch.uint8, device=packed.device)
    _lib.check(_lib.load().vq_bit_unpack(flat.data_ptr(), N, b, out.data_ptr(), _stream(packed)))
    return out


# ---------------------------------------------------------------------------
# VecInfer product VQ
# ---------------------------------------------------------------------------

def vecinfer_quantize_metal(x: torch.Tensor, codebook: torch.Tensor, sub_dim: int, *,
                            index_dtype: torch.dtype = torch.int32) -> torch.Tensor:
    """Nearest-centroid indices ``[..., D // sub_dim]``; drop-in for ``quantize_vq``
    (veloxquant_mlx/allocators/vecinfer.py:281-318) and ``vecinfer_quantize_metal``
    (veloxquant_mlx/metal/_vecinfer.py:181-222).  ``index_dtype=torch.uint8`` stores
    one byte per index (codebooks of at most 256 centroids)."""
    name = "vecinfer_quantize_metal"
    D = x.shape[-1]
    if D % sub_dim != 0:
        raise ValueError(f"{name}: D={D} not divisible by sub_dim={sub_dim}")
    if codebook.ndim != 2 or codebook.shape[1] != sub_dim:
        raise ValueError(f"{name}: codebook must be [n_centroids, {sub_dim}], got {tuple(codebook.shape)}")
    if index_dtype not in (torch.int32, torch.uint8):
        raise ValueError(f"{name}: index_dtype must be int32 or uint8")
    _need_gpu(name, x, codebook)
    if x.dtype not in _FLOAT_TAG:
        x = x.float()
    if codebook.dtype not in _FLOAT_TAG:
        codebook = codebook.float()
    xf, cb = x.contiguous(), codebook.contiguous()
    n_sub = D // sub_dim
    out = torch.empty(x.shape[:-1] + (n_sub,), dtype=index_dtype, device=x.device)
    rc = _lib.load().vq_vecinfer_assign(xf.data_ptr(), _FLOAT_TAG[xf.dtype], out.numel(), cb.data_ptr(),
                                        _FLOAT_TAG[cb.dtype], cb.shape[0], sub_dim, out.data_ptr(),
                                        VQ_U8 if index_dtype == torch.uint8 else VQ_I32, _stream(x))
    _lib.check(rc)
    return out


def vecinfer_dequant_metal(indices: torch.Tensor, codebook: torch.Tensor,
                           out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """Centroid gather ``[..., n_sub] -> [..., n_sub*sub_dim]``; drop-in for
    ``dequantize_vq`` (allocators/vecinfer.py:321-335) / ``vecinfer_dequant_metal``
    (metal/_vecinfer.py:144-178)."""
    name = "vecinfer_dequant_metal"
    if codebook.ndim != 2:
        raise ValueError(f"{name}: codebook must be 2D, got {tuple(codebook.shape)}")
    _need_gpu(name, indices, codebook)
    if out_dtype is None:
        out_dtype = codebook.dtype
    if out_dtype not in _FLOAT_TAG:
        raise ValueError(f"{name}: unsupported out dtype {out_dtype}")
    if codebook.dtype not in _FLOAT_TAG:
        codebook = codebook.float()
    if indices.dtype not in (torch.int32, torch.uint8):
        indices = indices.to(torch.int32)
    idx, cb = indices.contiguous(), codebook.contiguous()
    sub = cb.shape[1]
    out = torch.empty(indices.shape[:-1] + (indices.shape[-1] * sub,), dtype=out_dtype, device=indices.device)
    rc = _lib.load().vq_vecinfer_dequant(idx.data_ptr(), VQ_U8 if idx.dtype == torch.uint8 else VQ_I32,
                                         idx.numel(), cb.data_ptr(), _FLOAT_TAG[cb.dtype], cb.shape[0], sub,
                                         out.data_ptr(), _FLOAT_TAG[out_dtype], _stream(indices))
    _lib.check(rc)
    return out


vecinfer_quantize_hip = vecinfer_quantize_metal
vecinfer_dequant_hip = vecinfer_dequant_metal


def _sylvester_scale(H_mat: torch.Tensor) -> float:
    """``|H[0, 0]|`` if ``H_mat`` is the orthonormal Sylvester-Hadamard matrix in natural order
    (every entry ``(-1)^popcount(a & b)`` times one magnitude), else 0.  Checked once per tensor
    object and version (the verdict rides on the tensor itself)."""
    memo = getattr(H_mat, "_vq_sylvester", None)
    if memo is None or memo[0] != H_mat._version:
        D = H_mat.shape[0]
        ok = H_mat.ndim == 2 and H_mat.shape[1] == D and D >= 1 and (D & (D - 1)) == 0
        h = 0.0
        if ok:
            Hf = H_mat.float()
            h = float(Hf[0, 0].abs())
            a = torch.arange(D, device=H_mat.device)
            par = a[:, None] & a[None, :]
            sign = torch.ones_like(Hf)
            for b in range(max(D.bit_length() - 1, 0)):
                sign = sign * (1 - 2 * ((par >> b) & 1)).to(Hf.dtype)
            ok = h > 0 and bool(torch.equal(Hf, sign * h))
        memo = (H_mat._version, h if ok else 0.0)
        H_mat._vq_sylvester = memo
    return memo[1]


def vecinfer_encode_decode_metal(keys: torch.Tensor, k_codebook: torch.Tensor, sub_dim: int, H_mat: torch.Tensor,
                                 smooth: torch.Tensor | None = None, *, index_dtype: torch.dtype = torch.int32,
                                 want_k_hat: bool = True, want_k_tilde: bool = False):
    """Fused key encode+decode, smooth -> WHT -> VQ -> dequant -> inverse WHT -> smooth, in one
    launch; drop-in for ``vecinfer_encode_decode_metal`` (veloxquant_mlx/metal/_vecinfer.py:225-293).
    Returns ``(k_hat [B,H,S,D] in the dtype of keys, k_indices [B,H,S,n_sub])``; with
    ``want_k_hat=False`` the first element is ``None`` (indices only, what the memory-bound
    cache needs), with ``want_k_tilde=True`` a third element holds the transformed keys (float32).
    ``H_mat`` must be the orthonormal Sylvester-Hadamard matrix (``walsh_hadamard_matrix(D)``),
    which is applied as a fast transform; any other matrix, or a shape the fused kernel does not
    cover, takes the matrix product followed by the assignment and gather kernels."""
    name = "vecinfer_encode_decode_metal"
    if keys.ndim != 4:
        raise ValueError(f"{name}: keys must be 4D, got {tuple(keys.shape)}")
    B, Hh, S, D = keys.shape
    if D % sub_dim != 0:
        raise ValueError(f"{name}: D={D} not divisible by sub_dim={sub_dim}")
    if D > 512:
        raise ValueError(f"{name}: D={D} > 512 (threadgroup limit)")
    if k_codebook.ndim != 2 or k_codebook.shape[1] != sub_dim or k_codebook.shape[0] == 0:
        raise ValueError(f"{name}: codebook must be non-empty [n_centroids, {sub_dim}], got {tuple(k_codebook.shape)}")
    if index_dtype not in (torch.int32, torch.uint8):
        raise ValueError(f"{name}: index_dtype must be int32 or uint8")
    _need_gpu(name, keys, k_codebook, H_mat)
    if keys.dtype not in _FLOAT_TAG:
        keys = keys.float()
    kk = keys.contiguous()
    cb = (k_codebook if k_codebook.dtype in _FLOAT_TAG else k_codebook.float()).contiguous()
    sm = None
    if smooth is not None:
        sm = smooth.reshape(1, D) if smooth.ndim == 1 else smooth
        sm = sm.to(device=keys.device, dtype=torch.float32)
        if sm.shape[0] not in (1, Hh):   # e.g. factors calibrated on query heads under GQA: one averaged row
            sm = sm.mean(dim=0, keepdim=True)
        sm = sm.contiguous()
    n_sub = D // sub_dim
    h = _sylvester_scale(H_mat)
    fused = h > 0 and sub_dim in (4, 8) and n_sub in (8, 16, 32, 64) and cb.shape[0] <= 256
    if fused:
        idx = torch.empty((B, Hh, S, n_sub), dtype=index_dtype, device=keys.device)
        k_hat = torch.empty_like(kk) if want_k_hat else None
        k_tilde = torch.empty((B, Hh, S, D), dtype=torch.float32, device=keys.device) if want_k_tilde else None
        rc = _lib.load().vq_vecinfer_encode_keys(
            kk.data_ptr(), _FLOAT_TAG[kk.dtype], B, Hh, S, D, sm.data_ptr() if sm is not None else None,
            sm.shape[0] if sm is not None else 1, h, cb.data_ptr(), _FLOAT_TAG[cb.dtype], cb.shape[0], sub_dim,
            idx.data_ptr(), VQ_U8 if index_dtype == torch.uint8 else VQ_I32,
            k_hat.data_ptr() if k_hat is not None else None, k_tilde.data_ptr() if k_tilde is not None else None,
            _stream(keys))
        _lib.check(rc)
    else:
        Hf = H_mat.float()
        x = kk.float()
        if sm is not None:
            x = x / (sm[:, None, :] if sm.shape[0] == Hh and Hh > 1 else sm[0])
        k_tilde = x @ Hf
        idx = vecinfer_quantize_metal(k_tilde, cb, sub_dim, index_dtype=index_dtype)
        k_hat = None
        if want_k_hat:
            k_hat = vecinfer_dequant_metal(idx, cb, out_dtype=torch.float32) @ Hf.T
            if sm is not None:
                k_hat = k_hat * (sm[:, None, :] if sm.shape[0] == Hh and Hh > 1 else sm[0])
            k_hat = k_hat.to(keys.dtype)
        if not want_k_tilde:
            k_tilde = None
    return (k_hat, idx, k_tilde) if want_k_tilde else (k_hat, idx)


def vecinfer_encode_decode_simple_metal(values: torch.Tensor, v_codebook: torch.Tensor, sub_dim: int, *,
                                        index_dtype: torch.dtype = torch.int32):
    """Value encode+decode: nearest centroid and its gather; drop-in for
    ``vecinfer_encode_decode_simple_metal`` (veloxquant_mlx/metal/_vecinfer.py:296-345).
    Returns ``(v_hat [B,H,S,D] in the dtype of values, v_indices [B,H,S,n_sub])``."""
    name = "vecinfer_encode_decode_simple_metal"
    if values.ndim != 4:
        raise ValueError(f"{name}: values must be 4D, got {tuple(values.shape)}")
    D = values.shape[-1]
    if D % sub_dim != 0:
        raise ValueError(f"{name}: D={D} not divisible by sub_dim={sub_dim}")
    if D > 512:
        raise ValueError(f"{name}: D={D} > 512 (threadgroup limit)")
    if v_codebook.ndim != 2 or v_codebook.shape[1] != sub_dim or v_codebook.shape[0] == 0:
        raise ValueError(f"{name}: codebook must be non-empty [n_centroids, {sub_dim}], got {tuple(v_codebook.shape)}")
    idx = vecinfer_quantize_metal(values, v_codebook, sub_dim, index_dtype=index_dtype)
    out_dtype = values.dtype if values.dtype in _FLOAT_TAG else torch.float32
    return vecinfer_dequant_metal(idx, v_codebook, out_dtype=out_dtype), idx


# ---------------------------------------------------------------------------
# attention over a packed cache
# ---------------------------------------------------------------------------

_workspaces: dict[tuple, torch.Tensor] = {}


def _workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    key = (device.type, device.index, _stream_of(device))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


_tile_scratches: dict[tuple, torch.Tensor] = {}
_TILE_SCRATCH_MAX = 2 << 30   # bytes; larger inputs are attended without tiles


def _tile_scratch(device: torch.device, rows: int, units: int) -> torch.Tensor:
    key = (device.type, device.index, _stream_of(device))
    t = _tile_scratches.get(key)
    if t is None or t.numel() < rows * units * PREFILL_TILE_BYTES:
        t = _tile_scratches[key] = torch.empty(rows * units * PREFILL_TILE_BYTES, dtype=torch.uint8, device=device)
    return t[: rows * units * PREFILL_TILE_BYTES].view(rows, units, PREFILL_TILE_BYTES)


def release_tile_scratch() -> int:
    """Give back the tile scratches :func:`kivi_packed_attend` keeps per device and stream for long causal calls
    over plain keys and values; returns the bytes released.  (A call with ``static_scratch=True`` never makes
    one: it allocates nothing, so it takes tiles only when the caller passes them.)"""
    n = sum(t.numel() for t in _tile_scratches.values())
    _tile_scratches.clear()
    return n


_sync_counters: dict[tuple, torch.Tensor] = {}


def _counters(device: torch.device) -> torch.Tensor:
    """Per-(device, stream) int32 counters the single-launch decode path needs: zero when a
    call is enqueued, left zero by it (65536 = the largest B*H_kv the MFMA path takes)."""
    key = (device.type, device.index, _stream_of(device))
    c = _sync_counters.get(key)
    if c is None:
        c = torch.zeros(65536, dtype=torch.int32, device=device)
        _sync_counters[key] = c
    return c


def _tail_layout(t: torch.Tensor):
    """Return ``(tensor, capacity)`` for a ``[B,H,n,D]`` tail that is either dense or
    a token slice of a dense ``[B,H,capacity,D]`` buffer (rows dense, uniform head
    stride); anything else is copied."""
    B, H, n, D = t.shape
    if t.stride(3) == 1 and t.stride(2) == D:
        hs = t.stride(1) if H > 1 else (t.stride(0) if B > 1 else n * D)
        if hs % D == 0 and hs >= n * D and (B == 1 or H == 1 or t.stride(0) == H * hs):
            return t, hs // D
    t = t.contiguous()
    return t, n


def _cache_side(name, a, keep, k_packed, k_scale, k_zero, v_packed, v_scale, v_zero, n_packed, bits, group_size,
                v_layout, k_tail, v_tail, n_tail):
    """Fill the cache fields of ``a`` (packed prefix and tail); returns ``(Hkv, k_tail)`` with the tail as passed
    to the library."""
    Hkv = None
    if n_packed > 0:
        for t in (k_packed, k_scale, k_zero, v_packed, v_scale, v_zero):
            if t is None or not t.is_contiguous():
                raise ValueError(f"{name}: packed-cache tensors must be given and contiguous")
        _need_gpu(name, k_packed, v_packed, k_scale, k_zero, v_scale, v_zero)
        Hkv = k_packed.shape[1]
        per = 32 // bits
        a.k_packed, a.k_scale, a.k_zero = k_packed.data_ptr(), k_scale.data_ptr(), k_zero.data_ptr()
        a.v_packed, a.v_scale, a.v_zero = v_packed.data_ptr(), v_scale.data_ptr(), v_zero.data_ptr()
        a.pack_bits, a.group = int(bits), int(group_size)
        if k_scale.dtype not in (torch.float16, torch.float32) or any(
                t.dtype != k_scale.dtype for t in (k_zero, v_scale, v_zero)):
            raise ValueError(f"{name}: scale/zero must share one dtype, float16 or float32")
        a.meta_dtype = VQ_F16 if k_scale.dtype == torch.float16 else VQ_F32
        a.v_layout = _V_LAYOUT[v_layout]
        a.cap_tokens = k_packed.shape[2]
        vcap = v_packed.shape[2] * per if v_layout == "token" else v_packed.shape[2]
        if vcap != a.cap_tokens:
            raise ValueError(f"{name}: key capacity {a.cap_tokens} != value capacity {vcap}")
        keep += [k_packed, k_scale, k_zero, v_packed, v_scale, v_zero]
    if n_tail > 0:
        if k_tail is None or v_tail is None:
            raise ValueError(f"{name}: n_tail > 0 needs k_tail and v_tail")
        _need_gpu(name, k_tail, v_tail)
        if k_tail.dtype != v_tail.dtype:
            raise ValueError(f"{name}: k_tail and v_tail dtypes differ")
        if Hkv is not None and k_tail.shape[1] != Hkv:
            raise ValueError(f"{name}: tail has {k_tail.shape[1]} kv heads, packed cache has {Hkv}")
        Hkv = k_tail.shape[1]
        k_tail, kcap = _tail_layout(k_tail)
        v_tail, vcap = _tail_layout(v_tail)
        if kcap != vcap:
            k_tail, v_tail = k_tail.contiguous(), v_tail.contiguous()
            kcap = vcap = k_tail.shape[2]
        a.k_tail, a.v_tail = k_tail.data_ptr(), v_tail.data_ptr()
        a.tail_dtype = _ftag(name, k_tail)
        a.tail_cap = kcap
        keep += [k_tail, v_tail]
    if Hkv is None:
        raise ValueError(f"{name}: no key/value slots to attend to")
    a.n_packed, a.n_tail = int(n_packed), int(n_tail)
    return Hkv, k_tail


PREFILL_TILE_BYTES = 19456


def _check_tiles(name, tiles, rows, device):
    if (tiles.dtype != torch.uint8 or tiles.ndim != 3 or tiles.shape[0] != rows or tiles.shape[2] != PREFILL_TILE_BYTES
            or not tiles.is_contiguous() or tiles.device != device):
        raise ValueError(f"{name}: tiles must be a contiguous uint8 [{rows}, units, {PREFILL_TILE_BYTES}] tensor on the device")


def prefill_tiles_empty(B: int, Hkv: int, tokens: int, device) -> torch.Tensor:
    """Room for the tiles of ``tokens`` slots per (sequence, kv head)."""
    return torch.empty((B * Hkv, (int(tokens) + 31) // 32, PREFILL_TILE_BYTES), dtype=torch.uint8, device=device)


def kivi_prefill_tiles(tiles: torch.Tensor, first_unit: int, n_units: int, *, k_packed=None, k_scale=None, k_zero=None,
                       v_packed=None, v_scale=None, v_zero=None, n_packed: int = 0, bits: int = 4, group_size: int = 32,
                       v_layout: str = "token", k_tail=None, v_tail=None, n_tail: int = 0) -> None:
    """Write units ``first_unit .. first_unit + n_units - 1`` (32 slots each) of ``[quantised prefix | tail]`` into
    ``tiles`` in the form the prefill blocks of :func:`kivi_packed_attend` read from on-chip memory: packed slots
    reconstructed and rounded to fp16 (what the reference's cache holds, cache/kivi_cache.py:198-201), tail slots
    as they are.  One launch; a caller that appends chunk by chunk rewrites only what changed."""
    name = "kivi_prefill_tiles"
    a = AttendArgs()
    keep = [tiles]
    Hkv, _ = _cache_side(name, a, keep, k_packed, k_scale, k_zero, v_packed, v_scale, v_zero, n_packed, bits, group_size,
                         v_layout, k_tail, v_tail, n_tail)
    src = k_packed if n_packed > 0 else k_tail
    B, D = src.shape[0], (k_tail.shape[3] if k_tail is not None else 128)
    _check_tiles(name, tiles, B * Hkv, src.device)
    a.B, a.Hq, a.Hkv, a.Sq, a.D = B, Hkv, Hkv, 1, D
    a.kv_tiles, a.tile_cap = tiles.data_ptr(), tiles.shape[1]
    a.stream = _stream(src)
    _lib.check(_lib.load().vq_kivi_prefill_tiles(a, int(first_unit), int(n_units)))


def attend_fixed_order(enable: bool) -> bool:
    """Deal the decode kernel's token chunks to its waves in a fixed order (bit-identical results
    from run to run, a few percent slower) instead of on demand.  Returns the previous setting."""
    return bool(_lib.load().vq_kivi_attend_fixed_order(1 if enable else 0))


def kivi_packed_attend(q: torch.Tensor, *, k_packed=None, k_scale=None, k_zero=None, v_packed=None,
                       v_scale=None, v_zero=None, n_packed: int = 0, bits: int = 4, group_size: int = 32,
                       v_layout: str = "channel", k_tail=None, v_tail=None, n_tail: int = 0,
                       scale: float = 1.0, causal: bool = False, out_dtype: torch.dtype | None = None,
                       num_splits: int = 0, packed_lens: torch.Tensor | None = None,
                       tail_lens: torch.Tensor | None = None, k_new: torch.Tensor | None = None,
                       v_new: torch.Tensor | None = None, fixed_order: bool | None = None,
                       out: torch.Tensor | None = None, static_scratch: bool = False, sliding_window: int = 0,
                       sinks: tuple | None = None, tiles: torch.Tensor | None = None, tiles_stale_from: int | None = None,
                       _plan_out: dict | None = None, _single_launch: bool = True) -> torch.Tensor:
    """softmax(q k^T * scale) v over ``[quantised prefix | fp16 tail]``.

    q ``[B,Hq,Sq,D]``; packed buffers as :func:`kivi_quant_pack` lays them out
    with capacity read from their shapes, of which the first ``n_packed`` tokens
    are live; tails ``[B,Hkv,tail_cap,D]`` with ``n_tail`` live tokens.  GQA by
    repeat-interleave.  ``causal`` aligns queries to the end of the slots.
    ``fixed_order`` (this call only): True deals the decode kernel's token chunks to its waves
    in a fixed order (identical bits from run to run), False on demand, None takes the process
    default set by :func:`attend_fixed_order`.  ``out`` receives the result when given (a
    contiguous ``[B,Hq,Sq,D]`` tensor).  ``static_scratch=True`` goes through
    ``vq_kivi_attend_static``: the library's built-in scratch instead of a torch workspace, for
    callers that may not allocate (give ``out`` too; calls on one GPU must not overlap).
    ``sliding_window > 0``: a query sees only that many last slots up to its own position.
    ``sinks=(sink_k, sink_v, sink_pos)``: exact rows ``[B,Hkv,cap,D]`` standing for the packed
    positions ``sink_pos`` (int32 ``[B,cap]``, -1 for an unused slot) whose packed stand-ins carry
    zero value scale / zero: the stand-ins' softmax weights are taken out and the exact rows put in.
    ``tiles``: the slots once more as ready-made tiles (:func:`kivi_prefill_tiles`); prefill-sized calls copy
    them instead of reconstructing the prefix in every block (same bits), other calls ignore them.  With
    ``tiles_stale_from`` a call that reads the tiles first rewrites them from that unit on (None: they are up to
    date).  A causal call over plain keys and values with two dozen row tiles or more per kv head makes such tiles
    itself, in a scratch kept per device and stream (``tiles=False``: not even then)."""
    name = "kivi_packed_attend"
    if q.ndim != 4:
        raise ValueError(f"{name}: q must be 4D, got {tuple(q.shape)}")
    _need_gpu(name, q)
    B, Hq, Sq, D = q.shape
    q = q.contiguous()
    if out_dtype is None:
        out_dtype = q.dtype
    a = AttendArgs()
    if out is None:
        out = torch.empty((B, Hq, Sq, D), dtype=out_dtype, device=q.device)
    elif tuple(out.shape) != (B, Hq, Sq, D) or not out.is_contiguous() or out.device != q.device:
        raise ValueError(f"{name}: out must be a contiguous [{B}, {Hq}, {Sq}, {D}] tensor on the device of q")
    else:
        out_dtype = out.dtype
    a.q, a.out = q.data_ptr(), out.data_ptr()
    a.q_dtype, a.out_dtype = _ftag(name, q), _FLOAT_TAG[out_dtype]
    keep = [q, out]
    Hkv, k_tail = _cache_side(name, a, keep, k_packed, k_scale, k_zero, v_packed, v_scale, v_zero, n_packed, bits,
                              group_size, v_layout, k_tail, v_tail, n_tail)
    a.B, a.Hq, a.Hkv, a.Sq, a.D = B, Hq, Hkv, Sq, D
    a.scale, a.causal, a.num_splits = float(scale), int(bool(causal)), int(num_splits)
    a.sliding_window = int(sliding_window or 0)
    if sinks is not None:
        sk, sv, sp = sinks
        cap_s = sk.shape[2]
        if (sk.ndim != 4 or tuple(sv.shape) != tuple(sk.shape) or sk.shape[0] != B or sk.shape[3] != D or sv.dtype != sk.dtype
                or tuple(sp.shape) != (B, cap_s) or sp.dtype != torch.int32
                or not (sk.is_contiguous() and sv.is_contiguous() and sp.is_contiguous() and sk.is_cuda and sp.is_cuda)):
            raise ValueError(f"{name}: sinks must be (k [B,Hkv,cap,D], v like k, positions int32 [B,cap]), contiguous, on the device")
        a.sink_k, a.sink_v, a.sink_pos = sk.data_ptr(), sv.data_ptr(), sp.data_ptr()
        a.sink_cap, a.sink_dtype = int(cap_s), _FLOAT_TAG[sk.dtype]
        keep += [sk, sv, sp]
    if (tiles is None and n_packed == 0 and causal and D == 128 and Hq % Hkv == 0 and 1 <= Hq // Hkv <= 8
            and (Hq // Hkv) * Sq >= 24 * 256 and k_tail.dtype in (torch.float16, torch.bfloat16)
            and packed_lens is None and sinks is None and k_new is None and not static_scratch
            and B * Hkv * -(-int(n_tail) // 32) * PREFILL_TILE_BYTES <= _TILE_SCRATCH_MAX):
        # Plain keys and values under so many row tiles that every unit is read two dozen times or more: written
        # once as tiles (a scratch kept per device and stream, 608 B per slot and kv head) they are copied into
        # on-chip memory instead of being converted and transposed by every block that reads them; same bits.
        tiles, tiles_stale_from = _tile_scratch(q.device, B * Hkv, -(-int(n_tail) // 32)), 0
    if tiles is False:   # no tiles, not even the scratch above
        tiles = None
    if tiles is not None:
        _check_tiles(name, tiles, B * Hkv, q.device)
        a.kv_tiles, a.tile_cap = tiles.data_ptr(), tiles.shape[1]
        a.tiles_stale_from = tiles.shape[1] if tiles_stale_from is None else int(tiles_stale_from)
        keep.append(tiles)
    a.fixed_order = 0 if fixed_order is None else (int(fixed_order) if fixed_order is not True and fixed_order is not False and int(fixed_order) > 2 else (1 if fixed_order else 2))
    if (packed_lens is None) != (tail_lens is None):
        raise ValueError(f"{name}: packed_lens and tail_lens go together")
    if packed_lens is not None:
        # sequences of different lengths: int32 [B] on the device; n_packed / n_tail are the maxima
        lens = []
        for nm, t in (("packed_lens", packed_lens), ("tail_lens", tail_lens)):
            if t.shape != (B,) or not t.is_cuda:
                raise ValueError(f"{name}: {nm} must be a device tensor of shape [{B}]")
            lens.append(t.to(torch.int32).contiguous())
        a.packed_lens, a.tail_lens = lens[0].data_ptr(), lens[1].data_ptr()
    if (k_new is None) != (v_new is None):
        raise ValueError(f"{name}: k_new and v_new go together")
    if k_new is not None:
        # the newest token's rows [B, Hkv, 1, D]: stored as the last tail row and attended in the same launch
        for nm, t in (("k_new", k_new), ("v_new", v_new)):
            if k_tail is None or t.dtype != k_tail.dtype or t.numel() != B * Hkv * D or not t.is_contiguous() or not t.is_cuda:
                raise ValueError(f"{name}: {nm} must be a contiguous [{B}, {Hkv}, 1, {D}] device tensor in the dtype of the tail")
        a.k_new, a.v_new = k_new.data_ptr(), v_new.data_ptr()
    lib = _lib.load()
    if _plan_out is not None:
        import ctypes
        pth, npt = ctypes.c_int(0), ctypes.c_int(0)
        _lib.check(lib.vq_kivi_attend_plan(a, ctypes.byref(pth), ctypes.byref(npt)))
        _plan_out["path"], _plan_out["nparts"] = pth.value, npt.value
    a.stream = _stream(q)
    if static_scratch:
        _lib.check(lib.vq_kivi_attend_static(a))
        return out
    need = lib.vq_kivi_attend_workspace(a)
    ws = _workspace(q.device, need)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    a.sync_counters = _counters(q.device).data_ptr() if _single_launch else None
    _lib.check(lib.vq_kivi_attend(a))
    return out


def _check_fused_args(name, q, k_codes, v_codes, ndim):
    if q.ndim != ndim:
        raise ValueError(f"{name}: q must be {ndim}D, got {tuple(q.shape)}")
    if k_codes.ndim != ndim or v_codes.ndim != ndim:
        raise ValueError(f"{name}: k_codes and v_codes must be {ndim}D, "
                         f"got k_codes={tuple(k_codes.shape)}, v_codes={tuple(v_codes.shape)}")


def scalar_fused_decode_attend(q, k_codes, k_scale, k_zero, v_codes, v_scale, v_zero, group_size: int,
                               scale: float, nsg: int | None = None) -> torch.Tensor:
    """Fused group-affine decode + attention over uint8 codes and fp32 scale/zero;
    drop-in for ``scalar_fused_decode_attend``
    (veloxquant_mlx/metal/_scalar_attend.py:370-493).  ``nsg`` (SIMD groups per
    threadgroup on Apple GPUs) is validated for range and otherwise unused: the
    token axis is split across workgroups instead."""
    name = "scalar_fused_decode_attend"
    _check_fused_args(name, q, k_codes, v_codes, 4)
    B, H, S_q, D = q.shape
    if D > 256:
        raise ValueError(f"{name}: D={D} must be <= 256")
    if nsg is not None and not (1 <= nsg <= 32):
        raise ValueError(f"{name}: nsg={nsg} must be in 1..32")
    Bk, H_kv, S_kv, Dk = k_codes.shape
    if Bk != B:
        raise ValueError(f"{name}: batch mismatch: q B={B} vs k_codes B={Bk}")
    if Dk != D:
        raise ValueError(f"{name}: head_dim mismatch: q D={D} vs k_codes D={Dk}")
    if v_codes.shape[1] != H_kv:
        raise ValueError(f"{name}: k_codes H_kv={H_kv} vs v_codes H_kv={v_codes.shape[1]} mismatch")
    if H % H_kv != 0:
        raise ValueError(f"{name}: H_q={H} must be a multiple of H_kv={H_kv} (k_codes.shape[1]) "
                         "for GQA head-packing")
    if H // H_kv > _MAX_HEADS_PER_KV:
        raise ValueError(f"{name}: heads_per_kv={H // H_kv} exceeds the supported maximum of {_MAX_HEADS_PER_KV}")
    if D % 4:
        raise ValueError(f"{name}: D={D} must be a multiple of 4")
    _need_gpu(name, q, k_codes, v_codes)
    kw = _bytes_as_words(k_codes)
    vw = _bytes_as_words(v_codes)
    return kivi_packed_attend(
        q.to(torch.float16), k_packed=kw, k_scale=k_scale.float().contiguous(), k_zero=k_zero.float().contiguous(),
        v_packed=vw, v_scale=v_scale.float().contiguous(), v_zero=v_zero.float().contiguous(),
        n_packed=S_kv, bits=8, group_size=group_size, scale=scale, causal=False, out_dtype=torch.float16)


def scalar_fused_decode_attend_batched(q, k_codes, k_scale, k_zero, v_codes, v_scale, v_zero, group_size: int,
                                       scale: float, nsg: int | None = None) -> torch.Tensor:
    """Layer-batched form: every tensor carries a leading ``NL`` axis, which folds
    into the batch axis (veloxquant_mlx/metal/_scalar_attend.py:496-647)."""
    name = "scalar_fused_decode_attend_batched"
    if q.ndim != 5:
        raise ValueError(f"{name}: q must be 5D [NL,B,H,S_q,D], got {tuple(q.shape)}")
    _check_fused_args(name, q, k_codes, v_codes, 5)
    NL, B = q.shape[0], q.shape[1]
    if NL < 1:
        raise ValueError(f"{name}: NL={NL} must be >= 1")
    if k_codes.shape[0] != NL:
        raise ValueError(f"{name}: NL mismatch: q NL={NL} vs k_codes NL={k_codes.shape[0]}")
    if k_codes.shape[1] != B:
        raise ValueError(f"{name}: batch mismatch: q B={B} vs k_codes B={k_codes.shape[1]}")
    if v_codes.shape != k_codes.shape:
        raise ValueError(f"{name}: k_codes shape={tuple(k_codes.shape)} vs v_codes shape={tuple(v_codes.shape)} mismatch")
    H_kv = k_codes.shape[2]
    for nm, arr in (("k_scale", k_scale), ("k_zero", k_zero), ("v_scale", v_scale), ("v_zero", v_zero)):
        if arr.ndim != 5 or arr.shape[0] != NL or arr.shape[1] != B or arr.shape[2] != H_kv:
            raise ValueError(f"{name}: {nm} shape={tuple(arr.shape)} must be 5D with leading "
                             f"[NL={NL}, B={B}, H_kv={H_kv}, ...]")
    fold = lambda t: t.reshape((NL * B,) + tuple(t.shape[2:]))
    out = scalar_fused_decode_attend(fold(q), fold(k_codes), fold(k_scale), fold(k_zero), fold(v_codes),
                                     fold(v_scale), fold(v_zero), group_size, scale, nsg)
    return out.view((NL, B) + tuple(out.shape[1:]))


def scalar_predecoded_attend(q, k_hat, v_hat, scale: float, nsg: int | None = None) -> torch.Tensor:
    """Decode attention over already reconstructed fp16 K/V
    (veloxquant_mlx/metal/_scalar_attend.py:702-779)."""
    name = "scalar_predecoded_attend"
    if q.ndim != 4:
        raise ValueError(f"{name}: q must be 4D, got {tuple(q.shape)}")
    if k_hat.ndim != 4 or v_hat.ndim != 4:
        raise ValueError(f"{name}: k_hat and v_hat must be 4D, got k_hat={tuple(k_hat.shape)}, v_hat={tuple(v_hat.shape)}")
    B, H, S_q, D = q.shape
    if D > 256:
        raise ValueError(f"{name}: D={D} must be <= 256")
    if nsg is not None and not (1 <= nsg <= 32):
        raise ValueError(f"{name}: nsg={nsg} must be in 1..32")
    if k_hat.shape[0] != B:
        raise ValueError(f"{name}: batch mismatch: q B={B} vs k_hat B={k_hat.shape[0]}")
    if k_hat.shape[3] != D:
        raise ValueError(f"{name}: head_dim mismatch: q D={D} vs k_hat D={k_hat.shape[3]}")
    if v_hat.shape != k_hat.shape:
        raise ValueError(f"{name}: k_hat shape={tuple(k_hat.shape)} vs v_hat shape={tuple(v_hat.shape)} mismatch")
    if H % k_hat.shape[1] != 0:
        raise ValueError(f"{name}: H_q={H} must be a multiple of H_kv={k_hat.shape[1]} (k_hat.shape[1])")
    return kivi_packed_attend(q.to(torch.float16), k_tail=k_hat.to(torch.float16).contiguous(),
                              v_tail=v_hat.to(torch.float16).contiguous(), n_tail=k_hat.shape[2], scale=scale,
                              causal=False, out_dtype=torch.float16)


def flash_prefill_attend(q, k, v, scale) -> torch.Tensor:
    """Causal, tail-aligned attention over plain fp16 K/V
    (veloxquant_mlx/metal/_flash_prefill.py:171-237); GQA is accepted as well."""
    name = "flash_prefill_attend"
    if q.ndim != 4:
        raise ValueError(f"{name}: q must be 4D, got {tuple(q.shape)}")
    B, H, S_q, D = q.shape
    if D % 8 != 0:
        raise ValueError(f"{name}: D={D} must be divisible by 8")
    if k.ndim != 4 or k.shape[0] != B or k.shape[3] != D or H % k.shape[1] != 0:
        raise ValueError(f"{name}: k must be [B, H, S_kv, {D}], got {tuple(k.shape)}")
    S_kv = k.shape[2]
    if tuple(v.shape) != tuple(k.shape):
        raise ValueError(f"{name}: v must be {tuple(k.shape)}, got {tuple(v.shape)}")
    if S_q > S_kv:
        raise ValueError(f"{name}: S_q={S_q} exceeds S_kv={S_kv}; queries align to the tail of the KV cache, "
                         "so every query needs a slot to attend to")
    s = float(scale.reshape(-1)[0].item()) if isinstance(scale, torch.Tensor) else float(scale)
    return kivi_packed_attend(q.to(torch.float16), k_tail=k.to(torch.float16).contiguous(),
                              v_tail=v.to(torch.float16).contiguous(), n_tail=S_kv, scale=s, causal=True,
                              out_dtype=torch.float16)


__all__ = [
    "hip_available", "release_tile_scratch", "kivi_group_quant_dequant", "kivi_group_quant_dequant_rows", "kivi_group_quant_dequant_mixed", "kivi_group_quant_dequant_grouplevels", "channel_variance", "channel_hi_mask", "row_norms", "zip_route", "kivi_quant_pack", "kivi_quant_pack_kv", "kivi_quant_codes", "kivi_dequant", "kivi_prefill_tiles", "prefill_tiles_empty",
    "scalar_decode_once", "pack_indices", "unpack_indices", "turboquant_bit_pack", "turboquant_bit_unpack",
    "vecinfer_quantize_metal", "vecinfer_dequant_metal", "vecinfer_quantize_hip", "vecinfer_dequant_hip",
    "vecinfer_encode_decode_metal", "vecinfer_encode_decode_simple_metal", "metal_fused_sdpa", "vecinfer_fused_sdpa",
    "kv_tail_append", "kivi_cache_append", "attend_fixed_order",
    "kivi_packed_attend", "scalar_fused_decode_attend", "scalar_fused_decode_attend_batched",
    "scalar_predecoded_attend", "flash_prefill_attend",
]


# ---------------------------------------------------------------------------
# attention over VecInfer indices
# ---------------------------------------------------------------------------

def metal_fused_sdpa(q_tilde: torch.Tensor, k_indices: torch.Tensor, k_codebook: torch.Tensor,
                     v_indices: torch.Tensor, v_codebook: torch.Tensor, scale: float, *, causal: bool = True,
                     sliding_window: int = 0, out_dtype: torch.dtype | None = None,
                     n_tokens: int | None = None, num_splits: int = 0) -> torch.Tensor:
    """``softmax((q_tilde @ K_tilde^T) * scale) @ V_hat`` from codebook indices, without
    materialising ``K_tilde`` or ``V_hat``.  Same contract as ``metal_fused_sdpa``
    (veloxquant_mlx/metal/fused_sdpa.py:200-299): ``q_tilde [B,H_q,S_q,D]`` already passed through
    ``apply_dual_transform_queries``; ``k_indices, v_indices [B,H_kv,S_kv,n_sub]`` (uint8 or
    32-bit); codebooks ``[n_centroids, sub_dim]``; queries align to the tail of ``S_kv``;
    ``sliding_window > 0`` keeps only that many last keys before each query position.
    ``n_tokens`` (this build) attends over the first ``n_tokens`` rows of longer index buffers."""
    name = "fused_sdpa"
    if q_tilde.ndim != 4 or k_indices.ndim != 4 or v_indices.ndim != 4:
        raise ValueError(f"{name}: q_tilde and the index tensors must be 4D")
    if k_codebook.ndim != 2 or v_codebook.ndim != 2:
        raise ValueError(f"{name}: codebooks must be 2D [n_centroids, sub_dim]")
    _need_gpu(name, q_tilde, k_indices, v_indices, k_codebook, v_codebook)
    B, H_q, S_q, D = q_tilde.shape
    _, H_kv, cap, n_sub = k_indices.shape
    n_centroids, sub_dim = k_codebook.shape
    n_sub_v = v_indices.shape[3]
    n_centroids_v, sub_dim_v = v_codebook.shape
    if n_sub * sub_dim != D:
        raise ValueError(f"{name}: D={D} must equal n_sub*sub_dim={n_sub * sub_dim}.")
    if n_sub_v * sub_dim_v != D:
        raise ValueError(f"{name}: D={D} must equal n_sub_v*sub_dim_v={n_sub_v * sub_dim_v}.")
    if n_centroids != n_centroids_v:
        raise ValueError(f"{name}: key and value codebooks must currently have the same n_centroids "
                         f"(got {n_centroids} vs {n_centroids_v}).")
    if H_q % H_kv != 0:
        raise ValueError(f"{name}: H_q={H_q} must be a multiple of H_kv={H_kv}.")
    if v_indices.shape[:3] != k_indices.shape[:3] or k_indices.shape[0] != B:
        raise ValueError(f"{name}: key and value indices must share [B,H_kv,S_kv]")
    S_kv = cap if n_tokens is None else int(n_tokens)
    if not 1 <= S_kv <= cap:
        raise ValueError(f"{name}: n_tokens={S_kv} outside 1..{cap}")
    if out_dtype is None:
        out_dtype = q_tilde.dtype
    if q_tilde.dtype not in _FLOAT_TAG:
        q_tilde = q_tilde.float()
    if out_dtype not in _FLOAT_TAG:
        raise ValueError(f"{name}: unsupported out dtype {out_dtype}")

    # the byte-index kernel is several times faster than the one for 32-bit indices: with at most
    # 256 centroids wider indices are narrowed first (one extra pass over them)
    byte_kernel = (n_centroids <= 256 and n_sub == n_sub_v and n_sub in (4, 8, 16, 32) and sub_dim % 4 == 0)

    def idx(t):
        if t.dtype != torch.uint8:
            t = t.to(torch.uint8 if byte_kernel else torch.int32)
        return t.contiguous()
    ki, vi = idx(k_indices), idx(v_indices)
    if ki.dtype != vi.dtype:
        ki, vi = ki.to(torch.int32), vi.to(torch.int32)
    cb_dtype = k_codebook.dtype if k_codebook.dtype in _FLOAT_TAG and k_codebook.dtype == v_codebook.dtype else torch.float32
    kcb, vcb = k_codebook.to(cb_dtype).contiguous(), v_codebook.to(cb_dtype).contiguous()
    q = q_tilde.contiguous()
    out = torch.empty((B, H_q, S_q, D), dtype=out_dtype, device=q.device)
    a = LutAttendArgs(q=q.data_ptr(), out=out.data_ptr(), q_dtype=_FLOAT_TAG[q.dtype], out_dtype=_FLOAT_TAG[out_dtype],
                      B=B, Hq=H_q, Hkv=H_kv, Sq=S_q, D=D, k_idx=ki.data_ptr(), v_idx=vi.data_ptr(),
                      idx_dtype=VQ_U8 if ki.dtype == torch.uint8 else VQ_I32, n_tokens=S_kv, cap_tokens=cap,
                      k_codebook=kcb.data_ptr(), v_codebook=vcb.data_ptr(), cb_dtype=_FLOAT_TAG[cb_dtype],
                      n_centroids=n_centroids, k_sub_dim=sub_dim, v_sub_dim=sub_dim_v, scale=float(scale),
                      causal=1 if causal else 0, sliding_window=int(sliding_window or 0), num_splits=int(num_splits))
    lib = _lib.load()
    need = lib.vq_vecinfer_attend_workspace(C.byref(a))
    if need == 0:
        _lib.check(lib.vq_vecinfer_attend(C.byref(a)))   # raises with the validation message
    ws = _workspace(q.device, need)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    a.stream = _stream(q)
    _lib.check(lib.vq_vecinfer_attend(C.byref(a)))
    return out


vecinfer_fused_sdpa = metal_fused_sdpa
