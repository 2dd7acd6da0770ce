"""ctypes binding of ``libveloxquant_hip.so`` (the C ABI in ``include/veloxquant_hip.h``).

The library is the only compute backend: if it cannot be loaded every kernel
call raises ``RuntimeError`` -- there is no CPU or eager-torch fallback.
"""

from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("VELOXQUANT_HIP_LIB", os.path.join(_HERE, "libveloxquant_hip.so"))

# element tags (include/veloxquant_hip.h)
VQ_F16, VQ_BF16, VQ_F32, VQ_U8, VQ_I32, VQ_U32 = 0, 1, 2, 3, 4, 5
VQ_AXIS_TOKEN, VQ_AXIS_CHANNEL = 0, 1
VQ_V_CHANNEL_PACKED, VQ_V_TOKEN_PACKED = 0, 1
VQ_ERR_INVALID, VQ_ERR_UNSUPPORTED, VQ_ERR_WORKSPACE, VQ_ERR_HIP = -1, -2, -3, -4

i64, i32, f32, vp, sz = C.c_int64, C.c_int, C.c_float, C.c_void_p, C.c_size_t


class AttendArgs(C.Structure):
    """Mirror of ``vq_attend_args``."""

    _fields_ = [
        ("q", vp), ("out", vp), ("q_dtype", i32), ("out_dtype", i32),
        ("B", i64), ("Hq", i64), ("Hkv", i64), ("Sq", i64), ("D", i64),
        ("k_packed", vp), ("k_scale", vp), ("k_zero", vp),
        ("v_packed", vp), ("v_scale", vp), ("v_zero", vp),
        ("pack_bits", i32), ("group", i32), ("meta_dtype", i32), ("v_layout", i32),
        ("n_packed", i64), ("cap_tokens", i64),
        ("k_tail", vp), ("v_tail", vp), ("tail_dtype", i32),
        ("n_tail", i64), ("tail_cap", i64),
        ("scale", f32), ("causal", i32), ("num_splits", i32),
        ("workspace", vp), ("workspace_bytes", sz), ("stream", vp),
        ("sync_counters", vp),
        ("packed_lens", vp), ("tail_lens", vp),
        ("k_new", vp), ("v_new", vp),
        ("fixed_order", C.c_int32),
        ("sliding_window", C.c_int64),
        ("sink_k", C.c_void_p), ("sink_v", C.c_void_p), ("sink_pos", C.c_void_p),
        ("sink_cap", C.c_int64), ("sink_dtype", C.c_int32),
        ("kv_tiles", C.c_void_p), ("tile_cap", C.c_int64), ("tiles_stale_from", C.c_int64),
    ]


class LutAttendArgs(C.Structure):
    """Mirror of ``vq_lut_attend_args``."""

    _fields_ = [
        ("q", vp), ("out", vp), ("q_dtype", i32), ("out_dtype", i32),
        ("B", i64), ("Hq", i64), ("Hkv", i64), ("Sq", i64), ("D", i64),
        ("k_idx", vp), ("v_idx", vp), ("idx_dtype", i32),
        ("n_tokens", i64), ("cap_tokens", i64),
        ("k_codebook", vp), ("v_codebook", vp), ("cb_dtype", i32),
        ("n_centroids", i32), ("k_sub_dim", i32), ("v_sub_dim", i32),
        ("scale", f32), ("causal", i32), ("sliding_window", i64), ("num_splits", i32),
        ("workspace", vp), ("workspace_bytes", sz), ("stream", vp),
    ]


class KiviAppendArgs(C.Structure):
    """Mirror of ``vq_kivi_append_args``."""

    _fields_ = [
        ("k_new", vp), ("v_new", vp), ("k_strides", i64 * 3), ("v_strides", i64 * 3),
        ("dtype", i32),
        ("B", i64), ("H", i64), ("S", i64), ("D", i64),
        ("k_tail", vp), ("v_tail", vp), ("tail_cap", i64), ("n_tail", i64),
        ("n_flush", i64),
        ("k_packed", vp), ("k_scale", vp), ("k_zero", vp), ("v_packed", vp), ("v_scale", vp), ("v_zero", vp),
        ("meta_dtype", i32),
        ("cap_tokens", i64), ("dst_tok0", i64),
        ("group", i32), ("levels", i32), ("eps", f32), ("pack_bits", i32), ("v_layout", i32),
        ("k_spare", vp), ("v_spare", vp), ("spare_cap", i64),
    ]


_SIGNATURES = {
    "vq_abi_version": (i32, []),
    "vq_last_error": (i32, [C.c_char_p, sz]),
    "vq_device_count": (i32, []),
    "vq_kivi_quant_dequant": (i32, [vp, vp, i32, i64, i64, i64, i32, i32, i32, f32, vp]),
    "vq_skvq_clipped_roundtrip": (i32, [vp, vp, i32, i64, i64, i64, i64, i64, i64, vp, vp, i32, i32, C.POINTER(f32), i32, vp]),
    "vq_kivi_quant_pack": (i32, [vp, i32, i64, i64, i64, i64, i32, i32, i32, f32, i32, i32, vp, vp, vp, i32, i64, i64, vp]),
    "vq_zip_route": (i32, [vp, i64, i64, i64, vp, vp]),
    "vq_row_norms": (i32, [vp, i32, i64, i64, vp, vp]),
    "vq_kivi_quant_dequant_mixed": (i32, [vp, vp, i32, i64, i64, i64, i32, i32, i32, vp, f32, vp]),
    "vq_channel_moments": (i32, [vp, i32, i64, i64, i64, i64, vp, i32, vp]),
    "vq_channel_variance": (i32, [vp, i64, i32, i64, i64, vp, vp]),
    "vq_channel_hi_mask": (i32, [vp, i64, i64, i64, vp, vp]),
    "vq_kivi_quant_dequant_grouplevels": (i32, [vp, vp, i32, i64, i64, i64, i32, vp, f32, vp]),
    "vq_kivi_quant_dequant_rows": (i32, [vp, vp, i32, i64, i64, i64, i64, vp, i64, i32, i32, f32, vp]),
    "vq_kivi_quant_pack_kv": (i32, [vp, vp, i32, i64, i64, i64, i64, i32, i32, f32, i32, i32, vp, vp, vp, vp, vp, vp, i32, i64, i64, vp]),
    "vq_kivi_dequant": (i32, [vp, vp, vp, i32, i64, i64, i64, i32, i32, i32, i32, i64, i64, vp, i32, vp]),
    "vq_kv_tail_append": (i32, [vp, vp, C.POINTER(i64), C.POINTER(i64), vp, vp, i32, i64, i64, i64, i64, i64, i64, vp]),
    "vq_kivi_cache_append": (i32, [C.POINTER(KiviAppendArgs), vp]),
    "vq_pack_words": (i32, [vp, i64, i64, i32, vp, vp]),
    "vq_unpack_words": (i32, [vp, i64, i64, i32, vp, vp]),
    "vq_bit_pack": (i32, [vp, i64, i32, vp, vp]),
    "vq_bit_unpack": (i32, [vp, i64, i32, vp, vp]),
    "vq_vecinfer_assign": (i32, [vp, i32, i64, vp, i32, i32, i32, vp, i32, vp]),
    "vq_vecinfer_dequant": (i32, [vp, i32, i64, vp, i32, i32, i32, vp, i32, vp]),
    "vq_vecinfer_encode_keys": (i32, [vp, i32, i64, i64, i64, i64, vp, i32, f32, vp, i32, i32, i32, vp, i32, vp, vp, vp]),
    "vq_kivi_attend_fixed_order": (i32, [i32]),
    "vq_kivi_attend_workspace": (sz, [C.POINTER(AttendArgs)]),
    "vq_kivi_attend_plan": (i32, [C.POINTER(AttendArgs), C.POINTER(i32), C.POINTER(i32)]),
    "vq_kivi_attend": (i32, [C.POINTER(AttendArgs)]),
    "vq_kivi_attend_static": (i32, [C.POINTER(AttendArgs)]),
    "vq_kivi_prefill_tiles": (i32, [C.POINTER(AttendArgs), i64, i64]),
    "vq_vecinfer_attend_workspace": (sz, [C.POINTER(LutAttendArgs)]),
    "vq_vecinfer_attend": (i32, [C.POINTER(LutAttendArgs)]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None
_load_error: str | None = None


def load():
    """Return the loaded library or raise ``RuntimeError``."""
    global _lib, _load_error
    if _lib is not None:
        return _lib
    if _load_error is None:
        try:
            lib = C.CDLL(LIB_PATH)
            for name, (res, args) in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = res
                fn.argtypes = args
            _lib = lib
            return _lib
        except (OSError, AttributeError) as e:  # missing file or symbol
            _load_error = f"{type(e).__name__}: {e}"
    raise RuntimeError(
        f"veloxquant_mlx_amd: the HIP kernel library could not be loaded from {LIB_PATH} "
        f"({_load_error}). Build it with `python -m veloxquant_mlx_amd.build`; there is no fallback path."
    )


def library_present() -> bool:
    try:
        load()
        return True
    except RuntimeError:
        return False


def last_error() -> str:
    buf = C.create_string_buffer(512)
    load().vq_last_error(buf, 512)
    return buf.value.decode("utf-8", "replace")


def check(rc: int) -> None:
    """Map a status code to the exception type the reference wrappers raise."""
    if rc == 0:
        return
    msg = last_error()
    if rc == VQ_ERR_INVALID or rc == VQ_ERR_UNSUPPORTED:
        raise ValueError(msg)
    raise RuntimeError(msg)
