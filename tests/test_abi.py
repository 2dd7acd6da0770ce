"""The C-ABI library loads and exports every symbol the header declares
(no compute calls: this runs without a GPU)."""

import ctypes
import os
import re

import pytest

from veloxquant_mlx_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "veloxquant_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vq_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared() == sorted(_lib.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} is missing: run `python -m veloxquant_mlx_amd.build`")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), name
    assert lib.vq_abi_version() == 16


def test_attend_args_struct_matches_header_field_order():
    text = open(os.path.join(ROOT, "include", "veloxquant_hip.h")).read()
    body = text[text.index("typedef struct vq_attend_args {"):text.index("} vq_attend_args;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.split("{")[-1].strip()
        if not decl:
            continue
        for part in decl.split(","):
            names.append(re.findall(r"[A-Za-z_][A-Za-z0-9_]*", part)[-1])
    assert names == [f[0] for f in _lib.AttendArgs._fields_]


def test_argument_errors_surface_without_a_gpu():
    lib = _lib.load()
    # invalid axis is rejected before any device work
    rc = lib.vq_kivi_quant_dequant(None, None, 0, 1, 4, 8, 7, 32, 3, 1e-8, None)
    assert rc == _lib.VQ_ERR_INVALID
    assert "axis must be -1 or -2" in _lib.last_error()
    with pytest.raises(ValueError, match="axis must be -1 or -2"):
        _lib.check(rc)
    a = _lib.AttendArgs()
    a.B, a.Hq, a.Hkv, a.Sq, a.D = 1, 6, 4, 1, 128
    a.n_tail = 4
    assert lib.vq_kivi_attend(a) == _lib.VQ_ERR_INVALID
    assert "multiple of H_kv" in _lib.last_error()
    # ready-made tiles: a missing or short buffer is refused by the writer and by the attention call
    t = _lib.AttendArgs()
    t.B, t.Hq, t.Hkv, t.Sq, t.D = 1, 4, 4, 1, 128
    t.n_tail = 64
    assert lib.vq_kivi_prefill_tiles(t, 0, 2) == _lib.VQ_ERR_INVALID
    assert "kv_tiles must be given" in _lib.last_error()
    t.kv_tiles, t.tile_cap = 4096, 1
    assert lib.vq_kivi_prefill_tiles(t, 0, 2) == _lib.VQ_ERR_INVALID
    assert "do not lie inside" in _lib.last_error()
    assert lib.vq_kivi_attend(t) == _lib.VQ_ERR_INVALID
    assert "room for all 64 slots" in _lib.last_error()

