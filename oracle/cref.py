"""ctypes front end of the plain-C oracle (oracle/c/kv_oracle.c).

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).
"""

from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libkv_oracle.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-s", "-C", os.path.join(_HERE, "c")], check=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
    return _lib


def _p(a, t):
    return a.ctypes.data_as(C.POINTER(t))


def group_quant(x, axis: int, group: int, levels: int, eps: float = 1e-8):
    x = np.ascontiguousarray(x, dtype=np.float32)
    S, D = x.shape[-2], x.shape[-1]
    BH = x.size // (S * D)
    lead = x.shape[:-2]
    codes = np.empty(x.shape, np.uint8)
    if axis == -2:
        mshape = lead + ((S + group - 1) // group, D)
    else:
        mshape = lead + (S, (D + group - 1) // group)
    scale = np.empty(mshape, np.float32)
    zero = np.empty(mshape, np.float32)
    rc = lib().kvo_group_quant(_p(x, C.c_float), C.c_int64(BH), C.c_int64(S), C.c_int64(D),
                               0 if axis == -2 else 1, group, levels, C.c_float(eps),
                               _p(codes, C.c_uint8), _p(scale, C.c_float), _p(zero, C.c_float))
    assert rc == 0
    return codes, scale, zero


def pack_words(codes, bits: int):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    D = codes.shape[-1]
    per = 32 // bits
    W = (D + per - 1) // per
    out = np.empty(codes.shape[:-1] + (W,), np.uint32)
    rc = lib().kvo_pack_words(_p(codes, C.c_uint8), C.c_int64(codes.size // D), C.c_int64(D), bits,
                              _p(out, C.c_uint32))
    assert rc == 0
    return out


def vq_assign(x, codebook, sub_dim: int):
    x = np.asarray(x)
    flat = np.ascontiguousarray(x.reshape(-1, sub_dim), dtype=np.float32)
    cb = np.ascontiguousarray(codebook, dtype=np.float32)
    out = np.empty(flat.shape[0], np.int32)
    rc = lib().kvo_vq_assign(_p(flat, C.c_float), C.c_int64(flat.shape[0]), _p(cb, C.c_float),
                             cb.shape[0], sub_dim, _p(out, C.c_int32))
    assert rc == 0
    return out.reshape(x.shape[:-1] + (x.shape[-1] // sub_dim,))


def attend(q, kc, ks, kz, vc, vs, vz, group: int, scale: float, k_tail=None, v_tail=None,
           causal: bool = False):
    q = np.ascontiguousarray(q, dtype=np.float32)
    B, Hq, Sq, D = q.shape
    kc = np.ascontiguousarray(kc, dtype=np.uint8)
    vc = np.ascontiguousarray(vc, dtype=np.uint8)
    Hkv, S = kc.shape[1], kc.shape[2]
    ks, kz, vs, vz = (np.ascontiguousarray(a, dtype=np.float32) for a in (ks, kz, vs, vz))
    if k_tail is None:
        k_tail = np.zeros((B, Hkv, 0, D), np.float32)
        v_tail = np.zeros((B, Hkv, 0, D), np.float32)
    k_tail = np.ascontiguousarray(k_tail, dtype=np.float32)
    v_tail = np.ascontiguousarray(v_tail, dtype=np.float32)
    T = k_tail.shape[2]
    out = np.empty(q.shape, np.float32)
    rc = lib().kvo_attend(_p(q, C.c_float), C.c_int64(B), C.c_int64(Hq), C.c_int64(Sq), C.c_int64(D),
                          _p(kc, C.c_uint8), _p(ks, C.c_float), _p(kz, C.c_float),
                          _p(vc, C.c_uint8), _p(vs, C.c_float), _p(vz, C.c_float),
                          C.c_int64(Hkv), C.c_int64(S), group,
                          _p(k_tail, C.c_float), _p(v_tail, C.c_float), C.c_int64(T),
                          C.c_float(scale), int(causal), _p(out, C.c_float))
    assert rc == 0
    return out
