"""HIP KIVI quantise / pack / dequant kernels against the CPU oracle: bit-exact.

Cases restate the reference's kernel tests
(veloxquant_mlx/tests/metal/test_kivi_quant.py:76-159) and add the packed forms."""

import numpy as np
import pytest
import torch

from oracle import kivi as ok
from tests._gpu import gpu, host, outlier_kv, require_gpu, to_dev, words
from veloxquant_mlx_amd import kernels as K

pytestmark = gpu


def _bf16_cast(a):
    return torch.from_numpy(a).to(torch.bfloat16).float().numpy()


def _roundtrip_exact(x_np, axis, b=2, g=32, dtype=None):
    require_gpu()
    x = to_dev(x_np, dtype)
    levels = (1 << b) - 1
    got = K.kivi_group_quant_dequant(x, axis=axis, group_size=g, levels=levels, eps=1e-8)
    assert got.dtype == x.dtype and got.shape == x.shape
    src = host(x)
    if x.dtype == torch.bfloat16:
        ref = ok.quant_dequant_along(src, axis, g, levels, cast=_bf16_cast)
    else:
        ref = ok.quant_dequant_along(src, axis, g, levels)
    np.testing.assert_array_equal(host(got), ref)


@pytest.mark.parametrize("axis", [-2, -1])
@pytest.mark.parametrize("b", [1, 2, 4, 8])
@pytest.mark.parametrize("g", [4, 32, 128])
def test_bit_exact_across_bits_and_group_sizes(axis, b, g):
    rng = np.random.default_rng(b * 100 + g)
    _roundtrip_exact(rng.standard_normal((1, 4, 64, 128)).astype(np.float16), axis, b, g)


@pytest.mark.parametrize("axis", [-2, -1])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
def test_bit_exact_across_dtypes(axis, dtype):
    rng = np.random.default_rng(5)
    _roundtrip_exact(rng.standard_normal((1, 4, 96, 128)).astype(np.float32), axis, dtype=dtype)


@pytest.mark.parametrize("axis", [-2, -1])
@pytest.mark.parametrize("shape", [(1, 8, 32, 128), (2, 2, 33, 64), (1, 1, 7, 16), (3, 1, 200, 128), (1, 2, 70, 256)])
def test_bit_exact_across_shapes(axis, shape):
    rng = np.random.default_rng(sum(shape))
    _roundtrip_exact(rng.standard_normal(shape).astype(np.float16), axis)


@pytest.mark.parametrize("axis", [-2, -1])
def test_ragged_group_uses_edge_replication_padding(axis):
    rng = np.random.default_rng(11)
    _roundtrip_exact((rng.standard_normal((1, 2, 50, 96)) + 8.0).astype(np.float16), axis)
    _roundtrip_exact((rng.standard_normal((1, 2, 50, 128)) + 8.0).astype(np.float16), axis)


@pytest.mark.parametrize("axis", [-2, -1])
def test_exact_half_codes_round_half_to_even(axis):
    _roundtrip_exact(np.tile(np.array([0, 1, 2, 3], np.float16), (1, 2, 64, 24)), axis)
    x = np.tile(np.array([0, 1, 2, 3, 4, 5, 6, 6], np.float16), (1, 2, 64, 16))
    _roundtrip_exact(x, axis)
    _roundtrip_exact(np.ascontiguousarray(x.swapaxes(-1, -2)), axis)


@pytest.mark.parametrize("axis", [-2, -1])
@pytest.mark.parametrize("b", [2, 4, 8])
def test_quotients_on_and_next_to_ties(axis, b):
    """Every group spans [lo, lo + levels * step] for steps with and without an exact reciprocal
    and holds, next to random values, the values whose quotient is k + 1/2 exactly and one fp16
    step either side of it: the kernels decide codes from a reciprocal product and must fall
    back to the true division wherever that product cannot tell the side of the tie."""
    rng = np.random.default_rng(100 + b)
    levels = (1 << b) - 1
    g, D, S = 32, 128, 64
    x = np.zeros((1, 4, S, D), np.float32)
    steps = [1.0, 0.5, 3.0, 0.75, 1.5, 0.375, 6.0, 0.046875]
    for h in range(4):
        for blk in range((S // g) if axis == -2 else (D // g)):
            for line in range(D if axis == -2 else S):
                step = steps[(h + blk + line) % len(steps)] * (2.0 if b == 2 else 1.0) * (1 / 16 if b == 8 else 1.0)
                lo = float(np.float16(rng.integers(-8, 8) * step))
                vals = lo + step * rng.uniform(0, levels, g)
                ks = rng.integers(0, levels, g // 2)
                vals[: g // 2] = lo + step * (ks + 0.5)
                vals[0], vals[1] = lo, lo + step * levels
                v16 = vals.astype(np.float16)
                v16[2:g // 2:3] = np.nextafter(v16[2:g // 2:3], np.float16(np.inf))
                v16[3:g // 2:3] = np.nextafter(v16[3:g // 2:3], np.float16(-np.inf))
                if axis == -2:
                    x[0, h, blk * g:(blk + 1) * g, line] = v16
                else:
                    x[0, h, line, blk * g:(blk + 1) * g] = v16
    x16 = x.astype(np.float16)
    _roundtrip_exact(x16, axis, b=b, g=g)
    _pack_exact(x16, axis, b, g, torch.float16)


@pytest.mark.parametrize("axis", [-2, -1])
def test_no_fma_contraction_in_reconstruction(axis):
    rng = np.random.default_rng(7)
    _roundtrip_exact(rng.standard_normal((1, 4, 128, 128)).astype(np.float16), axis, b=8, g=32)


@pytest.mark.parametrize("axis", [-2, -1])
def test_degenerate_group_uses_eps_floor(axis):
    require_gpu()
    x = np.full((1, 2, 64, 32), 3.5, np.float16)
    got = K.kivi_group_quant_dequant(to_dev(x), axis=axis, group_size=32, levels=3)
    assert bool(torch.isfinite(got).all())
    _roundtrip_exact(x, axis)
    _roundtrip_exact(np.full((1, 2, 64, 128), 3.5, np.float16), axis)


def test_single_element_groups_are_lossless():
    require_gpu()
    rng = np.random.default_rng(3)
    x = to_dev(rng.standard_normal((1, 2, 16, 32)).astype(np.float16))
    assert torch.equal(K.kivi_group_quant_dequant(x, axis=-2, group_size=1, levels=3), x)
    x = to_dev(rng.standard_normal((1, 2, 16, 128)).astype(np.float16))
    assert torch.equal(K.kivi_group_quant_dequant(x, axis=-2, group_size=1, levels=3), x)


def test_many_sequence_lengths_one_library():
    """Sequence length is a run-time argument: 55 lengths, no per-length state."""
    require_gpu()
    rng = np.random.default_rng(0)
    for L in range(16, 400, 7):
        x = rng.standard_normal((1, 4, L, 128)).astype(np.float16)
        for axis in (-2, -1):
            _roundtrip_exact(x, axis)


def test_wrapper_errors():
    require_gpu()
    x = to_dev(np.zeros((1, 1, 8, 8), np.float16))
    with pytest.raises(ValueError, match="axis must be -1 or -2"):
        K.kivi_group_quant_dequant(x, axis=0, group_size=4, levels=3)
    with pytest.raises(ValueError, match="at least 2D"):
        K.kivi_group_quant_dequant(x.reshape(-1), axis=-1, group_size=4, levels=3)
    with pytest.raises(ValueError, match="group_size must be >= 1"):
        K.kivi_group_quant_dequant(x, axis=-1, group_size=0, levels=3)
    with pytest.raises(ValueError, match="unsupported dtype"):
        K.kivi_group_quant_dequant(x.to(torch.int32), axis=-1, group_size=4, levels=3)
    e = to_dev(np.zeros((1, 1, 0, 8), np.float16))
    assert K.kivi_group_quant_dequant(e, axis=-2, group_size=4, levels=3).shape == e.shape


# ------------------------------------------------------------------ packed forms
def _pack_exact(x_np, axis, b, g, meta_dtype, v_layout="channel"):
    require_gpu()
    levels = (1 << b) - 1
    codes, scale, zero = ok.group_quant_codes(x_np, axis, g, levels)
    p, s, z = K.kivi_quant_pack(to_dev(x_np), axis, g, b, meta_dtype=meta_dtype, v_layout=v_layout)
    if axis == -1 and v_layout == "token":
        ref_words = ok.pack_indices(codes.swapaxes(-1, -2), b).swapaxes(-1, -2)
        scale, zero = scale.swapaxes(-1, -2), zero.swapaxes(-1, -2)
    else:
        ref_words = ok.pack_indices(codes, b)
    np.testing.assert_array_equal(words(p), ref_words)
    np_meta = np.float16 if meta_dtype == torch.float16 else np.float32
    np.testing.assert_array_equal(host(s), scale.astype(np_meta))
    np.testing.assert_array_equal(host(z), zero.astype(np_meta))
    # and back: reconstruction from the packed form, bit for bit
    S, D = x_np.shape[-2], x_np.shape[-1]
    back = K.kivi_dequant(p, s, z, axis, g, b, S, D, v_layout=v_layout, out_dtype=torch.float32)
    sm = scale.astype(np_meta).astype(np.float32)
    zm = zero.astype(np_meta).astype(np.float32)
    if axis == -1 and v_layout == "token":
        sm, zm = sm.swapaxes(-1, -2), zm.swapaxes(-1, -2)
    np.testing.assert_array_equal(host(back), ok.group_dequant(codes, sm, zm, axis, g))
    for dt in (torch.float16, torch.bfloat16):   # the same values rounded once to the output type
        low = K.kivi_dequant(p, s, z, axis, g, b, S, D, v_layout=v_layout, out_dtype=dt)
        assert torch.equal(low, back.to(dt))


@pytest.mark.parametrize("axis", [-2, -1])
@pytest.mark.parametrize("b", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("g", [32, 64])
@pytest.mark.parametrize("meta", [torch.float16, torch.float32])
def test_quant_pack_bit_exact(axis, b, g, meta):
    k, v = outlier_kv((2, 3, 128, 128), seed=b * 10 + g)
    _pack_exact(k if axis == -2 else v, axis, b, g, meta)


@pytest.mark.parametrize("shape,g,b", [((1, 2, 33, 64), 32, 2), ((1, 1, 7, 16), 4, 4), ((2, 1, 200, 96), 32, 3),
                                       ((1, 2, 70, 256), 32, 4), ((1, 2, 64, 64), 16, 2), ((1, 1, 40, 128), 128, 4)])
@pytest.mark.parametrize("axis", [-2, -1])
def test_quant_pack_odd_shapes(shape, g, b, axis):
    k, v = outlier_kv(shape, seed=sum(shape))
    _pack_exact(k if axis == -2 else v, axis, b, g, torch.float32)


@pytest.mark.parametrize("b,g,D", [(4, 32, 128), (2, 32, 128), (4, 64, 128), (2, 64, 128), (8, 32, 64), (3, 32, 96), (2, 64, 256),
                                   (2, 32, 256), (4, 32, 256), (2, 128, 256), (2, 32, 64), (1, 32, 128)])
def test_value_token_packed_layout(b, g, D):
    per = 32 // b
    S = per * 12
    _, v = outlier_kv((2, 2, S, D), seed=b + g + D)
    _pack_exact(v, -1, b, g, torch.float16, v_layout="token")


def test_quant_codes_split_form_matches_reference_layout():
    require_gpu()
    k, v = outlier_kv((1, 4, 96, 128), seed=1)
    for x, axis in ((k, -2), (v, -1)):
        c, s, z = K.kivi_quant_codes(to_dev(x), axis, 32, 3)
        rc, rs, rz = ok.group_quant_codes(x, axis, 32, 3)
        assert c.dtype == torch.uint8 and s.dtype == torch.float32
        np.testing.assert_array_equal(host(c), rc)
        np.testing.assert_array_equal(host(s), rs)
        np.testing.assert_array_equal(host(z), rz)
        dec = K.scalar_decode_once(c, s, z, 32, "K" if axis == -2 else "V")
        np.testing.assert_array_equal(host(dec), ok.group_dequant(rc, rs, rz, axis, 32).astype(np.float16))


def test_config0_layer_roundtrip_and_pack():
    """K and V [1,8,2048,128] fp16 with outlier channels, 4-bit, group 32."""
    k, v = outlier_kv((1, 8, 2048, 128), seed=0)
    _roundtrip_exact(k, -2, b=4, g=32)
    _roundtrip_exact(v, -1, b=4, g=32)
    _pack_exact(k, -2, 4, 32, torch.float16)
    _pack_exact(v, -1, 4, 32, torch.float16)
    _pack_exact(v, -1, 4, 32, torch.float16, v_layout="token")


def test_pack_into_preallocated_cache_at_offset():
    require_gpu()
    k, v = outlier_kv((2, 2, 256, 128), seed=4)
    B, H, cap, D, g, b = 2, 2, 512, 128, 32, 4
    dev = "cuda:0"
    kp = torch.zeros((B, H, cap, D * b // 32), dtype=torch.int32, device=dev)
    ks = torch.zeros((B, H, cap // g, D), dtype=torch.float16, device=dev)
    kz = torch.zeros_like(ks)
    vp = torch.zeros((B, H, cap * b // 32, D), dtype=torch.int32, device=dev)
    vs = torch.zeros((B, H, D // g, cap), dtype=torch.float16, device=dev)
    vz = torch.zeros_like(vs)
    src_k, src_v = to_dev(k), to_dev(v)
    # two flushes of 128 tokens taken as strided slices of the fp16 history
    for lo in (0, 128):
        K.kivi_quant_pack(src_k[:, :, lo:lo + 128], -2, g, b, out=(kp, ks, kz), dst_tok0=lo)
        K.kivi_quant_pack(src_v[:, :, lo:lo + 128], -1, g, b, v_layout="token", out=(vp, vs, vz), dst_tok0=lo)
    kc, ksc, kzr = ok.group_quant_codes(k, -2, g, 15)
    vc, vsc, vzr = ok.group_quant_codes(v, -1, g, 15)
    np.testing.assert_array_equal(words(kp)[:, :, :256], ok.pack_indices(kc, b))
    np.testing.assert_array_equal(host(ks)[:, :, :8], ksc.astype(np.float16))
    np.testing.assert_array_equal(words(vp)[:, :, :32], ok.pack_indices(vc.swapaxes(-1, -2), b).swapaxes(-1, -2))
    np.testing.assert_array_equal(host(vz)[:, :, :, :256], vzr.swapaxes(-1, -2).astype(np.float16))
    assert int(kp[:, :, 256:].abs().sum()) == 0 and int(vp[:, :, 32:].abs().sum()) == 0


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("n", [1, 7, 8, 15, 33, 128, 1000])
def test_pack_indices_round_trip(bits, n):
    require_gpu()
    rng = np.random.default_rng(bits * 1000 + n)
    idx = rng.integers(0, 1 << bits, size=(3, n), dtype=np.uint8)
    p = K.pack_indices(to_dev(idx), bits)
    np.testing.assert_array_equal(words(p), ok.pack_indices(idx, bits))
    np.testing.assert_array_equal(host(K.unpack_indices(p, bits, n)), idx)


@pytest.mark.parametrize("b", [1, 2, 4])
def test_byte_pack_round_trip(b):
    require_gpu()
    rng = np.random.default_rng(b)
    idx = rng.integers(0, 1 << b, size=4096, dtype=np.uint8)
    p = K.turboquant_bit_pack(to_dev(idx), b)
    np.testing.assert_array_equal(host(p), ok.pack_bytes(idx, b))
    np.testing.assert_array_equal(host(K.turboquant_bit_unpack(p, 4096, b)), idx)
    with pytest.raises(ValueError, match="must be 1, 2, or 4"):
        K.turboquant_bit_pack(to_dev(idx), 3)
    with pytest.raises(ValueError, match="not divisible"):
        K.turboquant_bit_pack(to_dev(idx[:4095]), b)
    with pytest.raises(ValueError, match="needs"):
        K.turboquant_bit_unpack(p[:10], 4096, b)


@pytest.mark.parametrize("dtype,b,g,D,S,v_layout,meta", [
    (torch.float16, 4, 32, 128, 2048, "token", torch.float16),     # config 0's layer
    (torch.bfloat16, 2, 64, 128, 320, "token", torch.float32),
    (torch.float16, 4, 128, 128, 384, "channel", torch.float16),   # the longest key group the tile kernel holds
    (torch.float16, 2, 32, 64, 96, "token", torch.float16),        # head_dim 64: the two single calls
    (torch.float16, 8, 32, 128, 100, "channel", torch.float16),    # ragged last key group
])
def test_keys_and_values_in_one_call_equal_the_single_calls(dtype, b, g, D, S, v_layout, meta):
    """``kivi_quant_pack_kv`` is ``kivi_quant_pack`` of keys and values (each checked bit for bit
    against the oracle above), in fresh buffers and at an offset of pre-allocated ones."""
    require_gpu()
    k, v = outlier_kv((2, 3, S, D), seed=S + b)
    kt, vt = to_dev(k, dtype), to_dev(v, dtype)
    (kp, ks, kz), (vp, vs, vz) = K.kivi_quant_pack_kv(kt, vt, g, b, meta_dtype=meta, v_layout=v_layout)
    want_k = K.kivi_quant_pack(kt, -2, g, b, meta_dtype=meta)
    want_v = K.kivi_quant_pack(vt, -1, g, b, meta_dtype=meta, v_layout=v_layout)
    for got, want in zip((kp, ks, kz, vp, vs, vz), (*want_k, *want_v)):
        assert got.shape == want.shape and torch.equal(got, want)
    if S % g == 0 and S % (32 // b) == 0:
        cap, off = 2 * S, S
        bufs = K.kivi_quant_pack_kv(torch.zeros((2, 3, cap, D), dtype=dtype, device=kt.device),
                                    torch.zeros((2, 3, cap, D), dtype=dtype, device=kt.device), g, b, meta_dtype=meta,
                                    v_layout=v_layout)
        K.kivi_quant_pack_kv(kt, vt, g, b, meta_dtype=meta, v_layout=v_layout, out=bufs, dst_tok0=off)
        per = 32 // b
        assert torch.equal(bufs[0][0][:, :, off:], kp) and torch.equal(bufs[0][1][:, :, off // g:], ks)
        if v_layout == "token":
            assert torch.equal(bufs[1][0][:, :, off // per:], vp) and torch.equal(bufs[1][1][..., off:], vs)
        else:
            assert torch.equal(bufs[1][0][:, :, off:], vp) and torch.equal(bufs[1][2][:, :, off:], vz)
