"""Pins the numpy / C oracle for KIVI group quantisation and packing against
facts that do not come from the oracle itself: hand-computed answers, closed
forms, invariants, and the special cases the reference's own tests single out
(veloxquant_mlx/tests/metal/test_kivi_quant.py:110-159,
veloxquant_mlx/tests/quantizers/test_kivi.py:87-122,
veloxquant_mlx/tests/dsa/test_bit_pack.py:11-54)."""

import numpy as np
import pytest

from oracle import cref, kivi


# ---------------------------------------------------------------- known answers
def test_hand_computed_half_to_even_codes():
    # one group of 8 along the token axis, one channel; range 6, levels 3 -> scale 2
    x = np.array([0, 1, 2, 3, 4, 5, 6, 6], np.float16).reshape(1, 1, 8, 1)
    codes, scale, zero = kivi.group_quant_codes(x, -2, 8, 3)
    assert scale.reshape(-1).tolist() == [2.0]
    assert zero.reshape(-1).tolist() == [0.0]
    # x/2 = 0, .5, 1, 1.5, 2, 2.5, 3, 3 ; ties go to the even neighbour
    assert codes.reshape(-1).tolist() == [0, 0, 1, 2, 2, 2, 3, 3]
    # round-half-away would have produced [0,1,1,2,2,3,3,3]
    recon = kivi.group_dequant(codes, scale, zero, -2, 8)
    assert recon.reshape(-1).tolist() == [0, 0, 2, 4, 4, 4, 6, 6]
    # same data along the channel axis
    xv = x.reshape(1, 1, 1, 8)
    cv, sv, zv = kivi.group_quant_codes(xv, -1, 8, 3)
    assert cv.reshape(-1).tolist() == [0, 0, 1, 2, 2, 2, 3, 3]
    assert sv.shape == (1, 1, 1, 1) and zv.shape == (1, 1, 1, 1)


def test_hand_computed_ragged_group_replicates_last_element():
    # L=5, g=4: second group holds only x[4]=10 (padding = copies of 10)
    x = np.array([1, 2, 3, 5, 10], np.float32).reshape(1, 5, 1)
    codes, scale, zero = kivi.group_quant_codes(x, -2, 4, 3)
    assert zero.reshape(-1).tolist() == [1.0, 10.0]
    np.testing.assert_array_equal(scale.reshape(-1), np.array([np.float32(4) / np.float32(3), 1e-8], np.float32))
    # (x-1)/(4/3) = 0, .75, 1.5, 3 -> 0,1,2,3 ; lone element -> code 0
    assert codes.reshape(-1).tolist() == [0, 1, 2, 3, 0]
    # zero padding would have made the last group's min 0 and its code 3
    out = kivi.quant_dequant_along(x, -2, 4, 3)
    assert out.reshape(-1)[-1] == 10.0


def test_hand_computed_shapes_of_parameters():
    x = np.zeros((2, 3, 50, 96), np.float16)
    c, s, z = kivi.group_quant_codes(x, -2, 32, 3)
    assert c.shape == x.shape and s.shape == (2, 3, 2, 96) and z.shape == s.shape
    c, s, z = kivi.group_quant_codes(x, -1, 32, 3)
    assert c.shape == x.shape and s.shape == (2, 3, 50, 3) and z.shape == s.shape


# ---------------------------------------------------------------- invariants
@pytest.mark.parametrize("axis", [-2, -1])
@pytest.mark.parametrize("b", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("g", [4, 32, 128])
def test_invariants(axis, b, g):
    rng = np.random.default_rng(b * 100 + g)
    x = rng.standard_normal((1, 4, 64, 128)).astype(np.float16)
    levels = (1 << b) - 1
    codes, scale, zero = kivi.group_quant_codes(x, axis, g, levels)
    assert codes.max() <= levels
    x32 = x.astype(np.float32)
    recon = kivi.group_dequant(codes, scale, zero, axis, g)
    L = x.shape[axis]
    gi = np.arange(L) // g
    s_full = scale[..., gi, :] if axis == -2 else scale[..., :, gi]
    z_full = zero[..., gi, :] if axis == -2 else zero[..., :, gi]
    # group minimum -> code 0, group maximum -> top code
    assert np.all(codes[x32 == z_full] == 0)
    gmax = z_full + s_full * levels
    top = np.isclose(x32, gmax, rtol=0, atol=0) & (s_full > 1e-8)
    assert np.all(codes[top] == levels)
    # reconstruction error at most half a step (plus float32 slack)
    assert np.all(np.abs(recon - x32) <= 0.5 * s_full * (1 + 1e-5) + 1e-6)


def test_single_element_groups_are_lossless():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((1, 2, 16, 32)).astype(np.float16)
    np.testing.assert_array_equal(kivi.quant_dequant_along(x, -2, 1, 3), x)
    np.testing.assert_array_equal(kivi.quant_dequant_along(x, -1, 1, 3), x)


@pytest.mark.parametrize("axis", [-2, -1])
def test_constant_group_hits_eps_floor_and_stays_exact(axis):
    x = np.full((1, 2, 64, 32), 3.5, np.float16)
    codes, scale, zero = kivi.group_quant_codes(x, axis, 32, 3)
    assert np.all(scale == np.float32(1e-8)) and np.all(zero == 3.5) and np.all(codes == 0)
    out = kivi.quant_dequant_along(x, axis, 32, 3)
    assert np.all(np.isfinite(out)) and np.array_equal(out, x)


def _unit_gaussian(n, d, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, d)).astype(np.float32)
    return x / np.linalg.norm(x, axis=-1, keepdims=True)


@pytest.mark.parametrize("b,thr", [(2, 0.90), (3, 0.96), (4, 0.99), (8, 0.999)])
@pytest.mark.parametrize("axis", [-2, -1])
def test_cosine_quality_thresholds(b, thr, axis):
    x = _unit_gaussian(256, 128, 0)
    xh = kivi.quant_dequant_along(x[None], axis, 32, (1 << b) - 1)[0]
    cos = (x * xh).sum(-1) / (np.linalg.norm(x, axis=-1) * np.linalg.norm(xh, axis=-1))
    assert cos.mean() >= thr


def test_b8_mse_small():
    x = _unit_gaussian(256, 128, 1)
    xh = kivi.quant_dequant_along(x[None], -2, 32, 255)[0]
    assert np.mean((x - xh) ** 2) < 1e-4


def test_two_roundings_not_fma():
    # exhibit one element where fused multiply-add differs from the two-step
    # form, so a contracted implementation cannot pass bit-exact parity
    rng = np.random.default_rng(7)
    x = rng.standard_normal((1, 4, 128, 128)).astype(np.float16)
    codes, scale, zero = kivi.group_quant_codes(x, -2, 32, 255)
    gi = np.arange(128) // 32
    s = scale[..., gi, :].astype(np.float64)
    z = zero[..., gi, :].astype(np.float64)
    fused = (codes.astype(np.float64) * s + z).astype(np.float32)
    two_step = kivi.group_dequant(codes, scale, zero, -2, 32)
    assert (fused != two_step).mean() > 1e-5


# ---------------------------------------------------------------- numpy vs C
@pytest.mark.parametrize("axis", [-2, -1])
@pytest.mark.parametrize("shape", [(1, 8, 32, 128), (2, 2, 33, 64), (1, 1, 7, 16), (3, 1, 200, 128)])
@pytest.mark.parametrize("b", [2, 4])
def test_numpy_and_c_restatements_agree(axis, shape, b):
    rng = np.random.default_rng(sum(shape) + b)
    x = (rng.standard_normal(shape) * np.exp(rng.standard_normal(shape[-1]))).astype(np.float16)
    n = kivi.group_quant_codes(x, axis, 32, (1 << b) - 1)
    c = cref.group_quant(x.astype(np.float32), axis, 32, (1 << b) - 1)
    for a, bb in zip(n, c):
        np.testing.assert_array_equal(a, bb)
    np.testing.assert_array_equal(kivi.pack_indices(n[0], b), cref.pack_words(n[0], b))


# ---------------------------------------------------------------- packing
def test_pack_known_words():
    assert kivi.pack_indices(np.array([1, 2, 3, 0], np.uint8), 2).tolist() == [0x39]
    assert kivi.pack_indices(np.arange(1, 9, dtype=np.uint8), 4).tolist() == [0x87654321]
    assert kivi.pack_indices(np.array([1, 0, 1, 1], np.uint8), 1).tolist() == [0b1101]
    # 3-bit: ten codes per word, two idle top bits
    w = kivi.pack_indices(np.array([7] * 10 + [5], np.uint8), 3)
    assert w.tolist() == [(1 << 30) - 1, 5]
    assert kivi.pack_indices(np.arange(16, dtype=np.uint8) % 4, 2).tolist() == [0xE4E4E4E4]


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("n", [1, 7, 8, 15, 16, 17, 31, 32, 33, 128, 1000])
def test_pack_round_trip_and_size(bits, n):
    rng = np.random.default_rng(bits * 1000 + n)
    idx = rng.integers(0, 1 << bits, size=(3, n), dtype=np.uint8)
    p = kivi.pack_indices(idx, bits)
    per = 32 // bits
    assert p.shape == (3, (n + per - 1) // per) and p.dtype == np.uint32
    np.testing.assert_array_equal(kivi.unpack_indices(p, bits, n), idx)


@pytest.mark.parametrize("bits", [1, 2, 4])
def test_byte_form_is_the_little_endian_image_of_the_word_form(bits):
    rng = np.random.default_rng(bits)
    idx = rng.integers(0, 1 << bits, size=256, dtype=np.uint8)
    by = kivi.pack_bytes(idx, bits)
    wd = kivi.pack_indices(idx, bits)
    np.testing.assert_array_equal(by, wd.astype("<u4").view(np.uint8))
    np.testing.assert_array_equal(kivi.unpack_bytes(by, 256, bits), idx)
    assert kivi.pack_bytes(np.array([1, 2, 3, 0], np.uint8), 2).tolist() == [0x39]


# ---------------------------------------------------------------- cache model
def test_boundary_arithmetic():
    assert kivi.quantization_boundary(100, 128, 32) == 0
    assert kivi.quantization_boundary(160, 128, 32) == 32
    assert kivi.quantization_boundary(191, 128, 32) == 32
    assert kivi.quantization_boundary(192, 128, 32) == 64
    assert kivi.quantization_boundary(8320, 128, 32) == 8192
    # prefill chunks of 512 over a 4096 prefix
    assert [kivi.quantization_boundary(4096 + 512 * (c + 1), 128, 32) for c in range(3)] == [4480, 4992, 5504]


def test_accounting_known_bytes():
    # 128 tokens, D=128, b=2, g=32, one head: codes 4096 B; key params 4*128*4 B; value params 128*4*4 B
    assert kivi.quantized_bytes(128, 1, 1, 128, 2, 32) == (4096 + 2048, 4096 + 2048)
    assert kivi.quantized_bytes(64, 2, 8, 128, 4, 64) == ((4096 + 512) * 16, (4096 + 512) * 16)


def _kv(B, H, S, D, seed):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((B, H, S, D)).astype(np.float16),
            rng.standard_normal((B, H, S, D)).astype(np.float16))


def test_cache_model_passthrough_and_alignment():
    c = kivi.KiviCacheModel(2, 32, 64)
    k, v = _kv(1, 2, 32, 128, 1)
    ko, vo = c.update_and_fetch(k, v)
    assert np.array_equal(ko, k) and np.array_equal(vo, v) and c.key_bytes_compressed == 0
    c = kivi.KiviCacheModel(2, 16, 8)
    k, v = _kv(1, 1, 5, 128, 12)
    c.update_and_fetch(k, v)
    for t in range(70):
        c.update_and_fetch(*_kv(1, 1, 1, 128, 400 + t))
        assert c.n_quantized % 16 == 0
        assert c.offset - c.n_quantized <= 8 + 16 - 1


def test_cache_model_one_shot_equals_streamed():
    k, v = _kv(1, 2, 48, 128, 13)
    a = kivi.KiviCacheModel(2, 8, 8)
    ka, va = a.update_and_fetch(k, v)
    b = kivi.KiviCacheModel(2, 8, 8)
    for t in range(48):
        kb, vb = b.update_and_fetch(k[:, :, t:t + 1], v[:, :, t:t + 1])
    assert np.array_equal(ka, kb) and np.array_equal(va, vb) and a.n_quantized == b.n_quantized == 40
    assert (a.key_bytes_compressed, a.value_bytes_compressed) == (b.key_bytes_compressed, b.value_bytes_compressed)


def test_cache_model_trim_equals_feeding_kept_tokens():
    k, v = _kv(1, 2, 100, 64, 5)
    a = kivi.KiviCacheModel(2, 8, 8)
    a.update_and_fetch(k, v)
    assert a.trim(36) == 36
    b = kivi.KiviCacheModel(2, 8, 8)
    b.update_and_fetch(k[:, :, :64], v[:, :, :64])
    # frontier snaps down to a group multiple no larger than the kept length
    assert a.offset == 64 and a.n_quantized == min(88, 64) and a.n_quantized % 8 == 0
    assert a.key_bytes_fp16 == b.key_bytes_fp16 and a.tokens_seen == b.tokens_seen


def test_sink_cache_model_pins():
    """SinkCacheModel (veloxquant_mlx/cache/sink_cache.py:62-256) against what the method fixes:
    without sinks it is the KIVI model; the protected positions are the brute-force top-k of the
    head-averaged key norms; protected rows keep their fp16 values; a 25x row no longer sets its
    group's range (the reference's tests/cache/test_sink_cache.py ask exactly for these:
    sink rows exact, neighbours better than under plain KIVI, per-batch positions)."""
    rng = np.random.default_rng(0)
    k = rng.standard_normal((2, 2, 300, 64)).astype(np.float16)
    v = rng.standard_normal((2, 2, 300, 64)).astype(np.float16)
    k[0, :, 17] *= 25
    k[1, :, 200] *= 25
    plain = kivi.KiviCacheModel(2, 32, 64)
    kp, vp = plain.update_and_fetch(k, v)
    none = kivi.SinkCacheModel(2, 32, 64, n_sink=0)
    k0, v0 = none.update_and_fetch(k, v)
    assert np.array_equal(k0, kp) and np.array_equal(v0, vp)
    assert none.key_bytes_compressed == plain.key_bytes_compressed and none.sink_fp16_bytes == 0
    m = kivi.SinkCacheModel(2, 32, 64, n_sink=3)
    ks, vs = m.update_and_fetch(k, v)
    norms = np.sqrt((k.astype(np.float32) ** 2).sum(-1)).mean(1)
    for b in range(2):
        assert sorted(m.sink_positions_for(b)) == sorted(np.argsort(-norms[b])[:3].tolist())
        for p in m.sink_positions_for(b):
            if p < m.n_quantized:
                assert np.array_equal(ks[b, :, p], k[b, :, p]) and np.array_equal(vs[b, :, p], v[b, :, p])
    # keys are grouped along tokens: the group of token 17 (tokens 0..31) of batch 0
    err_plain = np.abs(kp[0, :, :32].astype(np.float32) - k[0, :, :32].astype(np.float32))
    err_sink = np.abs(ks[0, :, :32].astype(np.float32) - k[0, :, :32].astype(np.float32))
    rows = [t for t in range(32) if t != 17]
    assert err_sink[:, rows].mean() < 0.25 * err_plain[:, rows].mean()
    # key groups (32 tokens) that hold no protected row are bit-identical to plain KIVI
    clean = [g for g in range(m.n_quantized // 32) if not any(g * 32 <= p < g * 32 + 32 for p in m.sink_positions_for(0))]
    assert len(clean) >= 4
    for g in clean:
        assert np.array_equal(ks[0, :, g * 32:g * 32 + 32], kp[0, :, g * 32:g * 32 + 32])
    # accounting: the sinks inside the quantised region moved from the compressed pool to the fp16 pool
    n_in = max(sum(1 for p in m.sink_positions_for(b) if p < m.n_quantized) for b in range(2))
    assert m.sink_fp16_bytes == n_in * 64 * 2 * 2 * 2 * 2
    kq, vq = kivi.quantized_bytes(m.n_quantized - n_in, 2, 2, 64, 2, 32)
    assert (m.key_bytes_compressed, m.value_bytes_compressed) == (kq, vq)
    # the stand-in row: nearest non-sink neighbour, left first
    nb = kivi.SinkCacheModel.neighbour
    assert nb(5, {5}, 32) == 4 and nb(0, {0}, 32) == 1 and nb(1, {0, 1}, 32) == 2 and nb(0, {0}, 1) is None
    # streaming: sinks found in a later block are protected from then on; earlier ones stay
    st = kivi.SinkCacheModel(2, 32, 64, n_sink=1)
    for s0 in range(0, 300, 50):
        st.update_and_fetch(k[:, :, s0:s0 + 50], v[:, :, s0:s0 + 50])
    assert st.sink_positions_for(0) == [17] and st.sink_positions_for(1) == [200]
    assert np.array_equal(st.keys[1, :, 200], k[1, :, 200])
