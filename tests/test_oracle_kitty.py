"""Pins of the Kitty oracle (``oracle/kitty.py``): the known answers of the reference's own tests
(veloxquant_mlx/tests/cache/test_kitty_cache.py) and what the arithmetic fixes."""

import numpy as np

from oracle import kitty as okt, kivi as ok


def _keys(B=1, H=2, S=32, D=64, seed=0):
    return np.random.default_rng(seed).standard_normal((B, H, S, D)).astype(np.float16)


def test_all_channels_high_is_the_plain_group_round_trip():
    """test_kitty_cache.py:266-283: hi_fraction = 1 equals ``_group_quant_dequant(k, b=4, group_size=32)``
    exactly -- here the already pinned KIVI key-axis round trip."""
    k = _keys(B=1, H=1, S=32, D=64)
    m = okt.KittyCacheModel(64, hi_fraction=1.0)
    out, _ = m.update_and_fetch(k, _keys(seed=1, H=1))
    ref = ok.quant_dequant_along(k[0, 0], -2, 32, 15)
    assert np.array_equal(out[0, 0], ref)


def test_ranking_picks_the_high_variance_channels():
    """test_kitty_cache.py:110-123, same seed and shape: channels 0-7 scaled by 10 are the eight kept high."""
    data = np.random.default_rng(7).standard_normal((128, 64)).astype(np.float32)
    data[:, :8] *= 10.0
    hi, lo = okt.rank_channels_by_sensitivity(data, hi_fraction=0.125)
    assert hi == list(range(8)) and lo == list(range(8, 64))


def test_ties_go_to_the_lower_channel():
    """A stable descending sort (kitty.py:61-64 and the docstring of :112-129): equal variances keep index order."""
    mask = okt.hi_mask_from_variance(np.array([[1.0, 3.0, 1.0, 3.0, 1.0, 3.0]], np.float32), 0.5)
    assert mask.tolist() == [[False, True, False, True, False, True]]
    mask = okt.hi_mask_from_variance(np.ones((1, 4), np.float32), 0.5)
    assert mask.tolist() == [[True, True, False, False]]
    assert okt.hi_mask_from_variance(np.ones((1, 64), np.float32), 0.0).sum() == 1   # never fewer than one


def test_running_sums_give_the_variance():
    """test_kitty_cache.py:178-200, same seed: sums over 64 rows against numpy's variance."""
    data = np.random.default_rng(55).standard_normal((64, 32)).astype(np.float32)
    s, sq = data.sum(axis=0, dtype=np.float32), (data * data).sum(axis=0, dtype=np.float32)
    np.testing.assert_allclose(okt.compute_running_variance(s, sq, 64), np.var(data, axis=0), rtol=1e-4, atol=1e-5)
    assert not okt.compute_running_variance(s, sq, 1).any()


def test_accounting_by_hand():
    """D = 64, 64 tokens, 2 heads, defaults: 16 channels at 4 bits = 512 B of codes + 2 groups x 16 x 4 B,
    48 channels at 2 bits = 768 B + 2 x 48 x 4 B; per head 640 + 1152 (kitty_cache.py:150-163)."""
    assert okt.key_bytes(64, 1, 2, 64, 0.25, 4, 2, 32) == 2 * (640 + 1152)
    m = okt.KittyCacheModel(64)
    m.update_and_fetch(_keys(S=64), _keys(S=64, seed=1))
    assert m.compressed_key_bytes == 3584 and m.fp16_key_bytes == 16384 and m.value_fp16_bytes == 16384
    # one token at a time: a code byte count rounded up per call and one parameter set per call
    assert okt.key_bytes(1, 1, 1, 64, 0.25, 4, 2, 32) == (8 + 64) + (12 + 192)


def test_single_tokens_are_stored_exactly_and_values_pass_through():
    """A group of one token has min = max: code 0, reconstruction = the token (both bit widths)."""
    m = okt.KittyCacheModel(64)
    m.update_and_fetch(_keys(S=20), _keys(S=20, seed=1))
    k, v = _keys(S=1, seed=200), _keys(S=1, seed=300)
    ko, vo = m.update_and_fetch(k, v)
    assert ko.shape[2] == 21 and np.array_equal(ko[:, :, 20:], k) and np.array_equal(vo[:, :, 20:], v)


def test_high_channels_err_less_and_mixed_beats_two_bits():
    """test_kitty_cache.py:128-172 in substance: on keys whose first channels carry the variance, those channels
    come back with the smaller relative error, and the mix has a lower error than 2 bits everywhere."""
    rng = np.random.default_rng(3)
    x = rng.standard_normal((1, 256, 64)).astype(np.float32)
    x[:, :, :16] *= 8.0
    x = x.astype(np.float16)
    var = np.var(x.astype(np.float32), axis=1)
    mask = okt.hi_mask_from_variance(var, 0.25)
    assert mask[0, :16].all() and not mask[0, 16:].any()
    mixed = okt.quantize_mixed_channels_batched(x, mask).astype(np.float32)
    two = okt.group_round_trip_fp16(x, 2, 32).astype(np.float32)
    x32 = x.astype(np.float32)
    rel = lambda a, sl: np.abs(a[..., sl] - x32[..., sl]).mean() / np.abs(x32[..., sl]).mean()
    assert rel(mixed, slice(0, 16)) < rel(mixed, slice(16, 64))
    assert ((mixed - x32) ** 2).mean() < ((two - x32) ** 2).mean()


def test_trim_takes_the_tokens_out_of_the_sums():
    m = okt.KittyCacheModel(64)
    m.update_and_fetch(_keys(S=40), _keys(S=40, seed=1))
    s0, q0, b0 = m.key_sum.copy(), m.key_sq_sum.copy(), m.compressed_key_bytes
    m.update_and_fetch(_keys(S=8, seed=2), _keys(S=8, seed=3))
    assert m.trim(8) == 8 and m.n_keys == 40 and m.keys.shape[2] == 40
    np.testing.assert_allclose(m.key_sum, s0, atol=1e-4)
    np.testing.assert_allclose(m.key_sq_sum, q0, rtol=1e-5, atol=1e-4)
    assert m.compressed_key_bytes == b0
    assert m.trim(100) == 40 and m.key_sum is None and m.n_keys == 0
