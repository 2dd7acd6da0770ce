"""Pins of ``oracle/age_tiered.py``: the known answers of veloxquant_mlx/tests/cache/test_age_tiered_cache.py."""

import numpy as np

from oracle import age_tiered as oat, kivi as ok


def _kv(S=4, H=2, D=32, seed=0):
    rng = np.random.default_rng(seed)
    return rng.standard_normal((1, H, S, D)).astype(np.float16), rng.standard_normal((1, H, S, D)).astype(np.float16)


def test_tier_partition_by_age():
    """test_age_tiered_cache.py:170-181: 15 tokens, boundaries 3 / 6 -> 3 recent, 3 mid, 9 old."""
    m = oat.AgeTieredCacheModel(32, 3, 6)
    m.update_and_fetch(*_kv(S=15, H=1))
    assert m.tier_counts() == {oat.RECENT: 3, oat.MID: 3, oat.OLD: 9}
    assert oat.assign_age_tiers([0, 2, 3, 5, 6, 100], 3, 6) == [0, 0, 1, 1, 2, 2]


def test_short_sequence_is_recent_and_counts_scale_with_heads():
    """test_age_tiered_cache.py:149-167."""
    m = oat.AgeTieredCacheModel(32)
    m.update_and_fetch(*_kv(S=10, H=1))
    assert m.tier_counts() == {0: 10, 1: 0, 2: 0}
    m = oat.AgeTieredCacheModel(32, 4, 8)
    m.update_and_fetch(*_kv(S=20, H=2))
    assert sum(m.tier_counts().values()) == m.tokens_seen == 40


def test_a_token_ages_through_the_tiers():
    """test_age_tiered_cache.py:184-207: boundaries 2 / 4, one token per call."""
    m = oat.AgeTieredCacheModel(32, 2, 4)
    seen = []
    for s in range(5):
        m.update_and_fetch(*_kv(S=1, H=1, seed=s + 1))
        seen.append(m.tier_counts())
    assert seen[0][0] == 1 and seen[1][0] == 2 and seen[2][1] == 1 and seen[3][1] >= 1 and seen[4][2] == 1


def test_bytes_by_hand():
    """Codes only, keys + values: D = 32 -> 32 / 16 / 8 bytes per token at 8 / 4 / 2 bits
    (age_tiered.py:177-196); 16 bits everywhere equals the fp16 cost (test_age_tiered_cache.py:221-225)."""
    m = oat.AgeTieredCacheModel(32, 3, 6)
    m.update_and_fetch(*_kv(S=15, H=1))
    assert m.age_tiered_bytes == 2 * (3 * 32 + 3 * 16 + 9 * 8) and m.full_seq_bytes == 15 * 32 * 4
    m = oat.AgeTieredCacheModel(32, 3, 6, bits=(16, 16, 16))
    k, v = _kv(S=15, H=1)
    ko, vo = m.update_and_fetch(k, v)
    assert m.age_tiered_bytes == m.full_seq_bytes and np.array_equal(ko, k) and np.array_equal(vo, v)
    assert oat.age_tiered_bytes({0: 1}, {0: 3}, 5) == 2 * 2   # 15 bits round up to 2 bytes


def test_a_window_is_the_pinned_group_round_trip_at_its_tier():
    """Windows are position-aligned and independent; a window's bit width is that of its FIRST token's tier
    (age_tiered_cache.py:283-287), also when the window spans a boundary."""
    m = oat.AgeTieredCacheModel(32, 40, 70, group_size=32)
    k, v = _kv(S=100, H=2, seed=4)
    ko, vo = m.update_and_fetch(k, v)
    # ages: token i has age 99 - i; window 0 (tokens 0-31) starts at age 99 -> OLD (2 bits); window 1 starts at
    # age 67 -> MID (4 bits) although its last tokens are RECENT; window 2 starts at age 35 -> RECENT (8 bits);
    # window 3 (tokens 96-99, ragged) RECENT
    for lo, hi, bits in ((0, 32, 2), (32, 64, 4), (64, 96, 8), (96, 100, 8)):
        assert np.array_equal(ko[0, :, lo:hi], ok.quant_dequant_along(k[0, :, lo:hi], -2, 32, (1 << bits) - 1))
        assert np.array_equal(vo[0, :, lo:hi], ok.quant_dequant_along(v[0, :, lo:hi], -2, 32, (1 << bits) - 1))


def test_no_compounding():
    """A token is always one round trip from its raw value however often its window was re-derived
    (test_age_tiered_cache.py:371-405): token by token equals one call."""
    k, v = _kv(S=90, H=1, seed=9)
    one = oat.AgeTieredCacheModel(32, 8, 40, group_size=16)
    want_k, want_v = one.update_and_fetch(k, v)
    m = oat.AgeTieredCacheModel(32, 8, 40, group_size=16)
    for t in range(90):
        got_k, got_v = m.update_and_fetch(k[:, :, t:t + 1], v[:, :, t:t + 1])
    assert np.array_equal(got_k, want_k) and np.array_equal(got_v, want_v)
