"""Pins for ``oracle.skvq``: the properties the reference's own tests state for SKVQ's clipped group
quantisation (veloxquant_mlx/tests/quantizers/test_skvq.py) on the same seeded generators, known
answers worked by hand, and the count of groups whose choice of clip factor hangs on the order of
the error sum."""

import numpy as np
import pytest

from oracle import skvq as o


def _rows(n, d, seed=0, channel_scales=None):   # test_skvq.py:38-43
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, d)).astype(np.float32)
    if channel_scales is not None:
        x = x * channel_scales[None, :].astype(np.float32)
    return x


def _het_scales(d, seed=3):   # test_skvq.py:46-53
    rng = np.random.default_rng(seed)
    scales = np.logspace(-2, 1, d)
    rng.shuffle(scales)
    return scales


def _rt(x, bits, gs, alphas=o.DEFAULT_ALPHA_GRID):
    c, lo, sc = o.clipped_group_quant(x, bits, gs, alphas)
    return o.clipped_group_dequant(c, lo, sc, gs, x.shape[1])


def test_alpha1_equals_plain_minmax():   # test_skvq.py:103-121
    x = _rows(64, 32, seed=5, channel_scales=_het_scales(32))
    codes, lo, scale = o.clipped_group_quant(x, 2, 8, (1.0,))
    xn = x.reshape(64, 4, 8)
    gmin, gmax = xn.min(axis=-1, keepdims=True), xn.max(axis=-1, keepdims=True)
    ref_scale = np.maximum((gmax - gmin) / 3.0, 1e-8)
    ref_codes = np.clip(np.round((xn - gmin) / ref_scale), 0, 3)
    got = codes.astype(np.float64).reshape(64, 4, 8)
    assert np.mean(got == ref_codes) > 0.999
    assert np.max(np.abs(got - ref_codes)) <= 1.0
    recon = o.clipped_group_dequant(codes, lo, scale, 8, 32).reshape(64, 4, 8)
    assert np.all(np.abs(recon - (ref_codes * ref_scale + gmin)) <= ref_scale + 1e-5)


def test_clip_search_never_worse_than_alpha1():   # test_skvq.py:124-140
    rng = np.random.default_rng(6)
    x = rng.standard_normal((128, 32)).astype(np.float32)
    x[rng.random((128, 32)) < 0.03] *= 20.0

    def per_group_mse(alphas):
        return np.square(_rt(x, 2, 8, alphas) - x).reshape(128, 4, 8).mean(axis=-1)

    searched, plain = per_group_mse(o.DEFAULT_ALPHA_GRID), per_group_mse((1.0,))
    assert np.all(searched <= plain + 1e-7)
    assert searched.sum() < plain.sum()


def test_error_monotone_in_bits():   # test_skvq.py:143-147
    x = _rows(128, 64, seed=7)
    errs = [float(np.mean(np.square(_rt(x, b, 16) - x))) for b in (2, 4, 8)]
    assert errs[0] > errs[1] > errs[2]
    assert errs[2] < 1e-4


def test_known_answer_by_hand():
    """Group [0, 1, 2, 3] at 2 bits: alpha = 1 reproduces it exactly (error 0), so it wins and the
    codes are 0..3 with lo = 0, scale = 1.  A group [0, 0, 0, 10] at 1 bit: every alpha keeps codes
    [0, 0, 0, 1]; alpha = 1 is exact and wins.  A ragged row is padded with its last channel."""
    c, lo, sc = o.clipped_group_quant(np.array([[0, 1, 2, 3]], np.float32), 2, 4)
    assert c.tolist() == [[0, 1, 2, 3]] and lo.tolist() == [[0.0]] and sc.tolist() == [[1.0]]
    c, lo, sc = o.clipped_group_quant(np.array([[0, 0, 0, 10]], np.float32), 1, 4)
    assert c.tolist() == [[0, 0, 0, 1]] and lo.tolist() == [[0.0]] and sc.tolist() == [[10.0]]
    # clip factor 0.5 alone on [0, 0, 0, 10] at 1 bit: window [2.5, 7.5], codes [0, 0, 0, 1]
    c, lo, sc = o.clipped_group_quant(np.array([[0, 0, 0, 10]], np.float32), 1, 4, (0.5,))
    assert c.tolist() == [[0, 0, 0, 1]] and lo.tolist() == [[2.5]] and sc.tolist() == [[5.0]]
    c, lo, sc = o.clipped_group_quant(np.array([[0, 3, 1, 2, 7]], np.float32), 2, 4)
    assert c.shape == (1, 8) and c[0, 4:].tolist() == [0, 0, 0, 0] and lo[0, 1] == 7.0   # constant padded group
    assert sc[0, 1] == np.float32(1e-8)
    assert np.array_equal(o.clipped_group_dequant(c, lo, sc, 4, 5), np.array([[0, 3, 1, 2, 7]], np.float32))


def test_clipping_wins_on_a_single_outlier_group():
    """Seven values spread over [0, 1] and one at 1.2, 2 bits: shrinking the window lowers the error
    of the seven by more than it costs on the outlier, so the chosen scale is below range / levels."""
    x = np.array([[0.0, 0.15, 0.3, 0.45, 0.6, 0.75, 0.9, 1.2]], np.float32)
    _, _, sc1 = o.clipped_group_quant(x, 2, 8, (1.0,))
    _, _, sc = o.clipped_group_quant(x, 2, 8)
    e1 = np.square(_rt(x, 2, 8, (1.0,)) - x).sum()
    e = np.square(_rt(x, 2, 8) - x).sum()
    assert e <= e1 and (sc < sc1 or e == e1)


def test_ties_keep_the_first_alpha():
    """A constant group has zero error under every alpha: the first one is kept (argmin)."""
    _, lo, sc = o.clipped_group_quant(np.full((1, 4), 2.5, np.float32), 2, 4, (0.9, 1.0))
    assert lo[0, 0] == 2.5 and sc[0, 0] == np.float32(1e-8)


def test_validation_and_bytes():   # test_skvq.py guards and byte helpers
    with pytest.raises(ValueError, match="bits"):
        o.clipped_group_quant(np.zeros((1, 4), np.float32), 0, 4)
    with pytest.raises(ValueError, match="group_size"):
        o.clipped_group_quant(np.zeros((1, 4), np.float32), 2, 0)
    with pytest.raises(ValueError, match="alpha"):
        o.clipped_group_quant(np.zeros((1, 4), np.float32), 2, 4, (1.5,))
    assert o.skvq_compressed_bytes(10, 64, 2, 16) == 160 + 10 * 4 * 4
    assert o.skvq_fp16_bytes(10, 64) == 1280


def test_sum_order_sensitivity_is_rare():
    """How often the order of the error sum changes the chosen clip factor (the part of the
    selection no reference test fixes): well under 1 % of groups on seeded data."""
    x = _rows(512, 128, seed=11, channel_scales=_het_scales(128))
    for bits in (2, 4):
        _, lo_a, _ = o.clipped_group_quant(x, bits, 32)
        _, lo_b, _ = o.clipped_group_quant(x, bits, 32, pairwise=True)
        changed = float(np.mean(lo_a != lo_b))
        print(f"bits={bits}: {changed:.4%} of groups pick another clip factor under pairwise summation")
        assert changed < 0.01


def test_permutation_rules():   # test_skvq_cache.py:204-256
    rng = np.random.default_rng(7)
    k = (rng.standard_normal((1, 2, 16, 64)) * _het_scales(64)).astype(np.float16)
    perm, inv, err_id, err_cand = o.per_head_perms(k, 2, 4, 16, o.DEFAULT_ALPHA_GRID)
    for h in range(2):
        assert sorted(perm[h].tolist()) == list(range(64))
        assert np.array_equal(np.argsort(perm[h]), inv[h])
        x = k[0, h, 4:].astype(np.float32)
        if err_cand[h] < err_id[h]:
            assert np.array_equal(perm[h], np.argsort(x.max(0) - x.min(0), kind="stable"))
        else:
            assert np.array_equal(perm[h], np.arange(64))
    # equal ranges keep their channel order (stable sort), equal errors keep the identity
    flat = np.ones((1, 1, 8, 16), np.float16)
    p, i, *_ = o.per_head_perms(flat, 2, 0, 4, (1.0,))
    assert np.array_equal(p[0], np.arange(16)) and np.array_equal(i[0], np.arange(16))


def test_cache_model_path_independence_and_sinks():   # test_skvq_cache.py:87-140
    rng = np.random.default_rng(5)
    S = 53
    k = (rng.standard_normal((1, 2, S, 64)) * _het_scales(64)).astype(np.float16)
    v = (rng.standard_normal((1, 2, S, 64)) * _het_scales(64)).astype(np.float16)
    a = o.SKVQCacheModel(2, 2, 16, 16, 4)
    ka, va = a.update_and_fetch(k, v)
    b = o.SKVQCacheModel(2, 2, 16, 16, 4)
    for t in range(S):
        kb, vb = b.update_and_fetch(k[:, :, t:t + 1], v[:, :, t:t + 1])
    assert np.array_equal(ka, kb) and np.array_equal(va, vb) and a.q_end == b.q_end == 48
    assert np.array_equal(ka[:, :, :4], k[:, :, :4]) and np.array_equal(ka[:, :, 48:], k[:, :, 48:])
    assert not np.array_equal(ka[:, :, 4:48], k[:, :, 4:48])
