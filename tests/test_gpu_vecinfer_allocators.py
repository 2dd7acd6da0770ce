"""The VecInfer building blocks of ``veloxquant_mlx_amd.allocators.vecinfer`` on the GPU:
smooth-factor calibration, the query look-up table and Lloyd training (whose assignment
step is the HIP nearest-centroid kernel).  Restates
veloxquant_mlx/tests/allocators/test_vecinfer.py:21-153 and the training checks of
veloxquant_mlx/allocators/vecinfer.py:190-278 on torch ROCm tensors; expected values come
from closed forms, from brute force in numpy and from the CPU oracle, never from the
functions under test."""

import numpy as np
import pytest
import torch

from oracle import vecinfer as ov
from tests._gpu import gpu, host, require_gpu, to_dev
from veloxquant_mlx_amd.allocators import vecinfer as A

pytestmark = gpu


def test_calibrate_smooth_factors_closed_form_and_floor():
    """lambda_i = sqrt(max_t |K[t, i]|), floored at sqrt(eps) (vecinfer.py:29-54)."""
    require_gpu()
    k = np.array([[1.0, -4.0, 0.0, 0.25],
                  [-9.0, 2.0, 0.0, -0.5],
                  [0.5, 3.0, 0.0, 0.125]], np.float32)
    got = host(A.calibrate_smooth_factors(to_dev(k)))
    np.testing.assert_allclose(got, [3.0, 2.0, 1e-2, np.sqrt(0.5)], rtol=1e-6)
    # an all-zero channel is floored at sqrt(eps), whatever eps
    got = host(A.calibrate_smooth_factors(to_dev(k), eps=1e-6))
    assert got[2] == pytest.approx(1e-3, rel=1e-6)
    # 3-D input [T, H, D]: the maximum runs over tokens only, one row of factors per head
    rng = np.random.default_rng(3)
    k3 = rng.standard_normal((50, 4, 32)).astype(np.float32)
    got3 = host(A.calibrate_smooth_factors(to_dev(k3)))
    assert got3.shape == (4, 32)
    np.testing.assert_allclose(got3, np.sqrt(np.abs(k3).max(axis=0)), rtol=1e-6)
    np.testing.assert_allclose(got3, ov.calibrate_smooth_factors(k3), rtol=1e-6)
    with pytest.raises(ValueError, match="2D or 3D"):
        A.calibrate_smooth_factors(to_dev(k3[0, 0]))


def test_compute_query_lut_matches_explicit_dot():
    """Summing LUT entries at a key's indices equals q . K_hat for the gathered keys
    (tests/allocators/test_vecinfer.py:133-153)."""
    require_gpu()
    rng = np.random.default_rng(0)
    sub, D = 4, 16
    cb = rng.standard_normal((8, sub)).astype(np.float32)
    q = rng.standard_normal((D,)).astype(np.float32)
    keys = rng.standard_normal((5, D)).astype(np.float32)
    idx = host(A.quantize_vq(to_dev(keys), to_dev(cb), sub))
    k_hat = host(A.dequantize_vq(to_dev(idx), to_dev(cb)))
    # the gather itself, by hand
    np.testing.assert_array_equal(k_hat, cb[idx].reshape(5, D))
    explicit = k_hat @ q
    lut = host(A.compute_query_lut(to_dev(q), to_dev(cb), sub))
    assert lut.shape == (D // sub, 8)
    via_lut = np.array([sum(lut[s, idx[t, s]] for s in range(D // sub)) for t in range(5)], np.float32)
    np.testing.assert_allclose(via_lut, explicit, atol=1e-4)
    # every entry is the dot product of one query slice with one centroid
    for s in range(D // sub):
        for c in range(8):
            assert lut[s, c] == pytest.approx(float(q[sub * s: sub * s + sub] @ cb[c]), abs=1e-5)


def test_compute_query_lut_batched_heads_and_errors():
    require_gpu()
    rng = np.random.default_rng(1)
    sub, D, C = 8, 64, 32
    cb = rng.standard_normal((C, sub)).astype(np.float32)
    q = rng.standard_normal((2, 6, 3, D)).astype(np.float32)
    lut = host(A.compute_query_lut(to_dev(q), to_dev(cb), sub))
    assert lut.shape == (2, 6, 3, D // sub, C)
    ref = np.einsum("bhqsd,cd->bhqsc", q.reshape(2, 6, 3, D // sub, sub), cb)
    np.testing.assert_allclose(lut, ref, atol=1e-4)
    np.testing.assert_allclose(lut, ov.compute_query_lut(q, cb, sub), atol=1e-4)
    with pytest.raises(ValueError, match="not divisible"):
        A.compute_query_lut(to_dev(q[..., :60]), to_dev(cb), sub)


def _inertia(x, cent):
    d2 = ((x[:, None, :] - cent[None, :, :]) ** 2).sum(-1)
    return float(d2.min(axis=1).sum())


def test_train_codebook_recovers_planted_clusters():
    """Well separated clusters: every centre is found to within the noise, and the inertia is the
    within-cluster scatter (vecinfer.py:190-278)."""
    require_gpu()
    rng = np.random.default_rng(5)
    centres = np.array([[10, 0, 0, 0], [0, 10, 0, 0], [0, 0, 10, 0], [0, 0, 0, 10],
                        [-10, 0, 0, 0], [0, -10, 0, 0], [0, 0, -10, 0], [0, 0, 0, -10]], np.float32)
    labels = rng.integers(0, 8, 4000)
    x = (centres[labels] + 0.1 * rng.standard_normal((4000, 4))).astype(np.float32)
    # Lloyd's iteration with a random start may merge two clusters; the planted optimum is a fixed
    # point, so a run that starts there must stay there
    best = None
    for seed in range(6):
        cent = host(A.train_codebook(to_dev(x), 8, max_iter=30, seed=seed))
        assert cent.shape == (8, 4) and np.isfinite(cent).all()
        val = _inertia(x, cent)
        best = val if best is None else min(best, val)
    planted = _inertia(x, np.stack([x[labels == c].mean(0) for c in range(8)]))
    assert best == pytest.approx(planted, rel=1e-3)
    assert planted < 4000 * 4 * 0.1 ** 2 * 1.2


def test_train_codebook_inertia_never_increases():
    """One more Lloyd iteration never raises the inertia: run the trainer with growing iteration
    caps from one start (same seed) and compare."""
    require_gpu()
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((3000, 8)) * np.exp(0.5 * rng.standard_normal(8))).astype(np.float32)
    vals = [_inertia(x, host(A.train_codebook(to_dev(x), 16, max_iter=it, seed=4))) for it in (1, 2, 4, 8, 16)]
    for a, b in zip(vals, vals[1:]):
        assert b <= a * (1 + 1e-6), vals
    assert vals[-1] < vals[0]
    # and the trained codebook beats a random one of the same size
    assert vals[-1] < _inertia(x, x[rng.permutation(3000)[:16]])


def test_train_codebook_fewer_samples_than_centroids():
    """n <= n_centroids: the samples are repeated to 2 n_centroids rows before the draw
    (vecinfer.py:236-243); every centroid ends up on a sample."""
    require_gpu()
    rng = np.random.default_rng(2)
    x = rng.standard_normal((5, 4)).astype(np.float32)
    cent = host(A.train_codebook(to_dev(x), 16, max_iter=5, seed=0))
    assert cent.shape == (16, 4) and np.isfinite(cent).all()
    d = np.abs(cent[:, None, :] - x[None, :, :]).max(-1).min(1)
    assert float(d.max()) < 1e-6
    with pytest.raises(ValueError, match="must be 2D"):
        A.train_codebook(to_dev(x[0]), 4)


def test_fp16_large_magnitudes_match_fp32_assignment():
    """Distances are float32 whatever the input type: keys of magnitude ~300 (whose squared
    distances overflow fp16) get the indices of their float32 copies
    (tests/allocators/test_vecinfer.py:122-130)."""
    require_gpu()
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((2000, 8)) * 300.0).astype(np.float32)
    cb = A.train_codebook(to_dev(x), 64, max_iter=10, seed=0)
    idx32 = host(A.quantize_vq(to_dev(x), cb, 8))
    idx16 = host(A.quantize_vq(to_dev(x, torch.float16), cb, 8))
    assert float((idx32 == idx16).mean()) > 0.99
    np.testing.assert_array_equal(idx32, ov.quantize_vq(x, host(cb), 8))
