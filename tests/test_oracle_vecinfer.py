"""Pins the VecInfer oracle against brute force, closed forms and the tie rule
of the reference's Metal twin (veloxquant_mlx/metal/src/vecinfer_quantize.metal:26,
veloxquant_mlx/tests/allocators/test_vecinfer.py:21-54,133-153)."""

import numpy as np
import pytest

from oracle import cref, vecinfer as vi


def test_brute_force_loop_equals_vectorised_and_c():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 5, 16)).astype(np.float16)
    cb = rng.standard_normal((32, 4)).astype(np.float16)
    a = vi.quantize_vq_loop(x, cb, 4)
    b = vi.quantize_vq(x, cb, 4)
    c = cref.vq_assign(x.astype(np.float32), cb.astype(np.float32), 4)
    np.testing.assert_array_equal(a, b)
    np.testing.assert_array_equal(a, c)
    assert b.shape == (2, 5, 4) and b.dtype == np.int32


def test_duplicate_centroid_lowest_index_wins():
    rng = np.random.default_rng(1)
    cb = rng.standard_normal((16, 8)).astype(np.float32)
    cb[11] = cb[3]           # exact tie between 3 and 11 for every point nearest to them
    cb[7] = cb[3]
    x = np.tile(cb[3], (6, 1)) + rng.standard_normal((6, 8)).astype(np.float32) * 1e-3
    assert set(vi.quantize_vq(x, cb, 8).reshape(-1).tolist()) == {3}
    assert set(cref.vq_assign(x, cb, 8).reshape(-1).tolist()) == {3}


def test_points_equal_to_centroids_map_to_themselves():
    rng = np.random.default_rng(2)
    cb = rng.standard_normal((256, 8)).astype(np.float16)
    idx = vi.quantize_vq(cb.reshape(1, 256 * 8), cb, 8).reshape(-1)
    # distinct centroids: each row is its own nearest neighbour at distance 0
    np.testing.assert_array_equal(idx, np.arange(256))


def test_scalar_case_reduces_to_nearest_value():
    rng = np.random.default_rng(3)
    cb = np.sort(rng.standard_normal(64).astype(np.float32)).reshape(64, 1)
    x = rng.standard_normal((1000, 1)).astype(np.float32)
    idx = vi.quantize_vq(x, cb, 1).reshape(-1)
    mids = (cb[1:, 0].astype(np.float64) + cb[:-1, 0]) / 2
    expect = np.searchsorted(mids, x[:, 0].astype(np.float64))
    # identical away from the decision boundaries
    far = np.min(np.abs(x[:, :1].astype(np.float64) - mids[None, :]), axis=1) > 1e-5
    np.testing.assert_array_equal(idx[far], expect[far])


def test_distance_is_sequential_float32_sum():
    # a vector whose pairwise-tree sum and left-to-right sum differ in float32:
    # the oracle must follow the left-to-right order of the Metal twin
    x = np.array([[4096.0, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0]], np.float32)
    x[0, 0] = np.float32(4096.0)
    cb = np.zeros((2, 8), np.float32)
    d = vi._seq_sqdist(x, cb)[0, 0]
    seq = np.float32(0)
    for i in range(8):
        seq = np.float32(seq + np.float32(x[0, i] * x[0, i]))
    assert d == seq == np.float32(16777216.0)          # every +1 is absorbed
    tree = np.float32(np.float32(16777216.0 + 1.0) + np.float32(2.0)) + np.float32(4.0)
    assert tree != seq


def test_dequantize_and_lut():
    rng = np.random.default_rng(4)
    cb = rng.standard_normal((16, 4)).astype(np.float32)
    idx = rng.integers(0, 16, size=(3, 7, 8))
    out = vi.dequantize_vq(idx, cb)
    assert out.shape == (3, 7, 32)
    np.testing.assert_array_equal(out[1, 2, 4:8], cb[idx[1, 2, 1]])
    q = rng.standard_normal((3, 32)).astype(np.float32)
    lut = vi.compute_query_lut(q, cb, 4)
    assert lut.shape == (3, 8, 16)
    # LUT scoring == explicit dot with the reconstruction
    tok = idx[0, 0]
    np.testing.assert_allclose(lut[0, np.arange(8), tok].sum(), q[0] @ vi.dequantize_vq(tok[None], cb)[0], rtol=1e-5)


@pytest.mark.parametrize("d", [1, 2, 8, 64, 128, 256])
def test_hadamard_is_orthonormal_and_symmetric(d):
    H = vi.walsh_hadamard_matrix(d)
    np.testing.assert_allclose(H @ H.T, np.eye(d), atol=1e-5)
    np.testing.assert_array_equal(H, H.T)
    assert np.all(np.isclose(np.abs(H), 1 / np.sqrt(d), atol=1e-6))


def test_hadamard_rejects_non_power_of_two():
    with pytest.raises(ValueError, match="power of 2"):
        vi.walsh_hadamard_matrix(96)


def test_dual_transform_preserves_scores_including_gqa():
    rng = np.random.default_rng(5)
    D, Hkv, Hq = 64, 2, 8
    K = rng.standard_normal((1, Hkv, 9, D)).astype(np.float32)
    q = rng.standard_normal((1, Hq, 1, D)).astype(np.float32)
    sm = (np.abs(rng.standard_normal((Hkv, D))) + 0.5).astype(np.float32)
    H = vi.walsh_hadamard_matrix(D)
    Kt = vi.apply_dual_transform_keys(K, sm, H)
    qt = vi.apply_dual_transform_queries(q, sm, H)
    ref = np.einsum("bhqd,bhsd->bhqs", q, np.repeat(K, Hq // Hkv, 1))
    got = np.einsum("bhqd,bhsd->bhqs", qt, np.repeat(Kt, Hq // Hkv, 1))
    np.testing.assert_allclose(got, ref, atol=1e-3)


def test_calibrate_smooth_factors():
    k = np.array([[1.0, -4.0], [0.25, 9.0]], np.float32)
    np.testing.assert_allclose(vi.calibrate_smooth_factors(k), [1.0, 3.0])
    np.testing.assert_allclose(vi.calibrate_smooth_factors(np.zeros((3, 2), np.float32)), [0.01, 0.01], rtol=1e-6)


def test_encode_decode_keys_is_the_composition_and_inverts_on_centroid_points():
    """encode_decode_keys = transform, assignment, gather, inverse transform
    (veloxquant_mlx/cache/vecinfer_cache.py:313-356).  Pins: the Hadamard entries follow
    (-1)^popcount(a & b); keys built as (c @ H^T) * smooth from centroids come back as those
    centroids' indices with k_hat == keys; the transform agrees with a plain float32 loop."""
    rng = np.random.default_rng(0)
    D, sub, C = 32, 4, 16
    H = vi.walsh_hadamard_matrix(D)
    a = np.arange(D)
    par = np.array([[bin(x & y).count("1") & 1 for y in a] for x in a])
    np.testing.assert_array_equal(np.sign(H), 1 - 2 * par)
    assert len(set(np.abs(H).reshape(-1).tolist())) == 1
    cb = rng.standard_normal((C, sub)).astype(np.float32) * 3
    want = rng.integers(0, C, (1, 2, 5, D // sub))
    smooth = np.exp(rng.standard_normal((2, D))).astype(np.float32)
    keys = (vi.dequantize_vq(want, cb).astype(np.float64) @ H.T.astype(np.float64)) * smooth[:, None, :]
    k_tilde, idx, k_hat = vi.encode_decode_keys(keys.astype(np.float32), smooth, H, cb, sub)
    np.testing.assert_array_equal(idx, want)
    np.testing.assert_allclose(k_hat, keys, rtol=2e-6, atol=2e-6)
    loop = np.zeros_like(k_tilde)
    x = keys.astype(np.float32) / smooth[:, None, :]
    for b in range(D):
        for aa in range(D):
            loop[..., b] += x[..., aa] * H[aa, b]
    np.testing.assert_allclose(k_tilde, loop, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(k_tilde, vi.apply_dual_transform_keys(keys.astype(np.float32), smooth, H), rtol=1e-5, atol=1e-5)
