"""HIP VecInfer assignment / gather against the CPU oracle: indices bit-exact
(float32 distances, left-to-right sum, lowest index on ties).  Restates
veloxquant_mlx/tests/cache/test_vecinfer_metal_parity.py:140-167 and the shapes
of blogs/metal-kernels.md:150-157."""

import numpy as np
import pytest
import torch

from oracle import cref, vecinfer as ov
from tests._gpu import gpu, host, require_gpu, to_dev
from veloxquant_mlx_amd import kernels as K

pytestmark = gpu


def _keys(shape, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(shape).astype(np.float32)
    return (x * np.exp(rng.standard_normal(shape[-1])).astype(np.float32)).astype(np.float16), rng


@pytest.mark.parametrize("sub,nc,D", [(8, 256, 256), (4, 256, 128), (4, 4096, 128), (2, 16, 64), (16, 64, 128),
                                      (3, 50, 96), (1, 7, 8)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
def test_assign_bit_exact(sub, nc, D, dtype):
    require_gpu()
    x, rng = _keys((2, 3, 37, D), seed=sub * 1000 + nc)
    cb = rng.standard_normal((nc, sub)).astype(np.float16)
    xt, cbt = to_dev(x, dtype), to_dev(cb)
    got = K.vecinfer_quantize_metal(xt, cbt, sub)
    assert got.dtype == torch.int32 and got.shape == (2, 3, 37, D // sub)
    ref = ov.quantize_vq(host(xt), cb, sub)
    np.testing.assert_array_equal(host(got), ref)
    if nc <= 256:
        got8 = K.vecinfer_quantize_metal(xt, cbt, sub, index_dtype=torch.uint8)
        np.testing.assert_array_equal(host(got8), ref.astype(np.uint8))


def test_exact_ties_take_the_lowest_index():
    require_gpu()
    rng = np.random.default_rng(1)
    cb = rng.standard_normal((64, 8)).astype(np.float32)
    cb[40] = cb[9]
    cb[63] = cb[9]
    x = np.tile(cb[9], (100, 1)) + rng.standard_normal((100, 8)).astype(np.float32) * 1e-3
    got = host(K.vecinfer_quantize_metal(to_dev(x), to_dev(cb), 8))
    assert set(got.reshape(-1).tolist()) == {9}
    # symmetric tie: x exactly between two centroids along one axis
    cb2 = np.zeros((4, 2), np.float32)
    cb2[1] = [2, 0]; cb2[2] = [0, 2]; cb2[3] = [2, 2]
    x2 = np.array([[1, 0], [0, 1], [1, 1], [2, 1]], np.float32)
    got2 = host(K.vecinfer_quantize_metal(to_dev(x2), to_dev(cb2), 2)).reshape(-1)
    np.testing.assert_array_equal(got2, ov.quantize_vq(x2, cb2, 2).reshape(-1))
    assert got2.tolist() == [0, 0, 0, 1]


def test_config2_falcon_shape_full_size():
    """keys [4,4096,256] fp16 with outlier channels, 256 fp16 centroids of 8 dims:
    524,288 sub-vectors, every index equal to the brute-force C oracle."""
    require_gpu()
    x, rng = _keys((4, 4096, 256), seed=2)
    cb = rng.standard_normal((256, 8)).astype(np.float16)
    got = host(K.vecinfer_quantize_metal(to_dev(x), to_dev(cb), 8, index_dtype=torch.uint8))
    ref = cref.vq_assign(x.astype(np.float32), cb.astype(np.float32), 8)
    assert got.shape == (4, 4096, 32)
    np.testing.assert_array_equal(got, ref.astype(np.uint8))
    # the numpy restatement agrees on a slice, with the near-tie census the parity report quotes
    sl, margin = ov.quantize_vq(x[:1, :512], cb, 8, return_margin=True)
    np.testing.assert_array_equal(got[:1, :512], sl.astype(np.uint8))
    print(f"near-ties (<= 4 ulp of the best distance): {(margin <= 4 * np.spacing(np.float32(8.0))).sum()} of {margin.size}")


def test_dequant_gather_and_clamp():
    require_gpu()
    rng = np.random.default_rng(3)
    cb = rng.standard_normal((256, 8)).astype(np.float32)
    idx = rng.integers(0, 256, size=(2, 5, 16)).astype(np.int32)
    out = K.vecinfer_dequant_metal(to_dev(idx), to_dev(cb))
    np.testing.assert_array_equal(host(out), ov.dequantize_vq(idx, cb))
    out16 = K.vecinfer_dequant_metal(to_dev(idx.astype(np.uint8)), to_dev(cb), out_dtype=torch.float16)
    np.testing.assert_array_equal(host(out16), ov.dequantize_vq(idx, cb).astype(np.float16))
    bad = idx.copy(); bad[0, 0, 0] = 9999
    outc = host(K.vecinfer_dequant_metal(to_dev(bad), to_dev(cb)))
    np.testing.assert_array_equal(outc[0, 0, :8], cb[255])


def test_round_trip_idempotent_at_scale():
    """assign(gather(assign(x))) == assign(x) whenever centroids are distinct."""
    require_gpu()
    x, rng = _keys((2, 2048, 128), seed=4)
    cb = to_dev(rng.standard_normal((256, 4)).astype(np.float16))
    i1 = K.vecinfer_quantize_metal(to_dev(x), cb, 4)
    i2 = K.vecinfer_quantize_metal(K.vecinfer_dequant_metal(i1, cb), cb, 4)
    assert torch.equal(i1, i2)


def test_wrapper_errors():
    require_gpu()
    x = to_dev(np.zeros((4, 10), np.float16))
    cb = to_dev(np.zeros((8, 4), np.float16))
    with pytest.raises(ValueError, match="not divisible by sub_dim"):
        K.vecinfer_quantize_metal(x, cb, 4)
    with pytest.raises(ValueError, match=r"codebook must be \[n_centroids, 5\]"):
        K.vecinfer_quantize_metal(x, cb, 5)
    with pytest.raises(ValueError, match="codebook must be 2D"):
        K.vecinfer_dequant_metal(to_dev(np.zeros((2, 2), np.int32)), cb.reshape(-1))


# ------------------------------------------------ the MFMA filter's undecided cases
@pytest.mark.parametrize("sub,nc", [(8, 256), (8, 200), (4, 256), (8, 5), (4, 17)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
def test_mfma_filter_near_ties_follow_the_exact_rule(sub, nc, dtype):
    """Sub-vectors placed (almost) on the bisector of two or more centroids, where only the
    float32 rounding of the sequential rule decides: one ulp nudges either way, clusters of
    near-identical centroids, exact duplicates in several tracker positions."""
    require_gpu()
    rng = np.random.default_rng(sub * 7 + nc)
    cb = rng.standard_normal((nc, sub)).astype(np.float16).astype(np.float32)
    if nc >= 17:
        cb[3] = cb[16]; cb[nc - 1] = cb[16]            # triple duplicate across tiles and rows
        cb[5] = cb[4] + np.float32(2.0 ** -10)           # a cluster of near-identical centroids
        cb[6] = cb[4] - np.float32(2.0 ** -10)
        cb[7] = cb[4]
    cbt = to_dev(cb, torch.float32 if dtype == torch.float32 else torch.float16)
    cbh = host(cbt).astype(np.float32)
    n = 4096 + 37
    a = rng.integers(0, nc, n)
    b = rng.integers(0, nc, n)
    mid = 0.5 * (cbh[a] + cbh[b])
    x = mid + rng.standard_normal((n, sub)).astype(np.float32) * np.float32(1e-4) * (rng.integers(0, 3, (n, 1)) > 0)
    x[::5] = cbh[a[::5]]                                 # exactly on a centroid (duplicates tie)
    xt = to_dev(x.astype(np.float32), dtype)
    got = host(K.vecinfer_quantize_metal(xt, cbt, sub)).reshape(-1)
    ref = ov.quantize_vq(host(xt).astype(np.float32), cbh, sub).reshape(-1)
    np.testing.assert_array_equal(got, ref)


def test_mfma_filter_large_magnitudes_and_ragged_count():
    require_gpu()
    rng = np.random.default_rng(11)
    cb = (rng.standard_normal((256, 8)) * 30).astype(np.float16)
    for n in (1, 63, 64, 65, 1000):
        x = (rng.standard_normal((n, 8)) * np.exp(2 * rng.standard_normal(8))).astype(np.float16)
        got = host(K.vecinfer_quantize_metal(to_dev(x), to_dev(cb), 8)).reshape(-1)
        np.testing.assert_array_equal(got, ov.quantize_vq(x, cb, 8).reshape(-1))


# ---------------------------------------------------------------------------
# attention straight from the indices (look-up table + centroid histogram)
# ---------------------------------------------------------------------------

LUT_TOL = 2e-3   # max-abs against the float64 oracle; the reference's own bar is 1e-2
                 # (veloxquant_mlx/tests/cache/test_vecinfer_fused_sdpa.py:20)


def _lut_case(B, Hq, Hkv, Sq, S, D, sub_k, sub_v, C, seed, idx_dtype=np.uint8, cap=None, q_scale=1.0):
    rng = np.random.default_rng(seed)
    cap = cap or S
    q = (rng.standard_normal((B, Hq, Sq, D)) * q_scale).astype(np.float32)
    kcb = rng.standard_normal((C, sub_k)).astype(np.float32)
    vcb = rng.standard_normal((C, sub_v)).astype(np.float32)
    ki = rng.integers(0, C, (B, Hkv, cap, D // sub_k)).astype(idx_dtype)
    vi = rng.integers(0, C, (B, Hkv, cap, D // sub_v)).astype(idx_dtype)
    return q, ki, kcb, vi, vcb


def _lut_run(q, ki, kcb, vi, vcb, scale, q_dtype=torch.float32, cb_dtype=torch.float32, **kw):
    return host(K.metal_fused_sdpa(to_dev(q, q_dtype), to_dev(ki), to_dev(kcb, cb_dtype), to_dev(vi),
                                   to_dev(vcb, cb_dtype), scale, **kw)).astype(np.float32)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,Hq,Hkv,Sq,S,D,sub,C", [
    (1, 4, 4, 1, 128, 64, 4, 256),       # the reference's default case (test_vecinfer_fused_sdpa.py:120-131)
    (1, 32, 8, 1, 256, 128, 8, 256),     # GQA 32/8 (ibid. 172-184)
    (1, 4, 4, 8, 128, 64, 4, 256),       # S_q = 8 (ibid. 218-228)
    (1, 4, 4, 1, 4096, 64, 4, 256),      # long context (ibid. 206-216)
    (2, 8, 2, 5, 777, 128, 8, 256),      # ragged length, several query rows per kv head
    (1, 8, 8, 1, 1500, 256, 16, 200),    # D = 256, fewer centroids
    (1, 2, 1, 3, 300, 96, 8, 17),        # n_sub = 12
])
def test_lut_attention_matches_the_gather_oracle(B, Hq, Hkv, Sq, S, D, sub, C, causal):
    require_gpu()
    q, ki, kcb, vi, vcb = _lut_case(B, Hq, Hkv, Sq, S, D, sub, sub, C, seed=S + D + Sq)
    scale = 1.0 / np.sqrt(D)
    ref = ov.fused_sdpa(q, ki, kcb, vi, vcb, scale, causal=causal)
    got = _lut_run(q, ki, kcb, vi, vcb, scale, causal=causal)
    assert got.shape == ref.shape
    assert np.max(np.abs(got - ref)) < LUT_TOL
    # 32-bit indices take the word path; same answer
    got32 = _lut_run(q, ki.astype(np.int32), kcb, vi.astype(np.int32), vcb, scale, causal=causal)
    assert np.max(np.abs(got32 - ref)) < LUT_TOL


@pytest.mark.parametrize("S", [1, 2])
def test_lut_attention_one_and_two_tokens(S):
    """veloxquant_mlx/tests/cache/test_vecinfer_fused_sdpa.py:186-204"""
    require_gpu()
    q, ki, kcb, vi, vcb = _lut_case(1, 4, 4, 1, S, 64, 4, 4, 256, seed=S)
    ref = ov.fused_sdpa(q, ki, kcb, vi, vcb, 0.125)
    assert np.max(np.abs(_lut_run(q, ki, kcb, vi, vcb, 0.125) - ref)) < LUT_TOL
    if S == 1:   # one token: the output is that token's value, whatever the query
        np.testing.assert_allclose(_lut_run(q, ki, kcb, vi, vcb, 0.125), ov.dequantize_vq(vi, vcb)[:, :, :1], atol=1e-6)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Sq,S,window", [(1, 256, 64), (8, 256, 64), (4, 1300, 100), (3, 40, 64), (2, 600, 1)])
def test_lut_attention_sliding_window(Sq, S, window, causal):
    """window mask of veloxquant_mlx/tests/cache/test_vecinfer_fused_sdpa.py:105-113, 155-170"""
    require_gpu()
    q, ki, kcb, vi, vcb = _lut_case(1, 4, 2, Sq, S, 64, 4, 4, 256, seed=window + Sq)
    ref = ov.fused_sdpa(q, ki, kcb, vi, vcb, 0.125, causal=causal, sliding_window=window)
    got = _lut_run(q, ki, kcb, vi, vcb, 0.125, causal=causal, sliding_window=window)
    assert np.max(np.abs(got - ref)) < LUT_TOL
    if window == 1 and causal:   # each query sees only its own position
        vh = ov.dequantize_vq(vi, vcb)
        np.testing.assert_allclose(got[0, 0], vh[0, 0, S - Sq:], atol=1e-6)


def test_lut_attention_mixed_sub_dims_dtypes_and_a_prefix_of_the_buffer():
    require_gpu()
    # keys in 8-wide, values in 4-wide sub-vectors; only the first 333 of 512 rows are tokens
    q, ki, kcb, vi, vcb = _lut_case(2, 8, 4, 2, 333, 128, 8, 4, 64, seed=5, cap=512)
    scale = 0.1
    ref = ov.fused_sdpa(q, ki[:, :, :333], kcb, vi[:, :, :333], vcb, scale)
    assert np.max(np.abs(_lut_run(q, ki, kcb, vi, vcb, scale, n_tokens=333) - ref)) < LUT_TOL
    # fp16 queries, codebooks and output: compare on the rounded operands
    q16, kcb16, vcb16 = (x.astype(np.float16).astype(np.float32) for x in (q, kcb, vcb))
    ref16 = ov.fused_sdpa(q16, ki[:, :, :333], kcb16, vi[:, :, :333], vcb16, scale)
    got16 = _lut_run(q, ki, kcb, vi, vcb, scale, q_dtype=torch.float16, cb_dtype=torch.float16, n_tokens=333)
    assert np.max(np.abs(got16 - ref16)) < LUT_TOL
    gotbf = host(K.metal_fused_sdpa(to_dev(q16), to_dev(ki), to_dev(kcb16), to_dev(vi), to_dev(vcb16), scale,
                                    n_tokens=333, out_dtype=torch.bfloat16).float())
    assert np.max(np.abs(gotbf - ref16)) < 2e-2   # bf16 output rounding


def test_lut_attention_properties():
    require_gpu()
    q, ki, kcb, vi, vcb = _lut_case(1, 8, 2, 4, 2000, 128, 8, 8, 256, seed=9)
    scale = 1.0 / np.sqrt(128)
    base = _lut_run(q, ki, kcb, vi, vcb, scale)
    # the token split must not matter
    for ns in (1, 2, 3, 4):
        assert np.max(np.abs(_lut_run(q, ki, kcb, vi, vcb, scale, num_splits=ns) - base)) < 1e-4
    # causal: the first query position cannot see the last three tokens
    ki2, vi2 = ki.copy(), vi.copy()
    ki2[:, :, -3:] += 7      # uint8 wraps inside the 256 centroids
    vi2[:, :, -3:] += 11
    pert = _lut_run(q, ki2, kcb, vi2, vcb, scale)
    assert np.max(np.abs(pert[:, :, 0] - base[:, :, 0])) < 1e-5
    assert np.max(np.abs(pert[:, :, 3] - base[:, :, 3])) > 1e-4
    # zero query: uniform weights, so the mean of the decoded values
    z = _lut_run(np.zeros_like(q[:, :, :1]), ki, kcb, vi, vcb, scale)
    np.testing.assert_allclose(z[0, 0, 0], ov.dequantize_vq(vi, vcb)[0, 0].mean(0), atol=1e-5)
    # large logits: a softmax that does not overflow
    big = _lut_run(q * 40, ki, kcb, vi, vcb, 1.0)
    ref = ov.fused_sdpa(q * 40, ki, kcb, vi, vcb, 1.0)
    assert np.isfinite(big).all() and np.max(np.abs(big - ref)) < LUT_TOL


def test_lut_attention_errors():
    """messages of veloxquant_mlx/metal/fused_sdpa.py:229-248 plus this kernel's own limits"""
    require_gpu()
    q, ki, kcb, vi, vcb = _lut_case(1, 4, 4, 1, 32, 64, 4, 4, 256, seed=1)
    t = lambda *xs: [to_dev(x) for x in xs]
    with pytest.raises(ValueError, match="must equal n_sub"):
        K.metal_fused_sdpa(*t(q[..., :60], ki, kcb, vi, vcb), 0.1)
    with pytest.raises(ValueError, match="same n_centroids"):
        K.metal_fused_sdpa(*t(q, ki, kcb, vi, vcb[:128]), 0.1)
    with pytest.raises(ValueError, match="multiple of H_kv"):
        K.metal_fused_sdpa(*t(np.concatenate([q, q[:, :1]], 1), ki, kcb, vi, vcb), 0.1)
    big = np.random.default_rng(0).standard_normal((512, 4)).astype(np.float32)
    with pytest.raises(ValueError, match="exceeds 256"):
        K.metal_fused_sdpa(*t(q, ki.astype(np.int32), big, vi.astype(np.int32), big), 0.1)
    with pytest.raises(ValueError, match="S_q"):
        K.metal_fused_sdpa(*t(np.repeat(q, 40, 2), ki, kcb, vi, vcb), 0.1, causal=True)
    with pytest.raises(RuntimeError, match="ROCm device"):
        K.metal_fused_sdpa(torch.from_numpy(q), *t(ki, kcb, vi, vcb), 0.1)


def test_lut_attention_many_weights_below_one_unit_still_count():
    """One dominant token and thousands whose weights are each below the resolution of the
    integer histogram (2^-18 of the largest weight in blocks of 8192 tokens): their total is a
    few percent of the sum and must not be rounded away."""
    require_gpu()
    rng = np.random.default_rng(3)
    B, H, S, D, sub, C = 16, 8, 8192, 64, 4, 256
    kcb = (rng.standard_normal((C, sub)) * 0.05).astype(np.float32)
    kcb[7] = [3.0, -3.0, 3.0, -3.0]
    vcb = rng.standard_normal((C, sub)).astype(np.float32)
    ki = rng.integers(8, C, (B, H, S, D // sub)).astype(np.uint8)
    vi = rng.integers(0, C, (B, H, S, D // sub)).astype(np.uint8)
    ki[:, :, 100] = 7
    q = np.tile(kcb[7], D // sub)[None, None, None, :].repeat(B, 0).repeat(H, 1).astype(np.float32)
    # the dominant score is 16 * 36 * scale, the others are near zero: a gap of about 13.5 nats
    scale = 13.5 / (16 * 36)
    ref = ov.fused_sdpa(q, ki, kcb, vi, vcb, scale)
    w_small = np.exp(-13.5) * (S - 1)
    assert 0.005 < w_small < 0.05 and np.exp(-13.5) * 2 ** 18 < 0.5
    got = _lut_run(q, ki, kcb, vi, vcb, scale)
    dom = ov.dequantize_vq(vi, vcb)[:, :, 100:101]
    assert np.max(np.abs(ref - dom)) > 5e-3          # the small weights matter at the tolerance below
    assert np.max(np.abs(got - ref)) < 2e-4


# ---------------------------------------------------------------------------
# fused key encode (+ decode): smooth, Walsh-Hadamard transform, assignment, way back
# ---------------------------------------------------------------------------

def _gap_to_second(k_tilde, cb, sub):
    """relative gap between the two smallest squared distances of every sub-vector"""
    x = k_tilde.reshape(-1, sub).astype(np.float64)
    d = ((x[:, None, :] - cb[None].astype(np.float64)) ** 2).sum(-1)
    d.sort(axis=1)
    return ((d[:, 1] - d[:, 0]) / np.maximum(d[:, 1], 1e-30)).reshape(k_tilde.shape[:-1] + (-1,))


@pytest.mark.parametrize("D,sub", [(64, 8), (128, 8), (256, 8), (512, 8), (32, 4), (64, 4), (128, 4), (256, 4)])
def test_encode_keys_on_integer_keys_is_exact(D, sub):
    """Integer keys and power-of-two smoothing factors: every partial sum of the transform is
    exact in float32 whatever its order, so the transformed keys, hence the indices, must equal
    the oracle's bit for bit."""
    require_gpu()
    rng = np.random.default_rng(D + sub)
    B, Hh, S, C = 2, 3, 21, 200
    keys = rng.integers(-8, 9, (B, Hh, S, D)).astype(np.float16)
    smooth = (2.0 ** rng.integers(-2, 3, (Hh, D))).astype(np.float32)
    Hm = ov.walsh_hadamard_matrix(D)
    cb = rng.standard_normal((C, sub)).astype(np.float32)
    kt_ref, idx_ref, khat_ref = ov.encode_decode_keys(keys, smooth, Hm, cb, sub)
    k_hat, idx, k_tilde = K.vecinfer_encode_decode_metal(to_dev(keys), to_dev(cb), sub, to_dev(Hm), to_dev(smooth),
                                                          want_k_tilde=True)
    np.testing.assert_array_equal(host(k_tilde), kt_ref)
    np.testing.assert_array_equal(host(idx), idx_ref)
    assert k_hat.dtype == torch.float16 and k_hat.shape == keys.shape
    np.testing.assert_allclose(host(k_hat).astype(np.float32), khat_ref, rtol=1.5e-3, atol=1e-3)
    # indices only, one byte each
    none, idx8 = K.vecinfer_encode_decode_metal(to_dev(keys), to_dev(cb), sub, to_dev(Hm), to_dev(smooth),
                                                index_dtype=torch.uint8, want_k_hat=False)
    assert none is None
    np.testing.assert_array_equal(host(idx8), idx_ref.astype(np.uint8))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("smooth_rows", [None, 1, "heads", "vector"])
def test_encode_keys_random_keys(dtype, smooth_rows):
    require_gpu()
    rng = np.random.default_rng(11)
    B, Hh, S, D, sub, C = 2, 4, 333, 128, 8, 256
    keys_t = to_dev((rng.standard_normal((B, Hh, S, D)) * np.exp(rng.standard_normal(D))).astype(np.float32), dtype)
    keys = host(keys_t).astype(np.float32)
    smooth = {None: None, 1: np.exp(rng.standard_normal((1, D)) * 0.5), "heads": np.exp(rng.standard_normal((Hh, D)) * 0.5),
              "vector": np.exp(rng.standard_normal(D) * 0.5)}[smooth_rows]
    smooth = None if smooth is None else smooth.astype(np.float32)
    Hm = ov.walsh_hadamard_matrix(D)
    cb = rng.standard_normal((C, sub)).astype(np.float32)
    kt_ref, idx_ref, _ = ov.encode_decode_keys(keys, smooth, Hm, cb, sub)
    k_hat, idx, k_tilde = K.vecinfer_encode_decode_metal(keys_t, to_dev(cb), sub, to_dev(Hm),
                                                          None if smooth is None else to_dev(smooth), want_k_tilde=True)
    kt, idx = host(k_tilde), host(idx)
    # the transform: float32 butterflies against the float64 product
    assert np.max(np.abs(kt - kt_ref)) <= 2e-6 * np.max(np.abs(kt_ref))
    # the assignment is exact on the kernel's own transformed keys
    np.testing.assert_array_equal(idx, ov.quantize_vq(kt, cb, sub))
    # against the oracle's transformed keys only near ties may differ
    diff = idx != idx_ref
    assert diff.mean() < 1e-3
    if diff.any():
        assert _gap_to_second(kt_ref, cb, sub)[diff].max() < 1e-4
    # the way back, from the kernel's own indices
    sm = 1.0 if smooth is None else (smooth[:, None, :] if smooth.ndim == 2 and smooth.shape[0] == Hh else smooth.reshape(-1, D)[0])
    back = (ov.dequantize_vq(idx, cb).astype(np.float64) @ Hm.T.astype(np.float64)) * sm
    tol = {torch.float16: 1.5e-3, torch.bfloat16: 1e-2, torch.float32: 1e-5}[dtype]
    assert k_hat.dtype == dtype
    np.testing.assert_allclose(host(k_hat).astype(np.float64), back, rtol=tol, atol=tol)


def test_encode_keys_other_shapes_take_the_composition():
    """sub_dim 16, a non-Hadamard matrix, more than 256 centroids: same contract through the
    matrix product and the assignment / gather kernels."""
    require_gpu()
    rng = np.random.default_rng(2)
    keys = rng.standard_normal((1, 2, 40, 64)).astype(np.float16)
    Hm = ov.walsh_hadamard_matrix(64)
    for sub, C, Hmat in ((16, 64, Hm), (8, 300, Hm), (8, 64, np.linalg.qr(rng.standard_normal((64, 64)))[0].astype(np.float32))):
        cb = rng.standard_normal((C, sub)).astype(np.float32)
        k_hat, idx, k_tilde = K.vecinfer_encode_decode_metal(to_dev(keys), to_dev(cb), sub, to_dev(Hmat), want_k_tilde=True)
        np.testing.assert_array_equal(host(idx), ov.quantize_vq(host(k_tilde), cb, sub))
        np.testing.assert_allclose(host(k_tilde), keys.astype(np.float32) @ Hmat, rtol=1e-4, atol=1e-4)
        back = ov.dequantize_vq(host(idx), cb) @ Hmat.T
        np.testing.assert_allclose(host(k_hat).astype(np.float32), back, rtol=2e-3, atol=2e-3)
    v_hat, v_idx = K.vecinfer_encode_decode_simple_metal(to_dev(keys), to_dev(cb), 8)
    np.testing.assert_array_equal(host(v_idx), ov.quantize_vq(keys, cb, 8))
    np.testing.assert_allclose(host(v_hat).astype(np.float32), ov.dequantize_vq(host(v_idx), cb), rtol=1e-3, atol=1e-3)
    with pytest.raises(ValueError, match="must be 4D"):
        K.vecinfer_encode_decode_metal(to_dev(keys[0]), to_dev(cb), 8, to_dev(Hm))
    with pytest.raises(ValueError, match="not divisible"):
        K.vecinfer_encode_decode_metal(to_dev(keys), to_dev(cb), 7, to_dev(Hm))
