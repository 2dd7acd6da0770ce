"""Pins the attention oracle against library SDPA, closed-form special cases
and the causal properties the reference tests
(veloxquant_mlx/tests/metal/test_scalar_attend.py:85-115,
veloxquant_mlx/tests/metal/test_flash_prefill.py:34-44,100-115)."""

import numpy as np
import pytest
import torch

from oracle import attend, cref, kivi


def _inputs(B, H, Hkv, S, D, b, g, seed=0):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((B, H, 1, D)).astype(np.float16)
    kf = rng.standard_normal((B, Hkv, S, D)).astype(np.float32)
    vf = rng.standard_normal((B, Hkv, S, D)).astype(np.float32)
    kq = kivi.group_quant_codes(kf, -2, g, (1 << b) - 1)
    vq = kivi.group_quant_codes(vf, -1, g, (1 << b) - 1)
    return q, kq, vq, kf, vf


def test_single_slot_returns_its_value():
    q, kq, vq, _, _ = _inputs(1, 4, 2, 1, 64, 2, 32)
    out = attend.reference_attend(q, *kq, *vq, 32, 0.125)
    v_hat = kivi.group_dequant(*vq, -1, 32)
    np.testing.assert_allclose(out, np.repeat(v_hat, 2, axis=1), rtol=1e-6)


def test_zero_query_gives_mean_of_values():
    q, kq, vq, _, _ = _inputs(1, 4, 4, 96, 64, 4, 32)
    out = attend.reference_attend(np.zeros_like(q), *kq, *vq, 32, 0.125)
    v_hat = kivi.group_dequant(*vq, -1, 32)
    np.testing.assert_allclose(out[:, :, 0], v_hat.mean(axis=2), atol=1e-5)


@pytest.mark.parametrize("H,Hkv", [(8, 2), (32, 4), (32, 8), (4, 4)])
def test_matches_library_sdpa_on_reconstruction(H, Hkv):
    q, kq, vq, _, _ = _inputs(2, H, Hkv, 130, 128, 3, 32, seed=H + Hkv)
    out = attend.reference_attend(q, *kq, *vq, 32, 1 / np.sqrt(128))
    k_hat = torch.from_numpy(kivi.group_dequant(*kq, -2, 32)).repeat_interleave(H // Hkv, 1)
    v_hat = torch.from_numpy(kivi.group_dequant(*vq, -1, 32)).repeat_interleave(H // Hkv, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q.astype(np.float32)), k_hat, v_hat, scale=1 / np.sqrt(128))
    np.testing.assert_allclose(out, ref.numpy(), atol=2e-5)


def test_eight_bit_reduces_to_plain_attention():
    q, kq, vq, kf, vf = _inputs(1, 8, 2, 256, 128, 8, 32, seed=9)
    out = attend.reference_attend(q, *kq, *vq, 32, 1 / np.sqrt(128))
    plain = attend.sdpa(q, kf, vf, 1 / np.sqrt(128))
    assert np.max(np.abs(out - plain)) < 6e-3  # step ~7/255, averaged over many slots


def test_numpy_and_c_restatements_agree_with_tail_and_causal():
    rng = np.random.default_rng(11)
    q, kq, vq, _, _ = _inputs(2, 8, 2, 64, 64, 2, 32, seed=3)
    q = rng.standard_normal((2, 8, 5, 64)).astype(np.float16)
    kt = rng.standard_normal((2, 2, 7, 64)).astype(np.float16)
    vt = rng.standard_normal((2, 2, 7, 64)).astype(np.float16)
    for causal in (False, True):
        a = attend.kivi_attend(q, *kq, *vq, 32, kt, vt, 0.125, causal=causal)
        c = cref.attend(q, *kq, *vq, 32, 0.125, kt, vt, causal=causal)
        np.testing.assert_allclose(a, c, atol=1e-6)


def test_causal_matches_library_and_ignores_future_keys():
    rng = np.random.default_rng(5)
    B, H, Sq, Skv, D = 1, 2, 24, 40, 32
    q = rng.standard_normal((B, H, Sq, D)).astype(np.float16)
    k = rng.standard_normal((B, H, Skv, D)).astype(np.float16)
    v = rng.standard_normal((B, H, Skv, D)).astype(np.float16)
    out = attend.sdpa(q, k, v, 0.2, causal=True)
    mask = torch.ones(Sq, Skv, dtype=torch.bool).tril(diagonal=Skv - Sq)
    ref = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q.astype(np.float32)), torch.from_numpy(k.astype(np.float32)),
        torch.from_numpy(v.astype(np.float32)), attn_mask=mask, scale=0.2)
    np.testing.assert_allclose(out, ref.numpy(), atol=2e-5)
    k2, v2 = k.copy(), v.copy()
    k2[:, :, 30:] += 3.0
    v2[:, :, 30:] -= 2.0
    out2 = attend.sdpa(q, k2, v2, 0.2, causal=True)
    # query i sees slots <= 16 + i, so rows 0..13 cannot see slot 30
    np.testing.assert_array_equal(out[:, :, :14], out2[:, :, :14])
    assert np.abs(out[:, :, 14:] - out2[:, :, 14:]).max() > 1e-3


def test_chunked_prefill_sees_quantised_prefix_and_fp16_window():
    rng = np.random.default_rng(8)
    B, H, S, D = 1, 2, 96, 32
    q = rng.standard_normal((B, H, S, D)).astype(np.float16)
    k = rng.standard_normal((B, H, S, D)).astype(np.float16)
    v = rng.standard_normal((B, H, S, D)).astype(np.float16)
    out = attend.chunked_prefill(q, k, v, chunk=32, bits=2, group_size=8, residual_length=16, scale=0.2)
    # first chunk: boundary floor((32-16)/8)*8 = 16 -> rows 0..15 quantised, 16..31 exact
    kq = k.copy(); vq = v.copy()
    kq[:, :, :16] = kivi.quant_dequant_along(k[:, :, :16], -2, 8, 3)
    vq[:, :, :16] = kivi.quant_dequant_along(v[:, :, :16], -1, 8, 3)
    ref0 = attend.sdpa(q[:, :, :32], kq[:, :, :32], vq[:, :, :32], 0.2, causal=True, acc=np.float64)
    np.testing.assert_allclose(out[:, :, :32], ref0, atol=1e-6)
    # with a residual window longer than the sequence nothing is quantised
    out_fp = attend.chunked_prefill(q, k, v, chunk=32, bits=2, group_size=8, residual_length=512, scale=0.2)
    np.testing.assert_allclose(out_fp, attend.sdpa(q, k, v, 0.2, causal=True, acc=np.float64), atol=1e-6)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("window", [1, 5, 64])
def test_sliding_window_and_index_attention_match_library_sdpa(causal, window):
    """The window keeps slots q_abs-window+1 .. (veloxquant_mlx/tests/cache/test_vecinfer_fused_sdpa.py:105-113);
    the index form is plain attention over the gathered centroids (ibid. 80-115)."""
    from oracle import vecinfer
    rng = np.random.default_rng(window)
    B, Hq, Hkv, Sq, Skv, D, sub, C = 1, 4, 2, 6, 33, 16, 4, 32
    q = rng.standard_normal((B, Hq, Sq, D)).astype(np.float32)
    kcb = rng.standard_normal((C, sub)).astype(np.float32)
    vcb = rng.standard_normal((C, sub)).astype(np.float32)
    ki = rng.integers(0, C, (B, Hkv, Skv, D // sub))
    vi = rng.integers(0, C, (B, Hkv, Skv, D // sub))
    out = vecinfer.fused_sdpa(q, ki, kcb, vi, vcb, 0.3, causal=causal, sliding_window=window)
    k = torch.from_numpy(kcb)[torch.from_numpy(ki)].reshape(B, Hkv, Skv, D).repeat_interleave(Hq // Hkv, 1)
    v = torch.from_numpy(vcb)[torch.from_numpy(vi)].reshape(B, Hkv, Skv, D).repeat_interleave(Hq // Hkv, 1)
    mask = torch.zeros(Sq, Skv, dtype=torch.bool)
    for i in range(Sq):
        qa = Skv - Sq + i
        for j in range(Skv):
            mask[i, j] = (j <= qa or not causal) and j >= qa - window + 1
    ref = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q), k, v, attn_mask=mask, scale=0.3)
    np.testing.assert_allclose(out, ref.numpy(), atol=2e-5)
