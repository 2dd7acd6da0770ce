"""``method="kitty"`` on the GPU against ``oracle.kitty`` (cases of
veloxquant_mlx/tests/cache/test_kitty_cache.py and tests/quantizers/test_kitty_batched.py)."""

import numpy as np
import pytest
import torch

from oracle import kitty as okt
from tests._gpu import gpu, host, require_gpu, to_dev
from veloxquant_mlx_amd import kernels as K
from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory
from veloxquant_mlx_amd.cache.kitty_cache import KittyKVCache
from veloxquant_mlx_amd.core.exceptions import QuantizerConfigError
from veloxquant_mlx_amd.quantizers import kitty as qk

pytestmark = gpu


def _kv(B, H, S, D, seed):
    """Keys whose channels differ in spread by clear margins (the ranking is then not a matter of
    the last bits of a float32 variance), values plain."""
    rng = np.random.default_rng(seed)
    spread = np.exp(np.random.default_rng(99).permutation(D) / D * 3.0).astype(np.float32)
    return ((rng.standard_normal((B, H, S, D)) * spread).astype(np.float16),
            rng.standard_normal((B, H, S, D)).astype(np.float16))


@pytest.mark.parametrize("B,H,D,prefill,kw", [
    (1, 2, 64, 20, {}),                                                    # ragged last group
    (2, 2, 128, 100, {}),
    (1, 4, 128, 64, dict(kitty_hi_fraction=0.5, kitty_hi_bit=8, kitty_lo_bit=3, kitty_group_size=16)),
    (1, 1, 64, 32, dict(kitty_hi_fraction=0.0)),
    (1, 1, 64, 32, dict(kitty_hi_fraction=1.0)),
])
def test_cache_matches_the_model_bit_for_bit(B, H, D, prefill, kw):
    require_gpu()
    c = KVCacheFactory.create(KVCacheConfig(method="kitty", head_dim=D, **kw))
    assert isinstance(c, KittyKVCache)
    m = okt.KittyCacheModel(D, kw.get("kitty_hi_fraction", 0.25), kw.get("kitty_hi_bit", 4), kw.get("kitty_lo_bit", 2),
                            kw.get("kitty_group_size", 32))
    k, v = _kv(B, H, prefill, D, 1)
    ko, vo = c.update_and_fetch(to_dev(k), to_dev(v))
    km, vm = m.update_and_fetch(k, v)
    assert np.array_equal(host(ko), km) and np.array_equal(host(vo), vm)
    for step in range(6):
        k, v = _kv(B, H, 1, D, 10 + step)
        ko, vo = c.update_and_fetch(to_dev(k), to_dev(v))
        km, vm = m.update_and_fetch(k, v)
        assert ko.shape[2] == prefill + step + 1
        assert np.array_equal(host(ko), km) and np.array_equal(host(vo), vm)
    k, v = _kv(B, H, 40, D, 30)   # a later multi-token call is ranked by the running sums
    ko, _ = c.update_and_fetch(to_dev(k), to_dev(v))
    km, _ = m.update_and_fetch(k, v)
    assert np.array_equal(host(ko), km)
    np.testing.assert_allclose(host(c._key_sum), m.key_sum, rtol=1e-5, atol=1e-3)
    np.testing.assert_allclose(host(c._key_sq_sum), m.key_sq_sum, rtol=1e-5, atol=1e-2)
    assert (c.compressed_key_bytes, c.fp16_key_bytes, c.value_fp16_bytes) == \
        (m.compressed_key_bytes, m.fp16_key_bytes, m.value_fp16_bytes)
    assert c.compressed_key_bytes < c.fp16_key_bytes
    assert c.trim(40) == m.trim(40) == 40 and c.offset == m.keys.shape[2]
    np.testing.assert_allclose(host(c._key_sum), m.key_sum, rtol=1e-5, atol=1e-3)
    assert c.compressed_key_bytes == m.compressed_key_bytes
    assert c.trim(10 ** 6) == prefill + 6 and c._key_sum is None and c._n_keys == 0


def test_bfloat16_keys_round_through_float16():
    """The reference builds the reconstruction as float16 and casts it to the keys' dtype (kitty_cache.py:141-148)."""
    require_gpu()
    k, v = _kv(1, 2, 64, 128, 5)
    kb = torch.from_numpy(k.astype(np.float32)).to(torch.bfloat16)
    c = KVCacheFactory.create(KVCacheConfig(method="kitty", head_dim=128))
    ko, _ = c.update_and_fetch(kb.cuda(), to_dev(v).to(torch.bfloat16))
    m = okt.KittyCacheModel(128)
    km, _ = m.update_and_fetch(kb.float().numpy(), v)
    want = torch.from_numpy(km).to(torch.bfloat16)
    assert ko.dtype == torch.bfloat16 and torch.equal(ko.cpu(), want)


def test_quantizer_functions():
    require_gpu()
    data = np.random.default_rng(7).standard_normal((128, 64)).astype(np.float32)
    data[:, :8] *= 10.0
    hi, lo = qk.rank_channels_by_sensitivity(torch.from_numpy(data).cuda(), hi_fraction=0.125)
    assert hi == list(range(8)) and lo == list(range(8, 64))          # test_kitty_cache.py:110-123
    x = data.astype(np.float16)
    out = qk.quantize_mixed_channels(to_dev(x), hi, lo)
    mask = np.zeros((1, 64), bool)
    mask[0, :8] = True
    assert np.array_equal(host(out), okt.quantize_mixed_channels_batched(x[None], mask)[0])
    tie = qk.hi_mask_from_variance_batched(torch.ones((1, 4), device="cuda"), 0.5)
    assert tie.tolist() == [[True, True, False, False]]
    s = torch.from_numpy(data.sum(0)).cuda()
    sq = torch.from_numpy((data * data).sum(0)).cuda()
    np.testing.assert_allclose(host(qk.compute_running_variance(s, sq, 128)), np.var(data, axis=0), rtol=1e-4, atol=1e-5)
    assert not qk.compute_running_variance(s, sq, 1).any()


def test_configuration():
    require_gpu()
    c = KittyKVCache(KVCacheConfig(method="kitty", head_dim=64))
    assert c.assigned_avg_bits == 2.5 and (c.hi_fraction, c.hi_bit, c.lo_bit, c.group_size) == (0.25, 4, 2, 32)
    c0 = KittyKVCache(KVCacheConfig(method="kitty", head_dim=64, kitty_hi_fraction=0.0))
    assert abs(c0.assigned_avg_bits - (4 + 63 * 2) / 64) < 1e-9          # test_kitty_cache.py:248-262
    for bad in (1.5, -0.1):
        with pytest.raises(QuantizerConfigError, match="kitty_hi_fraction"):
            KittyKVCache(KVCacheConfig(method="kitty", head_dim=64, kitty_hi_fraction=bad))


@pytest.mark.gpu
@pytest.mark.parametrize("g,S", [(32, 200), (64, 192), (32, 31)])
def test_one_launch_mixed_round_trip_equals_two_round_trips_and_a_select(g, S):
    """``vq_kivi_quant_dequant_mixed`` (a level count per channel) against what it replaces: the hi-bit and the lo-bit
    round trip of the whole tensor and a per-channel select (kitty.py:138-169), bit for bit, with ragged last groups,
    for the bit pairs the cache uses and one whose level counts take the plain division."""
    require_gpu()
    rng = np.random.default_rng(g + S)
    N, D = 5, 128
    x = (rng.standard_normal((N, S, D)) * np.exp(rng.standard_normal(D))).astype(np.float16)
    mask = rng.random((N, D)) < 0.3
    mask[0] = False
    mask[1] = True
    xt, mt = to_dev(x), to_dev(mask)
    for lo, hi in ((3, 15), (1, 255), (5, 10)):
        got = K.kivi_group_quant_dequant_mixed(xt, mt, g, lo, hi)
        want = torch.where(mt[:, None, :], K.kivi_group_quant_dequant(xt, -2, g, hi), K.kivi_group_quant_dequant(xt, -2, g, lo))
        assert torch.equal(got, want), (lo, hi)
    with pytest.raises(Exception):
        K.kivi_group_quant_dequant_mixed(xt, mt, 128, 3, 15)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("N,S,D", [(3, 1000, 128), (2, 77, 64), (1, 5000, 256)])
def test_channel_variance_in_one_pass(dtype, N, S, D):
    """``vq_channel_moments`` against numpy's float64 variance of the same values, with a large common offset in some
    channels (where a float32 sum of squares would lose the variance)."""
    require_gpu()
    rng = np.random.default_rng(N + S + D)
    x = rng.standard_normal((N, S, D)) * np.exp(rng.standard_normal(D))
    x[..., ::7] += 40.0
    xt = to_dev(x.astype(np.float32)).to(dtype)
    want = np.var(xt.double().cpu().numpy(), axis=1)
    got = host(K.channel_variance(xt)).astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-9)


@pytest.mark.gpu
def test_hi_mask_kernel_equals_the_double_stable_argsort():
    """``vq_channel_hi_mask`` against the definition it replaces (argsort of -variance, stable, then the rank of
    every channel, kitty.py:112-135) on rows with many exact ties, zeros of both signs, infinities and NaNs, for
    every n_hi at a small width and a few at the others; and the oracle's mask on the rows without NaN."""
    require_gpu()
    g = torch.Generator().manual_seed(9)
    for D in (1, 7, 64, 128, 200, 1024):
        v = torch.randint(0, 6, (6, D), generator=g).float() * 0.25
        v[1] = torch.rand(D, generator=g)
        v[2, ::3] = -0.0
        if D > 4:
            v[3, 1] = float("nan"); v[3, D - 2] = float("nan"); v[4, 2] = float("inf"); v[4, 0] = float("inf")
        for n_hi in (range(0, D + 1) if D <= 7 else (1, 2, D // 4, D // 2, D - 1, D)):
            order = torch.argsort(-v, dim=-1, stable=True)
            want = torch.argsort(order, dim=-1, stable=True) < n_hi
            got = K.channel_hi_mask(v.to("cuda:0"), n_hi).cpu()
            assert torch.equal(got, want), (D, n_hi)
    v = torch.rand((5, 128), generator=g)
    v[:, 10:20] = v[:, 30:40]
    for frac in (0.125, 0.25, 0.5):
        assert np.array_equal(host(qk.hi_mask_from_variance_batched(v.to("cuda:0"), frac)), okt.hi_mask_from_variance(v.numpy(), frac))
    with pytest.raises(ValueError):
        K.channel_hi_mask(torch.zeros((2, 2048), device="cuda:0"), 3)


@pytest.mark.parametrize("D", [64, 48])       # 64: one-pass variance kernel; 48: torch.var of the float32 copy
def test_near_tie_and_tied_variances_rank_alike_on_both_paths(D):
    """Channels that hold +a and -a on alternate tokens: mean 0 and variance a^2 in every arithmetic (sums of
    equal powers of two times a 22-bit square stay exact), so the ranking cannot depend on how a path forms
    the variance.  The amplitudes are neighbouring fp16 numbers with exact repeats; equal variances go to
    the lower channel (kitty.py:61-64, 112-135)."""
    require_gpu()
    rng = np.random.default_rng(D)
    S, N = 64, 3
    ladder = [np.float16(1.25)]
    for _ in range(5):
        ladder.append(np.nextafter(ladder[-1], np.float16(2)))
    ladder = np.array(ladder, np.float16)
    amp = ladder[rng.integers(0, 6, (N, D))]
    sign = np.where(np.arange(S) % 2 == 0, 1, -1).astype(np.float16)
    keys = (amp[:, None, :] * sign[None, :, None]).astype(np.float16)
    var = host(qk.channel_variance_batched(to_dev(keys)))
    assert np.array_equal(var, amp.astype(np.float32) ** 2)
    for frac in (0.125, 0.25, 0.5):
        got = host(qk.hi_mask_from_variance_batched(qk.channel_variance_batched(to_dev(keys)), frac))
        want = okt.hi_mask_from_variance(var, frac)
        assert np.array_equal(got, want)
        n_hi = max(1, int(D * frac))
        for n in range(N):
            beat = (var[n][None, :] > var[n][:, None]) | ((var[n][None, :] == var[n][:, None]) & (np.arange(D)[None, :] < np.arange(D)[:, None]))
            assert np.array_equal(want[n], beat.sum(1) < n_hi)
