"""``method="zipcache"`` on the GPU against ``oracle.zipcache`` (cases of
veloxquant_mlx/tests/cache/test_zipcache_cache.py); reconstructions bit for bit."""

import numpy as np
import pytest
import torch

from oracle import zipcache as oz
from tests._gpu import gpu, host, require_gpu, to_dev
from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory
from veloxquant_mlx_amd import kernels as K
from veloxquant_mlx_amd.cache.zipcache_cache import ZipCacheKVCache

pytestmark = gpu


def _kv(B, H, S, D, seed):
    rng = np.random.default_rng(seed)
    amp = (1.0 + 0.05 * rng.permutation(S)).astype(np.float32)[None, None, :, None]
    return ((rng.standard_normal((B, H, S, D)).astype(np.float32) * amp).astype(np.float16),
            rng.standard_normal((B, H, S, D)).astype(np.float16))


def _make(**kw):
    return KVCacheFactory.create(KVCacheConfig(method="zipcache", head_dim=kw.pop("head_dim", 64), **kw))


@pytest.mark.parametrize("B,H,S,D,kw", [
    (1, 2, 64, 64, {}),
    (2, 3, 50, 128, dict(zipcache_hi_bits=8, zipcache_lo_bits=3, zipcache_hi_fraction=0.5, zipcache_group_size=16)),
    (1, 2, 33, 64, dict(zipcache_hi_fraction=0.0)),
    (1, 2, 33, 64, dict(zipcache_hi_fraction=1.0)),
    (1, 4, 200, 128, dict(zipcache_quantize_values=False)),
])
def test_cache_matches_the_model_bit_for_bit(B, H, S, D, kw):
    require_gpu()
    c = _make(head_dim=D, **kw)
    assert isinstance(c, ZipCacheKVCache) and not hasattr(c, "bits")
    hb, lb = kw.get("zipcache_hi_bits", 4), kw.get("zipcache_lo_bits", 2)
    fr, gs = kw.get("zipcache_hi_fraction", 0.2), kw.get("zipcache_group_size", 32)
    k, v = _kv(B, H, S, D, seed=S)
    ko, vo = c.update_and_fetch(to_dev(k), to_dev(v))
    kr, _, (kc, kb, kf) = oz.compress(k, True, hb, lb, fr, gs)
    assert ko.dtype == torch.float16 and np.array_equal(host(ko).view(np.uint16), kr.view(np.uint16))
    assert (c.compressed_key_bytes, c.baseline_key_bytes, c.fp16_key_bytes) == (kc, kb, kf)
    if kw.get("zipcache_quantize_values", True):
        vr, _, (vc, vb, vf) = oz.compress(v, False, hb, lb, fr, gs)
        assert np.array_equal(host(vo).view(np.uint16), vr.view(np.uint16))
        assert (c.compressed_value_bytes, c.baseline_value_bytes, c.fp16_value_bytes) == (vc, vb, vf)
    else:
        assert np.array_equal(host(vo), v) and c.compressed_value_bytes == 0 and c.fp16_value_bytes > 0
    assert c.baseline_key_bytes <= c.compressed_key_bytes < c.fp16_key_bytes and c.compression_ratio > 1.0
    # decode steps: a single token is its own block (one group, exact at any bit width >= 1 only when constant)
    for t in range(3):
        k1, v1 = _kv(B, H, 1, D, seed=100 + t)
        ko, vo = c.update_and_fetch(to_dev(k1), to_dev(v1))
        assert np.array_equal(host(ko)[:, :, -1:].view(np.uint16), oz.compress(k1, True, hb, lb, fr, gs)[0].view(np.uint16))
    assert ko.shape[2] == S + 3 and len(c._runs) == 2 and (c._runs[-1].unit, c._runs[-1].end - c._runs[-1].start) == (1, 3)


def test_trim_takes_charges_back_and_nan_chunk_is_reported_by_the_next_call():
    require_gpu()
    c = _make()
    k, v = _kv(1, 2, 32, 64, seed=1)
    c.update_and_fetch(to_dev(k), to_dev(v))
    after_prefill = (c.compressed_key_bytes, c.fp16_key_bytes)
    for t in range(4):
        c.update_and_fetch(*map(to_dev, _kv(1, 2, 1, 64, seed=50 + t)))
    assert c.trim(4) == 4 and (c.compressed_key_bytes, c.fp16_key_bytes) == after_prefill and c.offset == 32
    assert c.trim(16) == 16 and c.fp16_key_bytes == after_prefill[1] // 2     # pro-rated
    bad = k.copy()
    bad[0, 0, 3, 5] = np.nan
    c2 = _make()
    c2.update_and_fetch(to_dev(bad), to_dev(v))
    with pytest.raises(ValueError, match="NaN or Inf"):
        c2.update_and_fetch(*map(to_dev, _kv(1, 2, 1, 64, seed=9)))
    assert c2.offset == 0 and c2.fp16_key_bytes == 0


def test_validation():
    require_gpu()
    for bad, what in ((dict(zipcache_hi_fraction=1.5), "zipcache_hi_fraction"), (dict(zipcache_hi_fraction=-0.1), "zipcache_hi_fraction"),
                      (dict(zipcache_hi_bits=9), "zipcache_hi_bits"), (dict(zipcache_lo_bits=0), "zipcache_lo_bits"),
                      (dict(zipcache_hi_bits=2, zipcache_lo_bits=4), "must not exceed"),
                      (dict(zipcache_group_size=0), "zipcache_group_size"), (dict(zipcache_quantize_values=1), "zipcache_quantize_values")):
        with pytest.raises(ValueError, match=what):
            _make(**bad)
    with pytest.raises(ValueError, match=r"\[B, H, S, D\]"):
        _make()._compress(torch.zeros((2, 4, 8), device="cuda:0"), True)


def test_row_norms_kernel_matches_float64():
    """``vq_row_norms``: float32 norms of fp16 / bf16 / float32 rows at the three head sizes, within float32
    rounding of the float64 value (the routing only needs their order; exact ties are broken by position)."""
    require_gpu()
    rng = np.random.default_rng(3)
    for D in (64, 128, 256):
        for dt in (torch.float16, torch.bfloat16, torch.float32):
            x = to_dev(rng.standard_normal((3, 5, 77, D)).astype(np.float32) * 4, dt)
            got = host(K.row_norms(x))
            want = np.sqrt((host(x).astype(np.float64) ** 2).sum(-1))
            assert got.shape == (3, 5, 77) and np.max(np.abs(got - want) / want) < 1e-6


def test_routing_kernel_equals_the_stable_sorts():
    """``vq_zip_route`` against the reference's definition (two stable argsorts for the mask, a third for the order,
    zipcache_cache.py:106-116, 186-190): norms with many exact ties, zeros, one NaN, lengths that do not divide the
    block, every block size from 1 to S - 1 at the small lengths."""
    require_gpu()
    g = torch.Generator().manual_seed(4)
    for S in (2, 7, 255, 256, 257, 1000, 2048, 2049, 5000, 8192, 8193):   # 8 and 32 norms a thread in registers, then the walk over memory
        norms = torch.randint(0, 9, (5, S), generator=g).float() * 0.37
        norms[1] = torch.rand(S, generator=g)
        if S > 10:
            norms[2, 5] = float("nan")
        for n_hi in (range(1, S) if S <= 7 else (1, 2, S // 5, S // 2, S - 1)):
            clean = torch.nan_to_num(norms, nan=float("inf"))       # the sorts put a NaN last, the bit order above inf
            rank = torch.argsort(torch.argsort(clean, dim=-1, stable=True), dim=-1, stable=True)
            want = torch.argsort((rank >= S - n_hi).to(torch.int32), dim=-1, stable=True)
            got = K.zip_route(norms.to("cuda:0"), n_hi).cpu().long()
            assert torch.equal(got, want), (S, n_hi)


@pytest.mark.parametrize("D", [128, 96])      # 128: norms and routing in the kernels; 96: the torch path
def test_near_tie_and_tied_norms_route_alike_on_both_paths(D):
    """Rows with one non-zero element: its square has 22 significant bits, so every summation order and
    float width gives the norm |x| exactly and the routing cannot depend on how a path rounds.  The values
    are neighbouring fp16 numbers (near ties, one unit in the last place apart) with exact repeats among
    them; on equal norms the later row goes to the high block (zipcache_cache.py:106-116), and both
    paths must reproduce the model's reconstruction bit for bit and its norms exactly."""
    require_gpu()
    B, H, S = 1, 3, 96
    rng = np.random.default_rng(D)
    base = np.float16(1.5)
    ladder = np.array([base] * 8, np.float16)
    for i in range(1, 8):
        ladder[i] = np.nextafter(ladder[i - 1], np.float16(2))
    k = np.zeros((B, H, S, D), np.float16)
    for h in range(H):
        vals = ladder[rng.integers(0, 8, S)]                       # many exact ties, neighbours everywhere
        cols = rng.integers(0, D, S)
        k[0, h, np.arange(S), cols] = vals * rng.choice(np.array([-1, 1], np.float16), S)
    c = _make(head_dim=D, zipcache_hi_fraction=0.3)
    got, norms, _ = c._compress(to_dev(k), True)
    want, wnorms, _ = oz.compress(k, True, 4, 2, 0.3, 32)
    assert np.array_equal(host(norms), wnorms)
    assert np.array_equal(host(norms).reshape(H, S), np.abs(k.astype(np.float32)).max(-1)[0])
    assert np.array_equal(host(got).view(np.uint16), want.view(np.uint16))
    # the tie rule itself, stated without a sort: a row is in the high block iff fewer than n_hi rows
    # beat it, where a later row with the same norm beats an earlier one
    n_hi = int(np.ceil(S * 0.3))
    nm = wnorms.reshape(H, S)
    for h in range(H):
        beat = (nm[h][None, :] > nm[h][:, None]) | ((nm[h][None, :] == nm[h][:, None]) & (np.arange(S)[None, :] > np.arange(S)[:, None]))
        assert np.array_equal(oz.saliency_mask(nm[h:h + 1], n_hi)[0], beat.sum(1) < n_hi)
