"""``method="age_tiered"`` on the GPU against ``oracle.age_tiered`` (cases of
veloxquant_mlx/tests/cache/test_age_tiered_cache.py and test_age_tiered_incremental_requantize.py)."""

import numpy as np
import pytest
import torch

from oracle import age_tiered as oat
from tests._gpu import gpu, host, require_gpu, to_dev
from veloxquant_mlx_amd import kernels as K
from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory
from veloxquant_mlx_amd.cache.age_tiered_cache import AgeTieredKVCache

pytestmark = gpu


def _kv(B, H, S, D, seed):
    rng = np.random.default_rng(seed)
    return rng.standard_normal((B, H, S, D)).astype(np.float16), rng.standard_normal((B, H, S, D)).astype(np.float16)


def _make(**kw):
    cfg = dict(method="age_tiered", head_dim=32)
    cfg.update(kw)
    return KVCacheFactory.create(KVCacheConfig(**cfg))


@pytest.mark.parametrize("B,H,D,rb,mb,g,bits,calls", [
    (1, 2, 32, 3, 6, 32, (8, 4, 2), [15]),
    (2, 2, 128, 40, 70, 32, (8, 4, 2), [100, 1, 1, 1, 30, 1]),       # windows that span a boundary, ragged tail
    (1, 4, 64, 8, 40, 16, (6, 3, 1), [5] + [1] * 60 + [17]),          # token by token through both boundaries
    (1, 1, 128, 128, 1024, 32, (8, 4, 2), [300, 1, 1]),               # the defaults
    (1, 2, 32, 50, 50, 32, (16, 4, 4), [70, 1]),                       # empty middle tier, 16 bits = untouched
])
def test_cache_matches_the_model_bit_for_bit(B, H, D, rb, mb, g, bits, calls):
    require_gpu()
    c = _make(head_dim=D, age_recent_boundary=rb, age_mid_boundary=mb, age_group_size=g, age_bits_recent=bits[0],
              age_bits_mid=bits[1], age_bits_old=bits[2])
    assert isinstance(c, AgeTieredKVCache) and not c.is_trimmable() and not hasattr(c, "bits")
    m = oat.AgeTieredCacheModel(D, rb, mb, bits, g)
    total = 0
    for i, S in enumerate(calls):
        k, v = _kv(B, H, S, D, 100 + i)
        ko, vo = c.update_and_fetch(to_dev(k), to_dev(v))
        km, vm = m.update_and_fetch(k, v)
        total += S
        assert ko.shape == (B, H, total, D) and ko.dtype == torch.float16
        assert np.array_equal(host(ko), km) and np.array_equal(host(vo), vm), (i, S)
        counts = m.tier_counts()
        assert (c.tokens_recent, c.tokens_mid, c.tokens_old) == (counts[0], counts[1], counts[2])
        assert c.age_tiered_bytes == m.age_tiered_bytes and c.full_seq_bytes == m.full_seq_bytes
    assert c.tokens_seen == B * H * total and c.tokens_kept == total
    assert c.compression_ratio == m.full_seq_bytes / m.age_tiered_bytes


def test_known_tier_counts():
    """test_age_tiered_cache.py:170-181."""
    require_gpu()
    c = _make(age_recent_boundary=3, age_mid_boundary=6)
    k, v = _kv(1, 1, 15, 32, 0)
    c.update_and_fetch(to_dev(k), to_dev(v))
    assert (c.tokens_recent, c.tokens_mid, c.tokens_old) == (3, 3, 9)


def test_only_changed_groups_are_recomputed(monkeypatch):
    """test_age_tiered_incremental_requantize.py:59-90 in substance: a decode step launches the round trip for
    the open group and for groups whose first token crossed a boundary, nothing else."""
    require_gpu()
    c = _make(head_dim=64, age_recent_boundary=64, age_mid_boundary=256, age_group_size=32)
    k, v = _kv(1, 2, 320, 64, 1)
    c.update_and_fetch(to_dev(k), to_dev(v))
    rows = []
    real = K.kivi_group_quant_dequant
    monkeypatch.setattr(K, "kivi_group_quant_dequant", lambda x, *a, **kw: (rows.append(x.shape[-2]), real(x, *a, **kw))[1])
    for step in range(3):
        k, v = _kv(1, 2, 1, 64, 50 + step)
        c.update_and_fetch(to_dev(k), to_dev(v))
    # 320 tokens = 10 full groups; each step re-derives the open 11th group (1-3 tokens); a first token crosses a
    # boundary only when position - (32 j + 1) hits 64 or 256, i.e. at position 321 for j = 8 (age 64) and
    # j = 2 (age 256): two one-group launches per tensor at the first step
    assert sorted(rows) == sorted([1, 1, 2, 2, 3, 3] + [32] * 4), rows


def test_bfloat16_storage_and_rejections():
    require_gpu()
    c = _make(head_dim=64, age_recent_boundary=8, age_mid_boundary=16)
    k, v = _kv(1, 2, 40, 64, 3)
    kb, vb = torch.from_numpy(k.astype(np.float32)).to(torch.bfloat16), torch.from_numpy(v.astype(np.float32)).to(torch.bfloat16)
    ko, vo = c.update_and_fetch(kb.cuda(), vb.cuda())
    cast = lambda a: torch.from_numpy(a).to(torch.bfloat16).float().numpy()
    m = oat.AgeTieredCacheModel(64, 8, 16, cast=cast)
    km, vm = m.update_and_fetch(kb.float().numpy(), vb.float().numpy())
    assert ko.dtype == torch.bfloat16 and np.array_equal(ko.float().cpu().numpy(), km) and np.array_equal(vo.float().cpu().numpy(), vm)
    for kw, pat in ((dict(age_recent_boundary=0), "age_recent_boundary"), (dict(age_recent_boundary=-5), "age_recent_boundary"),
                    (dict(age_recent_boundary=100, age_mid_boundary=50), "age_mid_boundary"),
                    (dict(age_bits_mid=0), "age_bits_mid"), (dict(age_bits_old=17), "age_bits_old")):
        with pytest.raises(ValueError, match=pat):
            _make(**kw)
    _make(age_recent_boundary=50, age_mid_boundary=50)


@pytest.mark.gpu
@pytest.mark.parametrize("g,n", [(32, 32 * 9), (64, 64 * 5 + 17), (32, 100)])
def test_one_launch_with_a_level_count_per_window_equals_a_launch_per_tier(g, n):
    """``vq_kivi_quant_dequant_grouplevels`` against what it replaces: every stretch of windows of one tier round-tripped
    on its own at that tier's bit width, 16-bit tiers copied (age_tiered.py:117-174) -- bit for bit, with a ragged last
    window and with tiers that alternate."""
    require_gpu()
    from veloxquant_mlx_amd import kernels as K
    rng = np.random.default_rng(g + n)
    G, D = 6, 128
    x = to_dev((rng.standard_normal((G, n, D)) * np.exp(rng.standard_normal(D))).astype(np.float16))
    n_groups = -(-n // g)
    for bits_of in ([16, 8, 4, 2], [4, 4, 2, 16], [2, 16, 2, 8]):
        per_group = [bits_of[j % len(bits_of)] for j in range(n_groups)]
        levels = torch.tensor([0.0 if b >= 16 else float((1 << b) - 1) for b in per_group], dtype=torch.float32, device=x.device)
        got = K.kivi_group_quant_dequant_grouplevels(x, levels, g)
        want = torch.empty_like(x)
        for j, b in enumerate(per_group):
            a, e = j * g, min((j + 1) * g, n)
            want[:, a:e] = x[:, a:e] if b >= 16 else K.kivi_group_quant_dequant(x[:, a:e].contiguous(), -2, g, (1 << b) - 1)
        assert torch.equal(got, want), bits_of
