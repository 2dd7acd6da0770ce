"""``method="skvq"`` and the clipped round-trip kernel on the GPU against ``oracle.skvq`` (cases of
veloxquant_mlx/tests/cache/test_skvq_cache.py and tests/quantizers/test_skvq.py).  The bar is
bit for bit: the kernel and the oracle add a group's squared errors in the same order."""

import numpy as np
import pytest
import torch

from oracle import skvq as o
from tests._gpu import gpu, host, require_gpu, to_dev
from veloxquant_mlx_amd import kernels as K
from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory
from veloxquant_mlx_amd.cache.skvq_cache import SKVQKVCache
from veloxquant_mlx_amd.quantizers.skvq import skvq_compressed_bytes

pytestmark = gpu


def _het_scales(d, seed=3):   # test_skvq_cache.py:32-36
    rng = np.random.default_rng(seed)
    scales = np.logspace(-2, 1, d)
    rng.shuffle(scales)
    return scales


def _kv(B, H, S, D, seed=0, channel_scales=None):   # test_skvq_cache.py:21-29
    rng = np.random.default_rng(seed)
    k = rng.standard_normal((B, H, S, D)).astype(np.float32)
    v = rng.standard_normal((B, H, S, D)).astype(np.float32)
    if channel_scales is not None:
        cs = channel_scales.astype(np.float32)[None, None, None, :]
        k, v = k * cs, v * cs
    return k.astype(np.float16), v.astype(np.float16)


def _make(**cfg):   # test_skvq_cache.py:39-52
    base = dict(method="skvq", head_dim=64, skvq_window=16, skvq_n_sink=4, skvq_group_size=16, skvq_bits_key=2,
                skvq_bits_value=2)
    base.update(cfg)
    return KVCacheFactory.create(KVCacheConfig(**base))


def _bits(a):
    a = np.ascontiguousarray(a)
    return a.view({2: np.uint16, 4: np.uint32}[a.dtype.itemsize])


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,H,r,D,bits,g,with_perm", [
    (1, 2, 16, 64, 2, 16, True),
    (2, 3, 37, 128, 4, 32, True),
    (1, 4, 128, 128, 4, 32, False),
    (1, 2, 9, 50, 3, 16, True),      # ragged last group: padded with the last permuted channel
    (1, 1, 5, 64, 8, 1, False),      # one channel per group
    (2, 2, 33, 256, 2, 256, True),   # one group per row
    (1, 2, 700, 128, 1, 64, False),
    (2, 2, 21, 80, 4, 32, True),     # ragged last group on the 16-byte path: the order's last channel fills it
    (1, 3, 50, 192, 2, 64, True),    # rows of a block in several heads, groups of 64
])
def test_round_trip_kernel_matches_the_oracle_bit_for_bit(dtype, B, H, r, D, bits, g, with_perm):
    require_gpu()
    rng = np.random.default_rng(B * 1000 + r + D + bits)
    x = (rng.standard_normal((B, H, r, D)) * _het_scales(D, seed=D)).astype(np.float32)
    x[rng.random(x.shape) < 0.02] *= 12.0   # outliers, so that clipped windows win somewhere
    xt = to_dev(x).to(dtype)
    xn = xt.float().cpu().numpy()           # the values the kernel sees
    perm = inv = None
    if with_perm:
        perm = np.stack([rng.permutation(D) for _ in range(H)]).astype(np.int32)
        inv = np.argsort(perm, axis=-1).astype(np.int32)
    ref32 = o.round_trip(xn, perm, inv, bits, g, o.DEFAULT_ALPHA_GRID)   # float32 reconstruction
    ref = torch.from_numpy(ref32).to(dtype)                               # cast as the cache does
    out = K.skvq_clipped_round_trip(xt, bits, g, o.DEFAULT_ALPHA_GRID, perm=None if perm is None else to_dev(perm))
    assert out.dtype == dtype and out.shape == xt.shape
    assert torch.equal(out.cpu().view(torch.int16 if dtype != torch.float32 else torch.int32),
                       ref.view(torch.int16 if dtype != torch.float32 else torch.int32))
    if with_perm:   # with the inverse order the rows move as 16-byte pieces; same bits
        out_inv = K.skvq_clipped_round_trip(xt, bits, g, o.DEFAULT_ALPHA_GRID, perm=to_dev(perm), inv=to_dev(inv))
        assert torch.equal(out_inv, out)
    # some group took a clipped window (the search is live), and a single alpha = 1 differs
    plain = K.skvq_clipped_round_trip(xt, bits, g, (1.0,), perm=None if perm is None else to_dev(perm))
    if bits <= 4 and g > 1:
        assert not torch.equal(plain, out)


def test_round_trip_in_place_on_a_slice_of_a_larger_buffer():
    require_gpu()
    k, _ = _kv(2, 3, 40, 64, seed=2, channel_scales=_het_scales(64))
    buf = torch.zeros((2, 3, 256, 64), dtype=torch.float16, device="cuda:0")
    buf[:, :, :40] = to_dev(k)
    rows = buf[:, :, 8:24]
    K.skvq_clipped_round_trip(rows, 2, 16, o.DEFAULT_ALPHA_GRID, out=rows)
    ref = o.round_trip(k[:, :, 8:24], None, None, 2, 16, o.DEFAULT_ALPHA_GRID)
    got = host(buf)
    assert np.array_equal(_bits(got[:, :, 8:24]), _bits(ref))
    assert np.array_equal(got[:, :, :8], k[:, :, :8]) and np.array_equal(got[:, :, 24:40], k[:, :, 24:40])
    assert not got[:, :, 40:].any()


def test_wrapper_rejects_bad_arguments():
    require_gpu()
    x = torch.zeros((1, 2, 4, 64), dtype=torch.float16, device="cuda:0")
    with pytest.raises(ValueError, match="bits"):
        K.skvq_clipped_round_trip(x, 0, 16, (1.0,))
    with pytest.raises(ValueError, match="group_size"):
        K.skvq_clipped_round_trip(x, 2, 0, (1.0,))
    with pytest.raises(ValueError, match="alphas"):
        K.skvq_clipped_round_trip(x, 2, 16, (1.2,))
    with pytest.raises(ValueError, match="perm"):
        K.skvq_clipped_round_trip(x, 2, 16, (1.0,), perm=torch.zeros((2, 64), dtype=torch.int64, device="cuda:0"))
    with pytest.raises(ValueError, match="inv"):
        K.skvq_clipped_round_trip(x, 2, 16, (1.0,), inv=torch.zeros((2, 64), dtype=torch.int32, device="cuda:0"))
    with pytest.raises(ValueError, match="token slice"):
        K.skvq_clipped_round_trip(x.transpose(1, 2), 2, 16, (1.0,))
    assert K.skvq_clipped_round_trip(x[:, :, :0], 2, 16, (1.0,)).shape == (1, 2, 0, 64)


@pytest.mark.parametrize("kw,B,H,S,D,het", [
    ({}, 1, 2, 53, 64, True),
    ({}, 2, 2, 40, 64, False),
    (dict(skvq_reorder=False), 1, 2, 35, 64, True),
    (dict(skvq_clip_search=False, skvq_clip_alpha=0.9), 1, 2, 32, 64, False),
    (dict(skvq_window=128, skvq_n_sink=5, skvq_group_size=32, skvq_bits_key=4, skvq_bits_value=4, head_dim=128),
     2, 4, 300, 128, True),
    (dict(skvq_n_sink=0, skvq_bits_key=4, skvq_bits_value=2), 1, 3, 64, 64, True),
])
def test_cache_matches_the_model_bit_for_bit(kw, B, H, S, D, het):
    """One prefill, then token-by-token decode; the permutation decisions are checked to be clear of
    ties (relative margin) so that the comparison does not hang on the order of a mean."""
    require_gpu()
    c = _make(**kw)
    assert isinstance(c, SKVQKVCache) and not hasattr(c, "bits")
    alphas = o.DEFAULT_ALPHA_GRID if kw.get("skvq_clip_search", True) else (kw.get("skvq_clip_alpha", 1.0),)
    m = o.SKVQCacheModel(c._bits_k, c._bits_v, c._group_size, c._window, c._n_sink, c._reorder, alphas)
    k, v = _kv(B, H, S, D, seed=S, channel_scales=_het_scales(D) if het else None)
    ko, vo = c.update_and_fetch(to_dev(k), to_dev(v))
    km, vm = m.update_and_fetch(k, v)
    for err_id, err_cand in m.margins:
        assert np.all(np.abs(err_cand - err_id) > 1e-6 * err_id), "permutation decision too close to a tie"
    if c._reorder and c.quantized_tokens:
        assert np.array_equal(host(c.key_perms), m.perm_k) and np.array_equal(host(c.value_perms), m.perm_v)
    assert np.array_equal(_bits(host(ko)), _bits(km)) and np.array_equal(_bits(host(vo)), _bits(vm))
    for t in range(c._window + 3):
        k1, v1 = _kv(B, H, 1, D, seed=1000 + t)
        ko, vo = c.update_and_fetch(to_dev(k1), to_dev(v1))
        km, vm = m.update_and_fetch(k1, v1)
    assert c.quantized_tokens == m.q_end and c.offset == m.offset
    assert np.array_equal(_bits(host(ko)), _bits(km)) and np.array_equal(_bits(host(vo)), _bits(vm))


def test_prefill_decode_bit_for_bit_equivalence_and_frozen_chunks():   # test_skvq_cache.py:127-160
    require_gpu()
    r, S = 16, 53
    k, v = _kv(1, 2, S, 64, seed=5, channel_scales=_het_scales(64))
    a = _make()
    ka, va = a.update_and_fetch(to_dev(k), to_dev(v))
    b = _make()
    for t in range(S):
        kb, vb = b.update_and_fetch(to_dev(k[:, :, t:t + 1]), to_dev(v[:, :, t:t + 1]))
    assert torch.equal(ka, kb) and torch.equal(va, vb) and a.quantized_tokens == b.quantized_tokens == 48
    first = ka[:, :, :r].clone()
    pk = a.key_perms.clone()
    k2, v2 = _kv(1, 2, 32, 64, seed=8)
    ko, _ = a.update_and_fetch(to_dev(k2), to_dev(v2))
    assert torch.equal(ko[:, :, :r], first) and torch.equal(a.key_perms, pk)


def test_window_sinks_accounting_and_guards():   # test_skvq_cache.py:66-125, 268-330
    require_gpu()
    c = _make()
    k, v = _kv(1, 2, 10, 64, seed=1)
    ko, vo = c.update_and_fetch(to_dev(k), to_dev(v))
    assert np.array_equal(host(ko), k) and np.array_equal(host(vo), v)
    assert c.quantized_tokens == 0 and c.compressed_key_bytes == 0 and c.assigned_avg_bits == 16.0
    assert c.key_perms is None and c.perm_bytes == 0 and not c.is_trimmable()

    B, H, D, r, n_sink, gs = 1, 2, 64, 16, 4, 16
    c = _make()
    k, v = _kv(B, H, 2 * r + 3, D, seed=12)
    ko, vo = c.update_and_fetch(to_dev(k), to_dev(v))
    assert np.array_equal(host(ko)[:, :, :n_sink], k[:, :, :n_sink]) and np.array_equal(host(ko)[:, :, 2 * r:], k[:, :, 2 * r:])
    assert not np.array_equal(host(ko)[:, :, n_sink:2 * r], k[:, :, n_sink:2 * r])
    expect = (skvq_compressed_bytes(r - n_sink, D, 2, gs) + skvq_compressed_bytes(r, D, 2, gs)) * B * H
    assert c.compressed_key_bytes == expect and c.compressed_value_bytes == expect
    assert c.fp16_key_bytes == B * H * (2 * r + 3) * D * 2
    assert c.residual_fp16_bytes == (3 + n_sink) * D * 2 * 2 * B * H
    assert c.perm_bytes == 2 * H * D * 4 and 2.0 < c.assigned_avg_bits < 16.0 and c.tokens_seen == 2 * r + 3

    with pytest.raises(ValueError, match="skvq_max_ctx"):
        _make(skvq_max_ctx=32).update_and_fetch(*map(to_dev, _kv(1, 2, 33, 64, seed=15)))
    for bad, what in ((dict(skvq_bits_key=0), "skvq_bits_key"), (dict(skvq_bits_value=9), "skvq_bits_value"),
                      (dict(skvq_group_size=0), "skvq_group_size"), (dict(skvq_window=1, skvq_n_sink=0), "skvq_window"),
                      (dict(skvq_n_sink=16), "skvq_n_sink"), (dict(skvq_clip_alpha=0.0), "skvq_clip_alpha")):
        with pytest.raises(ValueError, match=what):
            _make(**bad)


def test_reorder_beats_identity_on_heterogeneous_channels():   # test_skvq_cache.py:191-202
    require_gpu()
    k, v = _kv(1, 2, 64, 64, seed=10, channel_scales=_het_scales(64))

    def mse(reorder):
        c = _make(skvq_reorder=reorder, skvq_n_sink=0)
        ko, _ = c.update_and_fetch(to_dev(k), to_dev(v))
        q = c.quantized_tokens
        return float(np.mean((host(ko)[:, :, :q].astype(np.float32) - k[:, :, :q].astype(np.float32)) ** 2))

    assert mse(True) < mse(False)
