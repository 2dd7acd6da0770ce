"""Pins for ``oracle.zipcache``: reductions to the pinned KIVI round trip, routing on hand-picked
norms, byte counts by hand, and the orderings the reference's tests state
(veloxquant_mlx/tests/cache/test_zipcache_cache.py:76-100)."""

import numpy as np

from oracle import kivi as ok, zipcache as oz


def _kv(B, H, S, D, seed):
    """Rows whose norms differ by clear margins (the routing is then not a matter of the last bits)."""
    rng = np.random.default_rng(seed)
    amp = (1.0 + 0.05 * rng.permutation(S)).astype(np.float32)[None, None, :, None]
    return (rng.standard_normal((B, H, S, D)).astype(np.float32) * amp).astype(np.float16)


def test_all_high_and_all_low_reduce_to_the_kivi_round_trip():
    k = _kv(1, 2, 50, 64, 0)
    for frac, bits in ((1.0, 4), (0.0, 2)):
        out, _, _ = oz.compress(k, True, 4, 2, frac, 32)
        ref = ok.quant_dequant_along(k.reshape(2, 50, 64).astype(np.float32), -2, 32, (1 << bits) - 1)
        assert np.array_equal(out.reshape(2, 50, 64), ref.astype(np.float16))
    v_out, _, _ = oz.compress(k, False, 4, 2, 0.2, 32)   # values: everything at hi_bits
    assert np.array_equal(v_out, oz.compress(k, True, 4, 2, 1.0, 32)[0])


def test_routing_by_hand():
    """Six tokens with norms 1, 5, 2, 6, 3, 4 (times sqrt(D)), hi_fraction 1/3: tokens 1 and 3 go high;
    each block is quantised in original order, so the result equals two separate round trips."""
    D = 8
    amp = np.array([1, 5, 2, 6, 3, 4], np.float32)
    rng = np.random.default_rng(1)
    x = (np.sign(rng.standard_normal((1, 1, 6, D))).astype(np.float32) * amp[None, None, :, None]).astype(np.float16)
    out, norms, _ = oz.compress(x, True, 8, 1, 1 / 3, 4)
    assert np.allclose(norms[0], amp * np.sqrt(D))
    assert np.array_equal(oz.saliency_mask(norms, 2)[0], [False, True, False, True, False, False])
    hi = ok.quant_dequant_along(x[0, :, [1, 3]].transpose(1, 0, 2).astype(np.float32), -2, 4, 255)
    lo = ok.quant_dequant_along(x[0, :, [0, 2, 4, 5]].transpose(1, 0, 2).astype(np.float32), -2, 4, 1)
    assert np.array_equal(out[0, :, [1, 3]].transpose(1, 0, 2), hi.astype(np.float16))
    assert np.array_equal(out[0, :, [0, 2, 4, 5]].transpose(1, 0, 2), lo.astype(np.float16))
    # equal norms: the later token ranks higher (stable sort of the norms, top ranks taken)
    assert np.array_equal(oz.saliency_mask(np.ones((1, 4), np.float32), 1)[0], [False, False, False, True])


def test_bytes_by_hand_and_orderings():
    k = _kv(1, 2, 64, 64, 2)
    _, _, (stored, base, fp16) = oz.compress(k, True, 4, 2, 0.2, 32)
    # 13 high tokens (ceil(12.8)): 13*64*4/8 = 416 B codes + 1 group * 64 * 4 B; 51 low: 816 B + 2 groups * 256 B; 64 B mask
    assert stored == (416 + 256 + 816 + 512 + 64) * 2 and base == (64 * 64 * 2 // 8 + 2 * 256) * 2 and fp16 == 2 * 64 * 64 * 2
    assert base <= stored < fp16 and 2.0 <= 16.0 * stored / fp16 <= 4.0 + 1.0
    assert oz.base_only_bytes(10, 64, 2, 32) == 160 + 256


def test_sort_free_routing_equals_the_stable_sorts():
    """The cache's routing helpers (threshold + prefix sums) against the reference's definition by stable argsorts
    (zipcache_cache.py:106-116, 186-190), on norms with many ties and every block size."""
    import torch
    from veloxquant_mlx_amd.cache.zipcache_cache import ZipCacheKVCache as Z
    torch.manual_seed(0)
    for S in (1, 5, 64, 257):
        for n_hi in range(0, S + 1, max(1, S // 7)):
            norms = torch.randint(0, 6, (9, S)).float()
            rank = torch.argsort(torch.argsort(norms, dim=-1, stable=True), dim=-1, stable=True)
            want = rank >= (S - n_hi)
            got = Z._batched_saliency_mask(norms, n_hi, S)
            assert torch.equal(got, want), (S, n_hi)
            if 0 < n_hi < S:
                assert torch.equal(Z._routing_order(got, n_hi).long(), torch.argsort(got.to(torch.int32), dim=-1, stable=True))
