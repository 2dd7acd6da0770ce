"""Cache classes on the GPU against the oracle's cache model.

KIVI cases restate veloxquant_mlx/tests/cache/test_kivi_cache.py:60-221 and
veloxquant_mlx/tests/metal/test_kivi_quant.py:200-235; VecInfer cases restate
veloxquant_mlx/tests/cache/test_vecinfer_memory_bound_state.py:72-146."""

import math

import numpy as np
import pytest
import torch

from oracle import attend as oa, kivi as ok, vecinfer as ov
from tests._gpu import gpu, host, outlier_kv, require_gpu, to_dev
from veloxquant_mlx_amd import kernels as K
from veloxquant_mlx_amd.cache import KVCacheConfig, KVCacheFactory
from veloxquant_mlx_amd.quantizers import KIVIQuantizer

pytestmark = gpu


def _kv(B, H, S, D, seed):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((B, H, S, D)).astype(np.float16),
            rng.standard_normal((B, H, S, D)).astype(np.float16))


def _make(**kw):
    cfg = dict(method="kivi", head_dim=128, bit_width_inlier=2, kivi_group_size=32, residual_length=128)
    cfg.update(kw)
    return KVCacheFactory.create(KVCacheConfig(**cfg))


def test_residual_window_passthrough():
    require_gpu()
    c = _make(residual_length=64)
    k, v = _kv(1, 2, 32, 128, 1)
    ko, vo = c.update_and_fetch(to_dev(k), to_dev(v))
    assert np.array_equal(host(ko), k) and np.array_equal(host(vo), v) and c.compressed_key_bytes == 0


@pytest.mark.parametrize("fused", [False, True])
def test_prefill_plus_decode_matches_cache_model_bit_for_bit(fused):
    require_gpu()
    c = _make(residual_length=32, fused_sdpa=fused)
    m = ok.KiviCacheModel(2, 32, 32)
    rng = np.random.default_rng(3)
    k = rng.standard_normal((1, 8, 200, 128)).astype(np.float16)
    v = rng.standard_normal((1, 8, 200, 128)).astype(np.float16)
    ko, vo = c.update_and_fetch(to_dev(k), to_dev(v))
    mk, mv = m.update_and_fetch(k, v)
    for _ in range(40):
        k1 = rng.standard_normal((1, 8, 1, 128)).astype(np.float16)
        v1 = rng.standard_normal((1, 8, 1, 128)).astype(np.float16)
        ko, vo = c.update_and_fetch(to_dev(k1), to_dev(v1))
        mk, mv = m.update_and_fetch(k1, v1)
    assert np.array_equal(host(ko), mk) and np.array_equal(host(vo), mv)
    assert c.offset == 240 and c._n_quantized == m.n_quantized == 192
    assert c.compressed_key_bytes == m.key_bytes_compressed
    assert c.compressed_value_bytes == m.value_bytes_compressed
    assert c.residual_fp16_bytes == m.residual_fp16_bytes and c.fp16_key_bytes == m.key_bytes_fp16
    total_fp16 = m.key_bytes_fp16 + m.value_bytes_fp16
    assert c.effective_compression_ratio == total_fp16 / (m.key_bytes_compressed + m.value_bytes_compressed
                                                          + m.residual_fp16_bytes)


def test_one_shot_equals_token_by_token():
    require_gpu()
    k, v = _kv(1, 2, 48, 128, 13)
    a = _make(residual_length=8, kivi_group_size=8)
    ka, va = a.update_and_fetch(to_dev(k), to_dev(v))
    b = _make(residual_length=8, kivi_group_size=8)
    for t in range(48):
        kb, vb = b.update_and_fetch(to_dev(k[:, :, t:t + 1]), to_dev(v[:, :, t:t + 1]))
        assert b._n_quantized % 8 == 0 and b.offset - b._n_quantized <= 8 + 8 - 1
    assert torch.equal(ka, kb) and torch.equal(va, vb) and a._n_quantized == b._n_quantized == 40


def test_trim_equals_model_and_requantises():
    require_gpu()
    k, v = _kv(1, 2, 100, 64, 5)
    c = _make(head_dim=64, residual_length=8, kivi_group_size=8)
    m = ok.KiviCacheModel(2, 8, 8)
    c.update_and_fetch(to_dev(k), to_dev(v)); m.update_and_fetch(k, v)
    assert c.trim(36) == m.trim(36) == 36
    assert (c.offset, c._n_quantized) == (m.offset, m.n_quantized) == (64, 64)
    assert c.compressed_key_bytes == m.key_bytes_compressed and c.fp16_key_bytes == m.key_bytes_fp16
    k2, v2 = _kv(1, 2, 30, 64, 6)
    ko, vo = c.update_and_fetch(to_dev(k2), to_dev(v2)); mk, mv = m.update_and_fetch(k2, v2)
    assert np.array_equal(host(ko), mk) and np.array_equal(host(vo), mv)


@pytest.mark.parametrize("bits,g", [(2, 32), (4, 64), (3, 32)])
def test_decode_at_head_size_256_through_the_cache_and_the_layer_stack(bits, g):
    """Head size 256 (configuration 2's own model: 12 query / 4 kv heads): a memory-bound cache decodes through the
    matrix-unit kernel's 256-channel form (2 and 4 bits) or the vector kernel (3 bits) over steps that cross a flush,
    against the oracle; the layer-stacked cache gives the per-layer results under ``fixed_order``."""
    require_gpu()
    from veloxquant_mlx_amd.cache import LayerStackedKIVICache
    B, Hq, Hkv, D, R, NL = 2, 12, 4, 256, 64, 2
    cfg = KVCacheConfig(method="kivi", head_dim=D, bit_width_inlier=bits, kivi_group_size=g, residual_length=R,
                        fused_sdpa=True, fused_sdpa_memory_bound=True, fused_sdpa_max_ctx=1280, kivi_code_field="tight")
    solo = [KVCacheFactory.create(cfg) for _ in range(NL)]
    stack = LayerStackedKIVICache(cfg, NL)
    n0 = 960 if bits == 3 else 1000
    ks = [outlier_kv((B, Hkv, n0 + 80, D), seed=31 * l + bits) for l in range(NL)]
    rng = np.random.default_rng(5)
    scale = 1 / math.sqrt(D)
    for l in range(NL):
        for c in (solo[l], stack[l]):
            c.update_and_fetch(to_dev(ks[l][0][:, :, :n0]), to_dev(ks[l][1][:, :, :n0]))
    levels = (1 << bits) - 1
    for t in range(n0, n0 + 80):
        q = rng.standard_normal((NL, B, Hq, 1, D)).astype(np.float16)
        for l in range(NL):
            for c in (solo[l], stack[l]):
                c.update_and_fetch(to_dev(ks[l][0][:, :, t:t + 1]), to_dev(ks[l][1][:, :, t:t + 1]))
        if t % 9 and t < n0 + 76:
            continue
        outs = [solo[l].fused_sdpa(to_dev(q[l]), scale, fixed_order=True) for l in range(NL)]
        all_out = stack.fused_sdpa_all(to_dev(q), scale, fixed_order=True)
        for l in range(NL):
            nq = solo[l]._n_quantized
            assert nq == ok.quantization_boundary(t + 1, R, g) and stack[l]._n_quantized == nq
            k, v = ks[l]
            kq = ok.group_quant_codes(k[:, :, :nq], -2, g, levels)
            vq = ok.group_quant_codes(v[:, :, :nq], -1, g, levels)
            ref = oa.kivi_attend(q[l], kq[0], kq[1].astype(np.float16), kq[2].astype(np.float16), vq[0], vq[1].astype(np.float16),
                                 vq[2].astype(np.float16), g, k[:, :, nq:t + 1], v[:, :, nq:t + 1], scale)
            err = float(np.max(np.abs(host(outs[l]).astype(np.float32) - ref)))
            assert err < 2e-3, (t, l, err)
            # the stacked launch may cut the context differently (its batch axis is NL times as long): values, not bits
            assert float((all_out[l].float() - outs[l].float()).abs().max()) < 1e-3, (t, l)


@pytest.mark.parametrize("memory_bound", [False, True])
@pytest.mark.parametrize("bits,g,meta", [(2, 32, "float16"), (4, 64, "float16"), (4, 32, "float32")])
def test_fused_sdpa_over_packed_prefix(memory_bound, bits, g, meta):
    """Decode through the packed store: the same positions are quantised with the
    same groups as the cache model, and attention matches the oracle."""
    require_gpu()
    R = 64
    c = _make(bit_width_inlier=bits, kivi_group_size=g, residual_length=R, fused_sdpa=True,
              fused_sdpa_memory_bound=memory_bound, kivi_meta_dtype=meta)
    k, v = outlier_kv((2, 2, 300, 128), seed=bits + g)
    rng = np.random.default_rng(9)
    c.update_and_fetch(to_dev(k[:, :, :257]), to_dev(v[:, :, :257]))
    for t in range(257, 300):
        ko, vo = c.update_and_fetch(to_dev(k[:, :, t:t + 1]), to_dev(v[:, :, t:t + 1]))
    nq = ok.quantization_boundary(300, R, g)
    assert c._n_quantized == nq and ko.shape == (2, 2, 300, 128)
    q = rng.standard_normal((2, 8, 1, 128)).astype(np.float16)
    out = c.fused_sdpa(to_dev(q), 1 / math.sqrt(128))
    assert out.dtype == torch.float16
    levels = (1 << bits) - 1
    npm = np.float16 if meta == "float16" else np.float32
    kq = ok.group_quant_codes(k[:, :, :nq], -2, g, levels)
    vq = ok.group_quant_codes(v[:, :, :nq], -1, g, levels)
    ref = oa.kivi_attend(q, kq[0], kq[1].astype(npm), kq[2].astype(npm), vq[0], vq[1].astype(npm),
                         vq[2].astype(npm), g, k[:, :, nq:], v[:, :, nq:], 1 / math.sqrt(128))
    assert np.max(np.abs(host(out).astype(np.float32) - ref)) < 2e-3
    if memory_bound:
        # packed store plus the two pairs of fp16 tail buffers (the kept rows move between them at a flush)
        assert c.nbytes < 0.6 * (2 * 2 * 2 * c._packed_cap * 128 * 2) + 8 * c._tail_k.numel()
        assert float(ko.abs().sum()) == 0.0 and not c.empty()
    else:
        # stash mode still returns the reference's fp16 history
        mk, _ = ok.KiviCacheModel(bits, g, R).update_and_fetch(k, v)
        assert np.array_equal(host(ko), mk)


def test_memory_bound_trim_restores_reconstruction():
    require_gpu()
    c = _make(bit_width_inlier=4, kivi_group_size=32, residual_length=32, fused_sdpa=True,
              fused_sdpa_memory_bound=True, kivi_meta_dtype="float32")
    m = ok.KiviCacheModel(4, 32, 32)
    k, v = outlier_kv((1, 2, 200, 128), seed=2)
    c.update_and_fetch(to_dev(k), to_dev(v)); mk, mv = m.update_and_fetch(k, v)
    assert c.trim(90) == m.trim(90) == 90 and c._n_quantized == m.n_quantized == 96
    live = c.offset - c._n_quantized
    assert np.array_equal(host(c._tail_k[:, :, :live]), mk[:, :, 96:110])
    assert np.array_equal(host(c._tail_v[:, :, :live]), mv[:, :, 96:110])
    q = np.random.default_rng(0).standard_normal((1, 4, 1, 128)).astype(np.float16)
    out = c.fused_sdpa(to_dev(q), 0.09)
    ref = oa.sdpa(q, mk[:, :, :110], mv[:, :, :110], 0.09)
    assert np.max(np.abs(host(out).astype(np.float32) - ref)) < 2e-3


@pytest.mark.parametrize("mode", ["memory_bound", "stash", "standard"])
@pytest.mark.parametrize("bits,g,layout", [(4, 32, "auto"), (2, 32, "auto"), (4, 64, "channel")])
def test_packed_state_round_trip_and_prompt_cache_file(mode, bits, g, layout, tmp_path):
    """A cache rebuilt from (state, meta_state), directly and through a prompt-cache file,
    is the cache it came from: same frontier, same bytes, same attention now and after
    further tokens."""
    require_gpu()
    from veloxquant_mlx_amd.cache import load_prompt_cache, save_prompt_cache
    kw = dict(bit_width_inlier=bits, kivi_group_size=g, residual_length=128, kivi_value_layout=layout,
              fused_sdpa=mode != "standard", fused_sdpa_memory_bound=mode == "memory_bound")
    prev_order = K.attend_fixed_order(True)   # the process default, restored below
    try:
        c = _make(**kw)
        k, v = outlier_kv((2, 2, 333, 128), seed=bits + g)
        c.update_and_fetch(to_dev(k[:, :, :300]), to_dev(v[:, :, :300]))
        st, meta = c.state, c.meta_state
        assert meta[0] == "300" and int(meta[1]) == c._n_quantized == ((300 - 128) // g) * g
        c2 = type(c).from_state(KVCacheConfig(method="kivi", head_dim=128, **kw), st, meta)
        f = str(tmp_path / "prompt.safetensors")
        save_prompt_cache(f, [c], metadata={"model": "synthetic"})
        (c3,), user = load_prompt_cache(f, lambda i, name: _make(**kw), return_metadata=True)
        assert user == {"model": "synthetic"}
        q = to_dev(np.random.default_rng(1).standard_normal((2, 8, 1, 128)).astype(np.float16))
        for step in range(2):
            for other in (c2, c3):
                assert other.offset == c.offset and other._n_quantized == c._n_quantized
                assert other.meta_state == c.meta_state
                for name in ("compressed_key_bytes", "compressed_value_bytes", "fp16_key_bytes", "residual_fp16_bytes"):
                    assert getattr(other, name) == getattr(c, name), name
                assert len(other.state) == len(c.state)
                for a, b in zip(other.state, c.state):
                    assert a.shape == b.shape and torch.equal(a, b)
                if mode != "standard":
                    assert torch.equal(other.fused_sdpa(q, 0.09), c.fused_sdpa(q, 0.09))
            if step == 0:   # 33 more tokens: at least one group ages out of the residual window in all three
                for cc in (c, c2, c3):
                    cc.update_and_fetch(to_dev(k[:, :, 300:]), to_dev(v[:, :, 300:]))
        assert c._n_quantized > int(meta[1])
        # what must be refused
        with pytest.raises(ValueError, match="configured as"):
            _make(**{**kw, "bit_width_inlier": 8 if bits != 8 else 4}).meta_state = meta
        if mode != "standard":
            with pytest.raises(ValueError, match="arrays"):
                _make(**kw).state = st[:3]
            with pytest.raises(ValueError, match="do not fit|must be"):
                _make(**{**kw, "kivi_group_size": 2 * g}).state = st
        empty = _make(**kw)
        empty.state = ()
        assert empty.offset == 0 and empty.empty()
    finally:
        K.attend_fixed_order(prev_order)


@pytest.mark.parametrize("n_sink", [0, 3])
def test_sink_protected_cache_matches_model(n_sink):
    """method="kivi_sink" (veloxquant_mlx/cache/sink_cache.py): prefill, decode steps and a trim
    against the numpy model, bit for bit; two sequences with their outliers at different places."""
    require_gpu()
    rng = np.random.default_rng(7)
    B, H, D = 2, 2, 128
    k = rng.standard_normal((B, H, 330, D)).astype(np.float16)
    v = rng.standard_normal((B, H, 330, D)).astype(np.float16)
    k[0, :, 3] *= 25
    k[1, :, 150] *= 25
    k[1, :, 310] *= 30
    c = KVCacheFactory.create(KVCacheConfig(method="kivi_sink", head_dim=D, bit_width_inlier=2, kivi_group_size=32,
                                            residual_length=64, n_sink_tokens=n_sink))
    m = ok.SinkCacheModel(2, 32, 64, n_sink)
    steps = [(0, 200)] + [(s, s + 1) for s in range(200, 260)] + [(260, 330)]
    for s0, s1 in steps:
        ko, vo = c.update_and_fetch(to_dev(k[:, :, s0:s1]), to_dev(v[:, :, s0:s1]))
        km, vm = m.update_and_fetch(k[:, :, s0:s1], v[:, :, s0:s1])
    assert np.array_equal(host(ko), km) and np.array_equal(host(vo), vm)
    assert c._n_quantized == m.n_quantized and c.offset == 330
    for b in range(B):
        assert c.sink_positions_for(b) == m.sink_positions_for(b)
    assert c.sink_positions == m.sink_positions_for(0)
    for name, want in (("compressed_key_bytes", m.key_bytes_compressed), ("compressed_value_bytes", m.value_bytes_compressed),
                       ("sink_fp16_bytes", m.sink_fp16_bytes), ("residual_fp16_bytes", m.residual_fp16_bytes)):
        assert getattr(c, name) == want, name
    if n_sink:
        assert 3 in c.sink_positions_for(0) and 150 in c.sink_positions_for(1) and 310 in c.sink_positions_for(1)
        assert np.array_equal(host(ko)[0, :, 3], k[0, :, 3])
    assert c.trim(100) == m.trim(100) == 100 and c.offset == 230 and c._n_quantized == m.n_quantized == (230 // 32) * 32
    assert all(p < 230 for b in range(B) for p in c.sink_positions_for(b))
    for b in range(B):
        assert c.sink_positions_for(b) == m.sink_positions_for(b)
    for name, want in (("compressed_key_bytes", m.key_bytes_compressed), ("sink_fp16_bytes", m.sink_fp16_bytes),
                       ("residual_fp16_bytes", m.residual_fp16_bytes)):
        assert getattr(c, name) == want, name
    with pytest.raises(ValueError, match="n_sink_tokens"):
        KVCacheFactory.create(KVCacheConfig(method="kivi_sink", head_dim=D, n_sink_tokens=-1))


@pytest.mark.parametrize("mode", ["memory_bound", "stash"])
@pytest.mark.parametrize("bits,g,v_layout", [(4, 32, "token"), (2, 32, "token"), (4, 64, "channel")])
def test_sink_protected_cache_on_packed_storage(mode, bits, g, v_layout, tmp_path):
    """``kivi_sink`` with ``fused_sdpa``: the packed store holds stand-ins at the protected positions and
    the attention call swaps the exact rows in.  The oracle is attention over the history the numpy
    model of the reference's cache returns (sink_cache.py:117-198: protected rows exact, the rest
    round-tripped with the stand-ins setting the group parameters), at every stage of prefill,
    decode steps that flush, a trim and more decode; queries are aimed at the protected keys, so
    the weights that are swapped are the large ones.  Accounting and protected positions equal the
    model's as in the unpacked cache."""
    require_gpu()
    rng = np.random.default_rng(17)
    B, Hq, H, D, R = 2, 8, 2, 128, 64
    n = 420
    k = rng.standard_normal((B, H, n, D)).astype(np.float16)
    v = rng.standard_normal((B, H, n, D)).astype(np.float16)
    for b, p, f in ((0, 3, 12), (0, 40, 9), (1, 150, 12), (1, 151, 10), (1, 310, 14), (0, 333, 8)):
        k[b, :, p] *= f
    cfg = KVCacheConfig(method="kivi_sink", head_dim=D, bit_width_inlier=bits, kivi_group_size=g,
                        residual_length=R, n_sink_tokens=3, fused_sdpa=True,
                        fused_sdpa_memory_bound=(mode == "memory_bound"), kivi_meta_dtype="float32",
                        kivi_value_layout=v_layout)
    c = KVCacheFactory.create(cfg)
    m = ok.SinkCacheModel(bits, g, R, 3)
    scale = 1 / math.sqrt(D)

    def check(Sq, tag):
        km, vm = m.keys[:, :, : m.offset], m.values[:, :, : m.offset]
        q = rng.standard_normal((B, Hq, Sq, D)).astype(np.float16)
        # half of the query heads look at a protected key of their sequence
        for b in range(B):
            for p in m.sink_positions_for(b)[:2]:
                q[b, ::2, -1] += (0.4 * km[b, 0, p] / np.linalg.norm(km[b, 0, p].astype(np.float32)) * 8).astype(np.float16)
        for causal, w in ((Sq > 1, 0), (Sq > 1, 130)):
            got = host(c.fused_sdpa(to_dev(q), scale, causal=causal, sliding_window=w)).astype(np.float32)
            ref = oa.sdpa(q, km, vm, scale, causal=causal, sliding_window=w)
            err = float(np.max(np.abs(got - ref)))
            print(f"{tag}: Sq={Sq} window={w}: {len(c._side_pos[0]) if c._side_pos else 0}+{len(c._side_pos[1]) if len(c._side_pos) > 1 else 0} "
                  f"rows in the side store, max err {err:.2e}")
            assert err < 2e-3, (tag, Sq, causal, w, err)

    steps = [(0, 200)] + [(s, s + 1) for s in range(200, 300)] + [(300, 420)]
    for i, (s0, s1) in enumerate(steps):
        c.update_and_fetch(to_dev(k[:, :, s0:s1]), to_dev(v[:, :, s0:s1]))
        m.update_and_fetch(k[:, :, s0:s1], v[:, :, s0:s1])
        if i in (0, 40, 100):
            check(1, f"step {i}")
        if i in (0, 101):
            check(s1 - s0 if s1 - s0 < 100 else 24, f"chunk {i}")
    assert c._n_quantized == m.n_quantized and c.offset == m.offset
    for b in range(B):
        assert c.sink_positions_for(b) == m.sink_positions_for(b)
    for name, want in (("compressed_key_bytes", m.key_bytes_compressed), ("compressed_value_bytes", m.value_bytes_compressed),
                       ("sink_fp16_bytes", m.sink_fp16_bytes), ("residual_fp16_bytes", m.residual_fp16_bytes)):
        assert getattr(c, name) == want, name
    assert any(c._side_pos[b] for b in range(B))
    assert c.trim(130) == m.trim(130)
    assert c._n_quantized == m.n_quantized and all(p < c._n_quantized for ps in c._side_pos for p in ps)
    check(1, "after trim")
    for s in range(290, 330):
        c.update_and_fetch(to_dev(k[:, :, s:s + 1]), to_dev(v[:, :, s:s + 1]))
        m.update_and_fetch(k[:, :, s:s + 1], v[:, :, s:s + 1])
    check(1, "decode after trim")
    check(16, "chunk after trim")
    assert c.sink_fp16_bytes == m.sink_fp16_bytes and c.compressed_key_bytes == m.key_bytes_compressed

    # a cache rebuilt from the state (directly and through a prompt-cache file) protects the same rows:
    # same attention output now, and after both have taken the same further tokens and flushes
    from veloxquant_mlx_amd.cache.prompt_cache import load_prompt_cache, save_prompt_cache
    path = str(tmp_path / "sink.safetensors")
    save_prompt_cache(path, [c])
    twins = [type(c).from_state(cfg, c.state, c.meta_state), load_prompt_cache(path, lambda i, name: KVCacheFactory.create(cfg))[0]]
    q = to_dev(rng.standard_normal((B, Hq, 1, D)).astype(np.float16))
    for t in twins:
        assert (t.offset, t._n_quantized, t._side_pos) == (c.offset, c._n_quantized, c._side_pos)
        assert [t.sink_positions_for(b) for b in range(B)] == [c.sink_positions_for(b) for b in range(B)]
        assert torch.equal(t.fused_sdpa(q, scale), c.fused_sdpa(q, scale))
    for s in range(330, 420):
        for t in (c, *twins):
            t.update_and_fetch(to_dev(k[:, :, s:s + 1]), to_dev(v[:, :, s:s + 1]))
        m.update_and_fetch(k[:, :, s:s + 1], v[:, :, s:s + 1])
    for t in twins:
        assert t._side_pos == c._side_pos and torch.equal(t.fused_sdpa(q, scale), c.fused_sdpa(q, scale))
    check(1, "decode after restore")
    with pytest.raises(ValueError):
        KVCacheFactory.create(cfg).state = c.state[:-1]


def test_chunked_prefill_through_the_cache_matches_oracle():
    """Quantise-on-write prefill: chunks of 64 through a cache with R=32, g=32."""
    require_gpu()
    B, Hq, Hkv, S, D = 1, 8, 2, 256, 128
    k, v = outlier_kv((B, Hkv, S, D), seed=12)
    q = np.random.default_rng(5).standard_normal((B, Hq, S, D)).astype(np.float16)
    c = _make(bit_width_inlier=4, kivi_group_size=32, residual_length=32, fused_sdpa=True,
              fused_sdpa_memory_bound=True, kivi_meta_dtype="float32")
    outs = []
    for s0 in range(0, S, 64):
        c.update_and_fetch(to_dev(k[:, :, s0:s0 + 64]), to_dev(v[:, :, s0:s0 + 64]))
        outs.append(host(c.fused_sdpa(to_dev(q[:, :, s0:s0 + 64]), 1 / math.sqrt(D), causal=True)))
    got = np.concatenate(outs, axis=2).astype(np.float32)
    ref = oa.chunked_prefill(q, k, v, 64, 4, 32, 32, 1 / math.sqrt(D))
    assert np.max(np.abs(got - ref)) < 2e-3


def test_config4_prefill_mfma_kernel_agrees_with_vector_kernel_at_full_size():
    """Benchmark configuration 4: 4096 bf16 queries in chunks of 512 over a 4-bit packed prefix of 4096
    tokens plus their own tokens (32 query / 8 kv heads, D=128, group 32, residual 128).  The
    oracle is too slow at this size, so the two independent GPU implementations (each checked
    against the oracle at small sizes) are compared on the chunks with the shortest and the
    longest visible history; chunks in between only advance the cache."""
    require_gpu()
    B, Hq, Hkv, D, P, C = 1, 32, 8, 128, 4096, 512
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(4)
    f = torch.exp(torch.randn(D, generator=g, device=dev))
    c = _make(bit_width_inlier=4, kivi_group_size=32, residual_length=128, fused_sdpa=True,
              fused_sdpa_memory_bound=True)
    mk = lambda n: ((torch.randn((B, Hkv, n, D), generator=g, device=dev) * f).to(torch.bfloat16),
                    torch.randn((B, Hkv, n, D), generator=g, device=dev).to(torch.bfloat16))
    c.update_and_fetch(*mk(P))
    scale = 1 / math.sqrt(D)
    for ci in range(8):
        c.update_and_fetch(*mk(C))
        q = torch.randn((B, Hq, C, D), generator=g, device=dev).to(torch.bfloat16)
        if ci not in (0, 7):
            continue
        nq, n_tail = c._n_quantized, c.offset - c._n_quantized
        assert nq == (P + C * (ci + 1) - 128) // 32 * 32
        kw = dict(k_packed=c._kp, k_scale=c._ks, k_zero=c._kz, v_packed=c._vp, v_scale=c._vs, v_zero=c._vz,
                  n_packed=nq, bits=4, group_size=32, v_layout="token", k_tail=c._tail_k, v_tail=c._tail_v,
                  n_tail=n_tail, scale=scale, causal=True, out_dtype=torch.float32)
        p1, p0 = {}, {}
        o1 = K.kivi_packed_attend(q, _plan_out=p1, **kw)
        # the vector kernel over the reconstruction rounded to fp16: what the reference's cache holds
        # (kivi_cache.py:198-201) and what the 256-row MFMA blocks attend over
        o0 = K.kivi_packed_attend(q, num_splits=-2, _plan_out=p0, **kw)
        assert p1["path"] == 2 and p0["path"] == 0
        err = float((o1 - o0).abs().max())
        print(f"chunk {ci}: {nq} packed + {n_tail} tail slots, max |mfma - vector| = {err:.2e}")
        assert err < 2e-3
        # against the float32 reconstruction the fp16 rounding of keys and values shows
        assert float((o1 - K.kivi_packed_attend(q, num_splits=-1, **kw)).abs().max()) < 1e-2
        # the cache's own entry point returns the same numbers in the query dtype
        assert torch.equal(c.fused_sdpa(q, scale, causal=True), o1.to(torch.bfloat16))


@pytest.mark.parametrize("bits,g,dtype", [(4, 32, torch.bfloat16), (2, 64, torch.float16)])
def test_prefill_tiles_change_no_bit_and_follow_the_cache(bits, g, dtype):
    """Chunked quantise-on-write prefill with the ready-made tiles (the default) and without them: every chunk's
    output is identical.  The tiles follow the cache through flushes (only the units that changed are rewritten), a
    trim below the packed frontier (rewritten from the start) and growth of the packed store; the first decode step
    gives the scratch back."""
    require_gpu()
    B, Hq, Hkv, D, C = 1, 16, 4, 128, 256
    dev = "cuda:0"
    gen = torch.Generator(device=dev).manual_seed(bits + g)
    mk = lambda n: (torch.randn((B, Hkv, n, D), generator=gen, device=dev).to(dtype) * 1.5,
                    torch.randn((B, Hkv, n, D), generator=gen, device=dev).to(dtype))
    caches = []
    for on in (True, False):
        c = _make(bit_width_inlier=bits, kivi_group_size=g, residual_length=128, fused_sdpa=True, fused_sdpa_memory_bound=True)
        c.prefill_tiles = on
        caches.append(c)
    scale = 1 / math.sqrt(D)
    written = []
    for ci in range(7):
        k, v = mk(C if ci != 3 else 96)          # one ragged chunk: the tail then ends inside a unit
        q = torch.randn((B, Hq, k.shape[2], D), generator=gen, device=dev).to(dtype)
        if ci == 5:                               # drop tokens below the packed frontier, then go on
            for c in caches:
                c.trim(300)
        outs = []
        for c in caches:
            c.update_and_fetch(k, v)
            outs.append(c.fused_sdpa(q, scale, causal=True))
        if (Hq // Hkv) * k.shape[2] >= 256:
            assert caches[0]._tiles is not None and caches[1]._tiles is None
            written.append(caches[0]._tiles_packed)
        assert torch.equal(outs[0], outs[1]), (ci, float((outs[0].float() - outs[1].float()).abs().max()))
    assert written[0] < written[-1] and caches[0]._tiles_packed == caches[0]._n_quantized // 32
    assert caches[0].nbytes > caches[1].nbytes
    k, v = mk(1)
    q = torch.randn((B, Hq, 1, D), generator=gen, device=dev).to(dtype)
    outs = []
    for c in caches:
        c.update_and_fetch(k.clone(), v.clone())
        outs.append(c.fused_sdpa(q, scale, fixed_order=True))
    assert torch.equal(outs[0], outs[1]) and caches[0]._tiles is None and caches[0].nbytes == caches[1].nbytes
    # a prefill that would need more tile memory than the cache allows goes on without tiles, same bits
    k, v = mk(C)
    q = torch.randn((B, Hq, C, D), generator=gen, device=dev).to(dtype)
    caches[0].prefill_tiles_max_bytes = 1 << 20
    outs = []
    for c in caches:
        c.update_and_fetch(k, v)
        outs.append(c.fused_sdpa(q, scale, causal=True))
    assert torch.equal(outs[0], outs[1]) and caches[0]._tiles is None


@pytest.mark.parametrize("bits,g,Hq,Sq", [(4, 32, 8, 64), (2, 32, 8, 64), (4, 32, 6, 96), (2, 32, 14, 40)])
def test_sink_protected_cache_with_prefill_sized_query_blocks(bits, g, Hq, Sq):
    """Protected rows under a prefill-sized call (64 positions x 4 query heads = 256 rows a kv head, the
    256-row attention blocks; groups of 3 and 7 heads, which run as groups of 4 and 8): the stand-ins' weights are
    taken out of sums the matrix unit formed from fp16-rounded reconstructions, so the queries here are aimed at the
    stand-ins themselves and at the rows next to them, where those weights carry most of a row's mass."""
    require_gpu()
    rng = np.random.default_rng(23)
    B, H, D, R, n = 1, 2, 128, 64, 448
    k = rng.standard_normal((B, H, n, D)).astype(np.float16)
    v = rng.standard_normal((B, H, n, D)).astype(np.float16)
    for p, f in ((5, 12), (77, 10), (200, 14), (201, 9)):
        k[0, :, p] *= f
    cfg = KVCacheConfig(method="kivi_sink", head_dim=D, bit_width_inlier=bits, kivi_group_size=g, residual_length=R,
                        n_sink_tokens=3, fused_sdpa=True, fused_sdpa_memory_bound=True, kivi_meta_dtype="float32")
    c = KVCacheFactory.create(cfg)
    m = ok.SinkCacheModel(bits, g, R, 3)
    for s0, s1 in ((0, 256), (256, 384), (384, 448)):
        c.update_and_fetch(to_dev(k[:, :, s0:s1]), to_dev(v[:, :, s0:s1]))
        m.update_and_fetch(k[:, :, s0:s1], v[:, :, s0:s1])
    assert c._n_quantized == m.n_quantized and any(c._side_pos[b] for b in range(B))
    km, vm = m.keys[:, :, : m.offset], m.values[:, :, : m.offset]
    q = rng.standard_normal((B, Hq, Sq, D)).astype(np.float16)
    sinks = m.sink_positions_for(0)
    for i, p in enumerate(sinks):
        for dp in (0, 1):                              # the protected row, and its neighbour
            row = km[0, 0, min(p + dp, m.offset - 1)].astype(np.float32)
            q[0, i % Hq, -(1 + 2 * i + dp) % Sq] += (row / np.linalg.norm(row) * 6).astype(np.float16)
    scale = 1 / math.sqrt(D)
    for w in (0, 130):
        plan = {}
        got = host(c.fused_sdpa(to_dev(q), scale, causal=True, sliding_window=w)).astype(np.float32)
        ref = oa.sdpa(q, km, vm, scale, causal=True, sliding_window=w)
        err = float(np.max(np.abs(got - ref)))
        print(f"bits {bits}: window {w}: protected rows {sinks}, max err {err:.2e}")
        assert err < 2e-3, (w, err)


@pytest.mark.parametrize("bits,D,g,Hq,meta", [(3, 128, 32, 8, "float16"), (1, 128, 32, 8, "float32"), (3, 128, 64, 4, "float32"),
                                              (3, 256, 32, 6, "float16"), (1, 256, 64, 2, "float16")])
def test_odd_code_widths_in_the_next_even_field(bits, D, g, Hq, meta, tmp_path):
    """3-bit codes in 4-bit fields and 1-bit codes in 2-bit fields (``kivi_code_field="auto"``, the default): the same
    levels, hence the same codes, scale and zero as the tight packing, on the kernels of the even widths -- a prefill in
    chunks, decode steps across flushes, a trim, the saved state -- against the oracle and against a tight-packed cache."""
    require_gpu()
    B, H, R = 2, 2, 64
    kw = dict(head_dim=D, bit_width_inlier=bits, kivi_group_size=g, residual_length=R, fused_sdpa=True,
              fused_sdpa_memory_bound=True, kivi_meta_dtype=meta)
    c, tight = _make(**kw), _make(**kw, kivi_code_field="tight")
    assert c._field == {3: 4, 1: 2}[bits] and tight._field == bits and c._v_layout == "token"
    n0, n1 = 700, 790
    k, v = outlier_kv((B, H, n1, D), seed=bits * 100 + D + g)
    rng = np.random.default_rng(bits + D)
    scale, levels = 1 / math.sqrt(D), (1 << bits) - 1
    for x in (c, tight):
        for lo in range(0, n0, 256):
            hi = min(lo + 256, n0)
            x.update_and_fetch(to_dev(k[:, :, lo:hi]), to_dev(v[:, :, lo:hi]))

    def check(t_end, Sq=1, oracle=True):
        nq = c._n_quantized
        assert nq == tight._n_quantized and c.offset == tight.offset == t_end
        q = rng.standard_normal((B, Hq, Sq, D)).astype(np.float16)
        got = host(c.fused_sdpa(to_dev(q), scale, causal=True)).astype(np.float32)
        ref_t = host(tight.fused_sdpa(to_dev(q), scale, causal=True)).astype(np.float32)
        assert float(np.max(np.abs(got - ref_t))) < 2e-3, (t_end, Sq)
        if not oracle:
            return
        md = np.float16 if meta == "float16" else np.float32
        kq = ok.group_quant_codes(k[:, :, :nq], -2, g, levels)
        vq = ok.group_quant_codes(v[:, :, :nq], -1, g, levels)
        ref = oa.kivi_attend(q, kq[0], kq[1].astype(md), kq[2].astype(md), vq[0], vq[1].astype(md), vq[2].astype(md), g,
                             k[:, :, nq:t_end], v[:, :, nq:t_end], scale, causal=True)
        assert float(np.max(np.abs(got - ref))) < 2e-3, (t_end, Sq)
        # the codes themselves: what the wide fields hold is what the tight words hold
        kd = K.kivi_dequant(c._kp, c._ks, c._kz, -2, g, c._field, nq, D)
        kt = K.kivi_dequant(tight._kp, tight._ks, tight._kz, -2, g, bits, nq, D)
        vd = K.kivi_dequant(c._vp, c._vs, c._vz, -1, g, c._field, nq, D, v_layout=c._v_layout)
        vt = K.kivi_dequant(tight._vp, tight._vs, tight._vz, -1, g, bits, nq, D, v_layout=tight._v_layout)
        assert torch.equal(kd, kt) and torch.equal(vd, vt)

    check(n0)
    check(n0, Sq=3)
    for t in range(n0, n1):
        for x in (c, tight):
            x.update_and_fetch(to_dev(k[:, :, t:t + 1]), to_dev(v[:, :, t:t + 1]))
        if t % 13 == 0 or t == n1 - 1:
            check(t + 1)
    # saved and restored: the width of the field travels in meta_state, and a cache of the other packing refuses the file
    assert c.meta_state[2] == f"{bits}/{c._field}" and tight.meta_state[2] == str(bits)
    r = type(c).from_state(KVCacheConfig(method="kivi", **kw), c.state, c.meta_state)
    q = rng.standard_normal((B, Hq, 1, D)).astype(np.float16)
    assert torch.equal(r.fused_sdpa(to_dev(q), scale, fixed_order=True), c.fused_sdpa(to_dev(q), scale, fixed_order=True))
    with pytest.raises(ValueError):
        _make(**kw, kivi_code_field="tight").meta_state = c.meta_state
    # a trim into the packed rows brings them back as their reconstruction, the same one from either packing
    for x in (c, tight):
        assert x.trim(120) == 120
    check(n1 - 120, oracle=False)
    assert torch.equal(c._tail_k[:, :, : c.offset - c._n_quantized], tight._tail_k[:, :, : c.offset - c._n_quantized])


@pytest.mark.parametrize("bits,g,Hq,H,meta", [(4, 32, 32, 8, "float16"), (2, 64, 8, 2, "float32"), (2, 32, 14, 2, "float16"),
                                              (4, 64, 12, 4, "float16"), (3, 32, 4, 4, "float32"), (4, 32, 9, 3, "float16"),
                                              (2, 32, 5, 5, "float32")])
def test_heads_of_64_channels_are_kept_in_pairs(bits, g, Hq, H, meta):
    """A memory-bound cache of 64-channel heads keeps kv heads 2m and 2m+1 as one head of 128 channels (the head size of
    the matrix-unit kernels; queries zero-padded into their half): the stored codes are those of the unpaired cache, and
    chunked prefill, decode across flushes, per-sequence lengths, a window, the saved state, a trim and the layer stack
    agree with the oracle and with an unpaired cache (the vector kernel)."""
    require_gpu()
    from veloxquant_mlx_amd.cache import LayerStackedKIVICache
    B, D, R = 2, 64, 64
    kw = dict(head_dim=D, bit_width_inlier=bits, kivi_group_size=g, residual_length=R, fused_sdpa=True,
              fused_sdpa_memory_bound=True, kivi_meta_dtype=meta)
    c, plain = _make(**kw), _make(**kw, kivi_pair_heads=False)
    stack = LayerStackedKIVICache(KVCacheConfig(method="kivi", **kw), 2)
    n0, n1 = 600, 680
    k, v = outlier_kv((B, H, n1, D), seed=bits * 10 + g + Hq)
    rng = np.random.default_rng(Hq + g)
    scale, levels = 1 / math.sqrt(D), (1 << bits) - 1
    md = np.float16 if meta == "float16" else np.float32

    def oracle(q, t_end, nq, **okw):
        kq = ok.group_quant_codes(k[:, :, :nq], -2, g, levels)
        vq = ok.group_quant_codes(v[:, :, :nq], -1, g, levels)
        return oa.kivi_attend(q, kq[0], kq[1].astype(md), kq[2].astype(md), vq[0], vq[1].astype(md), vq[2].astype(md), g,
                              k[:, :, nq:t_end], v[:, :, nq:t_end], scale, **okw)

    # chunked prefill: every chunk attends causally over what is cached, itself included
    for lo in range(0, n0, 200):
        hi = min(lo + 200, n0)
        for x in (c, plain, stack[0], stack[1]):
            ret = x.update_and_fetch(to_dev(k[:, :, lo:hi]), to_dev(v[:, :, lo:hi]))
        assert tuple(ret[0].shape) == (B, H, hi, D)
        q = rng.standard_normal((B, Hq, hi - lo, D)).astype(np.float16)
        got = host(c.fused_sdpa(to_dev(q), scale, causal=True)).astype(np.float32)
        # (blocks of 256 query rows attend over the reconstruction rounded to fp16, as the reference's cache holds it)
        ref = oracle(q, hi, c._n_quantized, causal=True)
        assert float(np.max(np.abs(got - ref))) < 1e-2, (lo, float(np.max(np.abs(got - ref))))
    P = (H + 1) // 2   # an odd count: the last head's partner is a head of zeros
    assert c._pair and not plain._pair and c._shape_bhd == (B, P, 128) and c._n_quantized == plain._n_quantized
    assert c._kp.shape[1] == P and c._tail_k.shape[-1] == 128
    # the stored codes: the paired head holds its two heads' channels side by side
    nq = c._n_quantized
    f = c._field
    kd = K.kivi_dequant(c._kp, c._ks, c._kz, -2, g, f, nq, 128)
    vd = K.kivi_dequant(c._vp, c._vs, c._vz, -1, g, f, nq, 128, v_layout=c._v_layout)
    kp_ = K.kivi_dequant(plain._kp, plain._ks, plain._kz, -2, g, f, nq, D)
    vp_ = K.kivi_dequant(plain._vp, plain._vs, plain._vz, -1, g, f, nq, D, v_layout=plain._v_layout)
    unpair = lambda x: x.view(B, P, nq, 2, D).transpose(2, 3).reshape(B, 2 * P, nq, D)[:, :H]
    assert torch.equal(unpair(kd), kp_) and torch.equal(unpair(vd), vp_)

    def step_checks(t_end):
        q = rng.standard_normal((2, B, Hq, 1, D)).astype(np.float16)
        got = host(c.fused_sdpa(to_dev(q[0]), scale)).astype(np.float32)
        other = host(plain.fused_sdpa(to_dev(q[0]), scale)).astype(np.float32)
        ref = oracle(q[0], t_end, c._n_quantized)
        assert got.shape == (B, Hq, 1, D)
        assert float(np.max(np.abs(got - ref))) < 2e-3 and float(np.max(np.abs(got - other))) < 2e-3, t_end
        both = stack.fused_sdpa_all(to_dev(q), scale)
        assert tuple(both.shape) == (2, B, Hq, 1, D)
        assert float((both[0].float().cpu() - torch.from_numpy(got)).abs().max()) < 1e-3
        assert float(np.max(np.abs(host(both[1]).astype(np.float32) - oracle(q[1], t_end, c._n_quantized)))) < 2e-3

    for t in range(n0, n1):
        for x in (c, plain, stack[0], stack[1]):
            x.update_and_fetch(to_dev(k[:, :, t:t + 1]), to_dev(v[:, :, t:t + 1]))
        if t % 11 == 0 or t == n1 - 1:
            step_checks(t + 1)
    # per-sequence lengths and a sliding window
    q = rng.standard_normal((B, Hq, 1, D)).astype(np.float16)
    lens = torch.tensor([n1 - 37, n1], dtype=torch.int32)
    got = host(c.fused_sdpa(to_dev(q), scale, lengths=lens)).astype(np.float32)
    other = host(plain.fused_sdpa(to_dev(q), scale, lengths=lens)).astype(np.float32)
    assert float(np.max(np.abs(got - other))) < 2e-3
    got = host(c.fused_sdpa(to_dev(q), scale, sliding_window=100)).astype(np.float32)
    ref = oracle(q, n1, c._n_quantized, sliding_window=100)
    assert float(np.max(np.abs(got - ref))) < 2e-3
    # saved and restored (the rows of the state are the paired ones), then trimmed
    r = type(c).from_state(KVCacheConfig(method="kivi", **kw), c.state, c.meta_state)
    assert r._pair and r._shape_bhd == c._shape_bhd and r.offset == c.offset
    assert torch.equal(r.fused_sdpa(to_dev(q), scale, fixed_order=True), c.fused_sdpa(to_dev(q), scale, fixed_order=True))
    for x in (c, plain):
        assert x.trim(100) == 100
    got = host(c.fused_sdpa(to_dev(q), scale)).astype(np.float32)
    other = host(plain.fused_sdpa(to_dev(q), scale)).astype(np.float32)
    assert c.offset == plain.offset == n1 - 100 and float(np.max(np.abs(got - other))) < 2e-3


@pytest.mark.parametrize("D,bits", [(64, 4), (256, 2), (128, 3)])
def test_sink_protected_cache_on_the_other_decode_kernels(D, bits):
    """Protected rows where the attention kernel is the vector one (head size 64, 3-bit codes) or the 256-channel form of
    the matrix-unit one: the patch pass works from the partials, whichever kernel wrote them."""
    require_gpu()
    rng = np.random.default_rng(D + bits)
    B, Hq, H, R, n = 2, 8, 2, 64, 420 if bits != 3 else 480
    k = rng.standard_normal((B, H, n, D)).astype(np.float16)
    v = rng.standard_normal((B, H, n, D)).astype(np.float16)
    for p, f in ((7, 11), (130, 9), (131, 13)):
        k[:, :, p] *= f
    cfg = KVCacheConfig(method="kivi_sink", head_dim=D, bit_width_inlier=bits, kivi_group_size=32, residual_length=R,
                        n_sink_tokens=3, fused_sdpa=True, fused_sdpa_memory_bound=True, kivi_meta_dtype="float32",
                        kivi_code_field="tight")
    c = KVCacheFactory.create(cfg)
    m = ok.SinkCacheModel(bits, 32, R, 3)
    c.update_and_fetch(to_dev(k[:, :, :320]), to_dev(v[:, :, :320]))
    m.update_and_fetch(k[:, :, :320], v[:, :, :320])
    for t in range(320, n):
        c.update_and_fetch(to_dev(k[:, :, t:t + 1]), to_dev(v[:, :, t:t + 1]))
        m.update_and_fetch(k[:, :, t:t + 1], v[:, :, t:t + 1])
    assert c._n_quantized == m.n_quantized and any(c._side_pos[b] for b in range(B))
    km, vm = m.keys[:, :, : m.offset], m.values[:, :, : m.offset]
    scale = 1 / math.sqrt(D)
    for Sq in (1, 3):
        q = rng.standard_normal((B, Hq, Sq, D)).astype(np.float16)
        row = km[0, 0, m.sink_positions_for(0)[0]].astype(np.float32)
        q[0, 0, -1] += (row / np.linalg.norm(row) * 5).astype(np.float16)
        got = host(c.fused_sdpa(to_dev(q), scale, causal=True)).astype(np.float32)
        ref = oa.sdpa(q, km, vm, scale, causal=True)
        err = float(np.max(np.abs(got - ref)))
        assert err < 2e-3, (Sq, err)


def test_prefill_tile_scratch_is_given_back_by_every_kind_of_decode_step():
    """The tile scratch of a memory-bound prefill lives only until decoding begins: a single-token append, a
    single-query attend with per-sequence ``lengths`` and the layer-stacked launch all return ``nbytes`` to the
    packed size."""
    require_gpu()
    from veloxquant_mlx_amd.cache import LayerStackedKIVICache
    B, Hq, Hkv, D, C = 2, 16, 4, 128, 256
    dev = "cuda:0"
    gen = torch.Generator(device=dev).manual_seed(9)
    scale = 1 / math.sqrt(D)

    def prefilled(tiles=True):
        c = _make(bit_width_inlier=4, kivi_group_size=32, residual_length=128, fused_sdpa=True, fused_sdpa_memory_bound=True)
        c.prefill_tiles = tiles
        for _ in range(3):
            k = torch.randn((B, Hkv, C, D), generator=gen, device=dev).to(torch.float16)
            v = torch.randn((B, Hkv, C, D), generator=gen, device=dev).to(torch.float16)
            q = torch.randn((B, Hq, C, D), generator=gen, device=dev).to(torch.float16)
            c.update_and_fetch(k, v)
            c.fused_sdpa(q, scale, causal=True)
        return c

    plain = prefilled(tiles=False).nbytes
    q1 = torch.randn((B, Hq, 1, D), generator=gen, device=dev).to(torch.float16)
    # (a) decode with per-sequence lengths, no append in between
    c = prefilled()
    assert c._tiles is not None and c.nbytes > plain
    c.fused_sdpa(q1, scale, lengths=torch.tensor([c.offset, c.offset - 5]))
    assert c._tiles is None and c.nbytes == plain
    # (b) the single-token append alone
    c = prefilled()
    c.update_and_fetch(torch.randn((B, Hkv, 1, D), generator=gen, device=dev).to(torch.float16),
                       torch.randn((B, Hkv, 1, D), generator=gen, device=dev).to(torch.float16))
    assert c._tiles is None
    # (c) the layer-stacked launch
    layers = [prefilled(), prefilled()]
    assert all(l._tiles is not None for l in layers)
    stack = LayerStackedKIVICache.from_layers(layers)
    stack.fused_sdpa_all(torch.stack([q1, q1]), scale)
    assert all(l._tiles is None for l in layers)


def test_config4_every_chunk_against_the_oracle_on_sampled_rows():
    """Benchmark configuration 4 at full size, every one of the 8 chunks: for one kv head the host
    quantises the same bf16 keys and values with the numpy oracle (one shot over the packed prefix:
    whole groups are independent of how the cache was flushed), and sampled query rows -- first,
    last and two inner positions of the chunk, all four query heads of the group -- are attended
    over (reconstruction | residual rows) in float64.  The 256-row MFMA blocks attend over the
    reconstruction rounded to fp16, which is the oracle's ``recon_dtype``."""
    require_gpu()
    B, Hq, Hkv, D, P, C, g = 1, 32, 8, 128, 4096, 512, 32
    dev = "cuda:0"
    gen = torch.Generator(device=dev).manual_seed(41)
    f = torch.exp(torch.randn(D, generator=gen, device=dev))
    c = _make(bit_width_inlier=4, kivi_group_size=g, residual_length=128, fused_sdpa=True,
              fused_sdpa_memory_bound=True)
    mk = lambda n: ((torch.randn((B, Hkv, n, D), generator=gen, device=dev) * f).to(torch.bfloat16),
                    torch.randn((B, Hkv, n, D), generator=gen, device=dev).to(torch.bfloat16))
    hk = 5                                        # the kv head the host follows
    k0, v0 = mk(P)
    c.update_and_fetch(k0, v0)
    k_all, v_all = [host(k0[:, hk:hk + 1])], [host(v0[:, hk:hk + 1])]
    scale = 1 / math.sqrt(D)
    rng = np.random.default_rng(8)
    worst = 0.0
    for ci in range(8):
        kc_, vc_ = mk(C)
        c.update_and_fetch(kc_, vc_)
        k_all.append(host(kc_[:, hk:hk + 1]))
        v_all.append(host(vc_[:, hk:hk + 1]))
        q = torch.randn((B, Hq, C, D), generator=gen, device=dev).to(torch.bfloat16)
        out = host(c.fused_sdpa(q, scale, causal=True))
        nq = c._n_quantized
        kh, vh = np.concatenate(k_all, axis=2), np.concatenate(v_all, axis=2)     # float32 views of the bf16 rows
        n_total = kh.shape[2]
        assert n_total == c.offset and nq == (n_total - 128) // g * g
        kcodes, ksc, kzr = ok.group_quant_codes(kh[:, :, :nq], -2, g, 15)
        vcodes, vsc, vzr = ok.group_quant_codes(vh[:, :, :nq], -1, g, 15)
        meta = [a.astype(np.float16) for a in (ksc, kzr, vsc, vzr)]
        heads = slice(hk * (Hq // Hkv), (hk + 1) * (Hq // Hkv))
        for pos in sorted({0, C - 1, *rng.integers(1, C - 1, 2).tolist()}):
            vis = n_total - C + pos + 1
            npk = min(vis, nq)
            ref = oa.kivi_attend(host(q[:, heads, pos:pos + 1]), kcodes[:, :, :npk], meta[0][:, :, : -(-npk // g)], meta[1][:, :, : -(-npk // g)],
                                 vcodes[:, :, :npk], meta[2][:, :, :npk], meta[3][:, :, :npk], g,
                                 kh[:, :, nq:vis], vh[:, :, nq:vis], scale, recon_dtype=np.float16)
            err = float(np.max(np.abs(out[:, heads, pos:pos + 1] - ref)))
            worst = max(worst, err)
            # the output is bf16 (8 significant bits): half an ulp of values up to ~1 on top of the 2e-3 bar
            assert err < 2e-3 + 2.0 ** -9, (ci, pos, err)
    print(f"8 chunks, sampled rows: max |out - oracle| = {worst:.2e}")


@pytest.mark.parametrize("chunk,g", [(128, 32), (80, 32), (96, 64)])
def test_chunked_prefill_with_no_residual_window(chunk, g):
    """The other reading of quantise-on-write: ``residual_length=0``, every whole group is packed
    as soon as it is complete, so a chunk's queries see (nearly) all tokens, their own included, in
    quantised form and the causal edge runs through the packed prefix."""
    require_gpu()
    B, Hq, Hkv, S, D = 1, 8, 2, 480, 128
    k, v = outlier_kv((B, Hkv, S, D), seed=14)
    q = np.random.default_rng(6).standard_normal((B, Hq, S, D)).astype(np.float16)
    c = _make(bit_width_inlier=4, kivi_group_size=g, residual_length=0, fused_sdpa=True,
              fused_sdpa_memory_bound=True, kivi_meta_dtype="float32")
    outs, refs = [], []
    kc_, ks_, kz_ = ok.group_quant_codes(k, -2, g, 15)     # whole groups do not depend on when they were flushed
    vc_, vs_, vz_ = ok.group_quant_codes(v, -1, g, 15)
    for s0 in range(0, S, chunk):
        s1 = min(S, s0 + chunk)
        c.update_and_fetch(to_dev(k[:, :, s0:s1]), to_dev(v[:, :, s0:s1]))
        nq = s1 // g * g
        assert c._n_quantized == nq and c.offset - nq < g
        outs.append(host(c.fused_sdpa(to_dev(q[:, :, s0:s1]), 1 / math.sqrt(D), causal=True)))
        refs.append(oa.kivi_attend(q[:, :, s0:s1], kc_[:, :, :nq], ks_[:, :, : nq // g], kz_[:, :, : nq // g], vc_[:, :, :nq],
                                   vs_[:, :, :nq], vz_[:, :, :nq], g, k[:, :, nq:s1], v[:, :, nq:s1], 1 / math.sqrt(D), causal=True))
    got = np.concatenate(outs, axis=2).astype(np.float32)
    # every chunk here has 256 query rows or more per kv head and runs on the 256-row prefill blocks,
    # which attend over the reconstruction rounded to fp16: what the cache model holds
    # (kivi_cache.py:198-201) and the oracle at the usual bar.  With every token quantised that
    # rounding shows against code * scale + zero itself, inside the 1e-2 bar of the reference's own
    # fused-attention tests.
    assert np.max(np.abs(got - oa.chunked_prefill(q, k, v, chunk, 4, g, 0, 1 / math.sqrt(D)))) < 2e-3
    assert np.max(np.abs(got - np.concatenate(refs, axis=2))) < 1e-2


def test_bf16_history_holds_the_reconstruction_rounded_to_bf16():
    """Keys and values that arrive in bf16: the standard cache returns, below the frontier, the
    float32 reconstruction cast to bf16 -- ``recon.astype(x.dtype)``, kivi_cache.py:198-201 -- bit
    for bit; the packed cache never forms those rows: its attention works on code * scale + zero
    with scale / zero in the configured storage type, and differs from attention over the bf16
    history by less than bf16 rounding of keys and values allows."""
    require_gpu()
    B, Hq, Hkv, S, D, g = 1, 8, 2, 320, 128, 32
    k, v = outlier_kv((B, Hkv, S, D), seed=15)
    bf = lambda a: torch.from_numpy(a.astype(np.float32)).to(torch.bfloat16)
    kb, vb = bf(k), bf(v)
    cast = lambda a: torch.from_numpy(a).to(torch.bfloat16).float().numpy()
    std = _make(bit_width_inlier=4, kivi_group_size=g, residual_length=64)
    ko, vo = std.update_and_fetch(kb.to("cuda:0"), vb.to("cuda:0"))
    assert ko.dtype == torch.bfloat16
    nq = std._n_quantized
    assert nq == 256
    k32, v32 = kb.float().numpy(), vb.float().numpy()
    assert np.array_equal(host(ko)[:, :, :nq], ok.quant_dequant_along(k32[:, :, :nq], -2, g, 15, cast=cast))
    assert np.array_equal(host(vo)[:, :, :nq], ok.quant_dequant_along(v32[:, :, :nq], -1, g, 15, cast=cast))
    assert np.array_equal(host(ko)[:, :, nq:], k32[:, :, nq:])
    packed = _make(bit_width_inlier=4, kivi_group_size=g, residual_length=64, fused_sdpa=True, fused_sdpa_memory_bound=True,
                   kivi_meta_dtype="float32")
    packed.update_and_fetch(kb.to("cuda:0"), vb.to("cuda:0"))
    q = np.random.default_rng(7).standard_normal((B, Hq, 1, D)).astype(np.float16)
    got = host(packed.fused_sdpa(to_dev(q), 1 / math.sqrt(D), causal=False)).astype(np.float32)
    exact = oa.sdpa(q, np.concatenate([ok.quant_dequant_along(k32[:, :, :nq], -2, g, 15), k32[:, :, nq:]], axis=2),
                    np.concatenate([ok.quant_dequant_along(v32[:, :, :nq], -1, g, 15), v32[:, :, nq:]], axis=2), 1 / math.sqrt(D))
    over_bf16 = oa.sdpa(q, host(ko), host(vo), 1 / math.sqrt(D))
    assert np.max(np.abs(got - exact)) < 2e-3
    assert np.max(np.abs(got - over_bf16)) < 1e-2


@pytest.mark.parametrize("memory_bound", [True, False])
def test_cache_attention_under_a_window_and_with_sequence_lengths(memory_bound):
    """``KIVIKVCache.fused_sdpa`` with ``sliding_window`` (the parameter the fused dispatcher passes on)
    and with per-sequence ``lengths`` of a right-padded batch, in the packed-only and the stash mode,
    against the oracle over (reconstruction | fp16 rows)."""
    require_gpu()
    B, Hq, Hkv, D, g, n = 3, 8, 2, 128, 32, 700
    k, v = outlier_kv((B, Hkv, n, D), seed=44)
    c = _make(bit_width_inlier=4, kivi_group_size=g, residual_length=64, fused_sdpa=True,
              fused_sdpa_memory_bound=memory_bound, kivi_meta_dtype="float32")
    c.update_and_fetch(to_dev(k), to_dev(v))
    nq = c._n_quantized
    assert nq == (n - 64) // g * g
    kc_, ks_, kz_ = ok.group_quant_codes(k[:, :, :nq], -2, g, 15)
    vc_, vs_, vz_ = ok.group_quant_codes(v[:, :, :nq], -1, g, 15)
    scale = 1 / math.sqrt(D)
    rng = np.random.default_rng(45)
    for Sq, causal in ((1, False), (5, True), (40, True)):
        q = rng.standard_normal((B, Hq, Sq, D)).astype(np.float16)
        for w in (0, 17, 90, 400):
            got = host(c.fused_sdpa(to_dev(q), scale, causal=causal, sliding_window=w)).astype(np.float32)
            ref = oa.kivi_attend(q, kc_, ks_, kz_, vc_, vs_, vz_, g, k[:, :, nq:], v[:, :, nq:], scale, causal=causal,
                                 sliding_window=w)
            assert np.max(np.abs(got - ref)) < 2e-3, (Sq, w)
        lengths = [n, 655, 300]
        for lens in (torch.tensor(lengths), torch.tensor(lengths, device="cuda:0", dtype=torch.int32)):
            got = host(c.fused_sdpa(to_dev(q), scale, causal=causal, lengths=lens)).astype(np.float32)
            for b, nb in enumerate(lengths):
                npk = min(nb, nq)
                ref = oa.kivi_attend(q[b:b + 1], kc_[b:b + 1, :, :npk], ks_[b:b + 1, :, : -(-npk // g)], kz_[b:b + 1, :, : -(-npk // g)],
                                     vc_[b:b + 1, :, :npk], vs_[b:b + 1, :, :npk], vz_[b:b + 1, :, :npk], g,
                                     k[b:b + 1, :, nq:nb], v[b:b + 1, :, nq:nb], scale, causal=causal)
                assert np.max(np.abs(got[b:b + 1] - ref)) < 2e-3, (Sq, b)
    with pytest.raises(ValueError, match="lengths has"):
        c.fused_sdpa(to_dev(q), scale, lengths=torch.tensor([1, 2]))


def test_config3_decode_at_full_size_against_the_oracle_and_the_vector_kernel():
    """Benchmark configuration 3, one layer: batch 16, 32 query / 8 kv heads, D=128, 32768 tokens of
    context in a 4-bit group-64 packed cache plus the fp16 residual, one query token.  The last
    sequence is checked against the scalar C oracle (about a second of CPU), every sequence
    against the independent vector kernel."""
    require_gpu()
    from oracle import cref
    B, Hq, Hkv, D, ctx, g, bits = 16, 32, 8, 128, 32768, 64, 4
    dev = "cuda:0"
    gen = torch.Generator(device=dev).manual_seed(33)
    f = torch.exp(torch.randn(D, generator=gen, device=dev))
    c = _make(bit_width_inlier=bits, kivi_group_size=g, residual_length=128, fused_sdpa=True,
              fused_sdpa_memory_bound=True)
    n_total = ctx + 128 + 37                      # packed prefix of ctx tokens, 165 in the residual
    for s0 in range(0, n_total, 4096):
        n = min(4096, n_total - s0)
        c.update_and_fetch((torch.randn((B, Hkv, n, D), generator=gen, device=dev) * f).half(),
                           torch.randn((B, Hkv, n, D), generator=gen, device=dev).half())
    nq, n_tail = c._n_quantized, c.offset - c._n_quantized
    assert nq == ctx and n_tail == 165
    q = torch.randn((B, Hq, 1, D), generator=gen, device=dev).half()
    scale = 1 / math.sqrt(D)
    kw = dict(k_packed=c._kp, k_scale=c._ks, k_zero=c._kz, v_packed=c._vp, v_scale=c._vs, v_zero=c._vz,
              n_packed=nq, bits=bits, group_size=g, v_layout="token", k_tail=c._tail_k, v_tail=c._tail_v,
              n_tail=n_tail, scale=scale, out_dtype=torch.float32)
    p1, p0 = {}, {}
    o1 = K.kivi_packed_attend(q, _plan_out=p1, **kw)
    o0 = K.kivi_packed_attend(q, num_splits=-1, _plan_out=p0, **kw)
    assert p1["path"] == 1 and p0["path"] == 0
    err = float((o1 - o0).abs().max())
    print(f"max |mfma - vector| over 16 sequences = {err:.2e}")
    assert err < 2e-3
    # chunks handed out on demand: repeated runs agree to rounding; dealt in a fixed order: bit for bit
    assert float((c.fused_sdpa(q, scale).float() - o1).abs().max()) < 2e-3   # fp16 output
    f1, f2 = K.kivi_packed_attend(q, fixed_order=True, **kw), K.kivi_packed_attend(q, fixed_order=True, **kw)
    assert torch.equal(f1, f2) and float((f1 - o1).abs().max()) < 2e-3

    b, per = B - 1, 32 // bits
    kp = c._kp[b:b + 1, :, :nq].cpu().numpy().view(np.uint32)
    codes_k = ok.unpack_indices(kp, bits, D)
    vp = c._vp[b:b + 1, :, : nq // per].cpu().numpy().view(np.uint32)
    codes_v = np.ascontiguousarray(ok.unpack_indices(np.ascontiguousarray(vp.swapaxes(-1, -2)), bits, nq).swapaxes(-1, -2))
    ks, kz = (t[b:b + 1, :, : nq // g].float().cpu().numpy() for t in (c._ks, c._kz))
    vs, vz = (np.ascontiguousarray(t[b:b + 1, :, :, :nq].float().cpu().numpy().swapaxes(-1, -2)) for t in (c._vs, c._vz))
    ref = cref.attend(q[b:b + 1].float().cpu().numpy(), codes_k, ks, kz, codes_v, vs, vz, g, scale,
                      k_tail=c._tail_k[b:b + 1, :, :n_tail].float().cpu().numpy(),
                      v_tail=c._tail_v[b:b + 1, :, :n_tail].float().cpu().numpy())
    err = float(np.max(np.abs(o1[b:b + 1].cpu().numpy() - ref)))
    print(f"max |mfma - oracle| on the last sequence = {err:.2e}")
    assert err < 2e-3


def test_config3_all_36_layers_in_one_launch_equal_the_per_layer_calls_bit_for_bit():
    """Benchmark configuration 3 at full size through ``LayerStackedKIVICache``: 36 layers x 16 sequences x
    32768 tokens of 4-bit group-64 packed context plus the fp16 residual, the newest token appended by the
    launch itself.  With chunks dealt in a fixed order the one launch over all layers equals the 36
    per-layer launches bit for bit (the layer-batched call of veloxquant_mlx/metal/_scalar_attend.py:496-647
    against its per-layer loop, tests/metal/test_scalar_attend.py:660-707); one layer's last sequence is
    checked against the scalar C oracle."""
    require_gpu()
    from oracle import cref
    from veloxquant_mlx_amd.cache import LayerStackedKIVICache
    NL, B, Hq, Hkv, D, ctx, g, bits = 36, 16, 32, 8, 128, 32768, 64, 4
    dev = "cuda:0"
    gen = torch.Generator(device=dev).manual_seed(3)
    f = torch.exp(torch.randn(D, generator=gen, device=dev))
    n_total = ctx + 128 + 37
    layers = []
    for l in range(NL):
        c = _make(bit_width_inlier=bits, kivi_group_size=g, residual_length=128, fused_sdpa=True,
                  fused_sdpa_memory_bound=True, fused_sdpa_max_ctx=ctx + 4096)
        for s0 in range(0, n_total, 8192):
            n = min(8192, n_total - s0)
            c.update_and_fetch((torch.randn((B, Hkv, n, D), generator=gen, device=dev) * f).half(),
                               torch.randn((B, Hkv, n, D), generator=gen, device=dev).half())
        assert c._n_quantized == ctx
        layers.append(c)
    stack = LayerStackedKIVICache.from_layers(layers)
    q = torch.randn((NL, B, Hq, 1, D), generator=gen, device=dev).half()
    scale = 1 / math.sqrt(D)
    # (the same cut of the context on both sides: left to themselves 576 sequences take one run, 16 take two)
    all_at_once = stack.fused_sdpa_all(q, scale, fixed_order=True, num_splits=2)
    assert all_at_once.shape == (NL, B, Hq, 1, D)
    for l, c in enumerate(layers):
        one = c.fused_sdpa(q[l], scale, fixed_order=True, num_splits=2)
        assert torch.equal(one, all_at_once[l]), (l, float((one.float() - all_at_once[l].float()).abs().max()))
    # the default order (chunks handed out on demand) agrees to rounding
    assert float((stack.fused_sdpa_all(q, scale).float() - all_at_once.float()).abs().max()) < 2e-3
    # a decode step of all layers: 36 appends that launch nothing, one launch that stores and attends
    k_new, v_new = (torch.randn((NL, B, Hkv, 1, D), generator=gen, device=dev).half() for _ in range(2))
    for l, c in enumerate(layers):
        c.update_and_fetch(k_new[l], v_new[l])
    stepped = stack.fused_sdpa_all(q, scale)
    l, b, per = NL - 1, B - 1, 32 // bits
    c = layers[l]
    assert c._pending is None and c.offset == n_total + 1 and torch.equal(c._tail_k[:, :, n_total - ctx, :], k_new[l][:, :, 0, :])
    nq, n_tail = c._n_quantized, c.offset - c._n_quantized
    kp = c._kp[b:b + 1, :, :nq].cpu().numpy().view(np.uint32)
    codes_k = ok.unpack_indices(kp, bits, D)
    vp = c._vp[b:b + 1, :, : nq // per].cpu().numpy().view(np.uint32)
    codes_v = np.ascontiguousarray(ok.unpack_indices(np.ascontiguousarray(vp.swapaxes(-1, -2)), bits, nq).swapaxes(-1, -2))
    ks, kz = (t[b:b + 1, :, : nq // g].float().cpu().numpy() for t in (c._ks, c._kz))
    vs, vz = (np.ascontiguousarray(t[b:b + 1, :, :, :nq].float().cpu().numpy().swapaxes(-1, -2)) for t in (c._vs, c._vz))
    ref = cref.attend(q[l, b:b + 1].float().cpu().numpy(), codes_k, ks, kz, codes_v, vs, vz, g, scale,
                      k_tail=c._tail_k[b:b + 1, :, :n_tail].float().cpu().numpy(),
                      v_tail=c._tail_v[b:b + 1, :, :n_tail].float().cpu().numpy())
    err = float(np.max(np.abs(stepped[l, b:b + 1].float().cpu().numpy() - ref)))
    print(f"layer {l}, last sequence: max |one launch - oracle| = {err:.2e}")
    assert err < 2e-3


def test_kivi_quantizer_encode_decode():
    require_gpu()
    rng = np.random.default_rng(0)
    x = rng.standard_normal((96, 128)).astype(np.float16)
    for axis, ax in (("channel", -2), ("token", -1)):
        qz = KIVIQuantizer(d=128, b=2, group_size=32, axis=axis)
        ev = qz.encode(to_dev(x))
        codes, scale, zero = ok.group_quant_codes(x[None, None], ax, 32, 3)
        assert np.array_equal(host(ev.indices), codes[0, 0]) and np.array_equal(host(ev.norm), scale[0, 0])
        assert ev.memory_bytes() == codes.nbytes + scale.nbytes + zero.nbytes
        dec = qz.decode(ev)
        assert np.array_equal(host(dec), ok.group_dequant(codes, scale, zero, ax, 32)[0, 0].astype(np.float16))
        qv = rng.standard_normal(128).astype(np.float16)
        ip = qz.estimate_inner_product(to_dev(qv), ev)
        np.testing.assert_allclose(host(ip).astype(np.float32), host(dec).astype(np.float32) @ qv.astype(np.float32),
                                   rtol=2e-3, atol=2e-2)
    from veloxquant_mlx_amd.core import QuantizerConfigError
    bad = x.copy(); bad[0, 0] = np.inf
    with pytest.raises(QuantizerConfigError, match="NaN or Inf"):
        KIVIQuantizer(d=128).encode(to_dev(bad))


# ------------------------------------------------------------------ VecInfer
def _vi_cfg(**kw):
    rng = np.random.default_rng(7)
    base = dict(method="vecinfer", head_dim=128, key_sub_dim=8, value_sub_dim=8, key_codebook_bits=8,
                value_codebook_bits=8, key_codebook=rng.standard_normal((256, 8)).astype(np.float32),
                value_codebook=rng.standard_normal((256, 8)).astype(np.float32))
    base.update(kw)
    return KVCacheConfig(**base)


def test_vecinfer_standard_mode_matches_oracle_pipeline():
    require_gpu()
    rng = np.random.default_rng(1)
    smooth = (np.abs(rng.standard_normal((2, 128))) + 0.5).astype(np.float32)
    cfg = _vi_cfg(smooth_factors=smooth)
    c = KVCacheFactory.create(cfg)
    k, v = _kv(1, 2, 40, 128, 2)
    ko, vo = c.update_and_fetch(to_dev(k), to_dev(v))
    # values: plain VQ round trip, exact
    v_idx = ov.quantize_vq(v, cfg.value_codebook, 8)
    assert np.array_equal(host(vo), ov.dequantize_vq(v_idx, cfg.value_codebook).astype(np.float16))
    # keys: transform (BLAS) then VQ; compare the reconstruction within fp16 rounding
    H = ov.walsh_hadamard_matrix(128)
    kt = ov.apply_dual_transform_keys(k, smooth, H)
    k_hat = (ov.dequantize_vq(ov.quantize_vq(kt, cfg.key_codebook, 8), cfg.key_codebook) @ H.T) * smooth[:, None, :]
    close = np.isclose(host(ko).astype(np.float32), k_hat, atol=2e-2, rtol=2e-3)
    assert close.mean() > 0.995   # a near-tie may flip one sub-vector's centroid
    assert c.compressed_key_bytes == 16 * 2 * 40 and c.fp16_key_bytes == 2 * 40 * 128 * 2


@pytest.mark.parametrize("memory_bound", [False, True])
def test_vecinfer_fused_modes_and_state_round_trip(memory_bound):
    require_gpu()
    cfg = _vi_cfg(fused_sdpa=True, fused_sdpa_memory_bound=memory_bound)
    c = KVCacheFactory.create(cfg)
    k, v = _kv(2, 2, 70, 128, 3)
    c.update_and_fetch(to_dev(k[:, :, :64]), to_dev(v[:, :, :64]))
    for t in range(64, 70):
        ko, vo = c.update_and_fetch(to_dev(k[:, :, t:t + 1]), to_dev(v[:, :, t:t + 1]))
    assert c.offset == 70 and c._stored_S_kv == 70 and c._stored_k_indices.shape[2] == 256
    H = ov.walsh_hadamard_matrix(128)
    k_idx = host(c._stored_k_indices[:, :, :70])
    v_idx = host(c._stored_v_indices[:, :, :70])
    assert np.array_equal(v_idx, ov.quantize_vq(v, cfg.value_codebook, 8))
    kt_gpu = host(to_dev(k).float() @ to_dev(H))
    assert np.array_equal(k_idx, ov.quantize_vq(kt_gpu, cfg.key_codebook, 8))
    q = np.random.default_rng(4).standard_normal((2, 8, 1, 128)).astype(np.float16)
    out = c.fused_sdpa(to_dev(q), 0.09, causal=True)
    k_t_hat = ov.dequantize_vq(k_idx, cfg.key_codebook)
    v_hat = ov.dequantize_vq(v_idx, cfg.value_codebook)
    ref = oa.sdpa(q.astype(np.float32) @ H, k_t_hat, v_hat, 0.09)
    assert np.max(np.abs(host(out).astype(np.float32) - ref)) < 2e-3
    st = c.state
    if memory_bound:
        assert len(st) == 2 and st[0].shape == (2, 2, 70, 16) and float(ko.abs().sum()) == 0
        c2 = KVCacheFactory.create(cfg)
        c2.state = st
        assert c2.offset == 70 and c2._stored_S_kv == 70
        # the value histogram is summed in LDS in arrival order: equal up to float reassociation
        assert float((c2.fused_sdpa(to_dev(q), 0.09).float() - out.float()).abs().max()) < 2e-3
    else:
        assert len(st) == 4 and st[0].shape == (2, 2, 70, 128)
    assert c.trim(6) == 6 and c._stored_S_kv == 64 and c.offset == 64
    assert c.compressed_key_bytes == int(16 * 2 * 2 * 70 * (64 / 70))
    out_w = c.fused_sdpa(to_dev(q), 0.09, sliding_window=16)
    ref_w = oa.sdpa(q.astype(np.float32) @ H, k_t_hat[:, :, :64], v_hat[:, :, :64], 0.09, sliding_window=16)
    assert np.max(np.abs(host(out_w).astype(np.float32) - ref_w)) < 2e-3


@pytest.mark.parametrize("D,Hq,H,Sq,window", [(128, 8, 2, 100, 0), (128, 6, 2, 120, 64), (256, 12, 4, 100, 0), (128, 8, 2, 40, 0)])
def test_vecinfer_prefill_sized_queries_attend_over_gathered_rows(D, Hq, H, Sq, window):
    """256 query rows or more per kv head: the cache gathers the centroids once into 16-bit rows and runs the
    matrix-unit prefill blocks over them instead of building a look-up table per query row; fewer rows (the last case)
    stay on the table kernel.  Both against the oracle over the stored indices."""
    require_gpu()
    rng = np.random.default_rng(D + Sq)
    cfg = _vi_cfg(head_dim=D, fused_sdpa=True, fused_sdpa_memory_bound=True)
    c = KVCacheFactory.create(cfg)
    n = 700
    k, v = _kv(2, H, n, D, 5)
    c.update_and_fetch(to_dev(k[:, :, :400]), to_dev(v[:, :, :400]))
    c.update_and_fetch(to_dev(k[:, :, 400:]), to_dev(v[:, :, 400:]))
    q = rng.standard_normal((2, Hq, Sq, D)).astype(np.float16)
    out = host(c.fused_sdpa(to_dev(q), 0.09, causal=True, sliding_window=window)).astype(np.float32)
    Hm = ov.walsh_hadamard_matrix(D)
    k_t_hat = ov.dequantize_vq(host(c._stored_k_indices[:, :, :n]), cfg.key_codebook)
    v_hat = ov.dequantize_vq(host(c._stored_v_indices[:, :, :n]), cfg.value_codebook)
    gathered = (Hq // H) * Sq >= 256
    if gathered:   # the rows are rounded to the queries' type, as the reconstruction the cache hands out is
        k_t_hat, v_hat = k_t_hat.astype(np.float16).astype(np.float32), v_hat.astype(np.float16).astype(np.float32)
    ref = oa.sdpa(q.astype(np.float32) @ Hm, k_t_hat, v_hat, 0.09, causal=True, sliding_window=window)
    assert np.max(np.abs(out - ref)) < 2e-3, float(np.max(np.abs(out - ref)))
    # and against the table kernel on the same indices
    tab = K.metal_fused_sdpa(to_dev(q).float() @ to_dev(Hm), c._stored_k_indices, c._key_codebook, c._stored_v_indices,
                             c._value_codebook, 0.09, causal=True, sliding_window=window, out_dtype=torch.float16, n_tokens=n)
    assert float(np.max(np.abs(out - host(tab).astype(np.float32)))) < (4e-3 if gathered else 1e-6)


def test_vecinfer_max_ctx_cap():
    require_gpu()
    c = KVCacheFactory.create(_vi_cfg(fused_sdpa=True, fused_sdpa_max_ctx=100))
    k, v = _kv(1, 1, 90, 128, 1)
    c.update_and_fetch(to_dev(k), to_dev(v))
    with pytest.raises(RuntimeError, match="exceeded fused_sdpa_max_ctx=100"):
        c.update_and_fetch(to_dev(k[:, :, :20]), to_dev(v[:, :, :20]))


def test_decode_steps_store_the_new_token_in_the_attention_launch():
    """Memory-bound decode: a step with no flush due hands the new token to the attention launch
    (vq_attend_args.k_new / v_new), which stores it in the tail and attends in one go.  Sixty
    steps against the cache model + oracle, across two flushes, with a state read, a trim and a
    two-token step in between; the tail must hold every token afterwards."""
    require_gpu()
    B, Hq, Hkv, D, g, R = 2, 8, 2, 128, 32, 64
    k, v = outlier_kv((B, Hkv, 400, D), seed=21)
    rng = np.random.default_rng(3)
    c = _make(bit_width_inlier=4, kivi_group_size=g, residual_length=R, fused_sdpa=True, fused_sdpa_memory_bound=True)
    c.update_and_fetch(to_dev(k[:, :, :300]), to_dev(v[:, :, :300]))
    deferred = 0
    pos = 300
    levels = 15
    for step in range(60):
        n_new = 2 if step == 17 else 1
        c.update_and_fetch(to_dev(k[:, :, pos:pos + n_new]), to_dev(v[:, :, pos:pos + n_new]))
        pos += n_new
        deferred += c._pending is not None
        if step == 23:
            st = c.state            # reading the state stores the token first
            assert c._pending is None and st[-1].shape[2] == c.offset - c._n_quantized
            assert np.array_equal(host(st[-2][:, :, -1]), k[:, :, pos - 1])
        if step == 31:
            assert c.trim(3) == 3
            pos -= 3
        q = rng.standard_normal((B, Hq, 1, D)).astype(np.float16)
        out = host(c.fused_sdpa(to_dev(q), 0.09)).astype(np.float32)
        assert c._pending is None and c.offset == pos
        nq = c._n_quantized
        assert nq == ((pos - R) // g) * g
        kq = ok.group_quant_codes(k[:, :, :nq], -2, g, levels)
        vq = ok.group_quant_codes(v[:, :, :nq], -1, g, levels)
        f = np.float16
        ref = oa.kivi_attend(q, kq[0], kq[1].astype(f), kq[2].astype(f), vq[0], vq[1].astype(f), vq[2].astype(f), g,
                             k[:, :, nq:pos], v[:, :, nq:pos], 0.09)
        assert np.max(np.abs(out - ref)) < 2e-3, step
        n_tail = pos - nq
        assert np.array_equal(host(c._tail_k[:, :, :n_tail]), k[:, :, nq:pos]), step
        assert np.array_equal(host(c._tail_v[:, :, :n_tail]), v[:, :, nq:pos]), step
    assert deferred >= 50   # all but the flush steps, the two-token step and the one after the trim... took the fused path
    # the kernel refuses the pair where it cannot take it
    with pytest.raises(ValueError, match="k_new"):
        K.kivi_packed_attend(to_dev(rng.standard_normal((B, Hq, 4, D)).astype(np.float16)), k_packed=c._kp, k_scale=c._ks,
                             k_zero=c._kz, v_packed=c._vp, v_scale=c._vs, v_zero=c._vz, n_packed=c._n_quantized, bits=4,
                             group_size=g, v_layout="token", k_tail=c._tail_k, v_tail=c._tail_v, n_tail=8, scale=0.1,
                             k_new=to_dev(k[:, :, :1]), v_new=to_dev(v[:, :, :1]))


@pytest.mark.parametrize("dtype,bits,group,v_layout,D,n_tail,S,n_flush", [
    (torch.float16, 4, 32, "token", 128, 128, 512, 512),     # chunked prefill: the new rows split between store and tail
    (torch.bfloat16, 4, 64, "token", 128, 160, 96, 128),     # the flush stays inside the old tail
    (torch.bfloat16, 2, 32, "token", 128, 40, 200, 224),     # everything but a few rows leaves
    (torch.float16, 2, 32, "channel", 128, 0, 256, 256),     # empty tail, nothing kept
    (torch.float16, 4, 32, "token", 64, 64, 64, 96),         # head size the one-launch kernel does not take
    (torch.float32, 4, 32, "channel", 128, 32, 64, 64),      # float32 cache
    (torch.float16, 4, 32, "token", 128, 100, 7, 0),         # plain append
])
def test_cache_append_one_call_matches_the_single_steps(dtype, bits, group, v_layout, D, n_tail, S, n_flush):
    """``vq_kivi_cache_append`` against ``vq_kv_tail_append`` + two ``vq_kivi_quant_pack`` + a row
    move: packed words, scale, zero and the kept rows bit for bit."""
    require_gpu()
    B, H, cap_t, cap_p, tok0 = 2, 3, 768, 1024, 256
    g = torch.Generator(device="cuda").manual_seed(5)
    rnd = lambda *s: torch.randn(s, generator=g, device="cuda").to(dtype)
    tk, tv = rnd(B, H, cap_t, D), rnd(B, H, cap_t, D)
    kn, vn = rnd(B, H, S + 8, D)[:, :, 3:3 + S], rnd(B, H, S, D)   # the keys a strided view
    per = 32 // bits
    meta = torch.float16
    def store():
        W, GV = D // per, D // group
        z = lambda *s, dt=torch.int32: torch.zeros(s, dtype=dt, device="cuda")
        if v_layout == "token":
            return [z(B, H, cap_p, W), z(B, H, cap_p // group, D, dt=meta), z(B, H, cap_p // group, D, dt=meta),
                    z(B, H, cap_p // per, D), z(B, H, GV, cap_p, dt=meta), z(B, H, GV, cap_p, dt=meta)]
        return [z(B, H, cap_p, W), z(B, H, cap_p // group, D, dt=meta), z(B, H, cap_p // group, D, dt=meta),
                z(B, H, cap_p, W), z(B, H, cap_p, GV, dt=meta), z(B, H, cap_p, GV, dt=meta)]
    need, keep = n_tail + S, n_tail + S - n_flush
    # the single steps
    t1k, t1v, st1 = tk.clone(), tv.clone(), store()
    K.kv_tail_append(kn, vn, t1k, t1v, n_tail)
    if n_flush:
        K.kivi_quant_pack(t1k[:, :, :n_flush], -2, group, bits, meta_dtype=meta, out=tuple(st1[:3]), dst_tok0=tok0)
        K.kivi_quant_pack(t1v[:, :, :n_flush], -1, group, bits, meta_dtype=meta, v_layout=v_layout, out=tuple(st1[3:]),
                          dst_tok0=tok0)
    # one call
    t2k, t2v, st2 = tk.clone(), tv.clone(), store()
    spare = (torch.zeros_like(tk), torch.zeros_like(tv)) if n_flush else None
    K.kivi_cache_append(kn, vn, t2k, t2v, n_tail, n_flush, st2, tok0, spare, bits=bits, group_size=group,
                        levels=(1 << bits) - 1, eps=1e-8, v_layout=v_layout)
    torch.cuda.synchronize()
    if n_flush:
        for x, y in zip(st1, st2):
            assert torch.equal(x, y)
        assert torch.equal(spare[0][:, :, :keep], t1k[:, :, n_flush:need])
        assert torch.equal(spare[1][:, :, :keep], t1v[:, :, n_flush:need])
        assert not spare[0][:, :, keep:].any() and not spare[1][:, :, keep:].any()
    else:
        assert torch.equal(t1k, t2k) and torch.equal(t1v, t2v)


def test_cache_append_rejects_bad_arguments():
    require_gpu()
    z = lambda *s, dt=torch.float16: torch.zeros(s, dtype=dt, device="cuda")
    tk, tv, kn, vn = z(1, 1, 64, 128), z(1, 1, 64, 128), z(1, 1, 32, 128), z(1, 1, 32, 128)
    with pytest.raises(ValueError, match="tail capacity"):
        K.kivi_cache_append(kn, vn, tk, tv, 40, 0, None, 0, None, bits=4, group_size=32, levels=15, eps=1e-8,
                            v_layout="token")
    st = [z(1, 1, 64, 16, dt=torch.int32), z(1, 1, 2, 128), z(1, 1, 2, 128), z(1, 1, 8, 128, dt=torch.int32),
          z(1, 1, 4, 64), z(1, 1, 4, 64)]
    with pytest.raises(ValueError, match="spare"):   # the spare tails must not be the tails
        K.kivi_cache_append(kn, vn, tk, tv, 0, 32, st, 0, (tk, tv), bits=4, group_size=32, levels=15, eps=1e-8,
                            v_layout="token")
    with pytest.raises(ValueError, match="n_flush"):
        K.kivi_cache_append(kn, vn, tk, tv, 0, 64, st, 0, (z(1, 1, 64, 128), z(1, 1, 64, 128)), bits=4, group_size=32,
                            levels=15, eps=1e-8, v_layout="token")


def test_layer_stacked_cache_attends_for_all_layers_at_once():
    """``LayerStackedKIVICache``: per-layer updates through the ordinary cache API on slices of the
    stacked buffers, one attention launch for all layers; against separate per-layer caches fed the
    same tokens (the layer-batched call of veloxquant_mlx/metal/_scalar_attend.py:496-647 without its
    stacking step).  Outputs within 1e-3 (the launches may split the context differently), stored
    codes bit for bit."""
    require_gpu()
    from veloxquant_mlx_amd.cache import LayerStackedKIVICache
    NL, B, Hq, Hkv, D = 3, 2, 8, 2, 128
    cfg = KVCacheConfig(method="kivi", head_dim=D, bit_width_inlier=4, kivi_group_size=32, residual_length=64,
                        fused_sdpa=True, fused_sdpa_memory_bound=True, fused_sdpa_max_ctx=1024)
    stacked = LayerStackedKIVICache(cfg, NL)
    solo = [KVCacheFactory.create(cfg) for _ in range(NL)]
    g = torch.Generator(device="cuda").manual_seed(11)
    rnd = lambda *s: torch.randn(s, generator=g, device="cuda").to(torch.float16)
    scale = 1 / math.sqrt(D)

    def feed(layer, n):
        k, v = rnd(B, Hkv, n, D), rnd(B, Hkv, n, D)
        stacked[layer].update_and_fetch(k, v)
        solo[layer].update_and_fetch(k, v)

    def check(Sq=1):
        q = rnd(NL, B, Hq, Sq, D)
        out = stacked.fused_sdpa_all(q, scale)
        assert out.shape == (NL, B, Hq, Sq, D)
        for layer in range(NL):
            ref = solo[layer].fused_sdpa(q[layer], scale)
            assert (out[layer].float() - ref.float()).abs().max().item() <= 1e-3, layer

    for layer in range(NL):
        feed(layer, 200)
    check()
    kp = stacked._packed[0]
    assert all(stacked[layer]._kp.data_ptr() == kp[layer * B:].data_ptr() for layer in range(NL))   # the stack is the storage
    for step in range(80):   # crosses two flushes: tails swap inside the stack, nothing is copied back
        for layer in range(NL):
            feed(layer, 1)
        check()
    assert stacked._packed[0] is kp
    for layer in range(NL):
        a, b = stacked[layer], solo[layer]
        n = a._n_quantized
        assert a.offset == b.offset == 280 and n == b._n_quantized
        assert torch.equal(a._kp[:, :, :n], b._kp[:, :, :n]) and torch.equal(a._vp[:, :, :n // 8], b._vp[:, :, :n // 8])
        assert torch.equal(a._ks[:, :, :n // 32], b._ks[:, :, :n // 32]) and torch.equal(a._vz[..., :n], b._vz[..., :n])
        nt = a.offset - n
        assert torch.equal(a._tail_k[:, :, :nt], b._tail_k[:, :, :nt])
    # a forward pass in flight: layer 0 is one token ahead of the others
    feed(0, 1)
    check()
    check(Sq=4)
    # a layer whose buffers were replaced is copied back into the stack
    stacked[1].state = solo[1].state
    check()
    with pytest.raises(ValueError, match="NL=3"):
        stacked.fused_sdpa_all(rnd(2, B, Hq, 1, D), scale)


@pytest.mark.parametrize("bits,meta", [(4, "float16"), (2, "float32")])
def test_layer_stacked_cache_with_protected_rows_and_a_sliding_window(bits, meta):
    """``LayerStackedKIVICache`` over ``method="kivi_sink"`` layers: every layer protects its own rows (different
    positions and different counts per layer and sequence), the one launch patches all of them, with and without
    a sliding window; against separate ``SinkProtectedKVCache`` objects fed the same tokens, bit for bit under
    ``fixed_order`` with the same cut, and against the oracle's model of layer 0."""
    require_gpu()
    from veloxquant_mlx_amd.cache import LayerStackedKIVICache
    from veloxquant_mlx_amd.cache.sink_cache import SinkProtectedKVCache
    NL, B, Hq, Hkv, D, R = 3, 2, 8, 2, 128, 64
    cfg = KVCacheConfig(method="kivi_sink", head_dim=D, bit_width_inlier=bits, kivi_group_size=32, residual_length=R,
                        n_sink_tokens=3, fused_sdpa=True, fused_sdpa_memory_bound=True, fused_sdpa_max_ctx=1024,
                        kivi_meta_dtype=meta)
    stacked = LayerStackedKIVICache(cfg, NL)
    assert all(isinstance(c, SinkProtectedKVCache) for c in stacked.layers)
    solo = [KVCacheFactory.create(cfg) for _ in range(NL)]
    model = ok.SinkCacheModel(bits, 32, R, 3)
    rng = np.random.default_rng(101 + bits)
    scale = 1 / math.sqrt(D)
    pos = [0] * NL

    def feed(layer, n):
        k = rng.standard_normal((B, Hkv, n, D)).astype(np.float16)
        v = rng.standard_normal((B, Hkv, n, D)).astype(np.float16)
        for b in range(B):                     # loud rows at places that differ by layer and sequence
            for p in range(pos[layer], pos[layer] + n):
                if p % (37 + 11 * layer + 5 * b) == 3 + layer:
                    k[b, :, p - pos[layer]] *= 9 + (p % 5)
        pos[layer] += n
        stacked[layer].update_and_fetch(to_dev(k), to_dev(v))
        solo[layer].update_and_fetch(to_dev(k), to_dev(v))
        if layer == 0:
            model.update_and_fetch(k, v)

    def check(Sq=1, window=0):
        q = rng.standard_normal((NL, B, Hq, Sq, D)).astype(np.float16)
        # aim one head of every layer at one of its protected rows
        for layer in range(NL):
            ps = solo[layer]._side_pos[0] if solo[layer]._side_pos else []
            if ps:
                slot = len(ps) - 1
                row = host(solo[layer]._side_k[0, 0, slot]).astype(np.float32)
                q[layer, 0, 1, -1] += (row / np.linalg.norm(row) * 5).astype(np.float16)
        qd = to_dev(q)
        kw = dict(sliding_window=window, fixed_order=True, num_splits=2)
        out = stacked.fused_sdpa_all(qd, scale, **kw)
        for layer in range(NL):
            ref = solo[layer].fused_sdpa(qd[layer], scale, **kw)
            assert torch.equal(out[layer], ref), (layer, Sq, window)
        km, vm = model.keys[:, :, : model.offset], model.values[:, :, : model.offset]
        want = oa.sdpa(q[0], km, vm, scale, causal=Sq > 1, sliding_window=window)
        err = float(np.max(np.abs(host(out[0]).astype(np.float32) - want)))
        # the model keeps float32 group parameters; a store with fp16 ones adds their rounding (2^-11 of a
        # scale of ~0.5 on codes up to 15) to every reconstructed element
        assert err < (2e-3 if meta == "float32" else 6e-3), (Sq, window, err)

    for layer in range(NL):
        feed(layer, 300)
    assert any(any(c._side_pos[b] for b in range(B)) for c in stacked.layers)
    check()
    check(window=100)
    side = stacked._sinks[1][0]
    check()
    assert stacked._sinks[1][0] is side                      # nothing changed: the stacked side store is reused
    for step in range(70):                                   # crosses two flushes; protected rows age out on the way
        for layer in range(NL):
            feed(layer, 1)
        if step % 7 == 0 or step > 60:
            check(window=0 if step % 2 else 150)
    assert stacked._sinks[1][0] is not side
    for layer in range(NL):
        a, b = stacked[layer], solo[layer]
        assert a._side_pos == b._side_pos and a._n_quantized == b._n_quantized and a.sink_positions == b.sink_positions
    check(Sq=4)
    check(Sq=4, window=90)
    feed(0, 1)                                               # a forward pass in flight: ragged lengths
    check()
    # trimming a layer below a protected row takes the row out of the stacked side store as well
    n_side = [sum(len(ps) for ps in c._side_pos) for c in stacked.layers]
    stacked[2].trim(pos[2] - 150)
    solo[2].trim(pos[2] - 150)
    pos[2] = 150
    assert sum(len(ps) for ps in stacked[2]._side_pos) <= n_side[2] and stacked[2]._side_pos == solo[2]._side_pos
    q = to_dev(rng.standard_normal((NL, B, Hq, 1, D)).astype(np.float16))
    out = stacked.fused_sdpa_all(q, scale, fixed_order=True, num_splits=2)
    for layer in range(NL):
        assert torch.equal(out[layer], solo[layer].fused_sdpa(q[layer], scale, fixed_order=True, num_splits=2)), layer


def test_context_limit_error_leaves_the_cache_as_it_was():
    """An append whose flush would pass ``fused_sdpa_max_ctx`` raises before offset, rows or packed
    store change: the cache answers the same query with the same bits afterwards."""
    require_gpu()
    B, Hq, Hkv, D = 1, 8, 2, 128
    k, v = outlier_kv((B, Hkv, 600, D), seed=71)
    c = _make(bit_width_inlier=4, kivi_group_size=32, residual_length=64, fused_sdpa=True, fused_sdpa_memory_bound=True,
              fused_sdpa_max_ctx=256)
    c.update_and_fetch(to_dev(k[:, :, :300]), to_dev(v[:, :, :300]))
    q = to_dev(np.random.default_rng(72).standard_normal((B, Hq, 1, D)).astype(np.float16))
    before = c.fused_sdpa(q, 0.09, fixed_order=True)
    state = (c.offset, c._n_quantized, c.nbytes)
    with pytest.raises(RuntimeError, match="fused_sdpa_max_ctx"):
        c.update_and_fetch(to_dev(k[:, :, 300:600]), to_dev(v[:, :, 300:600]))
    assert (c.offset, c._n_quantized, c.nbytes) == state
    assert torch.equal(c.fused_sdpa(q, 0.09, fixed_order=True), before)
    c.update_and_fetch(to_dev(k[:, :, 300:310]), to_dev(v[:, :, 300:310]))      # a step that still fits goes through
    assert c.offset == 310
