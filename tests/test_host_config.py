"""Host-side configuration surface (no GPU work): option read-through, explicit
field priority, factory dispatch and rejections, builder validation.  Restates
veloxquant_mlx/tests/cache/test_kvcache_config_options.py:21-107 and
veloxquant_mlx/tests/cache/test_cache_factory.py:28-99 for the two methods built."""

import dataclasses
import warnings
from types import SimpleNamespace

import pytest

import veloxquant_mlx_amd.cache.options as opts
from veloxquant_mlx_amd.cache import KIVIOptions, KVCacheBuilder, KVCacheConfig, KVCacheFactory, VecInferOptions
from veloxquant_mlx_amd.cache.base import _CACHE_CLASS_BY_METHOD, _FIELD_TO_OPTIONS_CLASS
from veloxquant_mlx_amd.cache.kivi_cache import KIVIKVCache
from veloxquant_mlx_amd.cache.vecinfer_cache import VecInferKVCache
from veloxquant_mlx_amd.core import EncodedVector, QuantizerConfigError, QuantizerRegistry


def test_defaults_match_reference_values():
    c = KVCacheConfig()
    assert (c.head_dim, c.bit_width_inlier, c.kivi_group_size, c.residual_length) == (128, 2, 32, 128)
    assert (c.key_sub_dim, c.value_sub_dim, c.key_codebook_bits, c.value_codebook_bits) == (4, 8, 12, 8)
    assert c.use_metal_kernels is None and c.fused_sdpa is False and c.fused_sdpa_memory_bound is False
    assert c.fused_sdpa_max_ctx is None and c.seed == 42


def test_flat_field_construction_no_warning():
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        config = KVCacheConfig(method="kivi", kivi_group_size=64)
    assert config.kivi_group_size == 64
    assert not any(issubclass(w.category, DeprecationWarning) for w in caught)


def test_options_populate_flat_fields_and_explicit_wins():
    c = KVCacheConfig(method="vecinfer", options=VecInferOptions(key_sub_dim=8, key_codebook_bits=8))
    assert c.key_sub_dim == 8 and c.key_codebook_bits == 8 and c.value_sub_dim == 8
    c = KVCacheConfig(method="kivi", kivi_group_size=16, options=KIVIOptions(kivi_group_size=64))
    assert c.kivi_group_size == 16
    # an explicit value equal to the default still beats options
    c = KVCacheConfig(method="kivi", kivi_group_size=32, options=KIVIOptions(kivi_group_size=64))
    assert c.kivi_group_size == 32


def test_post_construction_set_warns_only_for_option_fields():
    c = KVCacheConfig(method="kivi")
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        c.kivi_group_size = 64
        c.seed = 7
    dep = [w for w in caught if issubclass(w.category, DeprecationWarning)]
    assert len(dep) == 1 and "KIVIOptions" in str(dep[0].message)
    assert c.kivi_group_size == 64 and c.seed == 7


def test_every_options_default_matches_config_default():
    flat = {f.name: f.default for f in dataclasses.fields(KVCacheConfig)}
    for cls_name in set(_FIELD_TO_OPTIONS_CLASS.values()):
        for f in dataclasses.fields(getattr(opts, cls_name)):
            assert f.default == flat[f.name], f"{cls_name}.{f.name}"


def test_inlier_bits_warning_for_methods_that_ignore_it():
    with pytest.warns(UserWarning, match="ignores bit_width_inlier"):
        KVCacheConfig(method="vecinfer", bit_width_inlier=3)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        KVCacheConfig(method="kivi", bit_width_inlier=3)
        dataclasses.replace(KVCacheConfig(method="vecinfer"), head_dim=64)


def test_factory_dispatch_and_rejections():
    assert set(_CACHE_CLASS_BY_METHOD) == {"kivi", "kivi_sink", "kitty", "age_tiered", "skvq", "zipcache", "vecinfer"}
    assert isinstance(KVCacheFactory.create(KVCacheConfig(method="kivi")), KIVIKVCache)
    with pytest.warns(UserWarning, match="random N"):
        assert isinstance(KVCacheFactory.create(KVCacheConfig(method="vecinfer")), VecInferKVCache)
    with pytest.raises(QuantizerConfigError, match="unknown method 'nope'. Choices: vecinfer, kivi"):
        KVCacheFactory.create(KVCacheConfig(method="nope"))
    with pytest.raises(QuantizerConfigError, match="observers"):
        KVCacheFactory.create(KVCacheConfig(method="kivi", observers=[object()]))
    with pytest.raises(QuantizerConfigError, match="bit_width_outlier"):
        KVCacheFactory.create(KVCacheConfig(method="kivi", bit_width_outlier=3))
    with pytest.raises(QuantizerConfigError, match="single int"):
        KVCacheFactory.create(KVCacheConfig(method="kivi", bit_width_inlier=[2, 4]))
    with pytest.raises(QuantizerConfigError, match="sliding_window"):
        KVCacheFactory.create(KVCacheConfig(method="kivi", sliding_window=64))


def test_kivi_cache_surface():
    c = KVCacheFactory.create(KVCacheConfig(method="kivi", bit_width_inlier=4))
    assert not hasattr(c, "bits") and c.assigned_avg_bits == 4.0
    assert c.offset == 0 and c.empty() and c.size() == 0 and c.nbytes == 0
    assert c.effective_compression_ratio == 1.0 and c.trim(3) == 0
    with pytest.raises(RuntimeError, match="fused_sdpa was not enabled"):
        c.fused_sdpa(None, 1.0)
    with pytest.raises(RuntimeError, match="requires fused_sdpa=True"):
        KIVIKVCache(KVCacheConfig(method="kivi", fused_sdpa_memory_bound=True))
    with pytest.raises(QuantizerConfigError, match="kivi_meta_dtype"):
        KIVIKVCache(KVCacheConfig(method="kivi", kivi_meta_dtype="int8"))
    # duck-typed configs work, as in the reference's tests
    c = KIVIKVCache(SimpleNamespace(head_dim=64, bit_width_inlier=2, kivi_group_size=8, residual_length=4))
    assert c._group_size == 8 and c._residual_length == 4 and c._v_layout == "channel"
    assert KIVIKVCache(KVCacheConfig(method="kivi"))._v_layout == "token"


def test_vecinfer_cache_validation():
    import numpy as np
    kw = dict(method="vecinfer", key_codebook=np.zeros((256, 8), np.float32), key_sub_dim=8, key_codebook_bits=8,
              value_codebook=np.zeros((256, 8), np.float32))
    with pytest.raises(QuantizerConfigError, match="power-of-2 head_dim"):
        KVCacheFactory.create(KVCacheConfig(head_dim=96, **kw))
    with pytest.raises(QuantizerConfigError, match="not divisible by key_sub_dim"):
        KVCacheFactory.create(KVCacheConfig(head_dim=128, **{**kw, "key_sub_dim": 3}))
    with pytest.raises(QuantizerConfigError, match="smooth_factors must be finite"):
        KVCacheFactory.create(KVCacheConfig(head_dim=128, smooth_factors=np.zeros(128, np.float32), **kw))
    with pytest.raises(RuntimeError, match="requires fused_sdpa=True"):
        KVCacheFactory.create(KVCacheConfig(head_dim=128, fused_sdpa_memory_bound=True, **kw))
    c = KVCacheFactory.create(KVCacheConfig(head_dim=128, fused_sdpa=True, fused_sdpa_memory_bound=True, **kw))
    assert c._memory_bound and c.empty() and c.state[0].shape == (1, 1, 0, 16)
    assert c.assigned_avg_bits == 1.0 and c.codebook_bytes == 2 * 256 * 8 * 2
    with pytest.raises(AttributeError):
        c.merge
    with pytest.raises(RuntimeError, match="before any tokens"):
        c.fused_sdpa(None, 1.0)
    c._smooth = __import__("torch").ones(3, 128)
    with pytest.raises(QuantizerConfigError, match="has 3 rows"):
        c._resolve_smooth_heads(2)


def test_builder_validation_and_for_model():
    with pytest.raises(QuantizerConfigError, match="power of 2"):
        KVCacheBuilder().with_method("kivi").with_head_dim(96).build()
    with pytest.raises(QuantizerConfigError, match="must be >= 1"):
        KVCacheBuilder().with_method("kivi").with_bit_width(0).build()
    with pytest.raises(QuantizerConfigError, match="must not be empty"):
        KVCacheBuilder().with_method("kivi").with_bit_width([]).build()
    assert isinstance(KVCacheBuilder().with_method("kivi").with_head_dim(64).with_bit_width(4).build(), KIVIKVCache)

    attn = SimpleNamespace(head_dim=64)
    layers = [SimpleNamespace(self_attn=attn), SimpleNamespace(mlp=1), SimpleNamespace(self_attn=SimpleNamespace(head_dim=None))]
    model = SimpleNamespace(layers=layers, args=SimpleNamespace(hidden_size=512, num_attention_heads=4, head_dim=None))
    caches = KVCacheBuilder.for_model(model, KVCacheConfig(method="kivi", bit_width_inlier=[2, 4], seed=5))
    assert [type(c).__name__ for c in caches] == ["KIVIKVCache", "FP16KVCache", "KIVIKVCache"]
    assert caches[0]._head_dim == 64 and caches[2]._head_dim == 128
    assert caches[0]._b == 2 and caches[2]._b == 4
    with pytest.raises(QuantizerConfigError, match="one entry per attention layer"):
        KVCacheBuilder.for_model(model, KVCacheConfig(method="kivi", bit_width_inlier=[2, 4, 8]))


def test_core_types():
    ev = EncodedVector("kivi", 2, 4)
    assert ev.memory_bytes() == 0 and "kivi" in repr(ev)
    import veloxquant_mlx_amd.quantizers  # registers
    assert "kivi" in QuantizerRegistry.names()
    q = QuantizerRegistry.create("kivi", d=16, b=4)
    assert "b=4" in repr(q)
    with pytest.raises(QuantizerConfigError, match=r"must be in \[1, 8\]"):
        QuantizerRegistry.create("kivi", d=16, b=9)
    with pytest.raises(QuantizerConfigError, match="'channel' or 'token'"):
        QuantizerRegistry.create("kivi", d=16, axis="rows")
    assert issubclass(QuantizerConfigError, ValueError)


def test_paired_heads_are_the_same_attention():
    """Two kv heads of 64 channels side by side as one head of 128, every query head zero-padded into the half of its own
    kv head and reading that half of the output: the attention of the single heads (the form a memory-bound KIVI cache
    keeps 64-channel heads in), here in plain float64 arithmetic."""
    import torch
    from veloxquant_mlx_amd.cache.kivi_cache import own_half_of_paired_output, pad_queries_for_paired_heads, pair_heads
    g = torch.Generator().manual_seed(0)
    B, H, S, D, Hq, Sq = 2, 4, 9, 64, 12, 3
    R = Hq // H
    k, v = (torch.randn((B, H, S, D), generator=g, dtype=torch.float64) for _ in range(2))
    q = torch.randn((B, Hq, Sq, D), generator=g, dtype=torch.float64)
    kp = pair_heads(k)
    assert kp.shape == (B, H // 2, S, 2 * D)
    for m in range(H // 2):
        assert torch.equal(kp[:, m, :, :D], k[:, 2 * m]) and torch.equal(kp[:, m, :, D:], k[:, 2 * m + 1])
    wide = pad_queries_for_paired_heads(q, H)
    for h in range(Hq):
        half = (h // R) % 2
        assert torch.equal(wide[:, h, :, half * D:(half + 1) * D], q[:, h])
        assert float(wide[:, h, :, (1 - half) * D:(2 - half) * D].abs().sum()) == 0.0
    assert torch.equal(own_half_of_paired_output(wide, H), q)
    # a buffer whose other halves are already zero is filled in place
    buf = torch.zeros_like(wide)
    assert pad_queries_for_paired_heads(q, H, buf) is buf and torch.equal(buf, wide)

    def attend(q_, k_, v_, ratio):
        k_, v_ = k_.repeat_interleave(ratio, 1), v_.repeat_interleave(ratio, 1)
        return torch.softmax(q_ @ k_.transpose(-1, -2) * 0.125, -1) @ v_

    got = own_half_of_paired_output(attend(wide, kp, pair_heads(v), 2 * R), H)
    assert float((got - attend(q, k, v, R)).abs().max()) < 1e-12
    # a leading layer axis (the layer stack) goes through unchanged
    q5 = torch.randn((3, B, Hq, 1, D), generator=g, dtype=torch.float64)
    assert torch.equal(own_half_of_paired_output(pad_queries_for_paired_heads(q5, H), H), q5)
    # an odd number of kv heads: the last one is paired with a head of zeros, whose query heads are zeros too
    for H3, Hq3 in ((3, 9), (5, 5)):
        k3, v3 = (torch.randn((B, H3, S, D), generator=g, dtype=torch.float64) for _ in range(2))
        q3 = torch.randn((B, Hq3, Sq, D), generator=g, dtype=torch.float64)
        R3 = Hq3 // H3
        assert pair_heads(k3).shape == (B, (H3 + 1) // 2, S, 2 * D) and float(pair_heads(k3)[:, -1, :, D:].abs().sum()) == 0.0
        w3 = pad_queries_for_paired_heads(q3, H3)
        assert w3.shape == (B, (H3 + 1) * R3, Sq, 2 * D) and torch.equal(own_half_of_paired_output(w3, H3), q3)
        got3 = own_half_of_paired_output(attend(w3, pair_heads(k3), pair_heads(v3), 2 * R3), H3)
        assert float((got3 - attend(q3, k3, v3, R3)).abs().max()) < 1e-12
        q35 = torch.randn((2, B, Hq3, 1, D), generator=g, dtype=torch.float64)
        assert torch.equal(own_half_of_paired_output(pad_queries_for_paired_heads(q35, H3), H3), q35)


def test_kivi_storage_options():
    """The additions that pick how a packed KIVI cache stores its codes: the width of a code's field and the pairing of
    64-channel heads (host-side decisions; the kernels are the same ones)."""
    def make(**kw):
        return KVCacheFactory.create(KVCacheConfig(method="kivi", fused_sdpa=True, fused_sdpa_memory_bound=True, **kw))
    assert [make(bit_width_inlier=b)._field for b in (1, 2, 3, 4, 8)] == [2, 2, 4, 4, 8]
    assert [make(bit_width_inlier=b, kivi_code_field="tight")._field for b in (1, 2, 3, 4)] == [1, 2, 3, 4]
    assert [make(bit_width_inlier=b)._levels for b in (1, 3)] == [1, 7]          # the levels stay the quantiser's
    assert make(bit_width_inlier=3)._v_layout == "token" and make(bit_width_inlier=3, kivi_code_field="tight")._v_layout == "channel"
    with pytest.raises(QuantizerConfigError, match="kivi_code_field"):
        make(kivi_code_field="wide")
    assert make(head_dim=64)._pair_wanted and not make(head_dim=64, kivi_pair_heads=False)._pair_wanted
    assert not make(head_dim=128)._pair_wanted
    assert not KVCacheFactory.create(KVCacheConfig(method="kivi", head_dim=64))._pair_wanted   # the fp16-history modes keep single heads
