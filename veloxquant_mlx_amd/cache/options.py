"""Per-method option dataclasses read through by ``KVCacheConfig``
(veloxquant_mlx/cache/options.py:36-50 in the reference)."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass
class VecInferOptions:
    """VecInfer-specific configuration."""

    key_sub_dim: int = 4
    value_sub_dim: int = 8
    key_codebook_bits: int = 12
    value_codebook_bits: int = 8
    residual_length: int = 128


@dataclass
class KIVIOptions:
    """KIVI configuration (asymmetric group quantization)."""

    kivi_group_size: int = 32  # min/max group size (KIVI default 32)


@dataclass
class KittyOptions:
    """Kitty configuration (channel-wise mixed-precision keys; options.py:66-73 in the reference)."""

    kitty_hi_fraction: float = 0.25  # fraction of channels kept at kitty_hi_bit
    kitty_hi_bit: int = 4
    kitty_lo_bit: int = 2
    kitty_group_size: int = 32


@dataclass
class AgeTieredKVOptions:
    """AgeTieredKV configuration (three precision tiers by token age; options.py in the reference)."""

    age_recent_boundary: int = 128
    age_mid_boundary: int = 1024
    age_bits_recent: int = 8
    age_bits_mid: int = 4
    age_bits_old: int = 2
    age_group_size: int = 32


@dataclass
class SKVQOptions:
    """SKVQ configuration (sliding window, channel reorder, clipped groups; options.py in the reference)."""

    skvq_bits_key: int = 4
    skvq_bits_value: int = 4
    skvq_group_size: int = 32
    skvq_window: int = 128
    skvq_n_sink: int = 5
    skvq_reorder: bool = True
    skvq_clip_search: bool = True
    skvq_clip_alpha: float = 1.0
    skvq_max_ctx: int | None = None


@dataclass
class ZipCacheOptions:
    """ZipCache-adapted configuration (per-token mixed precision by key norm; options.py in the reference)."""

    zipcache_hi_bits: int = 4
    zipcache_lo_bits: int = 2
    zipcache_hi_fraction: float = 0.20
    zipcache_group_size: int = 32
    zipcache_quantize_values: bool = True


__all__ = ["VecInferOptions", "KIVIOptions", "KittyOptions", "AgeTieredKVOptions", "SKVQOptions", "ZipCacheOptions"]
