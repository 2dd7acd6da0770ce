"""Cache API: ``KVCacheConfig(method=...)`` and the KIVI / VecInfer caches."""

from .base import KVCacheBuilder, KVCacheConfig, KVCacheFactory
from .options import AgeTieredKVOptions, KIVIOptions, KittyOptions, SKVQOptions, VecInferOptions, ZipCacheOptions
from .prompt_cache import load_prompt_cache, save_prompt_cache
from .stacked_cache import LayerStackedKIVICache

__all__ = ["KVCacheConfig", "KVCacheFactory", "KVCacheBuilder", "KIVIOptions", "VecInferOptions", "KittyOptions", "AgeTieredKVOptions", "SKVQOptions", "ZipCacheOptions",
           "save_prompt_cache", "load_prompt_cache", "LayerStackedKIVICache"]
