"""Cache API: ``KVCacheConfig(method=...)`` and the KIVI / VecInfer caches."""

from .base import KVCacheBuilder, KVCacheConfig, KVCacheFactory
from .options import KIVIOptions, VecInferOptions

__all__ = ["KVCacheConfig", "KVCacheFactory", "KVCacheBuilder", "KIVIOptions", "VecInferOptions"]
