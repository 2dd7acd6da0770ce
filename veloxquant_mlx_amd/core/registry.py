"""Name -> quantizer class registry (veloxquant_mlx/core/registry.py:91 in the reference)."""

from __future__ import annotations

import threading
from typing import Any, Callable


class QuantizerRegistry:
    _lock = threading.Lock()
    _classes: dict[str, type] = {}

    @classmethod
    def register(cls, name: str) -> Callable[[type], type]:
        def deco(klass: type) -> type:
            with cls._lock:
                cls._classes[name] = klass
            return klass
        return deco

    @classmethod
    def get(cls, name: str) -> type:
        with cls._lock:
            if name not in cls._classes:
                raise KeyError(f"QuantizerRegistry: unknown quantizer {name!r}; known: {sorted(cls._classes)}")
            return cls._classes[name]

    @classmethod
    def create(cls, name: str, **kwargs: Any) -> Any:
        return cls.get(name)(**kwargs)

    @classmethod
    def names(cls) -> list[str]:
        with cls._lock:
            return sorted(cls._classes)
