"""Small shared types of the hot path (veloxquant_mlx/core in the reference)."""

from .context import EncodedVector
from .exceptions import QuantizerConfigError
from .registry import QuantizerRegistry

__all__ = ["EncodedVector", "QuantizerConfigError", "QuantizerRegistry"]
