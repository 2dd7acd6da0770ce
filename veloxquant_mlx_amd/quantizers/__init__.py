"""Quantizers of the hot path."""

from .kivi import KIVIQuantizer

__all__ = ["KIVIQuantizer"]
