"""``EncodedVector``: the typed result of ``Quantizer.encode``
(veloxquant_mlx/core/context.py:71-138 in the reference).  Only the fields the
KIVI quantizer fills are kept."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any


@dataclass
class EncodedVector:
    """Codes plus the per-group parameters that decode them.

    For KIVI ``indices`` holds uint8 codes ``(batch, d)``, ``norm`` the per-group
    scale and ``residual_norm`` the per-group zero point."""

    quantizer_type: str
    batch_size: int
    dim: int
    indices: Any | None = None
    norm: Any | None = None
    residual_norm: Any | None = None

    def memory_bytes(self) -> int:
        total = 0
        for arr in (self.indices, self.norm, self.residual_norm):
            if arr is None:
                continue
            nb = getattr(arr, "nbytes", None)
            if nb is None and hasattr(arr, "numel"):
                nb = arr.numel() * arr.element_size()
            total += int(nb or 0)
        return total

    def __repr__(self) -> str:
        return (f"EncodedVector(type={self.quantizer_type!r}, batch={self.batch_size}, dim={self.dim}, "
                f"bytes={self.memory_bytes()})")
