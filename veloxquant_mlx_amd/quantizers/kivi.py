"""``KIVIQuantizer``: the 2-D ``(n, d)`` research API over the HIP group
quantiser (veloxquant_mlx/quantizers/kivi.py:49-202 in the reference).

``axis="channel"`` is the key scheme (groups run along the batch/token axis, one
scale per channel and group); ``axis="token"`` is the value scheme (groups run
along channels).  ``encode`` returns uint8 codes with float32 scale / zero in
``EncodedVector.norm`` / ``.residual_norm``.
"""

from __future__ import annotations

from typing import Any

import torch

from .. import kernels as K
from ..core.context import EncodedVector
from ..core.exceptions import QuantizerConfigError
from ..core.registry import QuantizerRegistry


@QuantizerRegistry.register("kivi")
class KIVIQuantizer:
    def __init__(self, d: int, b: int = 2, group_size: int = 32, axis: str = "channel", m: int | None = None,
                 seed: int = 42, store: Any = None, **kwargs: Any) -> None:
        if b < 1 or b > 8:
            raise QuantizerConfigError(f"KIVIQuantizer: b={b} must be in [1, 8] (uint8 codes).")
        if group_size < 1:
            raise QuantizerConfigError(f"KIVIQuantizer: group_size={group_size} must be >= 1.")
        if axis not in ("channel", "token"):
            raise QuantizerConfigError(f"KIVIQuantizer: axis={axis!r} must be 'channel' or 'token'.")
        self._d = int(d)
        self._b = int(b)
        self._group_size = int(group_size)
        self._axis = axis
        self._levels = (1 << self._b) - 1
        self._eps = 1e-8

    def encode(self, x: torch.Tensor) -> EncodedVector:
        """Encode ``(batch, d)`` vectors (quantizers/kivi.py:147-176)."""
        n, d = x.shape
        if d != self._d:
            raise QuantizerConfigError(f"KIVIQuantizer.encode: expected dim {self._d}, got {d}.")
        if not bool(torch.isfinite(x).all()):
            raise QuantizerConfigError("KIVIQuantizer.encode: input contains NaN or Inf.")
        x4 = x.reshape(1, 1, n, d)
        if x4.dtype not in (torch.float16, torch.bfloat16, torch.float32):
            x4 = x4.float()
        codes, scale, zero = K.kivi_quant_codes(x4, -2 if self._axis == "channel" else -1, self._group_size,
                                                self._levels, self._eps)
        return EncodedVector(quantizer_type="kivi", batch_size=n, dim=d, indices=codes[0, 0],
                             norm=scale[0, 0], residual_norm=zero[0, 0])

    def decode(self, ev: EncodedVector) -> torch.Tensor:
        """Reconstruct ``(batch, d)`` fp16 vectors (quantizers/kivi.py:178-189)."""
        codes = ev.indices.reshape(1, 1, ev.batch_size, ev.dim)
        return K.scalar_decode_once(codes, ev.norm[None, None], ev.residual_norm[None, None], self._group_size,
                                    "K" if self._axis == "channel" else "V")[0, 0]

    def estimate_inner_product(self, q: torch.Tensor, ev: EncodedVector) -> torch.Tensor:
        """``<q, k_hat>`` per encoded row via full reconstruction (quantizers/kivi.py:191-202)."""
        k_hat = self.decode(ev).float()
        return (k_hat @ q.reshape(-1).float().to(k_hat.device)).to(torch.float16)

    def __repr__(self) -> str:
        return f"KIVIQuantizer(d={self._d}, b={self._b}, group_size={self._group_size}, axis={self._axis!r})"


__all__ = ["KIVIQuantizer"]
