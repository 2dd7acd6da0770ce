"""MI355X-native KV-cache compression hot path (KIVI group quantisation, VecInfer
product VQ, fused dequant attention) behind the VeloxQuant-MLX cache API.

Compute runs in hand-written gfx950 HIP kernels reached through the C ABI of
``libveloxquant_hip.so``; this package is the host side on ``torch`` ROCm tensors.
"""

from ._lib import library_present
from .kernels import hip_available

__version__ = "0.1.0"

__all__ = ["hip_available", "library_present", "__version__"]
