"""Helpers shared by the GPU parity tests."""

import numpy as np
import pytest
import torch

gpu = pytest.mark.gpu


def require_gpu():
    from veloxquant_mlx_amd import kernels
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no ROCm device is visible")
    if not kernels.hip_available():
        pytest.fail("libveloxquant_hip.so is not loadable on this box (no fallback exists)")
    return torch.device("cuda:0")


def to_dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    return t if dtype is None else t.to(dtype)


def host(t):
    t = t.detach()
    if t.dtype == torch.bfloat16:
        return t.float().cpu().numpy()
    return t.cpu().numpy()


def words(t):
    """int32 storage of packed words -> uint32 numpy."""
    return t.detach().cpu().numpy().view(np.uint32)


def outlier_kv(shape, seed):
    """N(0,1) values with per-channel log-normal(0,1) factors on the keys."""
    rng = np.random.default_rng(seed)
    k = rng.standard_normal(shape).astype(np.float32)
    v = rng.standard_normal(shape).astype(np.float32)
    f = np.exp(rng.standard_normal(shape[-1])).astype(np.float32)
    return (k * f).astype(np.float16), v.astype(np.float16)
