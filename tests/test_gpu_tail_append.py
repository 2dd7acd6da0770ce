"""kv_tail_append on the GPU against slice assignment (the concatenation of
veloxquant_mlx/cache/kivi_cache.py:206-260 into a buffer with room): byte-exact."""

import pytest
import torch

from tests._gpu import gpu, require_gpu
from veloxquant_mlx_amd import kernels as K

pytestmark = gpu


def _case(B, H, S, D, cap, pos, dtype, layout="contiguous", seed=0):
    require_gpu()
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(seed)
    if layout == "transposed":      # [B,S,H,D] storage seen as [B,H,S,D], what a projection + transpose hands over
        k = torch.randn((B, S, H, D), generator=g, device=dev).to(dtype).transpose(1, 2)
        v = torch.randn((B, S, H, D), generator=g, device=dev).to(dtype).transpose(1, 2)
    elif layout == "sliced":        # a window of a longer sequence
        k = torch.randn((B, H, S + 5, D), generator=g, device=dev).to(dtype)[:, :, 3:3 + S]
        v = torch.randn((B, H, S + 5, D), generator=g, device=dev).to(dtype)[:, :, 2:2 + S]
    else:
        k = torch.randn((B, H, S, D), generator=g, device=dev).to(dtype)
        v = torch.randn((B, H, S, D), generator=g, device=dev).to(dtype)
    tk = torch.randn((B, H, cap, D), generator=g, device=dev).to(dtype)
    tv = torch.randn((B, H, cap, D), generator=g, device=dev).to(dtype)
    ek, ev = tk.clone(), tv.clone()
    ek[:, :, pos:pos + S] = k
    ev[:, :, pos:pos + S] = v
    K.kv_tail_append(k, v, tk, tv, pos)
    assert torch.equal(tk, ek) and torch.equal(tv, ev)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_single_token_decode_step(dtype):
    _case(16, 8, 1, 128, 192, 77, dtype)


@pytest.mark.parametrize("layout", ["contiguous", "transposed", "sliced"])
def test_chunk_append_layouts(layout):
    _case(2, 4, 37, 128, 64, 20, torch.float16, layout)


def test_odd_head_dim_and_ends_of_the_buffer():
    _case(1, 3, 5, 72, 8, 3, torch.float16)     # last rows of the buffer; 144-byte rows
    _case(1, 3, 8, 72, 8, 0, torch.bfloat16)    # fills the buffer
    _case(3, 1, 0, 128, 8, 8, torch.float16)    # nothing to append


def test_rejects_overflow_and_mismatch():
    require_gpu()
    k = torch.zeros((1, 2, 4, 128), dtype=torch.float16, device="cuda:0")
    t = torch.zeros((1, 2, 8, 128), dtype=torch.float16, device="cuda:0")
    with pytest.raises(ValueError):
        K.kv_tail_append(k, k, t, t.clone(), 5)
    with pytest.raises(ValueError):
        K.kv_tail_append(k, k.float(), t, t.clone(), 0)
    with pytest.raises(ValueError):
        K.kv_tail_append(k, k, t[:, :1], t[:, :1].clone(), 0)
