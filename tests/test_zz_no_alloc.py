"""``vq_kivi_attend_static`` (the entry point that allocates nothing: split partials and sync
counters live in a device array built into the library) against ``vq_kivi_attend`` with a
caller-provided workspace, through the C ABI.  Two calls in a row, the second on a smaller
input, so that what the first left in the shared scratch would show; token chunks dealt in a
fixed order, so the two entry points must agree bit for bit (the bar for the attention output
against the oracle is 2e-3 max-abs; the oracle check of these shapes is in test_gpu_attend.py)."""

import math

import numpy as np
import pytest
import torch

from tests._gpu import gpu, outlier_kv, require_gpu, to_dev
from veloxquant_mlx_amd import kernels as K

pytestmark = gpu


def _case(B, Hq, Hkv, n_packed, n_tail, bits, g, seed):
    D = 128
    k, v = outlier_kv((B, Hkv, n_packed + n_tail, D), seed=seed)
    kt, vt = to_dev(k), to_dev(v)
    kq = K.kivi_quant_pack(kt[:, :, :n_packed], -2, g, bits, meta_dtype=torch.float16)
    vq = K.kivi_quant_pack(vt[:, :, :n_packed], -1, g, bits, meta_dtype=torch.float16, v_layout="token")
    q = to_dev(np.random.default_rng(seed + 1).standard_normal((B, Hq, 1, D)).astype(np.float16))
    kw = dict(k_packed=kq[0], k_scale=kq[1], k_zero=kq[2], v_packed=vq[0], v_scale=vq[1], v_zero=vq[2],
              n_packed=n_packed, bits=bits, group_size=g, v_layout="token",
              k_tail=kt[:, :, n_packed:].contiguous(), v_tail=vt[:, :, n_packed:].contiguous(), n_tail=n_tail,
              scale=1 / math.sqrt(D), fixed_order=True)
    return q, kw


def test_static_scratch_entry_point_equals_the_workspace_entry_point():
    require_gpu()
    big = _case(2, 32, 8, 4096, 77, 2, 32, seed=5)       # 16 kv heads x 16 splits + tail partial
    small = _case(1, 8, 2, 512, 0, 4, 64, seed=9)        # fewer rows, fewer splits, no tail
    outs = [torch.empty_like(c[0]) for c in (big, small)]
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    for (q, kw), o in zip((big, small), outs):            # two calls in a row on the shared scratch
        plan = {}
        K.kivi_packed_attend(q, out=o, static_scratch=True, _plan_out=plan, **kw)
        assert plan["path"] == 1 and plan["nparts"] > 1, plan
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before        # torch's allocator was not touched either
    for (q, kw), o in zip((big, small), outs):
        ref = K.kivi_packed_attend(q, **kw)
        assert torch.equal(o, ref)
    # the multi-query and the vector-kernel plans go through the same scratch
    q, kw = small
    q4 = to_dev(np.random.default_rng(3).standard_normal((1, 8, 4, 128)).astype(np.float16))
    for extra in (dict(causal=True), dict(causal=True, num_splits=-1)):
        a = K.kivi_packed_attend(q4, static_scratch=True, **{**kw, **extra})
        b = K.kivi_packed_attend(q4, **{**kw, **extra})
        assert torch.equal(a, b)
    # a GQA group of three heads at a few positions runs filled up to four heads: queries and outputs in that form
    # sit in the scratch as well
    q3 = to_dev(np.random.default_rng(6).standard_normal((1, 6, 4, 128)).astype(np.float16))
    plan = {}
    a = K.kivi_packed_attend(q3, static_scratch=True, causal=True, _plan_out=plan, **kw)
    assert plan["path"] == 1 and torch.equal(a, K.kivi_packed_attend(q3, causal=True, **kw))
    # beyond the built-in scratch: refused with a clear error, nothing launched
    q512 = to_dev(np.random.default_rng(4).standard_normal((2, 32, 512, 128)).astype(np.float16))
    with pytest.raises(RuntimeError, match="built-in scratch"):   # 32768 query rows: 17 MB of partials
        K.kivi_packed_attend(q512, static_scratch=True, **{**big[1], "causal": True})


def test_static_scratch_makes_no_tile_scratch_for_long_plain_prefill():
    """A causal call over plain keys and values with thousands of query rows per kv head: the ordinary call
    writes the input once as tiles into a scratch it keeps; with ``static_scratch=True`` nothing may be
    allocated, the blocks convert the rows themselves, and the bits are the same."""
    require_gpu()
    B, Hq, Hkv, S, D = 1, 8, 2, 1536, 128                  # 4 query heads x 1536 positions = 6144 rows per kv head
    rng = np.random.default_rng(12)
    q, k, v = (to_dev(rng.standard_normal((B, h, S, D)).astype(np.float16)) for h in (Hq, Hkv, Hkv))
    # one part per block: the blocks write ``out`` themselves and no split partials are needed
    kw = dict(k_tail=k, v_tail=v, n_tail=S, scale=1 / math.sqrt(D), causal=True, num_splits=1)
    out = torch.empty_like(q)
    K.release_tile_scratch()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    K.kivi_packed_attend(q, out=out, static_scratch=True, **kw)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    ref = K.kivi_packed_attend(q, **kw)                   # makes and uses the tile scratch
    assert torch.cuda.memory_allocated() > before + out.numel() * 2
    assert torch.equal(out, ref)
    assert K.release_tile_scratch() > 0
