"""The mask recogniser and dispatcher of the fused attention path, on the accept / reject table of
veloxquant_mlx/tests/cache/test_vecinfer_memory_bound_masks.py:46-135 (restated on CPU tensors: the
recogniser is pure host logic) plus a brute-force sweep over every small window width."""

from types import SimpleNamespace

import pytest
import torch

from veloxquant_mlx_amd.fused_sdpa import make_fused_dispatcher, memory_bound_mask_parameters


def _causal(N, L, window=None):
    q = torch.arange(L - N, L)[:, None]
    k = torch.arange(L)[None, :]
    m = k <= q
    if window is not None:
        m &= k > q - window
    return m


@pytest.mark.parametrize("expanded", [False, True])
@pytest.mark.parametrize("kind", ["causal", "window", "additive", "additive-window", "all-visible"])
def test_accepted_masks(kind, expanded):
    offset = 0
    for N in (16, 4, 1):
        L = offset + N
        windowed = kind in ("window", "additive-window")
        mask = _causal(N, L, 8 if windowed else None)
        if N == 1 and not windowed:
            mask = torch.ones((N, L), dtype=torch.bool)
        if kind.startswith("additive"):
            mask = torch.where(mask, 0.0, float("-inf")).to(torch.float16)
        elif kind == "all-visible":
            mask = torch.ones_like(mask)
        if expanded:
            mask = mask.expand(2, 4, N, L)
        q = torch.zeros((2, 4, N, 64))
        causal, window = memory_bound_mask_parameters(mask, q, L)
        all_vis = bool((mask == 0).all()) if mask.dtype != torch.bool else bool(mask.all())
        if all_vis:
            assert (causal, window) == (False, 0)
        else:
            assert causal is True
            assert window == (8 if windowed and L > 8 else 0)
        offset = L
    assert memory_bound_mask_parameters(None, q, 5) == (False, 0)
    assert memory_bound_mask_parameters("causal", q, 5) == (True, 0)


def test_every_small_window_is_recovered():
    for L in range(1, 10):
        for N in range(1, L + 1):
            q = torch.zeros((1, 2, N, 8))
            for w in range(1, L + 2):
                mask = _causal(N, L, w)
                got = memory_bound_mask_parameters(mask, q, L)
                if bool(mask.all()):
                    assert got == (False, 0)
                else:
                    # a width that reaches the first key for the last row is a plain causal mask
                    assert got == (True, 0 if w >= L else w), (L, N, w)


@pytest.mark.parametrize("unsupported", ["hole", "padding", "head-specific", "bias", "empty", "shape", "string", "sinks",
                                         "row-shift", "int", "ragged-window"])
def test_rejected_without_fallback(unsupported):
    calls = []

    def original(*a, **k):
        pytest.fail("dense attention would read placeholder K/V")

    def fused(*a, **k):
        calls.append(k)
        pytest.fail("unsupported attention must not reach the fused kernel")

    cache = SimpleNamespace(_memory_bound=True, fused_sdpa=fused)
    q = torch.zeros((2, 4, 4, 64))
    kv = torch.zeros((2, 2, 8, 64))
    mask = _causal(4, 8).clone()
    sinks = None
    if unsupported == "hole":
        mask[0, 1] = False
    elif unsupported == "padding":
        mask[:, 0] = False
    elif unsupported == "head-specific":
        mask = mask.expand(2, 4, 4, 8).clone()
        mask[1, 2, 0, 1] = False
    elif unsupported == "bias":
        mask = torch.where(mask, 0.25, float("-inf"))
    elif unsupported == "empty":
        mask = torch.zeros_like(mask)
    elif unsupported == "shape":
        mask = torch.ones((4, 7), dtype=torch.bool)
    elif unsupported == "string":
        mask = "custom"
    elif unsupported == "sinks":
        mask, sinks = "causal", torch.zeros((4,))
    elif unsupported == "row-shift":      # causal, but aligned to the start of the keys
        mask = torch.arange(8)[None, :] <= torch.arange(4)[:, None]
    elif unsupported == "int":
        mask = mask.to(torch.int32)
    elif unsupported == "ragged-window":  # windows of different widths from row to row
        mask = _causal(4, 8, 3).clone()
        mask[0] = _causal(4, 8, 2)[0]
    with pytest.raises(ValueError, match="fused_sdpa_memory_bound=False"):
        make_fused_dispatcher(original)(q, kv, kv, cache=cache, scale=0.125, mask=mask, sinks=sinks)
    assert not calls


def test_dispatch_targets():
    q = torch.zeros((1, 1, 1, 64))
    with pytest.raises(RuntimeError, match="callable fused_sdpa"):
        make_fused_dispatcher(lambda *a, **k: pytest.fail("no"))(q, q, q, cache=SimpleNamespace(_memory_bound=True),
                                                                   scale=1, mask=None)
    seen = {}
    fused = lambda queries, **k: seen.update(k) or "fused"
    d = make_fused_dispatcher(lambda *a, **k: ("dense", k["mask"], k["sinks"]))
    qq, kv = torch.zeros((1, 2, 4, 8)), torch.zeros((1, 2, 12, 8))
    assert d(qq, kv, kv, cache=SimpleNamespace(_memory_bound=True, fused_sdpa=fused), scale=0.5, mask=_causal(4, 12, 5)) == "fused"
    assert seen == {"scale": 0.5, "causal": True, "sliding_window": 5}
    # a cache that holds real K/V keeps arbitrary masks and sinks on the host's own attention
    odd = torch.rand(4, 12)
    assert d(qq, kv, kv, cache=SimpleNamespace(_memory_bound=False), scale=0.5, mask=odd, sinks="s") == ("dense", odd, "s")
