"""Host dispatch of attention calls onto a cache's fused path.

Restates the part of veloxquant_mlx/metal/fused_sdpa.py that belongs to the attention path itself:
the recogniser that turns a caller's mask into the two parameters the fused kernels take
(``_memory_bound_mask_parameters``, fused_sdpa.py:332-396) and the dispatcher that a host model's
``scaled_dot_product_attention`` is replaced with (``_make_patched_sdpa``, fused_sdpa.py:399-416).
Patching a model library's modules is the host framework's business and is not done here.

A cache in memory-bound mode hands out zero-stride placeholders instead of K/V, so for such a cache
every call either reaches ``cache.fused_sdpa`` or raises; nothing may fall through to dense attention.
"""

from __future__ import annotations

from typing import Any, Callable

import torch

_UNSUPPORTED = ("Memory-bound VecInfer fused SDPA requires an unmasked, causal, or uniform sliding-window mask. "
                "This mask cannot be represented by the fused kernel. Set fused_sdpa_memory_bound=False to use "
                "standard SDPA.")


def memory_bound_mask_parameters(mask: Any, queries: torch.Tensor, kv_length: int) -> tuple[bool, int]:
    """``(causal, sliding_window)`` for a mask the fused kernels can honour exactly, else ``ValueError``.

    Accepted: ``None`` (all visible), the string ``"causal"``, and boolean or additive (0 / -inf)
    arrays of 1 to 4 dimensions broadcastable to ``[B, H, N, kv_length]`` that are the same for every
    batch element and head and are either all-visible or causal with the queries aligned to the end
    of the keys, optionally limited to a trailing window.  Every entry is checked: a mask with a
    hole, left padding, a per-head difference, a finite bias or no visible key is refused.

    The check is row-wise: a row qualifies when its visible keys form one run that ends at the row's
    own position and is ``min(width, position + 1)`` long, ``width`` being the run of the last row.
    One small device-to-host read delivers the verdict.
    """
    if mask is None:
        return False, 0
    if isinstance(mask, str):
        if mask == "causal":
            return True, 0
        raise ValueError(_UNSUPPORTED)
    if not isinstance(mask, torch.Tensor) or not 1 <= mask.dim() <= 4:
        raise ValueError(_UNSUPPORTED)
    B, H, N, _ = queries.shape
    L = int(kv_length)
    full = (B, H, N, L)
    shape4 = (1,) * (4 - mask.dim()) + tuple(mask.shape)
    if N < 1 or L < N or any(have != 1 and have != want for have, want in zip(shape4, full)):
        raise ValueError(_UNSUPPORTED)

    m = mask.reshape(shape4)
    if m.dtype == torch.bool:
        visible, well_formed = m, None
    elif m.dtype.is_floating_point:
        visible = m == 0
        well_formed = (visible | (m == float("-inf"))).all()
    else:
        raise ValueError(_UNSUPPORTED)

    same_everywhere = (visible == visible[:1, :1]).all()
    rows = visible[0, 0].expand(N, L)                                   # one [N, L] pattern
    n_visible = rows.sum(dim=-1)                                        # [N]
    key_index = torch.arange(L, device=rows.device)
    last_visible = torch.where(rows, key_index, -1).amax(dim=-1)        # -1 for an empty row
    first_visible = torch.where(rows, key_index, L).amin(dim=-1)
    one_run = n_visible == last_visible - first_visible + 1
    own_position = torch.arange(L - N, L, device=rows.device)
    width = n_visible[-1]
    windowed_causal = (one_run & (last_visible == own_position)
                       & (n_visible == torch.minimum(width, own_position + 1))).all()
    flags = [same_everywhere, (n_visible == L).all(), windowed_causal, width > 0]
    if well_formed is not None:
        flags.append(well_formed)
    verdict = torch.stack([f.to(torch.int64) for f in flags] + [width.to(torch.int64)]).tolist()
    same, everything, causal_ok, some = verdict[:4]
    entries_ok = verdict[4] if well_formed is not None else 1
    w = verdict[-1]
    if same and entries_ok:
        if everything:
            return False, 0
        if causal_ok and some:
            return True, (0 if w == L else w)
    raise ValueError(_UNSUPPORTED)


def make_fused_dispatcher(original: Callable) -> Callable:
    """``scaled_dot_product_attention(queries, keys, values, cache, scale, mask, sinks=None)`` that sends
    memory-bound caches to their fused path and everything else to ``original``."""

    def scaled_dot_product_attention(queries, keys, values, cache, scale, mask, sinks=None):
        if not getattr(cache, "_memory_bound", False):
            return original(queries, keys, values, cache=cache, scale=scale, mask=mask, sinks=sinks)
        if sinks is not None:
            raise ValueError("Memory-bound VecInfer fused SDPA does not support attention sinks. "
                             "Set fused_sdpa_memory_bound=False to use standard SDPA.")
        if not callable(getattr(cache, "fused_sdpa", None)):
            raise RuntimeError("Memory-bound cache requires a callable fused_sdpa method.")
        causal, window = memory_bound_mask_parameters(mask, queries, keys.shape[-2])
        return cache.fused_sdpa(queries, scale=scale, causal=causal, sliding_window=window)

    return scaled_dot_product_attention


__all__ = ["memory_bound_mask_parameters", "make_fused_dispatcher"]
