"""Prompt-cache files for the packed caches: every layer's ``state`` arrays and ``meta_state``
strings in one safetensors file, so a prefilled, compressed context can be put away and picked
up again without going back through fp16.  The layout follows what ``mlx_lm``'s
``save_prompt_cache`` / ``load_prompt_cache`` do with the reference's caches (arrays keyed by
layer and position, ``meta_state`` and class names in the file's metadata); the packed arrays
are stored as they are, so a file costs what the cache costs.

Only tensors and strings are written and read; loading executes nothing from the file."""

from __future__ import annotations

import json
from typing import Callable, Sequence

import torch
from safetensors import safe_open
from safetensors.torch import save_file

_FORMAT = "veloxquant-prompt-cache-1"


def save_prompt_cache(path: str, caches: Sequence, metadata: dict | None = None) -> None:
    """Write ``[c.state for c in caches]`` and their ``meta_state`` to ``path``."""
    tensors: dict[str, torch.Tensor] = {}
    layers = []
    for i, c in enumerate(caches):
        state = tuple(c.state)
        for j, t in enumerate(state):
            tensors[f"{i}.{j}"] = t.detach().contiguous().cpu()
        layers.append({"class": type(c).__name__, "n": len(state), "meta_state": list(getattr(c, "meta_state", ()) or ())})
    meta = {"format": _FORMAT, "layers": json.dumps(layers), "user": json.dumps(metadata or {})}
    if not tensors:   # safetensors needs at least the header; an empty cache list is still a valid file
        tensors["empty"] = torch.zeros(1, dtype=torch.uint8)
    save_file(tensors, path, metadata=meta)


def load_prompt_cache(path: str, make_cache: Callable[[int, str], object], device="cuda:0", return_metadata: bool = False):
    """Rebuild the caches of ``path``: ``make_cache(layer, class_name)`` returns an empty cache
    configured like the saved one; its ``state`` and then ``meta_state`` are assigned (the cache
    checks that bit width, group size and layout agree)."""
    with safe_open(path, framework="pt", device="cpu") as f:
        meta = f.metadata() or {}
        if meta.get("format") != _FORMAT:
            raise ValueError(f"load_prompt_cache: {path} is not a {_FORMAT} file")
        layers = json.loads(meta["layers"])
        caches = []
        for i, info in enumerate(layers):
            c = make_cache(i, info["class"])
            if type(c).__name__ != info["class"]:
                raise ValueError(f"load_prompt_cache: layer {i} was saved from {info['class']}, got {type(c).__name__}")
            c.state = tuple(f.get_tensor(f"{i}.{j}").to(device) for j in range(info["n"]))
            if info["meta_state"] and hasattr(type(c), "meta_state"):
                c.meta_state = tuple(info["meta_state"])
            caches.append(c)
    if return_metadata:
        return caches, json.loads(meta.get("user", "{}"))
    return caches


__all__ = ["save_prompt_cache", "load_prompt_cache"]
