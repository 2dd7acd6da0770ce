"""Plain growing fp16 KV cache on torch tensors.

Plays the role ``mlx_lm.models.cache.KVCache`` plays for the reference's cache
classes (their parent, veloxquant_mlx/cache/kivi_cache.py:76,248): a
``[B, H, capacity, D]`` buffer grown in steps of ``step`` tokens, an ``offset``
frontier, ``update_and_fetch`` / ``state`` / ``trim`` / ``size`` / ``empty`` /
``nbytes``.  It is memory management only; no arithmetic happens here.
"""

from __future__ import annotations

import torch


class FP16KVCache:
    step = 256

    def __init__(self) -> None:
        self.keys: torch.Tensor | None = None
        self.values: torch.Tensor | None = None
        self.offset = 0

    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        prev = self.offset
        S = keys.shape[2]
        if self.keys is None or prev + S > self.keys.shape[2]:
            B, H, _, Dk = keys.shape
            Dv = values.shape[3]
            n_steps = (self.step + S - 1) // self.step
            new_k = torch.zeros((B, H, n_steps * self.step, Dk), dtype=keys.dtype, device=keys.device)
            new_v = torch.zeros((B, H, n_steps * self.step, Dv), dtype=values.dtype, device=values.device)
            if self.keys is not None:
                self.keys = torch.cat([self.keys[:, :, :prev], new_k], dim=2)
                self.values = torch.cat([self.values[:, :, :prev], new_v], dim=2)
            else:
                self.keys, self.values = new_k, new_v
        self.offset += S
        self.keys[:, :, prev:self.offset] = keys
        self.values[:, :, prev:self.offset] = values
        return self.keys[:, :, : self.offset], self.values[:, :, : self.offset]

    def size(self) -> int:
        return self.offset

    def empty(self) -> bool:
        return self.keys is None

    def is_trimmable(self) -> bool:
        return True

    def trim(self, n: int) -> int:
        n = min(self.offset, max(int(n), 0))
        self.offset -= n
        return n

    @property
    def state(self):
        if self.keys is None:
            return ()
        return self.keys[:, :, : self.offset], self.values[:, :, : self.offset]

    @state.setter
    def state(self, v) -> None:
        if len(v) == 0:
            self.keys = self.values = None
            self.offset = 0
            return
        self.keys, self.values = v[0], v[1]
        self.offset = int(self.keys.shape[2])

    @property
    def nbytes(self) -> int:
        if self.keys is None:
            return 0
        return self.keys.numel() * self.keys.element_size() + self.values.numel() * self.values.element_size()
