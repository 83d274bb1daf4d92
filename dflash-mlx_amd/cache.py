"""Attention-layer KV cache with the two members the rollback path touches.

The reference trims mlx_lm ``KVCache`` objects (a third-party class, not part of
the reference tree) at dflash_mlx/runtime.py:895-900: ``cache.trim(offset - target_len)``.
Trimming is offset arithmetic only - ``n = min(offset, n); offset -= n`` - the
key/value buffers are left in place and later writes start again at ``offset``.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch


class KVCache:
    """Pre-allocated K/V buffers ``[B, H, capacity, D]`` plus a fill ``offset``."""

    step = 256

    def __init__(self):
        self.keys: Optional[torch.Tensor] = None
        self.values: Optional[torch.Tensor] = None
        self.offset = 0

    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """Append ``keys``/``values`` ``[B, H, S, D]`` at ``offset``; return the filled prefix."""
        prev = self.offset
        s = keys.shape[2]
        if self.keys is None or prev + s > self.keys.shape[2]:
            b, h, _, dk = keys.shape
            dv = values.shape[3]
            n_steps = (self.step + s - 1) // self.step
            new_k = torch.zeros((b, h, n_steps * self.step, dk), dtype=keys.dtype, device=keys.device)
            new_v = torch.zeros((b, h, n_steps * self.step, dv), dtype=values.dtype, device=values.device)
            if self.keys is not None:
                self.keys = torch.cat([self.keys[:, :, :prev], new_k], dim=2)
                self.values = torch.cat([self.values[:, :, :prev], new_v], dim=2)
            else:
                self.keys, self.values = new_k, new_v
        self.offset = prev + s
        self.keys[:, :, prev:self.offset] = keys
        self.values[:, :, prev:self.offset] = values
        return self.keys[:, :, :self.offset], self.values[:, :, :self.offset]

    def is_trimmable(self) -> bool:
        return True

    def trim(self, n: int) -> int:
        n = min(self.offset, int(n))
        self.offset -= n
        return n

    @property
    def state(self):
        if self.keys is None:
            return None, None
        return self.keys[:, :, :self.offset], self.values[:, :, :self.offset]

    def empty(self) -> bool:
        return self.keys is None
