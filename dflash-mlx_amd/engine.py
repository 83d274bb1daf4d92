"""Engine-level arm / rollback entry points (mirror of dflash_mlx/engine.py:12-65).

Only the two members on the rollback path are provided; ``verify`` needs a target
model forward, which is outside this package.
"""
from __future__ import annotations

from typing import Any, List

from . import runtime as runtime_mod


class _BaseEngine:
    def arm_rollback(self, target_cache: List[Any], *, prefix_len: int) -> None:
        runtime_mod._arm_target_rollback_with_prefix(target_cache, prefix_len=prefix_len)

    def rollback(self, target_cache: List[Any], *, target_len: int, acceptance_len: int,
                 drafted_tokens: int) -> int:
        return runtime_mod._restore_target_cache_after_acceptance(
            target_cache,
            target_len=target_len,
            acceptance_length=acceptance_len,
            drafted_tokens=drafted_tokens,
        )


class FullAttentionEngine(_BaseEngine):
    """Rollback backend for full-attention target models."""


class HybridGDNEngine(_BaseEngine):
    """Rollback backend for hybrid GDN target models."""
