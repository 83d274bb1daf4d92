"""Verify / rollback glue of the speculative cycle (host side).

Mirror of the parts of dflash_mlx/runtime.py that sit directly around the two
device kernels: the load-time decision to swap linears (:714-753), acceptance
matching (:101-108), arming (:833-846) and the per-layer restore after acceptance
(:849-907).  Index arithmetic is integer-exact with the reference.

Caches handed out by a ``RollbackArena`` are rolled back with one batched launch
instead of one launch per layer; everything else follows the per-layer loop.
"""
from __future__ import annotations

import os
import time
from typing import Any, List, Optional, Sequence

import torch

from .cache import KVCache
from .recurrent_rollback_cache import RecurrentRollbackCache, RollbackArena


def _verify_enabled_for(config: Any) -> bool:
    """``DFLASH_VERIFY_LINEAR`` = 1 / 0 forces the swap on / off; otherwise it is on for
    MoE targets (num_experts > 0) and dense targets with >= 40 layers."""
    override = os.environ.get("DFLASH_VERIFY_LINEAR", "").strip()
    if override == "1":
        return True
    if override == "0":
        return False
    try:
        text_cfg = config.get("text_config", config) if isinstance(config, dict) else config
        num_experts = int(text_cfg.get("num_experts", 0) or 0)
        num_layers = int(text_cfg.get("num_hidden_layers", 0) or 0)
    except Exception:
        return False
    if num_experts > 0:
        return True
    return num_layers >= 40


def enable_verify_linears(model: torch.nn.Module, config: Any, meta: Optional[dict] = None) -> int:
    """Load-time step of dflash_mlx/runtime.py:714-721: when the target qualifies, default
    ``DFLASH_VERIFY_QMM`` to "1" (an explicit user setting wins) and swap the linears.
    Beyond the reference: swapped projections that read the same input (gate/up, q/k/v, the
    input projections of a linear-attention layer) are then joined so that one launch serves
    them (``fuse_shared_input_linears``; ``DFLASH_VERIFY_FUSE_SHARED_INPUT=0`` keeps them apart)."""
    if not _verify_enabled_for(config):
        return 0
    os.environ.setdefault("DFLASH_VERIFY_QMM", "1")
    from .verify_linear import fuse_shared_input_linears, install_verify_linears

    n_swapped = install_verify_linears(model)
    n_groups = fuse_shared_input_linears(model) if n_swapped else 0
    if meta is not None:
        meta["verify_linear_swapped"] = n_swapped
        meta["verify_shared_input_groups"] = n_groups
    return n_swapped


def _match_acceptance_length(drafted_tokens: torch.Tensor, posterior_tokens: torch.Tensor) -> torch.Tensor:
    """Length of the longest prefix on which the draft and the target's greedy tokens
    agree, as an int32 scalar tensor on the inputs' device (no host sync)."""
    if int(drafted_tokens.shape[0]) == 0:
        return torch.zeros((), dtype=torch.int32, device=drafted_tokens.device)
    matches = torch.eq(drafted_tokens, posterior_tokens).to(torch.int32)
    return torch.sum(torch.cumprod(matches, dim=0)).to(torch.int32)


def make_target_cache(layer_is_linear: Sequence[bool], *, enable_speculative_linear_cache: bool = True,
                      conv_kernel_size: int = 4, arena: Optional[RollbackArena] = None) -> List[Any]:
    """One cache per layer (dflash_mlx/runtime.py:654-677): a RecurrentRollbackCache for a
    linear-attention layer, a KVCache for a full-attention layer.  With ``arena`` the
    recurrent caches are the arena's (stacked storage, batched rollback)."""
    caches: List[Any] = []
    arena_caches = iter(arena.caches()) if arena is not None else None
    for is_linear in layer_is_linear:
        if is_linear:
            if not enable_speculative_linear_cache:
                raise NotImplementedError("non-speculative recurrent cache is outside this package")
            if arena_caches is not None:
                caches.append(next(arena_caches))
            else:
                caches.append(RecurrentRollbackCache(size=2, conv_kernel_size=conv_kernel_size))
        else:
            caches.append(KVCache())
    return caches


def trim_cache_to(cache_entries: List[Any], size: int) -> int:
    if not cache_entries:
        return 0
    current_size = int(getattr(cache_entries[0], "offset", 0) or 0)
    if current_size <= size:
        return 0
    n = current_size - size
    trimmed = 0
    for c in cache_entries:
        if hasattr(c, "trim"):
            trimmed = c.trim(n)
    return int(trimmed or 0)


def _arm_target_rollback(cache_entries: List[Any]) -> None:
    for cache_entry in cache_entries:
        if hasattr(cache_entry, "arm_rollback"):
            cache_entry.arm_rollback()


def _arm_target_rollback_with_prefix(cache_entries: List[Any], *, prefix_len: int) -> None:
    for cache_entry in cache_entries:
        if hasattr(cache_entry, "arm_rollback"):
            cache_entry.arm_rollback(prefix_len=int(prefix_len))


def _clear_rollback_state(cache_entry: Any) -> None:
    if hasattr(cache_entry, "clear_transients"):
        cache_entry.clear_transients()
        return
    for name, value in (("_armed", False), ("_tape", None), ("_tape_k", None), ("_tape_g", None),
                        ("_tape_qkv", None), ("_snapshot", None)):
        if hasattr(cache_entry, name):
            setattr(cache_entry, name, value)


def _shared_arena(cache_entries: List[Any]) -> Optional[RollbackArena]:
    """The arena if every cache with a ``rollback`` method comes from one arena and they
    are exactly that arena's caches; None otherwise."""
    arena = None
    count = 0
    for c in cache_entries:
        if hasattr(c, "rollback"):
            a = getattr(c, "_arena", None)
            if a is None or (arena is not None and a is not arena):
                return None
            arena = a
            count += 1
    if arena is None or count != arena.L:
        return None
    return arena


def _restore_target_cache_after_acceptance(cache_entries: List[Any], *, target_len: int,
                                           acceptance_length: int, drafted_tokens: int = 0) -> int:
    """Per layer: recurrent caches roll back to ``acceptance_length`` accepted drafts (or
    just drop their transients when every draft was accepted); attention caches are
    trimmed to ``target_len``.  Returns the host nanoseconds spent issuing the work."""
    replay_ns_total = 0
    fully_accepted = drafted_tokens > 0 and acceptance_length == drafted_tokens
    arena = None if fully_accepted else _shared_arena(cache_entries)
    if arena is not None:
        replay_start_ns = time.perf_counter_ns()
        arena.rollback_all(int(acceptance_length), drafted_tokens=drafted_tokens)
        replay_ns_total += time.perf_counter_ns() - replay_start_ns
    for cache_entry in cache_entries:
        if hasattr(cache_entry, "rollback"):
            if arena is not None:
                continue
            if fully_accepted:
                _clear_rollback_state(cache_entry)
                continue
            replay_start_ns = time.perf_counter_ns()
            cache_entry.rollback(acceptance_length)
            replay_ns_total += time.perf_counter_ns() - replay_start_ns
        elif hasattr(cache_entry, "trim"):
            offset = int(getattr(cache_entry, "offset", 0) or 0)
            if offset > target_len:
                replay_start_ns = time.perf_counter_ns()
                cache_entry.trim(offset - target_len)
                replay_ns_total += time.perf_counter_ns() - replay_start_ns
        elif hasattr(cache_entry, "offset"):
            offset = int(getattr(cache_entry, "offset", 0) or 0)
            if offset > target_len:
                cache_entry.offset = target_len
        elif hasattr(cache_entry, "crop"):
            cache_entry.crop(target_len)
    return replay_ns_total
