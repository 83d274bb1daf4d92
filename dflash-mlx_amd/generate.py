"""The speculative cycle around the verify step (host side).

Mirror of the loop body of dflash_mlx/runtime.py:1290-1458 without its timers, prefetch and
streaming: stage the first token of a block, let the draft fill the rest, arm the rollback,
run the target over the block, take the target's greedy tokens, commit the staged token plus
the longest agreeing prefix of the draft, stage the target's token after it, roll the caches
back to the committed length.  Models come in as callables:

* ``target(ids [1, S], cache) -> logits [1, S, V]`` - one forward over S new tokens that
  appends to ``cache`` (``make_target_cache``: ``RecurrentRollbackCache`` / ``KVCache`` per layer);
* ``draft(staged_first [1], block_len, committed [n]) -> drafted [block_len - 1]``.

Whatever the draft proposes, the committed tokens are the target's own greedy continuation:
that is the invariant the tests hold this loop to.
"""
from __future__ import annotations

from typing import Any, Callable, List, Optional, Sequence

import torch

from .engine import HybridGDNEngine, _BaseEngine
from .runtime import _match_acceptance_length
from .verify_qmm import raise_on_device_errors

TargetFn = Callable[[torch.Tensor, List[Any]], torch.Tensor]
DraftFn = Callable[[torch.Tensor, int, torch.Tensor], torch.Tensor]


def greedy_tokens(logits: torch.Tensor) -> torch.Tensor:
    return torch.argmax(logits, dim=-1).to(torch.int64)


@torch.no_grad()
def generate_greedy(target: TargetFn, target_cache: List[Any], prompt_ids: torch.Tensor,
                    max_new_tokens: int) -> torch.Tensor:
    """Plain token-by-token greedy decoding: the sequence the speculative loop must reproduce."""
    logits = target(prompt_ids[None], target_cache)
    out = [greedy_tokens(logits[0, -1:])]
    while len(out) < max_new_tokens:
        logits = target(out[-1][None], target_cache)
        out.append(greedy_tokens(logits[0, -1:]))
    return torch.cat(out)[:max_new_tokens]


@torch.no_grad()
def generate_speculative(target: TargetFn, draft: DraftFn, target_cache: List[Any], prompt_ids: torch.Tensor,
                         max_new_tokens: int, *, block_tokens: int = 16, engine: Optional[_BaseEngine] = None,
                         stop_token_ids: Sequence[int] = (), acceptance_history: Optional[List[int]] = None
                         ) -> torch.Tensor:
    """dflash_mlx/runtime.py:1262-1458.  Returns the generated tokens (prompt excluded)."""
    engine = engine or HybridGDNEngine()
    device = prompt_ids.device
    prefill_logits = target(prompt_ids[None], target_cache)
    staged_first = greedy_tokens(prefill_logits[0, -1:])
    start = int(prompt_ids.shape[0])
    generated = torch.empty(max_new_tokens + block_tokens, dtype=torch.int64, device=device)
    count = 0
    stops = torch.tensor(list(stop_token_ids), dtype=torch.int64, device=device) if stop_token_ids else None
    while count < max_new_tokens:
        block_len = max(1, min(block_tokens, max_new_tokens - count))
        if block_len > 1:
            drafted = draft(staged_first, block_len, generated[:count]).to(torch.int64)
            verify_token_ids = torch.cat([staged_first[:1], drafted[: block_len - 1]])
        else:
            verify_token_ids = staged_first[:1]
        engine.arm_rollback(target_cache, prefix_len=start)
        verify_logits = target(verify_token_ids[None], target_cache)
        posterior = greedy_tokens(verify_logits[0])
        acceptance_len = int(_match_acceptance_length(verify_token_ids[1:], posterior[:-1]).item())
        if device.type == "cuda":
            raise_on_device_errors(device)  # the cycle's one wait for the device: a kernel that gave up a wait says so here
        if acceptance_history is not None:
            acceptance_history.append(acceptance_len)
        commit_count = 1 + acceptance_len
        committed = verify_token_ids[:commit_count]
        generated[count:count + commit_count] = committed
        count += commit_count
        staged_first = posterior[acceptance_len:acceptance_len + 1]
        start += commit_count
        engine.rollback(target_cache, target_len=start, acceptance_len=acceptance_len,
                        drafted_tokens=block_len - 1)
        if stops is not None and bool(torch.isin(committed, stops).any()):
            break
    return generated[:min(count, max_new_tokens)]
