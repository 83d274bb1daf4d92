"""GatedDeltaNet tape replay (host side).

Mirror of the replay half of dflash_mlx/kernels.py: ``tape_replay_kernel``
(:361-407) dispatches to the gfx950 kernel behind ``dflash_tape_replay``
(include/dflash_mi355.h); ``_tape_replay_ops`` (:328-358) is the same recurrence
in array ops, which the reference takes when the kernel does not cover a shape
(:374-375) and which this module takes for the same shapes and for host tensors.

Layouts: tape [B,T,Hv,Dv]; k [B,T,Hk,Dk]; g [B,T,Hv] or [B,T,Hv,Dk];
state [B,Hv,Dv,Dk]; mask [B,T] bool.
"""
from __future__ import annotations

import os
from typing import Optional, Union

import torch

from . import _native

_DTYPE_CODE = {torch.bfloat16: _native.BF16, torch.float16: _native.FP16, torch.float32: _native.FP32}


def _tape_replay_ops(tape: torch.Tensor, k: torch.Tensor, g: torch.Tensor, state: torch.Tensor,
                     mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    _, _, hk, _ = k.shape
    hv = tape.shape[2]
    if hv % hk != 0:
        raise ValueError(f"Cannot align K heads {hk} to tape heads {hv}")
    repeat_factor = hv // hk
    if repeat_factor > 1:
        k = torch.repeat_interleave(k, repeat_factor, dim=2)

    for t in range(int(tape.shape[1])):
        prev_state = state
        if g.ndim == 4:
            decay = g[:, t, :, None, :]
        elif g.ndim == 3:
            decay = g[:, t, :, None, None]
        else:
            raise ValueError(f"Unsupported gating shape {tuple(g.shape)}")
        delta = tape[:, t, :, :, None]
        k_t = k[:, t, :, None, :]
        state = state * decay
        state = state + delta * k_t
        if mask is not None:
            step_mask = mask[:, t][:, None, None, None]
            state = torch.where(step_mask, state, prev_state)
    return state


def _exact_order() -> bool:
    return os.environ.get("DFLASH_REPLAY_EXACT", "") == "1"


def _slot_major(t: torch.Tensor, inner: int) -> tuple:
    """Return (tensor, T_alloc) such that tensor's memory is [slots, T_alloc, inner...]
    densely packed and the logical tensor is its first ``t.shape[1]`` steps.  A prefix
    slice ``full[:, :steps]`` of a contiguous tensor qualifies without a copy."""
    if t.is_contiguous():
        return t, int(t.shape[1])
    st = t.stride()
    want = []
    acc = 1
    for d in reversed(t.shape[2:]):
        want.append(acc)
        acc *= int(d)
    inner_dense = tuple(st[2:]) == tuple(reversed(want)) and st[1] == inner
    if inner_dense and st[0] % inner == 0 and st[0] // inner >= t.shape[1]:
        return t, st[0] // inner
    t = t.contiguous()
    return t, int(t.shape[1])


def replay_launch(tape: torch.Tensor, k: torch.Tensor, g: torch.Tensor, state_in: torch.Tensor,
                  state_out: torch.Tensor, *, steps: Union[int, torch.Tensor], T_alloc: int,
                  mask: Optional[torch.Tensor] = None, slots: Optional[int] = None,
                  exact_order: Optional[bool] = None) -> None:
    """Enqueue one ``dflash_tape_replay`` on the current stream.

    The leading dimension(s) of every operand are flattened into ``slots``
    independent problems; ``steps`` is a host int applied to every slot or an int32
    device tensor with one entry per slot.  ``T_alloc`` is the number of step rows
    each slot's tape/k/g storage holds (>= any step count used)."""
    lib = _native.lib()
    if not state_in.is_cuda:
        raise _native.NativeLibraryError("tape replay kernel needs device tensors")
    Hv, Dv = int(tape.shape[-2]), int(tape.shape[-1])
    Hk, Dk = int(k.shape[-2]), int(k.shape[-1])
    if slots is None:
        slots = state_in.numel() // (Hv * Dv * Dk)
    g_per_dk = 1 if g.shape[-1] == Dk and g.ndim == tape.ndim else 0
    steps_dev, steps_host = None, 0
    if isinstance(steps, torch.Tensor):
        if steps.dtype != torch.int32 or not steps.is_cuda or steps.numel() != slots:
            raise ValueError("steps tensor must be int32, on the device, one entry per slot")
        steps_dev = steps.data_ptr()
    else:
        steps_host = int(steps)
    mask_ptr = None
    if mask is not None:
        mask = mask.to(torch.uint8).contiguous()
        mask_ptr = mask.data_ptr()
    stream = torch.cuda.current_stream(state_in.device).cuda_stream
    rc = lib.dflash_tape_replay(
        tape.data_ptr(), k.data_ptr(), g.data_ptr(), state_in.data_ptr(), state_out.data_ptr(),
        steps_dev, steps_host, mask_ptr, slots, T_alloc, Hk, Hv, Dk, Dv,
        _DTYPE_CODE[state_in.dtype], _DTYPE_CODE[tape.dtype], _DTYPE_CODE[k.dtype],
        _DTYPE_CODE[g.dtype], g_per_dk, 1 if (_exact_order() if exact_order is None else exact_order) else 0,
        stream)
    _native.check(rc, "dflash_tape_replay")


def tape_replay_kernel(tape: torch.Tensor, k: torch.Tensor, g: torch.Tensor, state: torch.Tensor,
                       mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Replay all ``tape.shape[1]`` steps onto ``state``; returns a new state tensor."""
    if not state.is_cuda:
        return _tape_replay_ops(tape, k, g, state, mask)

    bsz, steps, hk, dk = k.shape
    hv, dv = tape.shape[2:]
    if dk < 32 or dk % 32 != 0:
        return _tape_replay_ops(tape, k, g, state, mask)
    if g.ndim not in (3, 4):
        raise ValueError(f"Unsupported gating shape {tuple(g.shape)}")
    if hv % hk != 0:
        raise ValueError(f"Cannot align K heads {hk} to tape heads {hv}")
    if any(t.dtype not in _DTYPE_CODE for t in (tape, k, g, state)):
        return _tape_replay_ops(tape, k, g, state, mask)
    # LDS budget of the kernel: T*(Dv + 2*Dk + 1) floats
    if steps * (dv + 2 * dk + 1) * 4 + dk * 4 > 64 * 1024:
        return _tape_replay_ops(tape, k, g, state, mask)

    state_c = state.contiguous()
    tape_c, T_tape = _slot_major(tape, hv * dv)
    k_c, T_k = _slot_major(k, hk * dk)
    g_c, T_g = _slot_major(g, hv * (dk if g.ndim == 4 else 1))
    if not (T_tape == T_k == T_g):
        tape_c, k_c, g_c = tape.contiguous(), k.contiguous(), g.contiguous()
        T_tape = steps
    state_out = torch.empty_like(state_c)
    replay_launch(tape_c, k_c, g_c, state_c, state_out, steps=steps, T_alloc=T_tape, mask=mask,
                  slots=bsz)
    return state_out
