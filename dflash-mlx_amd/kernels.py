"""GatedDeltaNet forward-with-tape and tape replay (host side).

Mirror of the GatedDeltaNet half of dflash_mlx/kernels.py: ``gated_delta_kernel_with_tape``
(:176-224) and ``tape_replay_kernel`` (:361-407) dispatch to the gfx950 kernels behind
``dflash_gdn_forward_tape`` and ``dflash_tape_replay`` (include/dflash_mi355.h); the
``_..._ops`` functions (:131-173, :328-358) are the same recurrences in array ops, which
the reference takes when its kernels do not cover a shape (:187-188, :374-375) and which
this module takes for the same shapes and for host tensors.

Layouts: tape [B,T,Hv,Dv]; k [B,T,Hk,Dk]; g [B,T,Hv] or [B,T,Hv,Dk];
state [B,Hv,Dv,Dk]; mask [B,T] bool.
"""
from __future__ import annotations

import os
from typing import Optional, Union

import torch

from . import _native

_DTYPE_CODE = {torch.bfloat16: _native.BF16, torch.float16: _native.FP16, torch.float32: _native.FP32}


def _require_extents(who: str, device: torch.device, **operands) -> None:
    """``name=(tensor, shape)`` pairs: the kernels index with the extents the caller derived from
    one operand, so every other operand must have exactly the extents that follow from them, and
    live on the same device.  Anything else is an error here instead of a stray access there."""
    for name, (t, shape) in operands.items():
        if tuple(t.shape) != tuple(shape) or t.device != device:
            raise ValueError(f"{who}: {name} must be {list(shape)} on {device}, got {list(t.shape)} on {t.device}")


def _expand_heads(x: torch.Tensor, hv: int, what: str) -> torch.Tensor:
    hk = int(x.shape[2])
    if hv % hk != 0:
        raise ValueError(f"Cannot align K heads {hk} to {what} heads {hv}")
    return x if hk == hv else torch.repeat_interleave(x, hv // hk, dim=2)


def _gate_per_step(g: torch.Tensor) -> torch.Tensor:
    """g as [B, T, Hv, 1, Dk or 1], broadcastable against a state [B, Hv, Dv, Dk]."""
    if g.ndim == 4:
        return g.unsqueeze(-2)
    if g.ndim == 3:
        return g[..., None, None]
    raise ValueError(f"Unsupported gating shape {tuple(g.shape)}")


def _tape_replay_ops(tape: torch.Tensor, k: torch.Tensor, g: torch.Tensor, state: torch.Tensor,
                     mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The replay recurrence in array ops (what the reference does without its kernel,
    dflash_mlx/kernels.py:328-358): S <- g_t S + delta_t (x) k_t for every unmasked step."""
    kk = _expand_heads(k, int(tape.shape[2]), "tape")
    gate = _gate_per_step(g)
    keep = None if mask is None else mask.to(torch.bool)
    for t in range(int(tape.shape[1])):
        stepped = state * gate[:, t] + tape[:, t].unsqueeze(-1) * kk[:, t].unsqueeze(-2)
        state = stepped if keep is None else torch.where(keep[:, t].view(-1, 1, 1, 1), stepped, state)
    return state


def _gated_delta_ops_with_tape(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor,
                               beta: torch.Tensor, state: torch.Tensor,
                               mask: Optional[torch.Tensor] = None):
    """The forward recurrence in array ops (dflash_mlx/kernels.py:131-173): returns
    (y [B,T,Hv,Dv], state, tape [B,T,Hv,Dv] fp32)."""
    hv = int(v.shape[2])
    qq, kk = _expand_heads(q, hv, "V"), _expand_heads(k, hv, "V")
    gate = _gate_per_step(g)
    keep = None if mask is None else mask.to(torch.bool)
    ys, tape = [], []
    for t in range(int(k.shape[1])):
        decayed = state * gate[:, t]
        innovation = (v[:, t] - (decayed * kk[:, t].unsqueeze(-2)).sum(-1)) * beta[:, t].unsqueeze(-1)
        stepped = decayed + innovation.unsqueeze(-1) * kk[:, t].unsqueeze(-2)
        y_t = (stepped * qq[:, t].unsqueeze(-2)).sum(-1)
        if keep is not None:
            on = keep[:, t]
            stepped = torch.where(on.view(-1, 1, 1, 1), stepped, state)
            innovation = torch.where(on.view(-1, 1, 1), innovation, torch.zeros_like(innovation))
            y_t = torch.where(on.view(-1, 1, 1), y_t, torch.zeros_like(y_t))
        state = stepped
        ys.append(y_t)
        tape.append(innovation.to(torch.float32))
    return torch.stack(ys, dim=1), state, torch.stack(tape, dim=1)


def fused_output_norm_applies(q: torch.Tensor, v: torch.Tensor, state: torch.Tensor, z: torch.Tensor,
                              weight: torch.Tensor) -> bool:
    """Whether ``gated_delta_kernel_with_tape(..., output_norm=...)`` can be asked for: device
    tensors of the kernels' dtypes, z shaped like v, rows of a multiple of 64 up to 256."""
    dv = int(v.shape[-1])
    return (state.is_cuda and z.shape == v.shape and z.device == weight.device == state.device and
            z.dtype == q.dtype == v.dtype and weight.dtype in _DTYPE_CODE and
            q.dtype in _DTYPE_CODE and int(weight.numel()) == dv and dv % 64 == 0 and dv <= 256 and
            int(q.shape[-1]) >= 32 and int(q.shape[-1]) % 32 == 0 and int(q.shape[1]) > 0)


def gated_delta_kernel_with_tape(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor,
                                 beta: torch.Tensor, state: torch.Tensor,
                                 mask: Optional[torch.Tensor] = None, *,
                                 output_norm: Optional[tuple] = None):
    """GatedDeltaNet forward over a block that records the innovation tape (mirror of
    dflash_mlx/kernels.py:176-224): ``(y, state_out, tape)`` with y in q's dtype, the state in
    its own dtype and an fp32 tape.  Device tensors with Dk a multiple of 32 go to the gfx950
    kernel behind ``dflash_gdn_forward_tape``; host tensors and other shapes take the array
    ops, as the reference does without its kernel.

    ``output_norm=(z, weight, eps)`` (no counterpart in the reference, which calls the layer's
    norm right after): the first result is then ``silu(z) * rms_norm(y, weight, eps)``, computed
    by the same launch (``dflash_gdn_forward_tape_norm``); only for inputs the kernel takes -
    callers check ``fused_output_norm_applies`` first."""
    B, T, hk, dk = (int(d) for d in k.shape)
    hv, dv = int(v.shape[2]), int(v.shape[3])
    if g.ndim not in (3, 4):
        raise ValueError(f"Unsupported gating shape {tuple(g.shape)}")
    if hv % hk != 0:
        raise ValueError(f"Cannot align K heads {hk} to V heads {hv}")
    dtypes_ok = (q.dtype == k.dtype == v.dtype and
                 all(t.dtype in _DTYPE_CODE for t in (q, g, beta, state)))
    if not state.is_cuda or dk < 32 or dk % 32 != 0 or not dtypes_ok or T == 0:
        return _gated_delta_ops_with_tape(q, k, v, g, beta, state, mask)
    lib = _native.lib()
    _require_extents("gated_delta_kernel_with_tape", state.device, q=(q, (B, T, hk, dk)), k=(k, (B, T, hk, dk)),
                     v=(v, (B, T, hv, dv)), g=(g, (B, T, hv) + ((dk,) if g.ndim == 4 else ())),
                     beta=(beta, (B, T, hv)), state=(state, (B, hv, dv, dk)))
    if mask is not None and (mask.numel() != B * T or mask.device != state.device):
        raise ValueError(f"gated_delta_kernel_with_tape: mask must hold {B} x {T} entries on {state.device}")
    q_c, k_c, v_c, g_c, beta_c = (t.contiguous() for t in (q, k, v, g, beta))
    state_c = state.contiguous()
    y = torch.empty((B, T, hv, dv), dtype=q.dtype, device=q.device)
    tape = torch.empty((B, T, hv, dv), dtype=torch.float32, device=q.device)
    state_out = torch.empty_like(state_c)
    mask_ptr = None
    if mask is not None:
        mask = mask.to(torch.uint8).contiguous()
        mask_ptr = mask.data_ptr()
    if output_norm is not None:
        z, weight, eps = output_norm
        if not fused_output_norm_applies(q, v, state, z, weight):
            raise ValueError("output_norm: shapes or dtypes the fused kernel does not take")
        z_c, w_c = z.contiguous(), weight.contiguous()
        rc = lib.dflash_gdn_forward_tape_norm(
            q_c.data_ptr(), k_c.data_ptr(), v_c.data_ptr(), g_c.data_ptr(), beta_c.data_ptr(),
            state_c.data_ptr(), state_out.data_ptr(), z_c.data_ptr(), w_c.data_ptr(), y.data_ptr(), tape.data_ptr(),
            mask_ptr, B, T, hk, hv, dk, dv, _DTYPE_CODE[q.dtype], _DTYPE_CODE[g.dtype], _DTYPE_CODE[beta.dtype],
            _DTYPE_CODE[state.dtype], _DTYPE_CODE[weight.dtype], 1 if g.ndim == 4 else 0, float(eps),
            _native.raw_stream(q.device))
        _native.check(rc, "dflash_gdn_forward_tape_norm")
        return y, state_out, tape
    rc = lib.dflash_gdn_forward_tape(
        q_c.data_ptr(), k_c.data_ptr(), v_c.data_ptr(), g_c.data_ptr(), beta_c.data_ptr(),
        state_c.data_ptr(), state_out.data_ptr(), y.data_ptr(), tape.data_ptr(), mask_ptr,
        B, T, hk, hv, dk, dv, _DTYPE_CODE[q.dtype], _DTYPE_CODE[g.dtype], _DTYPE_CODE[beta.dtype],
        _DTYPE_CODE[state.dtype], 1 if g.ndim == 4 else 0,
        _native.raw_stream(q.device))
    _native.check(rc, "dflash_gdn_forward_tape")
    return y, state_out, tape


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
                  exact_order: Optional[bool] = None,
                  conv: Optional[tuple] = None) -> None:
    """Enqueue one ``dflash_tape_replay`` on the current stream.

    The leading dimension(s) of every operand are flattened into ``slots``
    independent problems; ``steps`` is a host int applied to every slot or an int32
    device tensor with one entry per slot.  ``T_alloc`` is the number of step rows
    each slot's tape/k/g storage holds (>= any step count used).

    ``conv = (conv_prev or None, qkv, conv_out)`` (contiguous, ``[slots.., keep | T_alloc, C]``, no
    mask): the same launch also rebuilds the conv windows (``dflash_rollback_layer``)."""
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
    stream = _native.raw_stream(state_in.device)
    exact = 1 if (_exact_order() if exact_order is None else exact_order) else 0
    if conv is not None:
        conv_prev, qkv, conv_out = conv
        if mask is not None or not (qkv.is_contiguous() and conv_out.is_contiguous()) or int(qkv.shape[-2]) != T_alloc:
            raise ValueError("conv windows ride along only without a mask, contiguous, with the tape's row count")
        # The kernel writes slots * keep rows of C elements into conv_out and reads slots * T_alloc
        # rows of qkv (and slots * keep of conv_prev): every one of those extents, the element
        # type and the device are checked here, since nothing behind this point can.
        keep, C = int(conv_out.shape[-2]), int(qkv.shape[-1])

        def leading(t: torch.Tensor) -> int:
            n = 1
            for d in t.shape[:-2]:
                n *= int(d)
            return n

        if (qkv.ndim < 3 or conv_out.ndim < 3 or int(conv_out.shape[-1]) != C or conv_out.dtype != qkv.dtype
                or leading(qkv) != slots or leading(conv_out) != slots
                or not (qkv.device == conv_out.device == state_in.device)):
            raise ValueError(f"conv windows: qkv must be [slots.., {T_alloc}, C] and conv_out [slots.., keep, C] with "
                             f"{slots} slots, one element type, on {state_in.device}; got {tuple(qkv.shape)} {qkv.dtype} "
                             f"on {qkv.device} and {tuple(conv_out.shape)} {conv_out.dtype} on {conv_out.device}")
        if conv_prev is not None and not (conv_prev.is_contiguous() and conv_prev.dtype == qkv.dtype
                                          and conv_prev.ndim >= 3 and tuple(conv_prev.shape[-2:]) == (keep, C)
                                          and leading(conv_prev) == slots and conv_prev.device == qkv.device):
            raise ValueError("conv_prev must be contiguous, [slots.., keep, C], in the dtype of qkv, on its device")
        rc = lib.dflash_rollback_layer(
            tape.data_ptr(), k.data_ptr(), g.data_ptr(), state_in.data_ptr(), state_out.data_ptr(),
            None if conv_prev is None else conv_prev.data_ptr(), qkv.data_ptr(), conv_out.data_ptr(),
            steps_dev, steps_host, slots, T_alloc, Hk, Hv, Dk, Dv,
            _DTYPE_CODE[state_in.dtype], _DTYPE_CODE[tape.dtype], _DTYPE_CODE[k.dtype], _DTYPE_CODE[g.dtype],
            g_per_dk, exact, int(conv_out.shape[-2]), int(qkv.shape[-1]), qkv.element_size(), stream)
        _native.check(rc, "dflash_rollback_layer")
        return
    rc = lib.dflash_tape_replay(
        tape.data_ptr(), k.data_ptr(), g.data_ptr(), state_in.data_ptr(), state_out.data_ptr(),
        steps_dev, steps_host, mask_ptr, slots, T_alloc, Hk, Hv, Dk, Dv,
        _DTYPE_CODE[state_in.dtype], _DTYPE_CODE[tape.dtype], _DTYPE_CODE[k.dtype],
        _DTYPE_CODE[g.dtype], g_per_dk, exact, stream)
    _native.check(rc, "dflash_tape_replay")


def tape_replay_kernel(tape: torch.Tensor, k: torch.Tensor, g: torch.Tensor, state: torch.Tensor,
                       mask: Optional[torch.Tensor] = None, steps: Optional[int] = None) -> torch.Tensor:
    """Replay all ``tape.shape[1]`` steps onto ``state``; returns a new state tensor.  ``steps``
    (no counterpart in the reference, which slices) replays only the first ``steps`` of them:
    the same as passing ``tape[:, :steps]``, ``k[:, :steps]``, ``g[:, :steps]`` (and the mask's
    first ``steps`` columns), without making the three views."""
    if steps is not None and (not state.is_cuda or steps >= tape.shape[1] or steps < 0):
        n = max(0, min(int(steps), int(tape.shape[1])))
        tape, k, g = tape[:, :n], k[:, :n], g[:, :n]
        mask = None if mask is None else mask.reshape(mask.shape[0], -1)[:, :n]
        steps = None
    if not state.is_cuda:
        return _tape_replay_ops(tape, k, g, state, mask)
    if steps is not None:
        # device tensors, fewer steps than rows: the rows are read in place where the kernel can
        # stage all of them, else through the sliced form
        bsz, rows, hk, dk = k.shape
        hv, dv = tape.shape[2:]
        direct = (dk >= 32 and dk % 32 == 0 and g.ndim == 3 and hv % hk == 0 and mask is None and
                  tape.is_contiguous() and k.is_contiguous() and g.is_contiguous() and
                  all(t.dtype in _DTYPE_CODE for t in (tape, k, g, state)) and
                  rows * (dv + 2 * dk + 1) * 4 + dk * 4 <= 64 * 1024)
        if not direct:
            n = int(steps)
            return tape_replay_kernel(tape[:, :n], k[:, :n], g[:, :n], state,
                                      None if mask is None else mask.reshape(mask.shape[0], -1)[:, :n])
        _require_extents("tape_replay_kernel", state.device, tape=(tape, (bsz, rows, hv, dv)), k=(k, (bsz, rows, hk, dk)),
                         g=(g, (bsz, rows, hv)), state=(state, (bsz, hv, dv, dk)))
        state_c = state.contiguous()
        state_out = torch.empty_like(state_c)
        replay_launch(tape, k, g, state_c, state_out, steps=int(steps), T_alloc=rows, slots=bsz)
        return state_out

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
    def fits_lds(rows: int) -> bool:  # the kernel stages T_alloc*(Dv + 2*Dk + 1) floats
        return rows * (dv + 2 * dk + 1) * 4 + dk * 4 <= 64 * 1024

    if not fits_lds(steps):
        return _tape_replay_ops(tape, k, g, state, mask)
    _require_extents("tape_replay_kernel", state.device, tape=(tape, (bsz, steps, hv, dv)), k=(k, (bsz, steps, hk, dk)),
                     g=(g, (bsz, steps, hv) + ((dk,) if g.ndim == 4 else ())), state=(state, (bsz, hv, dv, dk)))
    if mask is not None and (mask.numel() != bsz * steps or mask.device != state.device):
        raise ValueError(f"tape_replay_kernel: mask must hold {bsz} x {steps} entries on {state.device}")

    state_c = state.contiguous()
    tape_c, T_tape = _slot_major(tape, hv * dv)
    k_c, T_k = _slot_major(k, hk * dk)
    g_c, T_g = _slot_major(g, hv * (dk if g.ndim == 4 else 1))
    # prefix slices are read in place only when all three share one row count that the kernel
    # can stage; otherwise dense copies of the `steps` rows
    if not (T_tape == T_k == T_g) or not fits_lds(T_tape):
        tape_c, k_c, g_c = tape.contiguous(), k.contiguous(), g.contiguous()
        T_tape = steps
    if mask is not None:
        # the kernel reads the mask with the tape's row count per slot
        mask = mask.reshape(bsz, steps).to(torch.uint8)
        if T_tape != steps:
            mask = torch.nn.functional.pad(mask, (0, T_tape - steps))
    state_out = torch.empty_like(state_c)
    replay_launch(tape_c, k_c, g_c, state_c, state_out, steps=steps, T_alloc=T_tape, mask=mask,
                  slots=bsz)
    return state_out


_SDPA_WORKSPACE: dict = {}


def _sdpa_workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """Partial results of the key ranges, one buffer per device and stream, grown on demand."""
    key = (device, _native.raw_stream(device))
    buf = _SDPA_WORKSPACE.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _SDPA_WORKSPACE[key] = buf
    return buf


def batched_sdpa_2pass_exact(queries: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, scale: float,
                             mask: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """Exact attention of a 16-token verify block over a long KV cache (mirror of
    dflash_mlx/kernels.py:658-761): queries [B,Hq,16,D], keys / values [B,Hk,N,D] (views of a
    cache are read in place), mask None, bool or additive, broadcastable to [B,Hq,16,N].
    Query i attends to keys n <= N - 16 + i.  Returns None - the caller then takes its
    general attention - for everything the kernel does not cover, as the reference does:
    host tensors, q_len != 16, dtypes other than bf16 / fp16, head dims other than 128 / 256,
    more than 8 query heads per key/value head."""
    if queries.ndim != 4 or keys.ndim != 4 or values.ndim != 4 or not queries.is_cuda:
        return None
    bsz, hq, q_len, d = (int(x) for x in queries.shape)
    hk, n_kv = int(keys.shape[1]), int(keys.shape[2])
    vdim = int(values.shape[-1])
    if q_len != 16 or queries.dtype not in (torch.bfloat16, torch.float16):
        return None
    if d not in (128, 256) or d != vdim or hk <= 0 or hq % hk != 0 or hq // hk > 8 or n_kv < 16:
        return None
    if keys.dtype != queries.dtype or values.dtype != queries.dtype:
        return None
    if (tuple(keys.shape) != (bsz, hk, n_kv, d) or tuple(values.shape) != (bsz, hk, n_kv, d)
            or not (keys.device == values.device == queries.device)):
        return None

    def in_place(t: torch.Tensor) -> torch.Tensor:
        ok = t.stride(3) == 1 and all(s % 8 == 0 for s in t.stride()[:3]) and t.data_ptr() % 16 == 0
        return t if ok else t.contiguous()

    queries = queries.contiguous()
    keys, values = in_place(keys), in_place(values)
    mask_tensor = None
    if mask is not None:
        if mask.dtype == torch.bool:
            mask_tensor = torch.where(mask, torch.zeros((), dtype=queries.dtype, device=mask.device),
                                      torch.full((), torch.finfo(queries.dtype).min, dtype=queries.dtype,
                                                 device=mask.device))
        else:
            mask_tensor = mask.to(queries.dtype)
        mask_tensor = torch.broadcast_to(mask_tensor.to(queries.device), (bsz, hq, q_len, n_kv)).contiguous()

    lib = _native.lib()
    out = torch.empty_like(queries)
    need = int(lib.dflash_sdpa_q16_workspace_bytes(bsz, hq, hk, n_kv, d))
    ws = _sdpa_workspace(queries.device, need) if need else None
    rc = lib.dflash_sdpa_q16(
        queries.data_ptr(), keys.data_ptr(), values.data_ptr(),
        None if mask_tensor is None else mask_tensor.data_ptr(), out.data_ptr(),
        None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(), bsz, hq, hk, n_kv, d,
        keys.stride(0), keys.stride(1), keys.stride(2), values.stride(0), values.stride(1), values.stride(2),
        float(scale), _DTYPE_CODE[queries.dtype], _native.raw_stream(queries.device))
    _native.check(rc, "dflash_sdpa_q16")
    return out
