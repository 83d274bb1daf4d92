"""Per-layer recurrent cache of a GatedDeltaNet layer with tape-replay rollback.

Mirror of dflash_mlx/recurrent_rollback_cache.py: ``cache[0]`` is the conv window,
``cache[1]`` the recurrent state ``[B, Hv, Dv, Dk]``.  A verify step arms the cache
(snapshot by reference), the forward records the innovation tape, and ``rollback``
restores the snapshot and re-applies only ``n_accepted + 1`` steps (:148-171).

torch tensors are mutable where mlx arrays are not, so the snapshot only stays
valid if nothing writes into the snapshotted tensors in place: this class never
does (replay and conv rebuild write fresh tensors), and a forward that records a
tape must assign a *new* tensor to ``cache[1]`` rather than update it in place.

``RollbackArena`` is the batched form for a whole model: one allocation holds the
states (double-buffered), tapes and conv windows of all GDN layers, so that a
rollback of every layer is a single launch (replay and conv-window rebuild together)
whose accepted length may live on the device.
"""
from __future__ import annotations

from typing import Any, List, Optional, Union

import torch

from . import _native
from .kernels import _DTYPE_CODE, _exact_order, replay_launch, tape_replay_kernel


def conv_state_rebuild(conv_prev: Optional[torch.Tensor], qkv: torch.Tensor,
                       steps: Union[int, torch.Tensor], keep: int,
                       out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``concat([conv_prev or zeros, qkv], 1)[:, steps:steps+keep]`` as one device launch
    (dflash_mlx/recurrent_rollback_cache.py:129-146).  Leading dims are slots."""
    lead = qkv.shape[:-2]
    T, C = int(qkv.shape[-2]), int(qkv.shape[-1])
    slots = 1
    for d in lead:
        slots *= int(d)
    if out is None:
        out = torch.empty((*lead, keep, C), dtype=qkv.dtype, device=qkv.device)
    if not qkv.is_cuda:
        raise _native.NativeLibraryError("conv_state_rebuild needs device tensors")
    if (tuple(out.shape) != (*lead, keep, C) or out.dtype != qkv.dtype or out.device != qkv.device
            or not out.is_contiguous()):
        raise ValueError("out must be a contiguous [.., keep, C] tensor in the dtype of qkv, on its device")
    if isinstance(steps, torch.Tensor) and (steps.dtype != torch.int32 or steps.device != qkv.device
                                            or steps.numel() != slots or not steps.is_contiguous()):
        raise ValueError("steps tensor must be int32, on the device, one entry per slot")
    qkv = qkv.contiguous()
    prev_ptr = None
    if conv_prev is not None:
        conv_prev = conv_prev.contiguous()
        if (conv_prev.dtype != qkv.dtype or tuple(conv_prev.shape) != (*lead, keep, C)
                or conv_prev.device != qkv.device):
            raise ValueError("conv_prev must be [.., keep, C] in the dtype of qkv, on its device")
        prev_ptr = conv_prev.data_ptr()
    steps_dev, steps_host = None, 0
    if isinstance(steps, torch.Tensor):
        steps_dev = steps.data_ptr()
    else:
        steps_host = int(steps)
    stream = _native.raw_stream(qkv.device)
    rc = _native.lib().dflash_conv_state_rebuild(prev_ptr, qkv.data_ptr(), out.data_ptr(), steps_dev,
                                                 steps_host, slots, T, keep, C, qkv.element_size(),
                                                 stream)
    _native.check(rc, "dflash_conv_state_rebuild")
    return out


class RecurrentRollbackCache:
    def __init__(self, size: int = 2, *, conv_kernel_size: int = 4):
        self.cache: List[Any] = [None] * size
        self.conv_kernel_size = int(conv_kernel_size)
        self._armed = False
        self._tape = None
        self._tape_k = None
        self._tape_g = None
        self._tape_qkv = None
        self._snapshot = None
        self._arena: Optional["RollbackArena"] = None
        self._layer = -1
        # batched generation (dflash_mlx/recurrent_rollback_cache.py:18-19): per-row lengths of a
        # right-padded block, or per-row left padding, as `prepare` / a batching loop sets them
        self.lengths: Optional[torch.Tensor] = None
        self.left_padding: Optional[torch.Tensor] = None

    def __getitem__(self, idx: int):
        return self.cache[idx]

    def __setitem__(self, idx: int, value: Any) -> None:
        self.cache[idx] = value

    @property
    def state(self):
        return self.cache

    @state.setter
    def state(self, value) -> None:
        self.cache = value

    @property
    def nbytes(self):
        return sum(c.numel() * c.element_size() for c in self.cache if c is not None)

    # -- batch-cache protocol of the generation loops (recurrent_rollback_cache.py:46-94) ------
    # Rows of a batch come and go between steps, never inside a verify step: what a rollback
    # needs (snapshot, tapes) describes the batch as it was, so every change of the batch drops
    # it, and a cache that was a view into a RollbackArena stands on tensors of its own afterwards.
    def _leave_arena(self) -> None:
        self.clear_transients()
        self._arena, self._layer = None, -1

    def filter(self, batch_indices) -> None:
        """Keep the rows ``batch_indices`` (in that order)."""
        self._leave_arena()
        self.cache = [c[batch_indices] if c is not None else None for c in self.cache]
        if self.lengths is not None:
            self.lengths = self.lengths[batch_indices]
        if self.left_padding is not None:
            self.left_padding = self.left_padding[batch_indices]

    def extend(self, other: "RecurrentRollbackCache") -> None:
        """Append the rows of ``other``."""
        if len(self.cache) != len(other.cache):
            raise ValueError(f"caches of {len(self.cache)} and {len(other.cache)} entries cannot be joined")
        self._leave_arena()

        def joined(mine, theirs):
            if mine is None:
                return theirs
            if theirs is None:
                return mine
            return torch.cat([mine, theirs], dim=0)

        self.cache = [joined(a, b) for a, b in zip(self.cache, other.cache)]

    def extract(self, idx: int) -> "RecurrentRollbackCache":
        """A cache of its own holding row ``idx`` (batch dimension kept)."""
        one = RecurrentRollbackCache(len(self.cache), conv_kernel_size=self.conv_kernel_size)
        one.cache = [c[idx:idx + 1] if c is not None else None for c in self.cache]
        return one

    def prepare(self, lengths=None, **kwargs) -> None:
        del kwargs
        if lengths is None:
            self.lengths = None
            return
        device = next((c.device for c in self.cache if c is not None), None)
        self.lengths = torch.as_tensor(lengths, device=device)

    def finalize(self) -> None:
        self.lengths = None
        self.left_padding = None
        self.clear_transients()

    def advance(self, n: int) -> None:
        if self.lengths is not None:
            self.lengths = self.lengths - n
        if self.left_padding is not None:
            self.left_padding = self.left_padding - n

    def make_mask(self, n: int):
        """[B, n] bool, true where a position of the next ``n`` holds a token; None without padding."""
        ref = self.left_padding if self.left_padding is not None else self.lengths
        if ref is None:
            return None
        pos = torch.arange(n, device=ref.device)
        if self.left_padding is not None:
            return pos >= self.left_padding[:, None]
        return pos < self.lengths[:, None]

    def empty(self) -> bool:
        return self.cache[0] is None

    # -- rollback state machine (recurrent_rollback_cache.py:96-171)
    def checkpoint(self) -> None:
        self._snapshot = list(self.cache)

    def clear_transients(self) -> None:
        self._armed = False
        self._tape = None
        self._tape_k = None
        self._tape_g = None
        self._tape_qkv = None
        self._snapshot = None

    def arm_rollback(self, prefix_len: int = 0) -> None:
        del prefix_len
        self._armed = True
        self._tape = None
        self._tape_k = None
        self._tape_g = None
        self._tape_qkv = None
        self.checkpoint()

    def record_tape(self, *, tape: torch.Tensor, k: torch.Tensor, g: torch.Tensor,
                    qkv: torch.Tensor) -> None:
        if self._arena is not None:
            self._tape, self._tape_k, self._tape_g, self._tape_qkv = self._arena._store_tape(
                self._layer, tape, k, g, qkv)
            return
        self._tape = tape.contiguous()
        self._tape_k = k.contiguous()
        self._tape_g = g.contiguous()
        self._tape_qkv = qkv.contiguous()

    def _rebuild_conv_state(self, accepted_steps: int):
        if self._tape_qkv is None:
            return self.cache[0]
        keep = self.conv_kernel_size - 1
        if keep <= 0:
            return None
        conv_state = self._snapshot[0] if self._snapshot is not None else None
        if self._tape_qkv.is_cuda and accepted_steps <= int(self._tape_qkv.shape[1]):
            out = None if self._arena is None else self._arena._conv_out(self._layer)
            return conv_state_rebuild(conv_state, self._tape_qkv, accepted_steps, keep, out=out)
        if conv_state is None:
            prefix = torch.zeros((self._tape_qkv.shape[0], keep, self._tape_qkv.shape[-1]),
                                 dtype=self._tape_qkv.dtype, device=self._tape_qkv.device)
        else:
            prefix = conv_state
        conv_input = torch.cat([prefix, self._tape_qkv], dim=1)
        start = accepted_steps
        end = min(start + keep, int(conv_input.shape[1]))
        return conv_input[:, start:end, :].contiguous()

    def _rollback_in_one_call(self, accepted_steps: int) -> bool:
        """Replay and conv-window rebuild of this layer through one library call
        (``dflash_rollback_layer``): the common case of device tensors as ``record_tape`` keeps
        them.  False (nothing done) for anything else, which takes the two wrappers below."""
        tape, k, g, qkv, state = self._tape, self._tape_k, self._tape_g, self._tape_qkv, self.cache[1]
        keep = self.conv_kernel_size - 1
        if (qkv is None or keep <= 0 or not (state.is_cuda and qkv.is_cuda) or tape.ndim != 4 or k.ndim != 4
                or g.ndim != 3 or qkv.ndim != 3):
            return False
        bsz, rows, hv, dv = tape.shape
        hk, dk = k.shape[2], k.shape[3]
        # every extent the kernel indexes with is checked here: it reads what these numbers say
        if not (0 <= accepted_steps <= rows and k.shape[:2] == (bsz, rows) and g.shape == (bsz, rows, hv)
                and qkv.shape[:2] == (bsz, rows) and state.shape == (bsz, hv, dv, dk)
                and dk >= 32 and dk % 32 == 0 and hv % hk == 0
                and rows * (dv + 2 * dk + 1) * 4 + dk * 4 <= 64 * 1024
                and state.is_contiguous() and qkv.is_contiguous() and tape.is_contiguous()
                and k.is_contiguous() and g.is_contiguous()
                and tape.device == k.device == g.device == qkv.device == state.device):
            return False
        codes = _DTYPE_CODE
        if tape.dtype not in codes or k.dtype not in codes or g.dtype not in codes or state.dtype not in codes:
            return False
        prev = self._snapshot[0]
        prev_ptr = None
        if prev is not None:
            if not (prev.device == qkv.device and prev.is_contiguous() and prev.dtype == qkv.dtype
                    and prev.shape == (bsz, keep, qkv.shape[2])):
                return False
            prev_ptr = prev.data_ptr()
        state_out = torch.empty_like(state)
        conv_out = torch.empty((bsz, keep, qkv.shape[2]), dtype=qkv.dtype, device=qkv.device)
        rc = _native.lib().dflash_rollback_layer(
            tape.data_ptr(), k.data_ptr(), g.data_ptr(), state.data_ptr(), state_out.data_ptr(), prev_ptr,
            qkv.data_ptr(), conv_out.data_ptr(), None, accepted_steps, bsz, rows, hk, hv, dk, dv,
            codes[state.dtype], codes[tape.dtype], codes[k.dtype], codes[g.dtype], 0,
            1 if _exact_order() else 0, keep, qkv.shape[2], qkv.element_size(), _native.raw_stream(state.device))
        _native.check(rc, "dflash_rollback_layer")
        self.cache[1], self.cache[0] = state_out, conv_out
        return True

    def rollback(self, n_accepted: int) -> None:
        if self._snapshot is None:
            self.clear_transients()
            return

        self.cache = list(self._snapshot)
        if (self._tape is not None and self._tape_k is not None and self._tape_g is not None
                and self.cache[1] is not None):
            accepted_steps = int(n_accepted) + 1
            if self._arena is None and self._rollback_in_one_call(accepted_steps):
                self.clear_transients()
                return
            if self._arena is not None:
                state = self._arena._replay_layer(self._layer, self.cache[1], accepted_steps)
            else:
                # (the first accepted_steps rows of the three tapes, read in place)
                state = tape_replay_kernel(self._tape, self._tape_k, self._tape_g, self.cache[1], None,
                                           steps=accepted_steps)
            self.cache[1] = state
            self.cache[0] = self._rebuild_conv_state(accepted_steps)

        self.clear_transients()


class RollbackArena:
    """Stacked storage for the recurrent caches of all GDN layers of one model.

    Layout (L layers, B batch rows, T recorded steps):
      state [2, L, B, Hv, Dv, Dk]   double buffer: one half is the live / snapshot
                                    state, the other receives the next state
      conv  [2, L, B, keep, C]      same double buffering for the conv window
      tape  [L, B, T, Hv, Dv]   k [L, B, T, Hk, Dk]   g [L, B, T, Hv(, Dk)]   qkv [L, B, T, C]
      steps [L*B] int32             accepted step count per slot, device resident

    ``caches()`` hands out one ``RecurrentRollbackCache`` per layer whose tensors are
    views into this storage, so the per-layer API keeps working; ``rollback_all``
    replays every layer with one launch.
    """

    def __init__(self, num_layers: int, *, batch: int = 1, max_steps: int = 16, Hk: int, Hv: int,
                 Dk: int, Dv: int, conv_dim: int, conv_kernel_size: int = 4,
                 device: Union[str, torch.device] = "cuda", state_dtype=torch.float32,
                 tape_dtype=torch.float32, k_dtype=torch.bfloat16, g_dtype=torch.float32,
                 qkv_dtype=torch.bfloat16, g_per_dk: bool = False):
        self.L, self.B, self.T = int(num_layers), int(batch), int(max_steps)
        self.Hk, self.Hv, self.Dk, self.Dv, self.C = Hk, Hv, Dk, Dv, int(conv_dim)
        self.keep = int(conv_kernel_size) - 1
        self.conv_kernel_size = int(conv_kernel_size)
        L, B, T = self.L, self.B, self.T
        dev = torch.device(device)
        self.state = torch.zeros((2, L, B, Hv, Dv, Dk), dtype=state_dtype, device=dev)
        self.conv = torch.zeros((2, L, B, max(self.keep, 1), self.C), dtype=qkv_dtype, device=dev)
        self.tape = torch.zeros((L, B, T, Hv, Dv), dtype=tape_dtype, device=dev)
        self.k = torch.zeros((L, B, T, Hk, Dk), dtype=k_dtype, device=dev)
        gshape = (L, B, T, Hv, Dk) if g_per_dk else (L, B, T, Hv)
        self.g = torch.zeros(gshape, dtype=g_dtype, device=dev)
        self.qkv = torch.zeros((L, B, T, self.C), dtype=qkv_dtype, device=dev)
        self.steps = torch.zeros((L * B,), dtype=torch.int32, device=dev)
        self._caches: List[RecurrentRollbackCache] = []
        for layer in range(L):
            c = RecurrentRollbackCache(size=2, conv_kernel_size=conv_kernel_size)
            c._arena, c._layer = self, layer
            c.cache = [self.conv[0, layer], self.state[0, layer]]
            self._caches.append(c)

    def caches(self) -> List[RecurrentRollbackCache]:
        return list(self._caches)

    @staticmethod
    def _half_of(buf: torch.Tensor, layer: int, t: Optional[torch.Tensor]) -> int:
        """Which half of a double buffer tensor ``t`` is (0 when it is in neither)."""
        if t is not None and t.data_ptr() == buf[1, layer].data_ptr():
            return 1
        return 0

    def _reference_entry(self, layer: int, idx: int) -> Optional[torch.Tensor]:
        c = self._caches[layer]
        src = c._snapshot if c._snapshot is not None else c.cache
        return src[idx]

    def next_state(self, layer: int) -> torch.Tensor:
        """Where a verify forward of ``layer`` should write its new state: the half of the
        double buffer that does not hold the snapshot (or, un-armed, the current state)."""
        return self.state[1 - self._half_of(self.state, layer, self._reference_entry(layer, 1)), layer]

    def next_conv(self, layer: int) -> torch.Tensor:
        return self.conv[1 - self._half_of(self.conv, layer, self._reference_entry(layer, 0)), layer]

    def tape_slots(self, layer: int):
        """Views a tape producer may fill in place: (tape, k, g, qkv) of ``layer``."""
        return self.tape[layer], self.k[layer], self.g[layer], self.qkv[layer]

    # -- used by the per-layer cache objects
    def _store_tape(self, layer: int, tape, k, g, qkv):
        dst = self.tape_slots(layer)
        out = []
        for d, src, name in zip(dst, (tape, k, g, qkv), ("tape", "k", "g", "qkv")):
            steps = int(src.shape[1])
            if steps > self.T:
                raise ValueError(f"{name} has {steps} steps, arena holds {self.T}")
            view = d[:, :steps]
            if src.data_ptr() != view.data_ptr() or src.dtype != d.dtype:
                view.copy_(src)  # converts when the producer's dtype is not the arena's
            out.append(view)
        return tuple(out)

    def _conv_out(self, layer: int) -> torch.Tensor:
        return self.next_conv(layer)

    def _replay_layer(self, layer: int, state_in: torch.Tensor, steps: int) -> torch.Tensor:
        out = self.state[1 - self._half_of(self.state, layer, state_in), layer]
        replay_launch(self.tape[layer], self.k[layer], self.g[layer], state_in.contiguous(), out,
                      steps=steps, T_alloc=self.T, slots=self.B)
        return out

    # -- whole-model operations
    def arm_all(self, prefix_len: int = 0) -> None:
        for c in self._caches:
            c.arm_rollback(prefix_len=prefix_len)

    def _uniform_snapshot_half(self) -> Optional[int]:
        """Half (0/1) holding every layer's snapshot state and conv window, or None when
        the layers disagree, a snapshot or tape is missing, or a tensor is foreign."""
        half = None
        for layer, c in enumerate(self._caches):
            if c._snapshot is None or c._tape is None or c._tape_qkv is None:
                return None
            conv, st = c._snapshot[0], c._snapshot[1]
            if st is None or conv is None:
                return None
            h = self._half_of(self.state, layer, st)
            if st.data_ptr() != self.state[h, layer].data_ptr():
                return None
            if conv.data_ptr() != self.conv[h, layer].data_ptr():
                return None
            if c._tape.data_ptr() != self.tape[layer].data_ptr():
                return None
            if half is None:
                half = h
            elif half != h:
                return None
        return half

    def rollback_all(self, n_accepted: Union[int, torch.Tensor], *, drafted_tokens: int = 0) -> None:
        """Roll every layer back to ``n_accepted`` accepted draft tokens.

        ``n_accepted`` is a host int, or an int32 device tensor (a scalar, one entry per
        batch row, or one per layer and batch row) when the acceptance length has not been read back; in that case
        ``drafted_tokens`` cannot short-cut the fully-accepted case and the replay of
        all recorded steps reproduces the forward's state instead.
        """
        host = not isinstance(n_accepted, torch.Tensor)
        if host and drafted_tokens > 0 and int(n_accepted) == drafted_tokens:
            # everything accepted: keep what the forward produced (runtime.py:886-891)
            for c in self._caches:
                c.clear_transients()
            return
        snap = self._uniform_snapshot_half()
        if snap is None:
            if not host:
                raise ValueError("device-side acceptance needs every layer armed on the same half")
            for c in self._caches:
                c.rollback(int(n_accepted))
            return
        nxt = 1 - snap
        if host:
            steps: Union[int, torch.Tensor] = int(n_accepted) + 1
        else:
            acc = n_accepted.to(torch.int32).reshape(-1) + 1
            if acc.numel() == 1:
                acc = acc.expand(self.L * self.B)
            elif acc.numel() == self.B:  # one per batch row: slot = layer * B + row
                acc = acc.repeat(self.L)
            elif acc.numel() != self.L * self.B:
                raise ValueError(f"n_accepted has {acc.numel()} entries; expected 1, {self.B} (one per "
                                 f"batch row) or {self.L * self.B} (one per layer and batch row)")
            self.steps.copy_(acc)
            steps = self.steps
        # every layer's state and conv window in one launch
        replay_launch(self.tape, self.k, self.g, self.state[snap], self.state[nxt], steps=steps,
                      T_alloc=self.T, slots=self.L * self.B,
                      conv=(self.conv[snap], self.qkv, self.conv[nxt]) if self.keep > 0 else None)
        for layer, c in enumerate(self._caches):
            c.cache = [self.conv[nxt, layer], self.state[nxt, layer]]
            c.clear_transients()
