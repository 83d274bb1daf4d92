"""Module swap QuantizedLinear -> VerifyQuantizedLinear for the verify step.

Mirror of dflash_mlx/verify_linear.py on ``torch.nn.Module`` trees: the same
eligibility rules (:47-75), the same per-call dispatch - ``M == 16`` goes to
``verify_matmul``, everything else to the stock operator (:103-143) - and the
same install / uninstall entry points (:146-196).  A swapped module shares the
packed weight, scales and biases tensors with the module it replaces.

``fuse_shared_input_linears`` has no counterpart in the reference.  A verify call of
16 x K against N rows costs about 6 us on this part before and after its weights stream
(first-access latency, split-K hand-over, the gap to the next launch), whatever N is, so
projections that read the same activations - gate/up of an MLP, q/k/v of an attention
layer, the input projections of a linear-attention layer - are cheaper as one launch over
their rows laid end to end than as one launch each.  The joint launch is an explicit call:
the parent module asks for all of them at once (``shared_input_outputs(parent, names, x)``,
as the attention and linear-attention layers of this package do).  The module tree and every
module's own tensors (now views into the shared storage) stay as they were, and a member
called on its own still answers, from its rows, with a launch of its own.
"""
from __future__ import annotations

import os
from typing import Callable, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from .quantized import QuantizedLinear, stock_matmul
from .verify_qmm import (ChainProblem, QmmChain, _should_use_verify, pack_weights, packable, verify_matmul,
                         verify_matmul_packed)

_VERIFY_MAX_N_DEFAULT = 100_000


def _env_int(name: str, default: int) -> int:
    try:
        return int(os.environ.get(name, str(default)))
    except ValueError:
        return default


_PROJ_TAGS = {
    "mlp.gate_proj": "mlp_gate",
    "mlp.up_proj": "mlp_up",
    "mlp.down_proj": "mlp_down",
    "self_attn.q_proj": "attn_q",
    "self_attn.k_proj": "attn_k",
    "self_attn.v_proj": "attn_v",
    "self_attn.o_proj": "attn_o",
    "linear_attn.in_proj_qkv": "gdn_qkv",
    "linear_attn.in_proj_z": "gdn_z",
    "linear_attn.out_proj": "gdn_o",
}


def _path_tag(path: str) -> str:
    for suffix, tag in _PROJ_TAGS.items():
        if path.endswith(suffix):
            return tag
    return "other"


def is_verify_eligible(ql, path: str = "") -> bool:
    if not isinstance(ql, QuantizedLinear):
        return False
    if getattr(ql, "bits", None) != 4:
        return False
    if getattr(ql, "group_size", None) not in (32, 64, 128):
        return False
    if getattr(ql, "mode", "affine") != "affine":
        return False
    w = ql.weight
    N = int(w.shape[0])
    K = int(w.shape[1]) * (32 // ql.bits)
    if N % 32 != 0 or K % 32 != 0:
        return False
    if N >= _env_int("DFLASH_VERIFY_MAX_N", _VERIFY_MAX_N_DEFAULT):
        return False
    include = os.environ.get("DFLASH_VERIFY_INCLUDE", "all").strip().lower()
    if include not in ("", "all"):
        tag = _path_tag(path)
        allowed = {s.strip() for s in include.split(",") if s.strip()}
        if "mlp" in allowed:
            allowed.update({"mlp_gate", "mlp_up", "mlp_down"})
        if "attn" in allowed:
            allowed.update({"attn_q", "attn_k", "attn_v", "attn_o"})
        if "gdn" in allowed:
            allowed.update({"gdn_qkv", "gdn_z", "gdn_o"})
        if tag not in allowed:
            return False
    return True


# Sibling projections that read the same input in the decoder layers the reference serves.
SHARED_INPUT_GROUPS: Tuple[Tuple[str, ...], ...] = (
    ("gate_proj", "up_proj"),
    ("q_proj", "k_proj", "v_proj"),
    ("in_proj_qkv", "in_proj_z", "in_proj_b", "in_proj_a"),
    ("in_proj_qkvz", "in_proj_ba"),
)


class FusedProjections:
    """Rows of several projections of one parent module laid end to end: ``group(x)`` is one
    verify launch, ``x @ [W_0; W_1; ...]^T``, and returns every member's columns of it."""

    def __init__(self, names: Sequence[str], members: Sequence["VerifyQuantizedLinear"]):
        first = members[0]
        self.names = tuple(names)
        self.group_size, self.bits = first.group_size, first.bits
        self.weight = torch.cat([m.weight for m in members], dim=0).contiguous()
        self.scales = torch.cat([m.scales for m in members], dim=0).contiguous()
        self.biases = torch.cat([m.biases for m in members], dim=0).contiguous()
        self.bounds: List[Tuple[int, int]] = []
        row = 0
        for m in members:
            n = int(m.weight.shape[0])
            self.bounds.append((row, row + n))
            row += n
        self._packed = None  # the joint matrix in the streaming kernel's order (pack_verify_linears)
        self._packed_silu = None  # ... and in the order of the silu-mul epilogue, for silu_mul()
        self._silu_chain = None  # the planned launch of silu_mul(), made on first use

    def applies(self, parent: nn.Module, x: torch.Tensor) -> bool:
        """The joint launch gives what ``parent``'s members would give one by one: 16 rows on the
        verify path, on the device the joint matrix lives on, every member still a view into it
        (a module moved with ``.to()``, or replaced, has left) and behind no wrapper that would
        pad this input."""
        m = 1
        for d in x.shape[:-1]:
            m *= d
        if m != 16 or x.device != self.weight.device or not _should_use_verify(x, self.group_size, self.bits, True):
            return False
        for index, name in enumerate(self.names):
            mod = getattr(parent, name, None)
            if getattr(mod, "_dflash_exact_small_proj_wrapped", False):
                if x.ndim == 3 and x.shape[1] < mod.pad_m:
                    return False
                mod = mod.linear
            if getattr(mod, "_shared_input", None) != (self, index):
                return False
        return True

    def silu_mul_ready(self, x: torch.Tensor) -> bool:
        """Two members of equal height in a shape the chained kernel's epilogue covers."""
        if len(self.bounds) != 2 or not x.is_cuda or self.bits != 4 or self.group_size != 64:
            return False
        rows = self.bounds[0][1]
        k = int(self.weight.shape[1]) * 8
        return self.bounds[1] == (rows, 2 * rows) and rows % 64 == 0 and k % 1024 == 0 and x.is_contiguous()

    def silu_mul(self, x: torch.Tensor) -> torch.Tensor:
        """``silu(x @ W_0^T) * (x @ W_1^T)`` in one launch; a new tensor per call."""
        rows = self.bounds[0][1]
        out = torch.empty((*x.shape[:-1], rows), dtype=x.dtype, device=x.device)
        chain = self._silu_chain
        if chain is None:
            if self._packed_silu is not None:
                problem = ChainProblem(x.reshape(16, -1), self._packed_silu, epilogue="silu_mul", out=out.view(16, rows))
            else:
                problem = ChainProblem(x.reshape(16, -1), self.weight, self.scales, self.biases,
                                       epilogue="silu_mul", out=out.view(16, rows))
            chain = QmmChain([problem])
            self._silu_chain = chain
        else:
            chain.rebind(0, x=x.reshape(16, -1), out=out.view(16, rows))
        chain()
        return out

    def __call__(self, x: torch.Tensor) -> Tuple[torch.Tensor, ...]:
        if self._packed is not None and x.is_cuda:
            product = verify_matmul_packed(x, self._packed)
        else:
            product = verify_matmul(x, self.weight, self.scales, self.biases, transpose=True,
                                    group_size=self.group_size, bits=self.bits)
        return tuple(product[..., lo:hi] for lo, hi in self.bounds)


def silu_gate_up(parent: nn.Module, x: torch.Tensor, names: Tuple[str, str] = ("gate_proj", "up_proj")) -> torch.Tensor:
    """``silu(parent.gate_proj(x)) * parent.up_proj(x)``, the hidden activation of a gated MLP.

    Where ``fuse_shared_input_linears`` joined the two projections, they have the same number of
    rows and the chained kernel covers the shape (group 64, K a multiple of 1024, rows a multiple
    of 64), a 16-row block on the verify path takes ONE launch: the joint product with the
    activation and the product applied before anything is stored (``dflash_qmm_m16_chain`` with
    its silu-mul epilogue; every operator's rounding to the activation dtype is kept, the split
    of K between workgroups differs from the separate projections', so single results may
    differ by one rounding of the array dtype).  Everything else goes through
    ``shared_input_outputs`` and the array operators.  No counterpart in the reference, whose MLP
    is mlx-lm's ``down_proj(swiglu(gate_proj(x), up_proj(x)))``; 27B shape: gate/up/activation
    48 us with ``down_proj`` against 60 us for the four separate steps."""
    for group in getattr(parent, "_dflash_fused", ()):
        if group.names == tuple(names) and group.applies(parent, x) and group.silu_mul_ready(x):
            return group.silu_mul(x)
    gate, up = shared_input_outputs(parent, names, x)
    return (gate * torch.sigmoid(gate)) * up   # x * sigmoid(x): the operators the epilogue follows, one rounding each


def shared_input_outputs(parent: nn.Module, names: Sequence[str], x: torch.Tensor) -> Tuple[torch.Tensor, ...]:
    """``tuple(getattr(parent, n)(x) for n in names)``, with the projections that
    ``fuse_shared_input_linears`` joined under ``parent`` served by their one launch."""
    outs = {}
    for group in getattr(parent, "_dflash_fused", ()):
        if all(n in names for n in group.names) and group.applies(parent, x):
            outs.update(zip(group.names, group(x)))
    return tuple(outs[n] if n in outs else getattr(parent, n)(x) for n in names)


def _build_dispatch(obj: "VerifyQuantizedLinear"):
    w = obj.weight
    s = obj.scales
    b = obj.biases
    gs = obj.group_size
    bits = obj.bits
    mode = obj.mode
    bias = obj.bias
    packed = getattr(obj, "_packed", None)

    def call(x: torch.Tensor) -> torch.Tensor:
        m = 1
        for d in x.shape[:-1]:
            m *= d
        if m == 16 and packed is not None and x.is_cuda and _should_use_verify(x, gs, bits, True):
            y = verify_matmul_packed(x, packed)
        elif m == 16:
            y = verify_matmul(x, w, s, b, transpose=True, group_size=gs, bits=bits)
        else:
            y = stock_matmul(x, w, s, b, transpose=True, group_size=gs, bits=bits, mode=mode)
        return y if bias is None else y + bias

    return call


class VerifyQuantizedLinear(QuantizedLinear):
    """A QuantizedLinear whose M=16 calls go through ``verify_matmul``."""

    @classmethod
    def from_quantized(cls, ql: QuantizedLinear) -> "VerifyQuantizedLinear":
        obj = cls(ql.weight, ql.scales, getattr(ql, "biases", None), getattr(ql, "bias", None),
                  group_size=ql.group_size, bits=ql.bits, mode=getattr(ql, "mode", "affine"))
        object.__setattr__(obj, "_shared_input", None)
        object.__setattr__(obj, "_packed", None)
        object.__setattr__(obj, "_call_fn", _build_dispatch(obj))
        obj.requires_grad_(False)
        return obj

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self._call_fn(x)

    def _apply(self, fn, *args, **kwargs):
        # .to()/.cuda() replace the buffers; re-bind the dispatch closure to the new ones.
        # The new buffers are no longer views into a joint matrix: leave the group (its
        # ``applies`` sees that and stops serving the parent).
        out = super()._apply(fn, *args, **kwargs)
        object.__setattr__(self, "_shared_input", None)
        object.__setattr__(self, "_packed", None)  # a packed copy stays where it was made
        object.__setattr__(self, "_call_fn", _build_dispatch(self))
        return out


def _swap_modules(model: nn.Module, fn: Callable[[str, nn.Module], nn.Module]) -> None:
    for parent_path, parent in list(model.named_modules()):
        for name, child in list(parent.named_children()):
            path = f"{parent_path}.{name}" if parent_path else name
            new = fn(path, child)
            if new is not child:
                setattr(parent, name, new)


def install_verify_linears(model: nn.Module, *,
                           predicate: Optional[Callable[[str, QuantizedLinear], bool]] = None) -> int:
    if predicate is None:
        predicate = lambda path, m: is_verify_eligible(m, path=path)  # noqa: E731

    count = 0

    def _maybe_swap(path: str, m: nn.Module) -> nn.Module:
        nonlocal count
        if isinstance(m, VerifyQuantizedLinear):
            return m
        if isinstance(m, QuantizedLinear) and predicate(path, m):
            count += 1
            return VerifyQuantizedLinear.from_quantized(m)
        return m

    _swap_modules(model, _maybe_swap)
    return count


def pack_verify_linears(model: nn.Module) -> int:
    """Gives every swapped linear that stands alone, and every shared-input group (its joint
    matrix, counted once), whose shape the packed form covers (group 64, K a multiple of 1024, on the GPU) a second copy
    of its weights in the order the streaming kernel reads them; its 16-row calls then go through
    ``verify_matmul_packed`` and return the same bits as before, 3-8 % sooner.  A joined gate/up
    pair of equal heights gets one more copy, in the order of the chained kernel's silu-mul
    epilogue, which ``silu_gate_up`` then reads (same bits, about 10 % sooner).  The row-major
    buffers stay for every other call shape.  Call it after ``install_verify_linears`` (and
    after ``fuse_shared_input_linears``, if used) with the model on its device; moving a module
    afterwards drops its packed copy.  Returns the number of linears packed.  No counterpart in
    the reference."""
    count = 0
    for m in model.modules():
        shared = getattr(m, "_shared_input", None) if isinstance(m, VerifyQuantizedLinear) else None
        if shared is not None and shared[0]._packed is None and shared[0].bits == 4 \
                and packable(shared[0].weight, shared[0].scales, shared[0].biases, shared[0].group_size, 4):
            shared[0]._packed = pack_weights(shared[0].weight, shared[0].scales, shared[0].biases)
            group = shared[0]
            # a gate/up pair also in the order its one-launch activation reads (silu_gate_up)
            if (len(group.bounds) == 2 and group.bounds[1] == (group.bounds[0][1], 2 * group.bounds[0][1])
                    and group.bounds[0][1] % 64 == 0 and group._silu_chain is None):
                group._packed_silu = pack_weights(group.weight, group.scales, group.biases, gate_up=True)
            count += 1
        if (isinstance(m, VerifyQuantizedLinear) and getattr(m, "_shared_input", None) is None
                and getattr(m, "_packed", None) is None and m.biases is not None and m.mode == "affine"
                and packable(m.weight, m.scales, m.biases, m.group_size, m.bits)):
            object.__setattr__(m, "_packed", pack_weights(m.weight, m.scales, m.biases))
            object.__setattr__(m, "_call_fn", _build_dispatch(m))
            count += 1
    return count


def fuse_shared_input_linears(model: nn.Module, *,
                              groups: Sequence[Sequence[str]] = SHARED_INPUT_GROUPS) -> int:
    """Joins, under every parent module, the swapped projections named by one of ``groups``
    (those present, when at least two of them are and they agree in K, group size, dtype and
    device, K is a multiple of 512, the rows add up to a multiple of 32 and none adds a bias vector)
    into a ``FusedProjections`` kept in ``parent._dflash_fused`` for ``shared_input_outputs``; narrow
    projections left out of the swap (N a multiple of 16) join too.  Call it after
    ``install_verify_linears`` and after the model sits on its device.  Returns the number of
    groups formed.  ``DFLASH_VERIFY_FUSE_SHARED_INPUT=0`` turns it into a no-op."""
    if os.environ.get("DFLASH_VERIFY_FUSE_SHARED_INPUT", "1").strip() == "0":
        return 0
    formed = 0

    def candidate(parent: nn.Module, name: str):
        """(holder, attribute, module) of the projection ``parent.name`` if it can be a group
        member, else None.  A narrow projection that the N % 32 rule kept out of the swap (the
        48-row gates of a linear-attention layer) may still join - the joint product is what has
        to pass the gate; a pad-to-16 wrapper around it is looked through."""
        holder, attr, m = parent, name, getattr(parent, name, None)
        if m is not None and getattr(m, "_dflash_exact_small_proj_wrapped", False) and hasattr(m, "linear"):
            holder, attr, m = m, "linear", m.linear
        narrow = (type(m) is QuantizedLinear and m.bits == 4 and m.mode == "affine" and m.group_size in (32, 64, 128)
                  and int(m.weight.shape[0]) % 16 == 0 and m.biases is not None)
        if (narrow or (isinstance(m, VerifyQuantizedLinear) and getattr(m, "_shared_input", None) is None)) \
                and m.bias is None:
            return holder, attr, m
        return None

    for parent in list(model.modules()):
        for names in groups:
            found = [(n,) + c for n, c in ((n, candidate(parent, n)) for n in names) if c is not None]
            if len(found) < 2 or len({id(c[3]) for c in found}) != len(found):
                continue
            ref = found[0][3]
            same = all(m.weight.shape[1] == ref.weight.shape[1] and m.group_size == ref.group_size and
                       m.bits == ref.bits and m.mode == ref.mode and m.scales.dtype == ref.scales.dtype and
                       m.weight.dtype == ref.weight.dtype and m.weight.device == ref.weight.device
                       for _, _, _, m in found)
            rows = sum(int(m.weight.shape[0]) for _, _, _, m in found)
            # K a multiple of 512: no variant's divisibility guard can send the joint product
            # to the stock operator, whose rounding differs between one matrix and several
            k = int(ref.weight.shape[1]) * (32 // ref.bits)
            if not same or k % 512 != 0 or rows % 32 != 0 or \
                    rows >= _env_int("DFLASH_VERIFY_MAX_N", _VERIFY_MAX_N_DEFAULT):
                continue
            members = []
            for _, holder, attr, m in found:
                if not isinstance(m, VerifyQuantizedLinear):  # a narrow projection: swapped now that it has a group
                    m = VerifyQuantizedLinear.from_quantized(m)
                    setattr(holder, attr, m)
                members.append(m)
            group = FusedProjections([n for n, _, _, _ in found], members)
            object.__setattr__(parent, "_dflash_fused", tuple(getattr(parent, "_dflash_fused", ())) + (group,))
            for index, (m, (lo, hi)) in enumerate(zip(members, group.bounds)):
                # the module's own tensors become views: the stock path and state_dict see the
                # same values, and the separate copies are released
                m.weight, m.scales, m.biases = group.weight[lo:hi], group.scales[lo:hi], group.biases[lo:hi]
                object.__setattr__(m, "_shared_input", (group, index))
                object.__setattr__(m, "_call_fn", _build_dispatch(m))
            formed += 1
    return formed


def uninstall_verify_linears(model: nn.Module) -> int:
    count = 0

    def _maybe_unswap(path: str, m: nn.Module) -> nn.Module:
        nonlocal count
        if isinstance(m, VerifyQuantizedLinear):
            count += 1
            return QuantizedLinear(m.weight, m.scales, getattr(m, "biases", None),
                                   getattr(m, "bias", None), group_size=m.group_size,
                                   bits=m.bits, mode=m.mode)
        return m

    _swap_modules(model, _maybe_unswap)
    return count
