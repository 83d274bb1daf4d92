"""Module swap QuantizedLinear -> VerifyQuantizedLinear for the verify step.

Mirror of dflash_mlx/verify_linear.py on ``torch.nn.Module`` trees: the same
eligibility rules (:47-75), the same per-call dispatch - ``M == 16`` goes to
``verify_matmul``, everything else to the stock operator (:103-143) - and the
same install / uninstall entry points (:146-196).  A swapped module shares the
packed weight, scales and biases tensors with the module it replaces.
"""
from __future__ import annotations

import os
from typing import Callable, Optional

import torch
import torch.nn as nn

from .quantized import QuantizedLinear, quantized_matmul
from .verify_qmm import verify_matmul

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


def _build_dispatch(obj: "VerifyQuantizedLinear"):
    w = obj.weight
    s = obj.scales
    b = obj.biases
    gs = obj.group_size
    bits = obj.bits
    mode = obj.mode
    bias = obj.bias

    def call(x: torch.Tensor) -> torch.Tensor:
        m = 1
        for d in x.shape[:-1]:
            m *= d
        if m == 16:
            y = verify_matmul(x, w, s, b, transpose=True, group_size=gs, bits=bits)
        else:
            y = quantized_matmul(x, w, s, b, transpose=True, group_size=gs, bits=bits, mode=mode)
        return y if bias is None else y + bias

    return call


class VerifyQuantizedLinear(QuantizedLinear):
    """A QuantizedLinear whose M=16 calls go through ``verify_matmul``."""

    @classmethod
    def from_quantized(cls, ql: QuantizedLinear) -> "VerifyQuantizedLinear":
        obj = cls(ql.weight, ql.scales, getattr(ql, "biases", None), getattr(ql, "bias", None),
                  group_size=ql.group_size, bits=ql.bits, mode=getattr(ql, "mode", "affine"))
        object.__setattr__(obj, "_call_fn", _build_dispatch(obj))
        obj.requires_grad_(False)
        return obj

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self._call_fn(x)

    def _apply(self, fn, *args, **kwargs):
        # .to()/.cuda() replace the buffers; re-bind the dispatch closure to the new ones
        out = super()._apply(fn, *args, **kwargs)
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
