"""MLX affine int4 format on torch tensors: the *stock* (non-verify) operators.

These stand where the reference calls into the third-party mlx package:
``mx.quantized_matmul`` (dflash_mlx/verify_qmm.py:277-280, 300-304, 317-321;
dflash_mlx/verify_linear.py:124-127, 139-142), ``mx.quantize`` and
``mlx.nn.QuantizedLinear``.  They are ordinary torch ops on whatever device the
operands live on - the path every shape that is *not* an M=16 verify call takes.

Packed layout (dflash_mlx/verify_qmm.py:70-76): ``w[n, k >> 3]`` is a 32-bit word
holding elements ``8*(k>>3) .. +7`` of row n, element k in bits ``4*(k&7) .. +3``;
``scales`` / ``biases`` are ``[N, K/group_size]``; ``w~ = q * scale + bias``.
"""
from __future__ import annotations

import os

from typing import Optional, Tuple

import torch
import torch.nn as nn

_WORD_DTYPES = tuple(d for d in (torch.int32, getattr(torch, "uint32", None)) if d is not None)


def as_words_i32(w: torch.Tensor) -> torch.Tensor:
    """View packed words as int32 (bit-identical) so that shifts/masks are available."""
    if w.dtype == torch.int32:
        return w
    if w.dtype in _WORD_DTYPES:
        return w.view(torch.int32)
    raise TypeError(f"packed weights must be 32-bit words, got {w.dtype}")


def unpack_codes(w: torch.Tensor, bits: int = 4) -> torch.Tensor:
    """[..., N, K/8] words -> [..., N, K] uint8 codes (low nibble first)."""
    if bits != 4:
        raise NotImplementedError("only 4-bit codes are implemented")
    wi = as_words_i32(w)
    shifts = torch.arange(0, 32, 4, device=w.device, dtype=torch.int32)
    codes = (wi.unsqueeze(-1) >> shifts) & 0xF
    return codes.reshape(*wi.shape[:-1], wi.shape[-1] * 8).to(torch.uint8)


def pack_codes(codes: torch.Tensor) -> torch.Tensor:
    """[..., N, K] codes in 0..15 -> [..., N, K/8] int32 words (low nibble first)."""
    c = codes.to(torch.int64).reshape(*codes.shape[:-1], codes.shape[-1] // 8, 8)
    shifts = torch.arange(0, 32, 4, device=codes.device, dtype=torch.int64)
    words = (c << shifts).sum(dim=-1)
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words)
    return words.to(torch.int32)


def dequantize(w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
               group_size: int = 64, bits: int = 4, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Affine dequantisation to ``dtype`` (default: dtype of ``scales``); fp32 arithmetic."""
    q = unpack_codes(w, bits).to(torch.float32)
    n, k = q.shape[-2], q.shape[-1]
    qg = q.reshape(*q.shape[:-1], k // group_size, group_size)
    out = qg * scales.to(torch.float32).unsqueeze(-1) + biases.to(torch.float32).unsqueeze(-1)
    return out.reshape(*q.shape[:-2], n, k).to(dtype or scales.dtype)


def quantized_matmul(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
                     *, transpose: bool = True, group_size: int = 64, bits: int = 4,
                     mode: str = "affine") -> torch.Tensor:
    """Stock quantized matmul: dequantise to x.dtype, then an ordinary matmul."""
    if mode != "affine":
        raise NotImplementedError(f"quantisation mode {mode!r}")
    wd = dequantize(w, scales, biases, group_size, bits, dtype=x.dtype)
    return x @ (wd.transpose(-1, -2) if transpose else wd)


def stock_matmul(x: torch.Tensor, w: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
                 *, transpose: bool = True, group_size: int = 64, bits: int = 4, mode: str = "affine") -> torch.Tensor:
    """What a quantized module computes outside the verify switch: ``quantized_matmul``, except
    that at most 16 rows of device activations take the M=16 kernel on zero-padded rows
    (``verify_qmm.small_m_matmul``) instead of dequantising the whole matrix - one-token steps
    and the narrow projections that the verify gate does not admit.  ``DFLASH_STOCK_KERNEL=0``
    keeps every such call on the array-op form."""
    if transpose and mode == "affine" and x.is_cuda and os.environ.get("DFLASH_STOCK_KERNEL", "1") != "0":
        from .verify_qmm import small_m_matmul

        y = small_m_matmul(x, w, scales, biases, group_size=group_size, bits=bits)
        if y is not None:
            return y
    return quantized_matmul(x, w, scales, biases, transpose=transpose, group_size=group_size, bits=bits, mode=mode)


def quantize(w: torch.Tensor, group_size: int = 64, bits: int = 4) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Affine quantisation of ``w [N, K]`` per group of ``group_size`` along K.

    Follows what mlx's ``mx.quantize`` does as far as it is publicly described
    (min/max affine grid with the grid snapped so that the larger-magnitude edge
    is exactly representable); mlx itself is not available to compare against,
    so this only serves to make well-formed test data, not to reproduce mlx bit
    for bit.  Returns (packed int32 [N, K/8], scales, biases) with scales/biases
    in ``w.dtype``.
    """
    if bits != 4:
        raise NotImplementedError("only 4-bit codes are implemented")
    n, k = w.shape
    n_bins = float(2 ** bits - 1)
    wf = w.to(torch.float32).reshape(n, k // group_size, group_size)
    w_max = wf.amax(dim=-1, keepdim=True)
    w_min = wf.amin(dim=-1, keepdim=True)
    mask = w_min.abs() > w_max.abs()
    scales = torch.clamp((w_max - w_min) / n_bins, min=1e-7)
    scales = torch.where(mask, scales, -scales)
    edge = torch.where(mask, w_min, w_max)
    q0 = torch.round(edge / scales)
    scales = torch.where(q0 != 0, edge / q0, scales)
    biases = torch.where(q0 == 0, torch.zeros_like(edge), edge)
    # round scale/bias to the storage dtype first so that codes are chosen against
    # the values that will actually be used
    scales = scales.to(w.dtype)
    biases = biases.to(w.dtype)
    codes = torch.clamp(torch.round((wf - biases.to(torch.float32)) / scales.to(torch.float32)), 0, n_bins)
    packed = pack_codes(codes.reshape(n, k).to(torch.uint8))
    return packed, scales.squeeze(-1).contiguous(), biases.squeeze(-1).contiguous()


class QuantizedLinear(nn.Module):
    """torch counterpart of ``mlx.nn.QuantizedLinear`` (the module the reference swaps,
    dflash_mlx/verify_linear.py:47-60, 78-97): packed ``weight``, ``scales``, ``biases``,
    optional additive ``bias``; attributes ``group_size``, ``bits``, ``mode``."""

    def __init__(self, weight: torch.Tensor, scales: torch.Tensor, biases: Optional[torch.Tensor],
                 bias: Optional[torch.Tensor] = None, *, group_size: int = 64, bits: int = 4,
                 mode: str = "affine"):
        super().__init__()
        self.group_size = int(group_size)
        self.bits = int(bits)
        self.mode = mode
        self.register_buffer("weight", weight)
        self.register_buffer("scales", scales)
        self.register_buffer("biases", biases)
        self.register_buffer("bias", bias)

    @classmethod
    def from_linear(cls, linear: nn.Linear, group_size: int = 64, bits: int = 4) -> "QuantizedLinear":
        w, s, b = quantize(linear.weight.detach(), group_size, bits)
        bias = linear.bias.detach() if linear.bias is not None else None
        return cls(w, s, b, bias, group_size=group_size, bits=bits)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = stock_matmul(x, self.weight, self.scales, self.biases, transpose=True,
                         group_size=self.group_size, bits=self.bits, mode=self.mode)
        if self.bias is not None:
            y = y + self.bias
        return y

    def extra_repr(self) -> str:
        n = self.weight.shape[0]
        k = self.weight.shape[1] * (32 // self.bits)
        return f"in={k}, out={n}, group_size={self.group_size}, bits={self.bits}, mode={self.mode}"
