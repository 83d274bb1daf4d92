"""GatedDeltaNet layer glue of the verify step (host side).

Mirror of the layer-level hooks of dflash_mlx/runtime.py:

* ``_ExactSmallProjPad`` / ``_install_exact_small_proj_hooks`` (:243-285) - pad blocks shorter
  than 16 tokens to 16 in front of the two narrow projections, so that a single-token step and
  a 16-token verify step take the same matmul path and produce the same numbers;
* ``_install_speculative_linear_cache_hook`` (:344-455) - the layer call that, for an armed
  ``RecurrentRollbackCache``, runs the recurrence with the innovation tape and records
  tape, k, g and qkv for the rollback.

Between the projections and the recurrence the reference strings together about twenty array
operators (mask, conv, silu, split, two rms norms, gates); here device tensors take two
launches instead, ``dflash_gdn_prepare`` and ``dflash_gdn_gated_norm``
(include/dflash_mi355.h).  The ``*_ops`` functions are the same operators one by one, taken
for host tensors and for head sizes the kernels do not cover.

``GatedDeltaNet`` is a stand-in with the attribute names of the mlx-lm layer the reference
patches (in_proj_qkv / in_proj_z / in_proj_b / in_proj_a, conv1d, A_log, dt_bias, norm,
out_proj); its own ``forward`` is the plain, non-speculative call.
"""
from __future__ import annotations

import os
from typing import Any, Optional, Tuple

import torch
import torch.nn as nn

from . import _native
from .kernels import _DTYPE_CODE, fused_output_norm_applies, gated_delta_kernel_with_tape
from .recurrent_rollback_cache import RecurrentRollbackCache
from .verify_linear import shared_input_outputs

_EXACT_SMALL_PROJ_PAD_M = 16


# ---------------------------------------------------------------------------------------------
# array operators (one rounding to the array dtype per operator, fp32 inside)
# ---------------------------------------------------------------------------------------------
def silu_ops(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def rms_norm_ops(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    xf = x.to(torch.float32)
    y = xf * (1.0 / torch.sqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps))
    if weight is not None:
        y = y * weight.to(torch.float32)
    return y.to(x.dtype)


def compute_g(A_log: torch.Tensor, a: torch.Tensor, dt_bias: torch.Tensor) -> torch.Tensor:
    """exp(-exp(A_log) * softplus(a + dt_bias)) in fp32 (the gate of mlx-lm's gated_delta)."""
    apb = a + dt_bias                       # promoted dtype of the two
    wide = apb.to(torch.float32)
    softplus = (torch.clamp(wide, min=0) + torch.log1p(torch.exp(-wide.abs()))).to(apb.dtype)
    return torch.exp(-torch.exp(A_log.to(torch.float32)) * softplus.to(torch.float32))


def gdn_prepare_ops(qkv: torch.Tensor, conv_state: Optional[torch.Tensor], conv_w: torch.Tensor,
                    a: torch.Tensor, b: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor,
                    mask: Optional[torch.Tensor], *, Hk: int, Hv: int, Dk: int, Dv: int, eps: float = 1e-6):
    """dflash_mlx/runtime.py:381-407 operator by operator: (conv_next, q, k, v, g, beta)."""
    B, S, C = qkv.shape
    if conv_w.ndim == 3:            # mlx conv1d weight [C, K, 1]
        conv_w = conv_w.reshape(conv_w.shape[0], conv_w.shape[1])
    K = int(conv_w.shape[1])
    key_dim = Hk * Dk
    if mask is not None:
        qkv = torch.where(mask.to(torch.bool)[..., None], qkv, torch.zeros_like(qkv))
    if conv_state is None:
        conv_state = torch.zeros((B, K - 1, C), dtype=qkv.dtype, device=qkv.device)
    conv_input = torch.cat([conv_state, qkv], dim=1)
    conv_next = conv_input[:, conv_input.shape[1] - (K - 1):].contiguous()
    acc = torch.zeros((B, S, C), dtype=torch.float32, device=qkv.device)
    for j in range(K):
        acc = acc + conv_input[:, j:j + S].to(torch.float32) * conv_w[:, j].to(torch.float32)
    act = silu_ops(acc.to(qkv.dtype))
    q = act[..., :key_dim].reshape(B, S, Hk, Dk)
    k = act[..., key_dim:2 * key_dim].reshape(B, S, Hk, Dk)
    v = act[..., 2 * key_dim:].reshape(B, S, Hv, Dv).contiguous()
    inv_scale = Dk ** -0.5                  # a Python float meets the array in the array's dtype
    q = torch.tensor(inv_scale ** 2, dtype=q.dtype, device=q.device) * rms_norm_ops(q, None, eps)
    k = torch.tensor(inv_scale, dtype=k.dtype, device=k.device) * rms_norm_ops(k, None, eps)
    return conv_next, q, k, v, compute_g(A_log, a, dt_bias), torch.sigmoid(b)


def gated_norm_ops(x: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    return silu_ops(z) * rms_norm_ops(x, weight, eps)


# ---------------------------------------------------------------------------------------------
# device path
# ---------------------------------------------------------------------------------------------
def _kernel_covers(x: torch.Tensor, *dims: int) -> bool:
    return x.is_cuda and x.dtype in _DTYPE_CODE and all(0 < d <= 256 and d % 64 == 0 for d in dims)


def gdn_prepare(qkv: torch.Tensor, conv_state: Optional[torch.Tensor], conv_w: torch.Tensor, a: torch.Tensor,
                b: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor, mask: Optional[torch.Tensor] = None,
                *, Hk: int, Hv: int, Dk: int, Dv: int, eps: float = 1e-6
                ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Mask, conv, silu, split, norms and gates of a GatedDeltaNet call in one launch:
    (conv_next [B,K-1,C], q, k [B,S,Hk,Dk], v [B,S,Hv,Dv], g [B,S,Hv] fp32, beta [B,S,Hv])."""
    B, S, C = (int(d) for d in qkv.shape)
    if conv_w.ndim == 3:            # mlx conv1d weight [C, K, 1]
        conv_w = conv_w.reshape(conv_w.shape[0], conv_w.shape[1])
    K = int(conv_w.shape[1])
    if C != 2 * Hk * Dk + Hv * Dv or int(conv_w.shape[0]) != C:
        raise ValueError(f"conv_dim {C} does not match 2*{Hk}*{Dk} + {Hv}*{Dv}")
    same = (conv_w.dtype == a.dtype == b.dtype == qkv.dtype and A_log.dtype == dt_bias.dtype and
            A_log.dtype in _DTYPE_CODE and (conv_state is None or conv_state.dtype == qkv.dtype))
    if not (_kernel_covers(qkv, Dk, Dv) and same and S > 0 and 2 <= K <= 4):
        return gdn_prepare_ops(qkv, conv_state, conv_w, a, b, A_log, dt_bias, mask,
                               Hk=Hk, Hv=Hv, Dk=Dk, Dv=Dv, eps=eps)
    lib = _native.lib()
    dev, dt = qkv.device, qkv.dtype
    # the kernel indexes with B, S, C, K and the head counts: every operand must have the extents
    # that follow from them, on qkv's device
    expect = dict(a=(a, (B, S, Hv)), b=(b, (B, S, Hv)), A_log=(A_log, (Hv,)), dt_bias=(dt_bias, (Hv,)),
                  conv_w=(conv_w, (C, K)))
    if conv_state is not None:
        expect["conv_state"] = (conv_state, (B, K - 1, C))
    for name, (t, shape) in expect.items():
        if tuple(t.shape) != shape or t.device != dev:
            raise ValueError(f"gdn_prepare: {name} must be {list(shape)} on {dev}, got {list(t.shape)} on {t.device}")
    if mask is not None and (mask.numel() != B * S or mask.device != dev):
        raise ValueError(f"gdn_prepare: mask must hold {B} x {S} entries on {dev}")
    qkv_c, w_c, a_c, b_c = qkv.contiguous(), conv_w.contiguous(), a.contiguous(), b.contiguous()
    cs = None if conv_state is None else conv_state.contiguous()
    mask_c = None if mask is None else mask.to(torch.uint8).contiguous()
    conv_next = torch.empty((B, K - 1, C), dtype=dt, device=dev)
    q = torch.empty((B, S, Hk, Dk), dtype=dt, device=dev)
    k = torch.empty((B, S, Hk, Dk), dtype=dt, device=dev)
    v = torch.empty((B, S, Hv, Dv), dtype=dt, device=dev)
    g = torch.empty((B, S, Hv), dtype=torch.float32, device=dev)
    beta = torch.empty((B, S, Hv), dtype=dt, device=dev)
    rc = lib.dflash_gdn_prepare(
        qkv_c.data_ptr(), None if cs is None else cs.data_ptr(), w_c.data_ptr(), a_c.data_ptr(), b_c.data_ptr(),
        A_log.contiguous().data_ptr(), dt_bias.contiguous().data_ptr(),
        None if mask_c is None else mask_c.data_ptr(), conv_next.data_ptr(), q.data_ptr(), k.data_ptr(),
        v.data_ptr(), g.data_ptr(), beta.data_ptr(), B, S, Hk, Hv, Dk, Dv, K, _DTYPE_CODE[dt],
        _DTYPE_CODE[A_log.dtype], float(eps), _native.raw_stream(dev))
    _native.check(rc, "dflash_gdn_prepare")
    return conv_next, q, k, v, g, beta


def gated_norm(x: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """silu(z) * rms_norm(x, weight, eps) over the last axis."""
    D = int(x.shape[-1])
    if not (_kernel_covers(x, D) and z.dtype == x.dtype and z.shape == x.shape and weight.dtype in _DTYPE_CODE
            and tuple(weight.shape) == (D,) and z.device == x.device == weight.device):
        return gated_norm_ops(x, z, weight, eps)
    lib = _native.lib()
    x_c, z_c, w_c = x.contiguous(), z.contiguous(), weight.contiguous()
    y = torch.empty_like(x_c)
    rc = lib.dflash_gdn_gated_norm(x_c.data_ptr(), z_c.data_ptr(), w_c.data_ptr(), y.data_ptr(),
                                   x_c.numel() // D, D, _DTYPE_CODE[x.dtype], _DTYPE_CODE[weight.dtype],
                                   float(eps), _native.raw_stream(x.device))
    _native.check(rc, "dflash_gdn_gated_norm")
    return y


# ---------------------------------------------------------------------------------------------
# the layer
# ---------------------------------------------------------------------------------------------
class _ExactSmallProjPad(nn.Module):
    """dflash_mlx/runtime.py:246-274."""

    def __init__(self, linear: nn.Module, *, pad_m: int = _EXACT_SMALL_PROJ_PAD_M):
        super().__init__()
        self.linear = linear
        self.pad_m = int(pad_m)
        self._dflash_exact_small_proj_wrapped = True

    @property
    def weight(self) -> torch.Tensor:
        return self.linear.weight

    @weight.setter
    def weight(self, value: torch.Tensor) -> None:
        self.linear.weight = value

    @property
    def bias(self) -> Optional[torch.Tensor]:
        return getattr(self.linear, "bias", None)

    @bias.setter
    def bias(self, value: Optional[torch.Tensor]) -> None:
        self.linear.bias = value

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.ndim == 3 and x.shape[1] < self.pad_m:
            batch_size, seq_len, hidden_dim = x.shape
            pad = torch.zeros((batch_size, self.pad_m - seq_len, hidden_dim), dtype=x.dtype, device=x.device)
            out = self.linear(torch.cat([x, pad], dim=1))
            return out[:, :seq_len, :]
        return self.linear(x)


def _install_exact_small_proj_hooks(linear_attn: Any, *, pad_m: int = _EXACT_SMALL_PROJ_PAD_M) -> None:
    """dflash_mlx/runtime.py:277-285."""
    for attr_name in ("in_proj_b", "in_proj_a"):
        proj = getattr(linear_attn, attr_name, None)
        if proj is None or getattr(proj, "_dflash_exact_small_proj_wrapped", False):
            continue
        setattr(linear_attn, attr_name, _ExactSmallProjPad(proj, pad_m=pad_m))


class RMSNormGated(nn.Module):
    """silu(gate) * rms_norm(x, weight) - the output norm of the layer."""

    def __init__(self, hidden_size: int, eps: float = 1e-6, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.eps = float(eps)
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype), requires_grad=False)

    def forward(self, hidden_states: torch.Tensor, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        if gate is None:
            return rms_norm_ops(hidden_states, self.weight, self.eps)
        return gated_norm(hidden_states, gate, self.weight, self.eps)


class _DepthwiseConv1d(nn.Module):
    """Holder of the depthwise taps in the layout of an mlx conv1d weight, [C, K, 1]."""

    def __init__(self, channels: int, kernel_size: int, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros((channels, kernel_size, 1), dtype=dtype), requires_grad=False)


def _gdn_call(self, inputs: torch.Tensor, mask: Optional[torch.Tensor], cache: Optional[Any],
              record: bool) -> torch.Tensor:
    """The body shared by the plain and the speculative call (dflash_mlx/runtime.py:359-453)."""
    B, S, _ = inputs.shape
    # one launch for those of the four that fuse_shared_input_linears joined
    qkv, z, b, a = shared_input_outputs(self, ("in_proj_qkv", "in_proj_z", "in_proj_b", "in_proj_a"), inputs)
    z = z.reshape(B, S, self.num_v_heads, self.head_v_dim)

    conv_state = cache[0] if cache is not None else None
    conv_next, q, k, v, g, beta = gdn_prepare(
        qkv, conv_state, self.conv1d.weight, a, b, self.A_log, self.dt_bias, mask,
        Hk=self.num_k_heads, Hv=self.num_v_heads, Dk=self.head_k_dim, Dv=self.head_v_dim)
    if cache is not None:
        cache[0] = conv_next

    state = cache[1] if cache is not None else None
    if state is None:
        state = torch.zeros((B, self.num_v_heads, self.head_v_dim, self.head_k_dim), dtype=q.dtype, device=q.device)
    # the layer's output norm rides on the recurrence's launch where the kernel takes it
    norm = self.norm
    fused = (isinstance(norm, RMSNormGated) and os.environ.get("DFLASH_GDN_FUSED_NORM", "1") != "0" and
             fused_output_norm_applies(q, v, state, z, norm.weight))
    out, state, innovation_tape = gated_delta_kernel_with_tape(
        q, k, v, g, beta, state, mask, output_norm=(z, norm.weight, norm.eps) if fused else None)
    if record:
        if mask is not None:
            qkv = torch.where(mask.to(torch.bool)[..., None], qkv, torch.zeros_like(qkv))
        cache.record_tape(tape=innovation_tape, k=k, g=g, qkv=qkv)
    if cache is not None:
        cache[1] = state
    if not fused:
        out = self.norm(out, z)
    return self.out_proj(out.reshape(B, S, -1))


class GatedDeltaNet(nn.Module):
    """A GatedDeltaNet mixer with the attribute names the reference's hooks rely on."""

    def __init__(self, hidden_size: int, *, num_k_heads: int, num_v_heads: int, head_k_dim: int, head_v_dim: int,
                 conv_kernel_size: int = 4, in_proj_qkv: nn.Module, in_proj_z: nn.Module, in_proj_b: nn.Module,
                 in_proj_a: nn.Module, out_proj: nn.Module, dtype: torch.dtype = torch.bfloat16, eps: float = 1e-6):
        super().__init__()
        self.hidden_size = hidden_size
        self.num_k_heads, self.num_v_heads = num_k_heads, num_v_heads
        self.head_k_dim, self.head_v_dim = head_k_dim, head_v_dim
        self.key_dim = num_k_heads * head_k_dim
        self.value_dim = num_v_heads * head_v_dim
        self.conv_kernel_size = conv_kernel_size
        self.conv_dim = 2 * self.key_dim + self.value_dim
        self.in_proj_qkv, self.in_proj_z = in_proj_qkv, in_proj_z
        self.in_proj_b, self.in_proj_a = in_proj_b, in_proj_a
        self.conv1d = _DepthwiseConv1d(self.conv_dim, conv_kernel_size, dtype)
        self.A_log = nn.Parameter(torch.zeros(num_v_heads, dtype=dtype), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.ones(num_v_heads, dtype=dtype), requires_grad=False)
        self.norm = RMSNormGated(head_v_dim, eps, dtype)
        self.out_proj = out_proj

    def forward(self, inputs: torch.Tensor, mask: Optional[torch.Tensor] = None, cache: Optional[Any] = None):
        return _gdn_call(self, inputs, mask, cache, record=False)


def _install_speculative_linear_cache_hook(linear_attn: Any) -> None:
    """dflash_mlx/runtime.py:344-455: patch the layer class once so that a call with an armed
    ``RecurrentRollbackCache`` records the tape; every other call goes to the original."""
    cls = type(linear_attn)
    if getattr(cls, "_dflash_speculative_call_installed", False):
        return
    original_call = cls.forward

    def speculative_call(self, inputs: torch.Tensor, mask: Optional[torch.Tensor] = None,
                         cache: Optional[Any] = None) -> torch.Tensor:
        if not isinstance(cache, RecurrentRollbackCache) or not getattr(cache, "_armed", False):
            return original_call(self, inputs, mask=mask, cache=cache)
        return _gdn_call(self, inputs, mask, cache, record=True)

    cls.forward = speculative_call
    cls._dflash_speculative_call_installed = True
    cls._dflash_original_call = original_call
