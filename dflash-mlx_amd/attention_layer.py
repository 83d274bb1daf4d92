"""Full-attention layer glue of the verify step (host side).

Mirror of dflash_mlx/runtime.py:288-316 and :456-652: the attention call that, for a verify
block of 16 tokens over a long cached prefix, computes every query's softmax over exactly its
own keys - through ``batched_sdpa_2pass_exact`` (the gfx950 kernel behind ``dflash_sdpa_q16``)
when it applies, else query by query - so that a token's result does not depend on how many
tokens were verified with it.  ``GatedAttention`` is a stand-in with the attribute names of the
mlx-lm layer the reference patches (q_proj with an output gate, q_norm / k_norm, rope,
k_proj, v_proj, o_proj, scale, num_attention_heads, num_key_value_heads).
"""
from __future__ import annotations

from typing import Any, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .gdn_layer import rms_norm_ops
from .kernels import batched_sdpa_2pass_exact
from .verify_linear import shared_input_outputs

_HYBRID_SDPA_EXACT_KV_THRESHOLD = 1024


def _attention_num_heads(attn: Any) -> int:
    for attr in ("num_attention_heads", "n_heads"):
        value = getattr(attn, attr, None)
        if value is not None:
            return int(value)
    raise AttributeError(f"{type(attn).__name__} missing attention head count attribute")


def _attention_num_kv_heads(attn: Any) -> int:
    for attr in ("num_key_value_heads", "n_kv_heads"):
        value = getattr(attn, attr, None)
        if value is not None:
            return int(value)
    raise AttributeError(f"{type(attn).__name__} missing KV head count attribute")


def _attention_has_gated_q_proj(attn: Any) -> bool:
    """dflash_mlx/runtime.py:304-316: q_proj produces queries and a gate of the same width."""
    q_proj_weight = getattr(getattr(attn, "q_proj", None), "weight", None)
    q_norm_weight = getattr(getattr(attn, "q_norm", None), "weight", None)
    if q_proj_weight is None or q_norm_weight is None:
        return False
    try:
        num_attention_heads = _attention_num_heads(attn)
    except AttributeError:
        return False
    return int(q_proj_weight.shape[0]) == 2 * num_attention_heads * int(q_norm_weight.shape[0])


def scaled_dot_product_attention(queries: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, *,
                                 scale: float, mask: Any = None) -> torch.Tensor:
    """The general attention the reference falls back to: ``mask`` None, "causal" (queries are
    the last positions of the keys), a bool array (True = attend) or an additive array."""
    q_len, n_kv = int(queries.shape[2]), int(keys.shape[2])
    bias = None
    if isinstance(mask, str):
        if mask != "causal":
            raise ValueError(f"unknown mask {mask!r}")
        pos = torch.arange(n_kv - q_len, n_kv, device=queries.device)[:, None]
        bias = torch.arange(n_kv, device=queries.device)[None, :] <= pos
    elif mask is not None:
        bias = mask if mask.dtype == torch.bool else mask.to(queries.dtype)
    return F.scaled_dot_product_attention(queries, keys, values, attn_mask=bias, scale=scale,
                                          enable_gqa=keys.shape[1] != queries.shape[1])


def _split_sdpa_mask(mask: Optional[Any], *, query_start: int, query_end: int, key_end: int) -> Optional[Any]:
    if mask is None or (isinstance(mask, str) and mask == "causal"):
        return mask
    return mask[..., query_start:query_end, :key_end]


def _split_sdpa_output(*, queries: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, scale: float,
                       mask: Optional[Any], chunk_size: int, cached_prefix_len: int) -> torch.Tensor:
    """dflash_mlx/runtime.py:468-502: chunks of queries, each over the keys up to its own end."""
    q_len = int(queries.shape[2])
    if q_len <= chunk_size:
        return scaled_dot_product_attention(queries, keys, values, scale=scale, mask=mask)
    outputs = []
    for start in range(0, q_len, chunk_size):
        end = min(start + chunk_size, q_len)
        key_end = cached_prefix_len + end
        chunk_mask = _split_sdpa_mask(mask, query_start=start, query_end=end, key_end=key_end)
        outputs.append(scaled_dot_product_attention(queries[:, :, start:end, :], keys[:, :, :key_end, :],
                                                    values[:, :, :key_end, :], scale=scale, mask=chunk_mask))
    return torch.cat(outputs, dim=2)


class HeadRMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-6, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim, dtype=dtype), requires_grad=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return rms_norm_ops(x, self.weight, self.eps)


class RotaryEmbedding(nn.Module):
    """Rotation of the first ``dims`` features of every head, position = offset + index."""

    def __init__(self, dims: int, base: float = 10000.0):
        super().__init__()
        self.dims, self.base = dims, base

    def forward(self, x: torch.Tensor, offset: int = 0) -> torch.Tensor:
        L, half = int(x.shape[-2]), self.dims // 2
        freqs = self.base ** (-torch.arange(half, device=x.device, dtype=torch.float32) / half)
        angles = torch.arange(offset, offset + L, device=x.device, dtype=torch.float32)[:, None] * freqs
        cos, sin = torch.cos(angles), torch.sin(angles)
        x1, x2 = x[..., :half].float(), x[..., half:self.dims].float()
        rotated = torch.cat([x1 * cos - x2 * sin, x1 * sin + x2 * cos, x[..., self.dims:].float()], dim=-1)
        return rotated.to(x.dtype)


class GatedAttention(nn.Module):
    """Attention with an output gate carried by q_proj; ``forward`` is the plain call."""

    def __init__(self, *, num_attention_heads: int, num_key_value_heads: int, head_dim: int, q_proj: nn.Module,
                 k_proj: nn.Module, v_proj: nn.Module, o_proj: nn.Module, rope_dims: Optional[int] = None,
                 dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.num_attention_heads, self.num_key_value_heads = num_attention_heads, num_key_value_heads
        self.scale = head_dim ** -0.5
        self.q_proj, self.k_proj, self.v_proj, self.o_proj = q_proj, k_proj, v_proj, o_proj
        self.q_norm, self.k_norm = HeadRMSNorm(head_dim, dtype=dtype), HeadRMSNorm(head_dim, dtype=dtype)
        self.rope = RotaryEmbedding(rope_dims or head_dim)

    def forward(self, x: torch.Tensor, mask: Any = None, cache: Optional[Any] = None) -> torch.Tensor:
        queries, keys, values, gate, _ = _project(self, x, cache)
        output = scaled_dot_product_attention(queries, keys, values, scale=self.scale, mask=mask)
        return _finish(self, output, gate)


def _project(self, x: torch.Tensor, cache: Optional[Any]):
    """dflash_mlx/runtime.py:527-556: projections, head norms, rope, cache update."""
    B, L, _ = x.shape
    num_attention_heads = _attention_num_heads(self)
    num_key_value_heads = _attention_num_kv_heads(self)
    # one launch for the three where fuse_shared_input_linears joined them
    q_proj_output, keys, values = shared_input_outputs(self, ("q_proj", "k_proj", "v_proj"), x)
    queries, gate = torch.chunk(q_proj_output.reshape(B, L, num_attention_heads, -1), 2, dim=-1)
    gate = gate.reshape(B, L, -1)
    queries = self.q_norm(queries).transpose(1, 2)
    keys = self.k_norm(keys.reshape(B, L, num_key_value_heads, -1)).transpose(1, 2)
    values = values.reshape(B, L, num_key_value_heads, -1).transpose(1, 2)
    cached_prefix_len = int(getattr(cache, "offset", 0) or 0) if cache is not None else 0
    if cache is not None:
        queries = self.rope(queries, offset=cached_prefix_len)
        keys = self.rope(keys, offset=cached_prefix_len)
        keys, values = cache.update_and_fetch(keys, values)
    else:
        queries = self.rope(queries)
        keys = self.rope(keys)
    return queries, keys, values, gate, cached_prefix_len


def _finish(self, output: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    B, _, L, _ = output.shape
    output = output.transpose(1, 2).reshape(B, L, -1)
    return self.o_proj(output * torch.sigmoid(gate))


def _install_split_full_attention_hook(attn: Any) -> None:
    """dflash_mlx/runtime.py:508-616: patch the layer class once; layers with
    ``_dflash_split_sdpa_enabled`` take the exact path for long cached prefixes."""
    cls = type(attn)
    if getattr(cls, "_dflash_split_full_attention_installed", False):
        return
    original_call = cls.forward

    def split_call(self, x: torch.Tensor, mask: Any = None, cache: Optional[Any] = None) -> torch.Tensor:
        if not getattr(self, "_dflash_split_sdpa_enabled", False):
            return original_call(self, x, mask=mask, cache=cache)
        if not _attention_has_gated_q_proj(self):
            return original_call(self, x, mask=mask, cache=cache)
        queries, keys, values, gate, cached_prefix_len = _project(self, x, cache)
        exact_prefix_threshold = int(getattr(self, "_dflash_split_sdpa_exact_kv_threshold",
                                             _HYBRID_SDPA_EXACT_KV_THRESHOLD))
        is_array = isinstance(mask, torch.Tensor)
        should_split = (cache is not None and cached_prefix_len >= exact_prefix_threshold and
                        (mask is None or is_array or mask == "causal"))
        should_use_batched_2pass = (should_split and int(queries.shape[2]) == 16 and
                                    queries.dtype in (torch.bfloat16, torch.float16) and
                                    int(queries.shape[-1]) in (128, 256) and int(values.shape[-1]) in (128, 256))
        output = None
        if should_use_batched_2pass:
            output = batched_sdpa_2pass_exact(queries=queries, keys=keys, values=values, scale=self.scale,
                                              mask=mask if is_array else None)
        if output is None and should_split:
            output = _split_sdpa_output(queries=queries, keys=keys, values=values, scale=self.scale, mask=mask,
                                        chunk_size=1, cached_prefix_len=cached_prefix_len)
        if output is None:
            output = scaled_dot_product_attention(queries, keys, values, scale=self.scale, mask=mask)
        return _finish(self, output, gate)

    cls.forward = split_call
    cls._dflash_split_full_attention_installed = True
    cls._dflash_original_call = original_call


def configure_full_attention_split(layers, *, enabled: bool, chunk_size: int = 8) -> None:
    """dflash_mlx/runtime.py:633-652 for a list of decoder layers (``is_linear`` / ``self_attn``)."""
    for layer in layers:
        if not getattr(layer, "is_linear", False) and hasattr(layer, "self_attn"):
            _install_split_full_attention_hook(layer.self_attn)
            layer.self_attn._dflash_split_sdpa_enabled = enabled
            layer.self_attn._dflash_split_sdpa_chunk_size = int(chunk_size)
            layer.self_attn._dflash_split_sdpa_exact_kv_threshold = _HYBRID_SDPA_EXACT_KV_THRESHOLD
