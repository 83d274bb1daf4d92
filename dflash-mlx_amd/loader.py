"""MLX-format 4-bit checkpoints on torch: the on-disk side of the verify path.

An mlx-lm quantized checkpoint stores every quantized linear as a triple
``<path>.weight`` (uint32, 8 codes per word, low nibble first), ``<path>.scales`` and
``<path>.biases`` (``[N, K / group_size]``), plus ``<path>.bias`` where the layer has one, in
``*.safetensors`` shards, with ``"quantization": {"group_size": g, "bits": b}`` in
``config.json`` - the arrays ``VerifyQuantizedLinear.from_quantized`` shares with the module it
replaces (dflash_mlx/verify_linear.py:81-97).  This module reads such shards into
``QuantizedLinear`` modules, puts them into a torch module tree by path, and writes the same
format (for fixtures and tests; nothing here downloads anything).
"""
from __future__ import annotations

import glob
import json
import os
from typing import Dict, Iterable, Optional, Tuple

import torch
import torch.nn as nn

from .quantized import QuantizedLinear, as_words_i32

_TRIPLE = ("weight", "scales", "biases")


def read_quantization(config_path: str) -> Tuple[int, int]:
    """(group_size, bits) of a checkpoint's config.json; mlx-lm's defaults if it has none."""
    group_size, bits = 64, 4
    if os.path.isfile(config_path):
        with open(config_path) as f:
            q = json.load(f).get("quantization") or {}
        group_size, bits = int(q.get("group_size", group_size)), int(q.get("bits", bits))
    return group_size, bits


def _shards(path: str) -> Iterable[str]:
    if os.path.isdir(path):
        files = sorted(glob.glob(os.path.join(path, "*.safetensors")))
        if not files:
            raise FileNotFoundError(f"no *.safetensors under {path}")
        return files
    return [path]


def load_tensors(path: str, device: str = "cpu") -> Dict[str, torch.Tensor]:
    """All tensors of a safetensors file or of every shard in a directory."""
    from safetensors import safe_open

    out: Dict[str, torch.Tensor] = {}
    for shard in _shards(path):
        with safe_open(shard, framework="pt", device=device) as f:
            for key in f.keys():
                out[key] = f.get_tensor(key)
    return out


def quantized_linears(tensors: Dict[str, torch.Tensor], *, group_size: int = 64, bits: int = 4
                      ) -> Dict[str, QuantizedLinear]:
    """Every ``<path>.{weight,scales,biases}`` triple with packed 32-bit weights becomes a
    ``QuantizedLinear`` keyed by ``<path>``.  Shapes are checked against the format."""
    out: Dict[str, QuantizedLinear] = {}
    for key, scales in tensors.items():
        if not key.endswith(".scales"):
            continue
        path = key[: -len(".scales")]
        w, b = tensors.get(path + ".weight"), tensors.get(path + ".biases")
        if w is None or b is None:
            raise KeyError(f"{path}: scales without weight/biases")
        words = as_words_i32(w)
        n, k = int(words.shape[-2]), int(words.shape[-1]) * (32 // bits)
        if tuple(scales.shape[-2:]) != (n, k // group_size) or scales.shape != b.shape or k % group_size:
            raise ValueError(f"{path}: weight {tuple(w.shape)} does not fit scales {tuple(scales.shape)} "
                             f"at group_size {group_size}, bits {bits}")
        out[path] = QuantizedLinear(words, scales, b, tensors.get(path + ".bias"), group_size=group_size, bits=bits)
    return out


def load_quantized_linears(path: str, device: str = "cpu") -> Dict[str, QuantizedLinear]:
    """Read a checkpoint directory (shards + config.json) or a single file."""
    cfg = os.path.join(path if os.path.isdir(path) else os.path.dirname(path), "config.json")
    group_size, bits = read_quantization(cfg)
    return quantized_linears(load_tensors(path, device), group_size=group_size, bits=bits)


def assign_quantized_linears(model: nn.Module, linears: Dict[str, QuantizedLinear], *, prefix: str = "",
                             strict: bool = True) -> int:
    """Put each loaded linear at its path in ``model`` (``a.b.3.c`` walks attributes and
    indices); returns how many were placed.  ``strict``: unknown paths raise."""
    placed = 0
    for path, ql in linears.items():
        if prefix and not path.startswith(prefix):
            continue
        parts = path[len(prefix):].lstrip(".").split(".")
        parent = model
        try:
            for part in parts[:-1]:
                parent = parent[int(part)] if part.isdigit() else getattr(parent, part)
            if not hasattr(parent, parts[-1]) and not parts[-1].isdigit():
                raise AttributeError(parts[-1])
        except (AttributeError, IndexError, KeyError, TypeError):
            if strict:
                raise KeyError(f"{path}: no such module in the model")
            continue
        if parts[-1].isdigit():
            parent[int(parts[-1])] = ql
        else:
            setattr(parent, parts[-1], ql)
        placed += 1
    return placed


def save_quantized_linears(path: str, linears: Dict[str, QuantizedLinear],
                           extra: Optional[Dict[str, torch.Tensor]] = None) -> None:
    """Write ``model.safetensors`` and ``config.json`` in the layout above."""
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    tensors: Dict[str, torch.Tensor] = {}
    group_size = bits = None
    for name, ql in linears.items():
        u32 = getattr(torch, "uint32", None)
        w = ql.weight.detach().cpu().contiguous()
        tensors[name + ".weight"] = w.view(u32) if u32 is not None else w
        tensors[name + ".scales"] = ql.scales.detach().cpu().contiguous()
        tensors[name + ".biases"] = ql.biases.detach().cpu().contiguous()
        if ql.bias is not None:
            tensors[name + ".bias"] = ql.bias.detach().cpu().contiguous()
        if group_size not in (None, ql.group_size) or bits not in (None, ql.bits):
            raise ValueError("one checkpoint, one quantization")
        group_size, bits = ql.group_size, ql.bits
    for name, t in (extra or {}).items():
        tensors[name] = t.detach().cpu().contiguous()
    save_file(tensors, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump({"quantization": {"group_size": group_size or 64, "bits": bits or 4}}, f)
