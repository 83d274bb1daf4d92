"""Seeded synthetic inputs of the benchmark configurations.

Value distributions (all drawn from ``torch.Generator`` streams seeded with
``0xDF1A + 1000*config + layer``):

* qmm: x bf16 ~ N(0,1); packed words uniform over all 32-bit patterns (= 8
  independent codes uniform in 0..15); scales = bf16(|N(0, 0.02)| + 1e-4);
  biases = bf16(-8 * scale).
* replay: state fp32 ~ N(0, 0.1) laid out [.., Dv, Dk]; k bf16 = N(0,1) L2-normalised
  over Dk; delta bf16 ~ N(0, 0.05); g fp32 = exp(-softplus(N(0,1))).

Generating on the CPU (default) gives bit-identical tensors on every machine, so a
host oracle and the device kernel can be fed the same data.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple, Union

import torch

BASE_SEED = 0xDF1A
GROUP_SIZE = 64

# (name, K, N) per layer
STACK_9B: List[Tuple[str, int, int]] = [
    ("qkv_proj", 4096, 6144), ("o_proj", 4096, 4096),
    ("gate_proj", 4096, 12288), ("up_proj", 4096, 12288), ("down_proj", 12288, 4096),
]
STACK_27B: List[Tuple[str, int, int]] = [
    ("qkv_proj", 5120, 7168), ("o_proj", 5120, 5120),
    ("gate_proj", 5120, 17408), ("up_proj", 5120, 17408), ("down_proj", 17408, 5120),
]
STACKS: Dict[str, Tuple[List[Tuple[str, int, int]], int, int]] = {
    # name: (linears per layer, layers, config index in BASELINE.json)
    "9b": (STACK_9B, 32, 1),
    "27b": (STACK_27B, 64, 3),
}


def seed_for(config: int, layer: int = 0) -> int:
    return BASE_SEED + 1000 * config + layer


def _gen(seed: int, device: Union[str, torch.device]) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


@dataclass
class QmmCase:
    x: torch.Tensor        # [16, K]
    w: torch.Tensor        # [N, K/8] int32 words
    scales: torch.Tensor   # [N, K/gs]
    biases: torch.Tensor   # [N, K/gs]
    group_size: int

    @property
    def K(self) -> int:
        return int(self.x.shape[-1])

    @property
    def N(self) -> int:
        return int(self.w.shape[0])

    def to(self, device) -> "QmmCase":
        return QmmCase(self.x.to(device), self.w.to(device), self.scales.to(device),
                       self.biases.to(device), self.group_size)


def qmm_algorithmic_bytes(K: int, N: int, group_size: int = GROUP_SIZE, M: int = 16) -> Tuple[int, int]:
    """(weight bytes, total bytes) one call has to move: packed codes + scales + biases
    once, x once, y once."""
    weights = N * K // 2 + 2 * 2 * N * (K // group_size)
    return weights, weights + M * K * 2 + M * N * 2


def make_qmm_case(K: int, N: int, seed: int, *, group_size: int = GROUP_SIZE,
                  dtype: torch.dtype = torch.bfloat16, device: Union[str, torch.device] = "cpu",
                  M: int = 16) -> QmmCase:
    g = _gen(seed, device)
    x = torch.randn((M, K), generator=g, device=device, dtype=torch.float32).to(dtype)
    w = torch.randint(-2 ** 31, 2 ** 31, (N, K // 8), generator=g, device=device, dtype=torch.int32)
    s = (torch.randn((N, K // group_size), generator=g, device=device, dtype=torch.float32) * 0.02).abs() + 1e-4
    s = s.to(dtype)
    b = (-8.0 * s.to(torch.float32)).to(dtype)
    return QmmCase(x, w, s, b, group_size)


def stack_linears(stack: str) -> Tuple[List[Tuple[str, int, int]], int, int]:
    return STACKS[stack]


def stack_bytes(stack: str) -> Tuple[int, int]:
    """(weight bytes, total algorithmic bytes) of one pass over the whole stack."""
    linears, layers, _ = STACKS[stack]
    wb = tb = 0
    for _, K, N in linears:
        w_, t_ = qmm_algorithmic_bytes(K, N)
        wb += w_
        tb += t_
    return wb * layers, tb * layers


@dataclass
class ReplayCase:
    state: torch.Tensor   # [L, B, Hv, Dv, Dk] fp32
    tape: torch.Tensor    # [L, B, T, Hv, Dv]
    k: torch.Tensor       # [L, B, T, Hk, Dk]
    g: torch.Tensor       # [L, B, T, Hv] or [L, B, T, Hv, Dk]
    steps: torch.Tensor   # [L*B] int32

    def to(self, device) -> "ReplayCase":
        return ReplayCase(*(t.to(device) for t in (self.state, self.tape, self.k, self.g, self.steps)))


def replay_algorithmic_bytes(Dk: int, Dv: int, steps: int, *, tape_bytes: int = 2, k_bytes: int = 2,
                             g_bytes: int = 4, state_bytes: int = 4) -> int:
    """Bytes one (slot, head) has to move: state read + written, and per applied step
    one delta row, one k row and one gate."""
    return 2 * Dk * Dv * state_bytes + steps * (Dv * tape_bytes + Dk * k_bytes + g_bytes)


def make_replay_case(layers: int = 48, *, batch: int = 1, T: int = 16, Hk: int = 32, Hv: int = 32,
                     Dk: int = 128, Dv: int = 128, seed: Optional[int] = None,
                     steps: Optional[int] = None, g_per_dk: bool = False,
                     tape_dtype: torch.dtype = torch.bfloat16,
                     device: Union[str, torch.device] = "cpu") -> ReplayCase:
    """BASELINE config[2] by default; ``steps`` None draws one accepted count in 0..T
    for the cycle (the same for all layers, as in the engine)."""
    g = _gen(seed_for(2) if seed is None else seed, device)
    L, B = layers, batch
    state = torch.randn((L, B, Hv, Dv, Dk), generator=g, device=device, dtype=torch.float32) * 0.1
    k = torch.randn((L, B, T, Hk, Dk), generator=g, device=device, dtype=torch.float32)
    k = (k / k.norm(dim=-1, keepdim=True)).to(torch.bfloat16)
    tape = (torch.randn((L, B, T, Hv, Dv), generator=g, device=device, dtype=torch.float32) * 0.05).to(tape_dtype)
    gshape = (L, B, T, Hv, Dk) if g_per_dk else (L, B, T, Hv)
    gate = torch.exp(-torch.nn.functional.softplus(
        torch.randn(gshape, generator=g, device=device, dtype=torch.float32)))
    if steps is None:
        steps = int(torch.randint(0, T + 1, (1,), generator=g, device=device).item())
    st = torch.full((L * B,), int(steps), dtype=torch.int32, device=device)
    return ReplayCase(state, tape, k, gate, st)


@dataclass
class MoeCase:
    x: torch.Tensor           # [P, K] rows already gathered per (token, expert) pair
    expert_ids: torch.Tensor  # [P] int32
    w: torch.Tensor           # [E, N, K/8] int32 words
    scales: torch.Tensor      # [E, N, K/gs]
    biases: torch.Tensor      # [E, N, K/gs]
    group_size: int

    def to(self, device) -> "MoeCase":
        return MoeCase(self.x.to(device), self.expert_ids.to(device), self.w.to(device),
                       self.scales.to(device), self.biases.to(device), self.group_size)


def make_moe_case(K: int, N: int, seed: int, *, experts: int = 256, tokens: int = 16, top_k: int = 8,
                  group_size: int = GROUP_SIZE, device: Union[str, torch.device] = "cpu") -> MoeCase:
    """BASELINE config[4] routing: softmax over router logits ~ N(0,1), top-k experts per
    token; one row per (token, expert) pair, token-major."""
    g = _gen(seed, device)
    logits = torch.randn((tokens, experts), generator=g, device=device, dtype=torch.float32)
    ids = torch.topk(torch.softmax(logits, dim=-1), top_k, dim=-1).indices.to(torch.int32).reshape(-1)
    x = torch.randn((tokens * top_k, K), generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    w = torch.randint(-2 ** 31, 2 ** 31, (experts, N, K // 8), generator=g, device=device, dtype=torch.int32)
    s = ((torch.randn((experts, N, K // group_size), generator=g, device=device, dtype=torch.float32) * 0.02).abs()
         + 1e-4).to(torch.bfloat16)
    b = (-8.0 * s.to(torch.float32)).to(torch.bfloat16)
    return MoeCase(x, ids, w, s, b, group_size)
