"""Randomly drawn configurations of the recurrent kernels and of the 16-query attention against
the array-op forms of the same recurrences (the reference's own fallbacks,
dflash_mlx/kernels.py:131-173 and 328-358) evaluated in fp64 on the device: head counts, block
lengths, dtypes of every operand, per-element gates, masks and ragged key counts all vary.

Tolerances: states and tapes are fp32 results of at most 16 steps (rel-L2 <= 2e-5; the replay's
folded sweep <= 2e-6); outputs carry one rounding to the 16-bit type (<= 8e-3)."""
import pytest
import torch

from dflash_mlx_amd import kernels as K
from dflash_mlx_amd.workloads import seed_for

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()


@pytest.fixture()
def draws():
    gen = torch.Generator(device=DEV).manual_seed(seed_for(2, 501))
    host = torch.Generator().manual_seed(seed_for(2, 502))
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=host))
    normal = lambda *shape, scale=1.0: torch.randn(shape, generator=gen, device=DEV) * scale
    return gen, pick, normal


def test_recurrences(native_lib, draws):
    gen, pick, normal = draws
    for i in range(60):
        B, T, Hk = pick(1, 5), pick(1, 16), pick(1, 4)
        Hv, D = Hk * pick(1, 4), (128 if i % 5 else 64)
        tape_dt, k_dt, g_dt, dt = DTYPES[pick(0, 2)], DTYPES[pick(0, 2)], DTYPES[pick(0, 2)], DTYPES[pick(0, 1)]
        per_dk = bool(pick(0, 1))
        what = f"case {i}: B={B} T={T} Hk={Hk} Hv={Hv} D={D} {tape_dt} {k_dt} {g_dt} {dt} per_dk={per_dk}"
        tape = normal(B, T, Hv, D, scale=0.05).to(tape_dt)
        k = torch.nn.functional.normalize(normal(B, T, Hk, D), dim=-1).to(k_dt)
        g = torch.exp(-torch.nn.functional.softplus(normal(B, T, Hv, D) if per_dk else normal(B, T, Hv))).to(g_dt)
        state = normal(B, Hv, D, D, scale=0.1)
        mask = (torch.rand((B, T), generator=gen, device=DEV) > 0.3) if pick(0, 1) else None

        got = K.tape_replay_kernel(tape, k, g, state, mask)
        want = K._tape_replay_ops(tape.double(), k.double(), g.double(), state.double(), mask)
        assert _rel(got, want) <= 2e-6, "replay, " + what

        q = torch.nn.functional.normalize(normal(B, T, Hk, D), dim=-1).to(dt)
        kf = k.to(dt)
        v, beta, gf = normal(B, T, Hv, D).to(dt), torch.sigmoid(normal(B, T, Hv)).to(dt), g.float()
        y, state_out, recorded = K.gated_delta_kernel_with_tape(q, kf, v, gf, beta, state, mask)
        y64, state64, tape64 = K._gated_delta_ops_with_tape(q.double(), kf.double(), v.double(), gf.double(),
                                                            beta.double(), state.double(), mask)
        assert _rel(state_out, state64) <= 2e-5 and _rel(recorded, tape64) <= 2e-5, "forward, " + what
        assert _rel(y, y64) <= 8e-3, "forward output, " + what


def test_attention(native_lib, draws):
    gen, pick, normal = draws
    for i in range(60):
        Hk, D, B = pick(1, 4), (128 if i % 3 else 256), pick(1, 2)
        Hq, N = Hk * pick(1, 8), (pick(16, 6000) if i % 4 else pick(16, 600))
        dt, kind = DTYPES[pick(0, 1)], pick(0, 2)
        what = f"case {i}: B={B} Hq={Hq} Hk={Hk} N={N} D={D} {dt} mask kind {kind}"
        held = N + pick(0, 64)   # the cache buffer is longer than the keys in use
        cache_k, cache_v = normal(B, Hk, held, D).to(dt), normal(B, Hk, held, D).to(dt)
        q = normal(B, Hq, 16, D).to(dt)
        allowed = torch.ones((16, N), dtype=torch.bool, device=DEV).tril(N - 16).expand(B, 1, 16, N)
        mask, added = None, None
        if kind == 1:
            allowed = allowed & (torch.rand((B, 1, 16, N), generator=gen, device=DEV) > 0.2)
            allowed[..., 0] = True
            mask = allowed
        elif kind == 2:
            added = normal(B, Hq, 16, N, scale=0.5).to(dt)
            mask = added
        out = K.batched_sdpa_2pass_exact(q, cache_k[:, :, :N], cache_v[:, :, :N], D ** -0.5, mask=mask)
        assert out is not None, what
        keys = cache_k[:, :, :N].double().repeat_interleave(Hq // Hk, 1)
        values = cache_v[:, :, :N].double().repeat_interleave(Hq // Hk, 1)
        scores = (q.double() @ keys.transpose(-1, -2)) * D ** -0.5
        if added is not None:
            scores = scores + added.double()
        want = torch.softmax(scores.masked_fill(~allowed, float("-inf")), -1) @ values
        assert torch.isfinite(out.float()).all() and _rel(out, want) <= 6e-3, what
