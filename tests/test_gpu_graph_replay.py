"""The kernels of the verify step recorded into a HIP graph: every replay, with the inputs
rewritten and ordinary eager work in between, reproduces what the same calls give eagerly.

A serving loop replays the verify step rather than launching its kernels one by one, so the
kernels must not depend on host state from the time of capture: the split-K arrival counters
return to zero by themselves, accepted lengths are read from device memory, and the attention
workspace is owned by the stream."""
import pytest
import torch

from dflash_mlx_amd import kernels as K
from dflash_mlx_amd import verify_qmm as VQ
from dflash_mlx_amd.gdn_layer import gated_norm, gdn_prepare
from dflash_mlx_amd.graph_replay import record
from dflash_mlx_amd.workloads import make_qmm_case, make_replay_case, seed_for

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _capture(fn):
    return record(fn)


def _replays_match(graph, captured, eager_fn, refill, rounds=3):
    for r in range(rounds):
        refill(r)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = eager_fn()          # the program's own eager work between replays
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(captured, eager)):
            assert torch.equal(a, b), f"replay {r}: output {i} differs from the eager result"


def test_qmm_chain_replays(verify_env, native_lib):
    """Three dependent-size calls in a row (streaming kernel with split K, scale/bias chunks of 4
    and of 2, and the tile kernel for a group size the streaming kernel does not take)."""
    verify_env.setenv("DFLASH_QMM_KERNEL", "auto")
    cases = [make_qmm_case(2048, 1536, seed_for(0, 81)).to(DEV), make_qmm_case(1536, 4096 + 64, seed_for(0, 82)).to(DEV),
             make_qmm_case(1024, 512, seed_for(0, 83), group_size=32).to(DEV)]

    def run():
        return [VQ.verify_matmul(c.x, c.w, c.scales, c.biases, group_size=c.group_size, bits=4) for c in cases]

    graph, captured = _capture(run)
    gen = torch.Generator(device=DEV).manual_seed(5)

    def refill(r):
        for c in cases:
            c.x.copy_(torch.randn(c.x.shape, generator=gen, device=DEV).to(c.x.dtype))

    _replays_match(graph, captured, run, refill)


def test_chained_launches_replay(verify_env, native_lib):
    """Chained launches in a graph: the per-problem split, the joint split on packed weights and a
    gate/up problem with the activation epilogue, one after the other on one workspace; every
    replay with new inputs gives what the same launches give eagerly."""
    verify_env.setenv("DFLASH_QMM_KERNEL", "stream")
    cases = [make_qmm_case(2048, 1536, seed_for(0, 91)).to(DEV), make_qmm_case(1024, 4096, seed_for(0, 92)).to(DEV),
             make_qmm_case(3072, 512, seed_for(0, 93)).to(DEV)]
    gate, up = make_qmm_case(2048, 1024, seed_for(0, 94)).to(DEV), make_qmm_case(2048, 1024, seed_for(0, 95)).to(DEV)
    gu = (torch.cat([gate.w, up.w]), torch.cat([gate.scales, up.scales]), torch.cat([gate.biases, up.biases]))
    plain = VQ.QmmChain([VQ.ChainProblem(c.x, c.w, c.scales, c.biases) for c in cases])
    joint = VQ.QmmChain([VQ.ChainProblem(c.x, VQ.pack_weights(c.w, c.scales, c.biases)) for c in cases], joint_split=True)
    hidden = VQ.QmmChain([VQ.ChainProblem(gate.x, VQ.pack_weights(*gu, gate_up=True), epilogue="silu_mul")])

    def run():
        return [y.clone() for chain in (plain, joint, hidden) for y in chain()]

    graph, captured = _capture(run)
    gen = torch.Generator(device=DEV).manual_seed(6)

    def refill(r):
        for c in cases + [gate]:
            c.x.copy_(torch.randn(c.x.shape, generator=gen, device=DEV).to(c.x.dtype))

    _replays_match(graph, captured, run, refill)
    VQ.raise_on_device_errors(torch.device(DEV))


def test_rollback_replays_with_device_step_counts(native_lib):
    """Tape replay with the accepted length in device memory: one recorded launch serves every
    acceptance length."""
    case = make_replay_case(layers=3, Hk=4, Hv=8, seed=91, steps=16).to(DEV)
    L, B = case.state.shape[:2]
    tape, k, g = (t.reshape(L * B, *t.shape[2:]).contiguous() for t in (case.tape, case.k, case.g))
    state_in = case.state.reshape(L * B, *case.state.shape[2:]).contiguous()
    state_out = torch.empty_like(state_in)
    steps = torch.zeros(L * B, dtype=torch.int32, device=DEV)

    def run():
        K.replay_launch(tape, k, g, state_in, state_out, steps=steps, T_alloc=16)
        return [state_out]

    graph, captured = _capture(run)
    for r, lens in enumerate(([16, 0, 5], [1, 16, 9], [0, 0, 0], [7, 7, 7])):
        steps.copy_(torch.tensor(lens, dtype=torch.int32))
        graph.replay()
        torch.cuda.synchronize()
        got = captured[0].clone()
        for slot, n in enumerate(lens):
            one = torch.empty_like(state_in[slot:slot + 1])
            K.replay_launch(tape[slot:slot + 1], k[slot:slot + 1], g[slot:slot + 1], state_in[slot:slot + 1], one,
                            steps=n, T_alloc=16)
            torch.cuda.synchronize()
            assert torch.equal(got[slot:slot + 1], one), f"replay {r}, slot {slot}, {n} steps"


def test_gdn_layer_kernels_replay(native_lib):
    """Fused glue, forward with tape and gated norm of one GatedDeltaNet layer, chained."""
    B, S, Hk, Hv, D, Kc = 1, 16, 4, 8, 128, 4
    C = 2 * Hk * D + Hv * D
    gen = torch.Generator(device=DEV).manual_seed(17)
    rnd = lambda *shape, scale=1.0: (torch.randn(shape, generator=gen, device=DEV) * scale)
    qkv = rnd(B, S, C).to(torch.bfloat16)
    conv_state = rnd(B, Kc - 1, C).to(torch.bfloat16)
    conv_w = rnd(C, Kc, scale=0.5).to(torch.bfloat16)
    a, b = rnd(B, S, Hv).to(torch.bfloat16), rnd(B, S, Hv).to(torch.bfloat16)
    A_log, dt_bias = rnd(Hv).float(), rnd(Hv).float()
    z = rnd(B, S, Hv, D).to(torch.bfloat16)
    norm_w = (1 + rnd(D, scale=0.1)).to(torch.bfloat16)
    state = rnd(B, Hv, D, D, scale=0.1).float()

    def run():
        conv_next, q, k, v, g, beta = gdn_prepare(qkv, conv_state, conv_w, a, b, A_log, dt_bias, None,
                                                  Hk=Hk, Hv=Hv, Dk=D, Dv=D)
        y, state_out, tape = K.gated_delta_kernel_with_tape(q, k, v, g, beta, state)
        return [gated_norm(y, z, norm_w), state_out, tape, conv_next]

    graph, captured = _capture(run)

    def refill(r):
        qkv.copy_(rnd(B, S, C).to(torch.bfloat16))
        state.copy_(rnd(B, Hv, D, D, scale=0.1))
        a.copy_(rnd(B, S, Hv).to(torch.bfloat16))

    _replays_match(graph, captured, run, refill)


def test_attention_kernel_replays(native_lib):
    """16 queries over 1500 cached keys, read in place from a larger cache buffer."""
    Hq, Hk, D, N = 8, 2, 128, 1500
    gen = torch.Generator(device=DEV).manual_seed(23)
    cache_k = torch.randn((1, Hk, 2048, D), generator=gen, device=DEV).to(torch.bfloat16)
    cache_v = torch.randn((1, Hk, 2048, D), generator=gen, device=DEV).to(torch.bfloat16)
    q = torch.randn((1, Hq, 16, D), generator=gen, device=DEV).to(torch.bfloat16)
    mask = torch.ones((16, N), dtype=torch.bool, device=DEV).tril(N - 16)

    def run():
        out = K.batched_sdpa_2pass_exact(q, cache_k[:, :, :N], cache_v[:, :, :N], D ** -0.5, mask=mask)
        assert out is not None
        return [out]

    graph, captured = _capture(run)

    def refill(r):
        q.copy_(torch.randn(q.shape, generator=gen, device=DEV).to(torch.bfloat16))
        cache_k[:, :, N - 16:N].copy_(torch.randn((1, Hk, 16, D), generator=gen, device=DEV).to(torch.bfloat16))

    _replays_match(graph, captured, run, refill)
