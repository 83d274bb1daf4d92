"""The Python wrappers hand raw device pointers and a few integers to the kernels, which read
exactly what those integers say.  Operands whose extents do not follow from them, or that live on
another device, must be refused on the host, before anything is launched."""
import pytest
import torch

from dflash_mlx_amd import gdn_layer as G
from dflash_mlx_amd import kernels as K
from dflash_mlx_amd import verify_qmm as VQ
from dflash_mlx_amd.recurrent_rollback_cache import conv_state_rebuild
from dflash_mlx_amd.workloads import make_qmm_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_qmm_wrappers(native_lib, monkeypatch):
    monkeypatch.setenv("DFLASH_VERIFY_QMM", "1")
    c = make_qmm_case(1024, 256, 3, device=DEV)
    with pytest.raises(ValueError):
        VQ.verify_matmul(c.x, c.w, c.scales[:, :8], c.biases[:, :8])          # half the groups
    with pytest.raises(ValueError):
        VQ.verify_matmul(c.x, c.w, c.scales[:128], c.biases[:128])            # half the rows
    with pytest.raises(ValueError):
        VQ.verify_matmul(c.x, c.w, c.scales.cpu(), c.biases)                  # a host tensor among them
    with pytest.raises(ValueError):
        VQ.QmmChain([VQ.ChainProblem(c.x, c.w, c.scales[:128], c.biases[:128])])
    w3, s3, b3 = (t.unsqueeze(0).repeat(2, 1, 1) for t in (c.w, c.scales, c.biases))
    ids = torch.zeros(16, dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError):
        VQ.gather_qmm(c.x, w3, s3[:1], b3, ids)                               # scales of one expert only
    with pytest.raises(ValueError):
        VQ.gather_qmm(c.x, w3, s3, b3, ids.cpu())
    assert VQ.gather_qmm(c.x, w3, s3, b3, ids).shape == (16, 256)             # and the well-formed call runs


def _gdn_args(B=1, T=4, Hk=2, Hv=4, D=128):
    g = torch.Generator(device=DEV).manual_seed(5)
    q = torch.randn((B, T, Hk, D), generator=g, device=DEV).to(torch.bfloat16)
    k = torch.randn((B, T, Hk, D), generator=g, device=DEV).to(torch.bfloat16)
    v = torch.randn((B, T, Hv, D), generator=g, device=DEV).to(torch.bfloat16)
    gate = torch.rand((B, T, Hv), generator=g, device=DEV)
    beta = torch.rand((B, T, Hv), generator=g, device=DEV).to(torch.bfloat16)
    state = torch.randn((B, Hv, D, D), generator=g, device=DEV) * 0.1
    return q, k, v, gate, beta, state


def test_recurrence_wrappers(native_lib):
    q, k, v, gate, beta, state = _gdn_args()
    with pytest.raises(ValueError):
        K.gated_delta_kernel_with_tape(q, k, v, gate, beta[:, :2], state)         # fewer steps of beta
    with pytest.raises(ValueError):
        K.gated_delta_kernel_with_tape(q[:, :, :1], k, v, gate, beta, state)      # q of one head
    with pytest.raises(ValueError):
        K.gated_delta_kernel_with_tape(q, k, v, gate, beta, state[:, :2])         # state of two heads
    with pytest.raises(ValueError):
        K.gated_delta_kernel_with_tape(q, k, v, gate.cpu(), beta, state)
    y, s1, tape = K.gated_delta_kernel_with_tape(q, k, v, gate, beta, state)
    with pytest.raises(ValueError):
        K.tape_replay_kernel(tape, k, gate[:, :2], state)                          # gates of two steps
    with pytest.raises(ValueError):
        K.tape_replay_kernel(tape, k, gate, state[:, :2])
    with pytest.raises(ValueError):
        K.tape_replay_kernel(tape, k, gate, state, steps=2, mask=None) if False else K.tape_replay_kernel(
            tape[:, :, :2], k, gate, state, steps=2)                               # tape of two heads, rows read in place
    assert K.tape_replay_kernel(tape, k, gate, state).shape == state.shape

    # replay with the conv windows riding along: the kernel writes slots * keep rows of C elements
    B, T, C = int(tape.shape[0]), int(tape.shape[1]), 24
    qkv = torch.randn((B, T, C), device=DEV).to(torch.bfloat16)
    prev = torch.randn((B, 3, C), device=DEV).to(torch.bfloat16)
    out = torch.empty((B, 3, C), dtype=torch.bfloat16, device=DEV)
    s_in, s_out = state.contiguous(), torch.empty_like(state)

    def launch(conv):
        K.replay_launch(tape.contiguous(), k.contiguous(), gate.contiguous(), s_in, s_out, steps=2, T_alloc=T, slots=B, conv=conv)

    launch((prev, qkv, out))
    torch.cuda.synchronize()
    assert torch.equal(out, torch.cat([prev, qkv], dim=1)[:, 2:5])
    for bad in ((prev, qkv, out.float()),                                   # another element type
                (prev, qkv, torch.empty((B, 3, C - 8), dtype=torch.bfloat16, device=DEV)),   # narrower rows
                (prev, qkv, torch.empty((B + 1, 3, C), dtype=torch.bfloat16, device=DEV)),   # more slots than the launch
                (prev, torch.cat([qkv, qkv]), out),                         # qkv of more slots
                (prev, qkv, out.cpu()),                                     # host memory
                (prev[:, :2].contiguous(), qkv, out),                       # conv_prev of another window
                (torch.cat([prev, prev]), qkv, out),                        # conv_prev of more slots
                (prev.cpu(), qkv, out)):
        with pytest.raises(ValueError):
            launch(bad)


def test_attention_wrapper_declines(native_lib):
    q = torch.randn((1, 4, 16, 128), device=DEV).to(torch.bfloat16)
    kv = torch.randn((1, 2, 64, 128), device=DEV).to(torch.bfloat16)
    assert K.batched_sdpa_2pass_exact(q, kv.repeat(2, 1, 1, 1), kv.repeat(2, 1, 1, 1), 0.1) is None   # another batch size
    assert K.batched_sdpa_2pass_exact(q, kv, kv[..., :64], 0.1) is None                              # narrower values
    assert K.batched_sdpa_2pass_exact(q, kv, kv.cpu(), 0.1) is None
    host_mask = torch.zeros((16, 64), dtype=torch.bfloat16)                                          # a mask left on the host is moved
    with_mask, without = K.batched_sdpa_2pass_exact(q, kv, kv, 0.1, host_mask), K.batched_sdpa_2pass_exact(q, kv, kv, 0.1)
    assert torch.allclose(with_mask.float(), without.float(), atol=2e-2)   # (two kernels: equal up to rounding)


def test_glue_wrappers(native_lib):
    B, S, Hk, Hv, D = 1, 4, 2, 4, 128
    C = 2 * Hk * D + Hv * D
    g = torch.Generator(device=DEV).manual_seed(9)
    bf = lambda *shape: torch.randn(shape, generator=g, device=DEV).to(torch.bfloat16)  # noqa: E731
    qkv, conv_w, a, b = bf(B, S, C), bf(C, 4), bf(B, S, Hv), bf(B, S, Hv)
    A_log, dt_bias = bf(Hv), bf(Hv)
    args = dict(Hk=Hk, Hv=Hv, Dk=D, Dv=D)
    with pytest.raises(ValueError):
        G.gdn_prepare(qkv, None, conv_w, a[:, :2], b, A_log, dt_bias, **args)
    with pytest.raises(ValueError):
        G.gdn_prepare(qkv, bf(B, 2, C), conv_w, a, b, A_log, dt_bias, **args)      # a window of two rows for a kernel of four
    with pytest.raises(ValueError):
        G.gdn_prepare(qkv, None, conv_w, a, b, A_log[:2], dt_bias, **args)
    assert G.gdn_prepare(qkv, None, conv_w, a, b, A_log, dt_bias, **args)[1].shape == (B, S, Hk, D)
    with pytest.raises(ValueError):
        conv_state_rebuild(bf(B, 3, C // 2), qkv, 2, 3)                              # a narrower previous window
    with pytest.raises(ValueError):
        conv_state_rebuild(None, qkv, 2, 3, out=bf(B, 2, C))
    assert conv_state_rebuild(bf(B, 3, C), qkv, 2, 3).shape == (B, 3, C)
