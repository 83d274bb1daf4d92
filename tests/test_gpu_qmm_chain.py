"""dflash_qmm_m16_chain: several 16-row quantized matmuls in one launch.

Bars: every projection's output equals, bit for bit, what a launch of its own gives for the same
operands (streaming kernel: same unit ranges, same order of partial sums) - hence the oracle
parity of tests/test_gpu_qmm.py carries over, and is checked directly on one chain as well.  The
silu-mul epilogue equals silu(gate) * up computed operator by operator on separate launches'
outputs on at least 99.8 % of the elements (a launch of its own splits K elsewhere, which can
move the last bit of a factor), and meets the qmm bar (max-abs <= 2e-2 * row-inf, rel-L2 <= 5e-3)
against silu(g) * u of the exact fp64 products.  A projection that reads another's output gives what a separate launch gives on
that output, bit for bit.  The bounded wait is made to give up from the host: the launch still
ends and says which projection gave up."""
import ctypes

import numpy as np
import pytest
import torch

from dflash_mlx_amd.gdn_layer import silu_ops

import dflash_mlx_amd._native as nat
from dflash_mlx_amd import verify_qmm as VQ
from dflash_mlx_amd.workloads import make_qmm_case
from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def _env(verify_env):
    verify_env.setenv("DFLASH_QMM_KERNEL", "stream")


def _separate(x, c):
    return VQ.verify_matmul(x, c.w, c.scales, c.biases, group_size=64, bits=4)


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _exact(c_oracle, c, x=None):
    y32, _ = c_oracle.qmm_m16(_bits(c.x if x is None else x), c.w.cpu().numpy().view(np.uint32), _bits(c.scales), _bits(c.biases),
                              c.group_size, flavour=0)
    return y32


def _cases(shapes, seed, dtype=torch.bfloat16):
    return [make_qmm_case(K, N, seed + i, dtype=dtype).to(DEV) for i, (K, N) in enumerate(shapes)]


LAYER_27B = [(5120, 7168), (5120, 5120), (5120, 17408), (5120, 17408), (17408, 5120)]
LAYER_9B = [(4096, 6144), (4096, 4096), (4096, 12288), (4096, 12288), (12288, 4096)]


@pytest.mark.parametrize("shapes", [LAYER_27B, LAYER_9B, [(1024, 64), (2048, 32), (1024, 4096), (3072, 96)],
                                    [(5120, 5120)], [(1024, 32)] * 16],
                         ids=["27b-layer", "9b-layer", "small-and-ragged", "single", "sixteen-tiny"])
def test_independent_projections_equal_separate_launches(native_lib, shapes):
    cases = _cases(shapes, 700)
    print(f"chain of {len(shapes)}: {shapes[:5]}", flush=True)
    chain = VQ.QmmChain([VQ.ChainProblem(c.x, c.w, c.scales, c.biases) for c in cases])
    for rep in range(3):                      # the workspace is left ready for the next launch
        for y in chain.outputs:
            y.fill_(float("nan"))
        ys = chain()
        torch.cuda.synchronize()
        for i, (c, y) in enumerate(zip(cases, ys)):
            want = _separate(c.x, c)
            assert torch.equal(y.view(torch.int16), want.view(torch.int16)), (rep, i, shapes[i])
    assert chain.error_word() == 0


@pytest.mark.parametrize("shapes", [LAYER_27B, LAYER_9B, [(1024, 64), (2048, 32), (1024, 4096), (3072, 96)],
                                    [(5120, 5120)], [(1024, 32)] * 16, LAYER_27B * 3],
                         ids=["27b-layer", "9b-layer", "small-and-ragged", "single", "sixteen-tiny", "three-27b-layers"])
def test_joint_split_of_independent_projections(native_lib, c_oracle, shapes):
    """All units of all projections divided as one range: most row blocks are summed by one
    workgroup over all of K, so a sum is cut in other places than in a launch of its own.  Bars:
    the same bits from run to run; against the exact product the bar of the single launches
    (max-abs <= 2e-2 * row-inf, rel-L2 <= 5e-3, checked on the projections the oracle finishes
    quickly); against separate launches at most one step of the output type apart, and equal on at
    least 99 % of the elements; the workspace handed back zero-filled."""
    cases = _cases(shapes, 760)
    chain = VQ.QmmChain([VQ.ChainProblem(c.x, c.w, c.scales, c.biases) for c in cases], joint_split=True)
    runs = []
    for rep in range(3):
        for y in chain.outputs:
            y.fill_(float("nan"))
        ys = chain()
        torch.cuda.synchronize()
        runs.append([y.clone() for y in ys])
    assert chain.error_word() == 0
    assert int((chain._ws != 0).sum()) == 0
    for i, c in enumerate(cases):
        assert torch.equal(runs[0][i].view(torch.int16), runs[1][i].view(torch.int16)), (i, shapes[i])
        assert torch.equal(runs[0][i].view(torch.int16), runs[2][i].view(torch.int16)), (i, shapes[i])
        got = runs[0][i].float()
        want = _separate(c.x, c).float()
        assert torch.isfinite(got).all()
        # one bf16 step at that size; sums that cancel to next to nothing may differ by the fp32 rounding of their terms
        step = 2.0 ** -7 * torch.maximum(got.abs(), want.abs()) + 1e-5 * want.abs().max()
        assert bool(((got - want).abs() <= step).all()), (i, shapes[i])
        assert float((got == want).float().mean()) >= 0.99, (i, shapes[i])
    for i, c in enumerate(cases[:5]):
        if c.K * c.N > 5120 * 7168:
            continue
        exact = _exact(c_oracle, c).astype(np.float64)
        got = runs[0][i].float().cpu().numpy().astype(np.float64)
        assert np.all(np.abs(got - exact) <= 2e-2 * np.abs(exact).max(axis=1, keepdims=True)), (i, shapes[i])
        assert np.linalg.norm(got - exact) / np.linalg.norm(exact) <= 5e-3, (i, shapes[i])


def test_joint_split_with_the_activation_epilogue(native_lib):
    """Gate/up matrices with the silu-mul epilogue next to plain projections in a joint split:
    the hidden activation equals the per-projection split's on nearly every element."""
    K, I = 2048, 4096
    gate, up = make_qmm_case(K, I, 771).to(DEV), make_qmm_case(K, I, 772).to(DEV)
    other = make_qmm_case(2048, 1024, 773).to(DEV)
    w = torch.cat([gate.w, up.w]); sc = torch.cat([gate.scales, up.scales]); bi = torch.cat([gate.biases, up.biases])
    probs = lambda: [VQ.ChainProblem(other.x, other.w, other.scales, other.biases),
                     VQ.ChainProblem(gate.x, w, sc, bi, epilogue="silu_mul"),
                     VQ.ChainProblem(other.x, other.w, other.scales, other.biases)]
    joint = [y.clone() for y in VQ.QmmChain(probs(), joint_split=True)()]
    plain = [y.clone() for y in VQ.QmmChain(probs())()]
    torch.cuda.synchronize()
    for a, b in zip(joint, plain):
        assert torch.isfinite(a.float()).all()
        assert float((a == b).float().mean()) >= 0.99
        assert bool(((a.float() - b.float()).abs() <= 2.0 ** -6 * torch.maximum(a.float().abs(), b.float().abs())
                     + 1e-4 * b.float().abs().max()).all())


@pytest.mark.parametrize("joint", [False, True], ids=["per-problem", "joint-split"])
def test_packed_weights_in_a_chain(native_lib, joint):
    """A chain whose problems' weights are the packed images of `pack_weights`: bit for bit the
    chain on the row-major triples, in either split, and the packed single launches."""
    shapes = [(5120, 7168), (1024, 96), (5120, 5120), (2048, 4096), (17408, 5120)]
    cases = _cases(shapes, 790)
    packed = [VQ.pack_weights(c.w, c.scales, c.biases) for c in cases]
    rows = VQ.QmmChain([VQ.ChainProblem(c.x, c.w, c.scales, c.biases) for c in cases], joint_split=joint)
    want = [y.clone() for y in rows()]
    with pytest.raises(ValueError, match="for all projections"):
        VQ.QmmChain([VQ.ChainProblem(cases[0].x, packed[0]),
                     VQ.ChainProblem(cases[1].x, cases[1].w, cases[1].scales, cases[1].biases)])
    mixed = VQ.QmmChain([VQ.ChainProblem(c.x, pk) for c, pk in zip(cases, packed)], joint_split=joint)
    for rep in range(2):
        got = mixed()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), (rep, i, shapes[i])
    assert mixed.error_word() == 0 and int((mixed._ws != 0).sum()) == 0
    if not joint:
        for c, pk, y in zip(cases, packed, want):
            assert torch.equal(VQ.verify_matmul_packed(c.x, pk).view(torch.int16), y.view(torch.int16))
    with pytest.raises(ValueError, match="gate_up=True"):
        VQ.ChainProblem(cases[0].x, packed[0], epilogue="silu_mul")


def test_joint_split_on_packed_weights_with_fp16_activations(native_lib):
    """The remaining corner of the table: fp16 activations and scales, packed weights, joint split,
    outputs rebound between launches."""
    shapes = [(2048, 1024), (1024, 4096), (4096, 2048)]
    cases = _cases(shapes, 810, torch.float16)
    chain = VQ.QmmChain([VQ.ChainProblem(c.x, VQ.pack_weights(c.w, c.scales, c.biases)) for c in cases], joint_split=True)
    first = [y.clone() for y in chain()]
    elsewhere = torch.empty_like(first[1])
    chain.rebind(1, out=elsewhere)
    second = chain()
    torch.cuda.synchronize()
    assert chain.error_word() == 0
    assert torch.equal(elsewhere, first[1]) and torch.equal(second[0], first[0]) and torch.equal(second[2], first[2])
    for c, y in zip(cases, first):
        want = _separate(c.x, c).float()
        got = y.float()
        assert bool(((got - want).abs() <= 2.0 ** -10 * torch.maximum(got.abs(), want.abs()) + 1e-5 * want.abs().max()).all())
        # (fp16 keeps three more bits of the fp32 sum than bf16: another order of additions shows eight times as often)
        assert float((got == want).float().mean()) >= 0.95


@pytest.mark.parametrize("K,I", [(2048, 4096), (5120, 17408)])
def test_packed_gate_up_with_the_activation_epilogue(native_lib, K, I):
    """The gate/up matrix packed in the order of the epilogue's row blocks (64 gate rows, then the
    64 up rows of the same columns): the hidden activation bit for bit that of the row-major
    matrix, alone and next to another packed problem."""
    gate, up = make_qmm_case(K, I, 801).to(DEV), make_qmm_case(K, I, 802).to(DEV)
    other = make_qmm_case(1024, 2048, 803).to(DEV)
    w = torch.cat([gate.w, up.w]); sc = torch.cat([gate.scales, up.scales]); bi = torch.cat([gate.biases, up.biases])
    want = VQ.QmmChain([VQ.ChainProblem(gate.x, w, sc, bi, epilogue="silu_mul")])()[0].clone()
    images = VQ.pack_weights(w, sc, bi, gate_up=True)
    got = VQ.QmmChain([VQ.ChainProblem(gate.x, images, epilogue="silu_mul")])()[0].clone()
    both = VQ.QmmChain([VQ.ChainProblem(other.x, VQ.pack_weights(other.w, other.scales, other.biases)),
                        VQ.ChainProblem(gate.x, images, epilogue="silu_mul")])()
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert torch.equal(both[1].view(torch.int16), want.view(torch.int16))
    assert torch.equal(both[0].view(torch.int16), _separate(other.x, other).view(torch.int16))
    with pytest.raises(ValueError, match="ordered for the silu-mul epilogue"):
        VQ.verify_matmul_packed(gate.x, images)
    with pytest.raises(ValueError, match="gate_up=True"):
        VQ.ChainProblem(gate.x, images)


def test_chain_against_the_oracle(native_lib, c_oracle):
    cases = _cases([(1024, 512), (2048, 256), (1024, 1024)], 720)
    ys = VQ.QmmChain([VQ.ChainProblem(c.x, c.w, c.scales, c.biases) for c in cases])()
    torch.cuda.synchronize()
    for c, y in zip(cases, ys):
        exact = O.qmm_exact(c.x.float().cpu().numpy(), c.w.cpu().numpy().view(np.uint32),
                            c.scales.float().cpu().numpy(), c.biases.float().cpu().numpy(), 64)
        got = y.float().cpu().numpy()
        assert np.all(np.abs(got - exact) <= 2e-2 * np.abs(exact).max(axis=1, keepdims=True))
        assert np.linalg.norm(got - exact) / np.linalg.norm(exact) <= 5e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fp16_and_bf16_activations(native_lib, dtype):
    cases = _cases([(1024, 256), (2048, 2048)], 730, dtype)
    ys = VQ.QmmChain([VQ.ChainProblem(c.x, c.w, c.scales, c.biases) for c in cases])()
    torch.cuda.synchronize()
    for c, y in zip(cases, ys):
        assert torch.equal(y.view(torch.int16), _separate(c.x, c).view(torch.int16))


@pytest.mark.parametrize("shapes", [[(1024, 1024), (1024, 2048), (2048, 1024)],
                                    [(5120, 5120), (5120, 17408), (17408, 5120)],
                                    [(1024, 1024)] * 6],
                         ids=["small", "27b-sized", "six-in-a-row"])
def test_projection_reading_an_earlier_output(native_lib, shapes):
    """y0 = A x, y1 = B y0, y2 = C y1: every link waits for the one before it."""
    cases = _cases(shapes, 740)
    print(f"dependent chain {shapes}", flush=True)
    # keep the activations in range: outputs of one matmul feed the next
    for c in cases:
        c.scales.mul_(0.05); c.biases.mul_(0.05)
    problems, prev = [], cases[0].x
    for c in cases:
        pr = VQ.ChainProblem(prev, c.w, c.scales, c.biases)
        problems.append(pr)
        prev = pr
    chain = VQ.QmmChain(problems)
    for rep in range(3):
        for y in chain.outputs:
            y.fill_(float("nan"))
        ys = chain()
        torch.cuda.synchronize()
        assert chain.error_word() == 0
        x = cases[0].x
        for i, (c, y) in enumerate(zip(cases, ys)):
            want = _separate(x, c)
            assert torch.isfinite(want.float()).all()
            assert torch.equal(y.view(torch.int16), want.view(torch.int16)), (rep, i)
            x = y


@pytest.mark.parametrize("K,I", [(1024, 1024), (5120, 17408), (2048, 3072)])
def test_mlp_in_one_launch(native_lib, c_oracle, K, I):
    """gate/up with the silu-mul epilogue, then the down projection waiting for it."""
    gate, up = make_qmm_case(K, I, 750).to(DEV), make_qmm_case(K, I, 751).to(DEV)
    down = make_qmm_case(I, K, 752).to(DEV)
    for c in (gate, up, down):
        c.scales.mul_(0.1); c.biases.mul_(0.1)
    joint = [torch.cat([a, b], dim=0).contiguous() for a, b in
             ((gate.w, up.w), (gate.scales, up.scales), (gate.biases, up.biases))]
    x = gate.x
    print(f"mlp chain K={K} I={I}", flush=True)
    p0 = VQ.ChainProblem(x, *joint, epilogue="silu_mul")
    p1 = VQ.ChainProblem(p0, down.w, down.scales, down.biases)
    chain = VQ.QmmChain([p0, p1])
    for rep in range(2):
        for y in chain.outputs:
            y.fill_(float("nan"))
        h, y = chain()
        torch.cuda.synchronize()
        assert chain.error_word() == 0
        # operator by operator on separate launches: a launch of its own splits K elsewhere than
        # the gate/up pair does, so g and u may differ in their last bit where sums cancel - equal
        # on nearly all elements, and everywhere within the bar on the exact product below
        g, u = _separate(x, gate), _separate(x, up)
        want_h = silu_ops(g) * u
        assert float((h != want_h).float().mean()) <= 2e-3
        ge, ue = (_exact(c_oracle, c, x).astype(np.float64) for c in (gate, up))
        exact = ge / (1.0 + np.exp(-ge)) * ue
        got = h.float().cpu().numpy().astype(np.float64)
        assert np.all(np.abs(got - exact) <= 2e-2 * np.abs(exact).max(axis=1, keepdims=True))
        assert np.linalg.norm(got - exact) / np.linalg.norm(exact) <= 5e-3
        # the down projection read exactly the h the launch stored
        want_y = _separate(h, down)
        assert torch.equal(y.view(torch.int16), want_y.view(torch.int16))


def test_bounded_wait_gives_up_and_the_launch_still_ends(native_lib):
    """spin_limit = 1: a projection that waits polls twice at most.  Whether its input was ready
    by then is a matter of timing; either way every workgroup leaves, the launch ends, the error
    word names the projection when a wait was given up, and the next launch (default limit) is
    right again."""
    cases = _cases([(5120, 17408), (17408, 5120)], 760)
    for c in cases:
        c.scales.mul_(0.05); c.biases.mul_(0.05)
    p0 = VQ.ChainProblem(cases[0].x, cases[0].w, cases[0].scales, cases[0].biases)
    p1 = VQ.ChainProblem(p0, cases[1].w, cases[1].scales, cases[1].biases)
    hasty = VQ.QmmChain([p0, p1], spin_limit=1)
    hasty()
    torch.cuda.synchronize()                       # returns: nothing hangs
    word = hasty.error_word()
    assert word in (0, 2)
    y0 = _separate(cases[0].x, cases[0])
    assert torch.equal(hasty.outputs[0].view(torch.int16), y0.view(torch.int16))   # nothing waits for x0
    if word:
        with pytest.raises(nat.NativeLibraryError, match="projection 1 of a chained launch"):
            hasty.check()                          # says so, and hands the workspace back zero-filled
        assert hasty.error_word() == 0
    else:
        hasty.check()
    # the same for a word as the streaming kernel leaves it (its waits cannot be made to expire
    # from the host: written by hand)
    ws = VQ._workspace(cases[0].x.device, nat.raw_stream(cases[0].x.device), 1)
    ws[nat.QMM_ERROR_OFFSET:nat.QMM_ERROR_OFFSET + 4].view(torch.int32).fill_(-2147483648 + 7)
    with pytest.raises(nat.NativeLibraryError, match="row block 7"):
        VQ.raise_on_device_errors(cases[0].x.device)
    VQ.raise_on_device_errors()                    # cleared: nothing to report
    assert int((ws != 0).sum()) == 0
    patient = VQ.QmmChain([p0, p1])
    ys = patient()
    torch.cuda.synchronize()
    assert patient.error_word() == 0
    assert torch.equal(ys[1].view(torch.int16), _separate(ys[0], cases[1]).view(torch.int16))


def test_argument_errors(native_lib):
    L = native_lib
    tab = (nat.QmmProblem * 2)()
    one = 256
    for t in tab:
        t.x = t.w_q = t.scales = t.biases = t.y = one
        t.K, t.N, t.wait_for, t.epilogue = 1024, 64, -1, 0
    ws = ctypes.c_void_p(one)
    assert L.dflash_qmm_m16_chain(tab, 0, ws, 1 << 30, 64, 0, 0, 0, 0, None) == -1
    assert L.dflash_qmm_m16_chain(tab, 17, ws, 1 << 30, 64, 0, 0, 0, 0, None) == -2
    tab[1].K = 512
    assert L.dflash_qmm_m16_chain(tab, 2, ws, 1 << 30, 64, 0, 0, 0, 0, None) == -2      # K % 1024
    tab[1].K = 1024
    tab[1].wait_for = 1
    assert L.dflash_qmm_m16_chain(tab, 2, ws, 1 << 30, 64, 0, 0, 0, 0, None) == -1      # waits for itself
    tab[1].wait_for = 0
    assert L.dflash_qmm_m16_chain(tab, 2, ws, 1 << 30, 64, 0, 0, 0, 0, None) == -1      # x is not problem 0's y / K != N0
    assert b"waits for" in L.dflash_last_error()
    tab[1].wait_for = -1
    tab[0].epilogue = 1
    assert L.dflash_qmm_m16_chain(tab, 2, ws, 1 << 30, 64, 0, 0, 0, 0, None) == -2      # N % 128 with an epilogue
    tab[0].epilogue = 0
    assert L.dflash_qmm_m16_chain(tab, 2, None, 0, 64, 0, 0, 0, 0, None) == -3
    assert L.dflash_qmm_m16_chain_workspace_bytes(tab, 2, 64, 0) >= 64 * 1024 + 2 * 2 * 8192
    assert L.dflash_qmm_m16_chain_workspace_bytes(tab, 2, 32, 0) == 0
    assert L.dflash_qmm_m16_chain(tab, 2, ws, 1 << 30, 64, 0, 0, 0, 2, None) == -1      # unknown flag
    tab[0].layout = 2
    assert L.dflash_qmm_m16_chain(tab, 2, ws, 1 << 30, 64, 0, 0, 0, 0, None) == -2      # unknown layout
    tab[0].layout = nat.QMM_LAYOUT_PACKED
    assert L.dflash_qmm_m16_chain(tab, 2, ws, 1 << 30, 64, 0, 0, 0, 0, None) == -1      # two layouts in one launch
    assert b"one weight layout" in L.dflash_last_error()
    tab[0].layout = 0
    assert L.dflash_qmm_m16_pack_gate_up(one, one, one, one, one, one, 1024, 64, 64, None) == -2   # N % 128
    assert L.dflash_qmm_m16_pack_gate_up(one, one, one, None, one, one, 1024, 128, 64, None) == -1
    tab[1].wait_for = 0
    assert L.dflash_qmm_m16_chain(tab, 2, ws, 1 << 30, 64, 0, 0, 0, nat.QMM_CHAIN_JOINT_SPLIT, None) == -1
    assert b"independent" in L.dflash_last_error()
    tab[1].wait_for = -1
    assert (L.dflash_qmm_m16_chain_workspace_bytes(tab, 2, 64, nat.QMM_CHAIN_JOINT_SPLIT)
            >= L.dflash_qmm_m16_chain_workspace_bytes(tab, 2, 64, 0))


def test_hidden_activation_of_a_gated_mlp_in_one_launch(native_lib, c_oracle, monkeypatch):
    """verify_linear.silu_gate_up on joined gate/up projections: one chained launch with the
    silu-mul epilogue per call, a new output tensor per call, inputs rebound per call; within
    the north-star bar of the exact activation, and nearly everywhere the bits of the joint
    product followed by the array operators."""
    import dflash_mlx_amd.verify_linear as VL
    from dflash_mlx_amd.quantized import QuantizedLinear

    monkeypatch.setenv("DFLASH_VERIFY_QMM", "1")
    K, I = 1024, 1536
    gate, up = _cases([(K, I), (K, I)], 880)
    for c in (gate, up):
        c.scales.mul_(0.05); c.biases.mul_(0.05)
    mlp = torch.nn.Module()
    mlp.gate_proj = QuantizedLinear(gate.w.clone(), gate.scales.clone(), gate.biases.clone(), group_size=64, bits=4)
    mlp.up_proj = QuantizedLinear(up.w.clone(), up.scales.clone(), up.biases.clone(), group_size=64, bits=4)
    model = torch.nn.Module()
    model.mlp = mlp
    assert VL.install_verify_linears(model) == 2 and VL.fuse_shared_input_linears(model) == 1
    group = model.mlp.gate_proj._shared_input[0]
    launches = []
    real = VQ.QmmChain.__call__
    monkeypatch.setattr(VQ.QmmChain, "__call__", lambda self: (launches.append(self._count), real(self))[1])
    outs = []
    for seed in (1, 2, 3):
        x = (torch.randn(16, K, generator=torch.Generator().manual_seed(seed)) * 0.5).to(torch.bfloat16).to(DEV)
        assert group.silu_mul_ready(x)
        h = VL.silu_gate_up(model.mlp, x.reshape(1, 16, K))
        torch.cuda.synchronize()
        assert h.shape == (1, 16, I) and all(h.data_ptr() != o.data_ptr() for o in outs)
        outs.append(h)
        g, u = VL.shared_input_outputs(model.mlp, ("gate_proj", "up_proj"), x)
        ops = silu_ops(g) * u
        assert float((h.reshape(16, I) != ops).float().mean()) <= 2e-3
        ge, ue = (_exact(c_oracle, c, x).astype(np.float64) for c in (gate, up))
        exact = ge / (1.0 + np.exp(-ge)) * ue
        got = h.reshape(16, I).float().cpu().numpy().astype(np.float64)
        assert np.all(np.abs(got - exact) <= 2e-2 * np.abs(exact).max(axis=1, keepdims=True))
    assert launches == [1, 1, 1]
    # a block that is not a verify block: array operators on the members' own outputs
    x5 = torch.randn(5, K).to(torch.bfloat16).to(DEV)
    assert torch.equal(VL.silu_gate_up(model.mlp, x5),
                       silu_ops(model.mlp.gate_proj(x5)) * model.mlp.up_proj(x5))
    assert launches == [1, 1, 1]
    # rebinding is refused where it would break the chain, or where the tensor does not fit
    small = _cases([(1024, 64), (64, 32)], 881)[0]
    first = VQ.ChainProblem(small.x, small.w, small.scales, small.biases)
    w2 = torch.zeros((32, 64 // 8), dtype=small.w.dtype, device=DEV)
    with pytest.raises(ValueError):
        VQ.QmmChain([first, VQ.ChainProblem(first, w2, small.scales[:32, :1], small.biases[:32, :1])])   # K = 64
    two = _cases([(1024, 1024), (1024, 64)], 882)
    a = VQ.ChainProblem(two[0].x, two[0].w, two[0].scales, two[0].biases)
    b = VQ.ChainProblem(a, two[1].w, two[1].scales, two[1].biases)
    chain = VQ.QmmChain([a, b])
    with pytest.raises(ValueError, match="reads another"):
        chain.rebind(1, x=two[1].x)
    with pytest.raises(ValueError, match="reads this output"):
        chain.rebind(0, out=torch.empty_like(chain.outputs[0]))
    with pytest.raises(ValueError, match="contiguous"):
        chain.rebind(0, x=two[0].x.float())
    fresh = torch.empty_like(chain.outputs[1])
    chain.rebind(0, x=two[0].x.clone())
    chain.rebind(1, out=fresh)
    ys = chain()
    torch.cuda.synchronize()
    assert ys[1] is fresh and torch.equal(fresh, _separate(_separate(two[0].x, two[0]), two[1]))


def test_gated_mlp_activation_on_packed_weights(native_lib, monkeypatch):
    """pack_verify_linears gives a joined gate/up pair a copy in the order of the epilogue's row
    blocks as well: silu_gate_up then reads that copy and returns the bits it returned before."""
    import dflash_mlx_amd.verify_linear as VL
    from dflash_mlx_amd.quantized import QuantizedLinear

    monkeypatch.setenv("DFLASH_VERIFY_QMM", "1")
    K, I = 2048, 1536

    def build():
        gate, up = _cases([(K, I), (K, I)], 890)
        mlp = torch.nn.Module()
        mlp.gate_proj = QuantizedLinear(gate.w.clone(), gate.scales.clone(), gate.biases.clone(), group_size=64, bits=4)
        mlp.up_proj = QuantizedLinear(up.w.clone(), up.scales.clone(), up.biases.clone(), group_size=64, bits=4)
        model = torch.nn.Module()
        model.mlp = mlp
        assert VL.install_verify_linears(model) == 2 and VL.fuse_shared_input_linears(model) == 1
        return model

    x = (torch.randn(1, 16, K, generator=torch.Generator().manual_seed(9)) * 0.5).to(torch.bfloat16).to(DEV)
    plain = build()
    before = VL.silu_gate_up(plain.mlp, x).clone()
    packed = build()
    assert VL.pack_verify_linears(packed) == 1
    group = packed.mlp.gate_proj._shared_input[0]
    assert group._packed_silu is not None and group._packed_silu.gate_up and not group._packed.gate_up
    after = VL.silu_gate_up(packed.mlp, x)
    torch.cuda.synchronize()
    assert group._silu_chain._table[0].layout == nat.QMM_LAYOUT_PACKED
    assert torch.equal(after.view(torch.int16), before.view(torch.int16))
    g, u = VL.shared_input_outputs(packed.mlp, ("gate_proj", "up_proj"), x)          # the plain packed copy
    g0, u0 = VL.shared_input_outputs(plain.mlp, ("gate_proj", "up_proj"), x)
    assert torch.equal(g, g0) and torch.equal(u, u0)

