"""Shapes drawn at random through the M=16 qmm kernels.

The split of a launch (how many workgroups, which row blocks two of them share, who adds the
partial tiles) follows from K and N, so the shapes of the stacks exercise a handful of splits;
these draws exercise the rest: the streaming kernel on K any multiple of 512 up to 18 432 and N
any multiple of 16 up to 20 800, both activation types, a new shape after every launch and
earlier ones again without a wait in between; the chained kernel's joint split on random lists
of problems; packed weights alone, chained and in a joint split; chains whose links wait for
each other, with and without the MLP epilogue; gathered experts on skewed routings.  Results
are checked against the oracle's C restatement of the reference arithmetic (north-star bar of
tests/test_gpu_qmm.py) or, where a route is stated to give another route's bits, against that
route; they must repeat bit for bit; afterwards the error word is clear and the partial-tile
workspace is back at zero.
"""
import numpy as np
import pytest
import torch

import dflash_mlx_amd._native as nat
from dflash_mlx_amd import verify_qmm as VQ
from dflash_mlx_amd.workloads import make_qmm_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _exact(c_oracle, case):
    y32, _ = c_oracle.qmm_m16(_bits(case.x), case.w.cpu().numpy().view(np.uint32), _bits(case.scales),
                              _bits(case.biases), case.group_size, flavour=0)
    return y32.astype(np.float64)


def _close(y, exact):
    y = y.detach().cpu().float().numpy().astype(np.float64)
    row_inf = np.max(np.abs(exact), axis=1, keepdims=True)
    assert np.all(np.abs(y - exact) <= 2e-2 * row_inf + 1e-30)
    assert np.linalg.norm(y - exact) <= 5e-3 * max(np.linalg.norm(exact), 1e-30)


def _workspace_is_clean(device):
    VQ.raise_on_device_errors(device)
    ws = VQ._workspace(device, nat.raw_stream(device), 1)
    assert int((ws != 0).sum()) == 0


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_streaming_kernel_on_random_shapes(verify_env, native_lib, c_oracle, seed):
    verify_env.setenv("DFLASH_QMM_KERNEL", "stream")
    rng = np.random.default_rng(seed)
    earlier = []
    for i in range(24):
        K = 512 * int(rng.integers(1, 37))
        N = 16 * int(rng.integers(1, 1301)) if i % 3 else 64 * int(rng.integers(1, 321))
        case = make_qmm_case(K, N, 1000 * seed + i).to(DEV)
        runs = [VQ.verify_matmul(case.x, case.w, case.scales, case.biases, group_size=64, bits=4).clone()
                for _ in range(3)]
        torch.cuda.synchronize()
        assert torch.equal(runs[1], runs[0]) and torch.equal(runs[2], runs[0]), (K, N)
        _close(runs[0], _exact(c_oracle, case))
        earlier.append((case, runs[0]))
        if len(earlier) == 8:  # the same shapes again, back to back: the workspace is shared
            again = [VQ.verify_matmul(c.x, c.w, c.scales, c.biases, group_size=64, bits=4).clone() for c, _ in earlier]
            torch.cuda.synchronize()
            for (c, first), y in zip(earlier, again):
                assert torch.equal(y, first), (c.K, c.N)
            earlier = []
    _workspace_is_clean(torch.device(DEV))


@pytest.mark.parametrize("seed", [21, 22])
def test_joint_split_on_random_lists_of_problems(verify_env, native_lib, c_oracle, seed):
    verify_env.setenv("DFLASH_QMM_KERNEL", "stream")
    rng = np.random.default_rng(seed)
    for it in range(8):
        big = it % 3 == 0
        shapes = [(1024 * int(rng.integers(1, 18 if big else 5)), 32 * int(rng.integers(1, 541 if big else 41)))
                  for _ in range(int(rng.integers(1, 17)))]
        cases = [make_qmm_case(K, N, 100 * seed + 16 * it + i).to(DEV) for i, (K, N) in enumerate(shapes)]
        chain = VQ.QmmChain([VQ.ChainProblem(c.x, c.w, c.scales, c.biases) for c in cases], joint_split=True)
        first = [y.clone() for y in chain()]
        second = [y.clone() for y in chain()]
        torch.cuda.synchronize()
        assert chain.error_word() == 0 and int((chain._ws != 0).sum()) == 0, shapes
        for c, a, b in zip(cases, first, second):
            assert torch.equal(a, b), shapes
            _close(a, _exact(c_oracle, c))


@pytest.mark.parametrize("seed", [31, 32])
def test_packed_weights_on_random_shapes(verify_env, native_lib, seed):
    """The packed copy of a triple gives the bits of the row-major route, alone and in a chain
    with the joint split (K a multiple of 1024: whole scale/bias chunks; N of 32)."""
    verify_env.setenv("DFLASH_QMM_KERNEL", "stream")
    rng = np.random.default_rng(seed)
    cases, images = [], []
    for i in range(12):
        K = 1024 * int(rng.integers(1, 18))
        N = 32 * int(rng.integers(1, 350))
        case = make_qmm_case(K, N, 1000 * seed + i).to(DEV)
        image = VQ.pack_weights(case.w, case.scales, case.biases)
        want = VQ.verify_matmul(case.x, case.w, case.scales, case.biases, group_size=64, bits=4)
        assert torch.equal(VQ.verify_matmul_packed(case.x, image), want), (K, N)
        cases.append(case)
        images.append(image)
    separate = [VQ.verify_matmul(c.x, c.w, c.scales, c.biases, group_size=64, bits=4) for c in cases]
    chain = VQ.QmmChain([VQ.ChainProblem(c.x, im) for c, im in zip(cases, images)])
    for y, want in zip(chain(), separate):  # per-problem split: bit for bit the separate launches
        assert torch.equal(y, want)
    joint = VQ.QmmChain([VQ.ChainProblem(c.x, im) for c, im in zip(cases, images)], joint_split=True)
    first = [y.clone() for y in joint()]
    second = [y.clone() for y in joint()]
    torch.cuda.synchronize()
    for a, b, want in zip(first, second, separate):  # another split: within an output rounding, repeatable
        assert torch.equal(a, b)
        assert float((a == want).float().mean()) >= 0.97
        assert float((a.float() - want.float()).abs().max()) <= 2 ** -7 * float(want.float().abs().max())
    assert joint.error_word() == 0 and int((joint._ws != 0).sum()) == 0
    _workspace_is_clean(torch.device(DEV))


@pytest.mark.parametrize("seed", [41, 42, 43])
def test_gathered_experts_on_random_routings(native_lib, monkeypatch, seed):
    """Expert counts, rows per expert (none, one, more than sixteen) and shapes at random: every row
    is the product with its own expert whatever else shares the launch, twice the same bits."""
    from dflash_mlx_amd.verify_qmm import gather_qmm
    from dflash_mlx_amd.workloads import make_moe_case
    from oracle import dflash_oracle as O

    monkeypatch.setenv("DFLASH_QMM_KERNEL", "auto")
    rng = np.random.default_rng(seed)
    for i in range(6):
        K = 512 * int(rng.integers(1, 9))
        N = 16 * int(rng.integers(1, 80))
        E = int(rng.integers(1, 40))
        P = int(rng.integers(1, 257))
        case = make_moe_case(K, N, 100 * seed + i, experts=E, tokens=P, top_k=1)
        # a skewed routing: most rows on a few experts, some experts without rows
        weights = rng.random(E) ** 4
        ids = rng.choice(E, size=P, p=weights / weights.sum()).astype(np.int32)
        case.expert_ids = torch.from_numpy(ids)
        d = case.to(DEV)
        y = gather_qmm(d.x, d.w, d.scales, d.biases, d.expert_ids, group_size=64)
        assert torch.equal(y, gather_qmm(d.x, d.w, d.scales, d.biases, d.expert_ids, group_size=64)), (K, N, E, P)
        exact = O.qmm_gather_exact(case.x.float().numpy(), ids, case.w.numpy().view(np.uint32),
                                   case.scales.float().numpy(), case.biases.float().numpy(), 64)
        _close(y, exact)
        j = int(rng.integers(0, P))
        # (alone in a call the row's K range is cut at other places - the cut follows the number
        # of units of the whole launch - so its fp32 sums associate differently: the same value
        # to within an output rounding, not always the same bits)
        one = gather_qmm(d.x[j:j + 1], d.w, d.scales, d.biases, d.expert_ids[j:j + 1], group_size=64)
        assert float((one[0] == y[j]).float().mean()) >= 0.97, (K, N, E, P, j)
        assert float((one[0].float() - y[j].float()).abs().max()) <= 2 ** -7 * float(y[j].float().abs().max())
    VQ.raise_on_device_errors(torch.device(DEV))


@pytest.mark.parametrize("seed", [51, 52, 53])
def test_dependent_chains_of_random_widths(verify_env, native_lib, seed):
    """y0 = A0 x, y1 = A1 y0, ...: widths at random, every link waiting inside the launch for the one
    before it, now and then an MLP (gate/up with the silu-mul epilogue, then its down projection).
    Every link gives the bits of a separate launch on the input the chain actually stored."""
    from dflash_mlx_amd.gdn_layer import silu_ops

    verify_env.setenv("DFLASH_QMM_KERNEL", "stream")
    rng = np.random.default_rng(seed)
    for it in range(4):
        width = 1024 * int(rng.integers(1, 7))
        x = make_qmm_case(width, 16, 7000 + 10 * seed + it).to(DEV).x
        problems, links, prev = [], [], x
        for i in range(int(rng.integers(2, 7))):
            nxt = 1024 * int(rng.integers(1, 7))
            if rng.random() < 0.3:  # an MLP of inner width `inner` in the place of a plain link
                inner = 1024 * int(rng.integers(1, 9))
                gate_up = make_qmm_case(width, 2 * inner, 100 * seed + 10 * it + i).to(DEV)
                down = make_qmm_case(inner, nxt, 100 * seed + 10 * it + i + 5000).to(DEV)
                for c in (gate_up, down):
                    c.scales.mul_(0.05); c.biases.mul_(0.05)
                p0 = VQ.ChainProblem(prev, gate_up.w, gate_up.scales, gate_up.biases, epilogue="silu_mul")
                p1 = VQ.ChainProblem(p0, down.w, down.scales, down.biases)
                problems += [p0, p1]
                links += [("mlp", gate_up), ("plain", down)]
                prev = p1
            else:
                c = make_qmm_case(width, nxt, 100 * seed + 10 * it + i).to(DEV)
                c.scales.mul_(0.05); c.biases.mul_(0.05)
                pr = VQ.ChainProblem(prev, c.w, c.scales, c.biases)
                problems.append(pr)
                links.append(("plain", c))
                prev = pr
            width = nxt
        chain = VQ.QmmChain(problems)
        for rep in range(2):
            for y in chain.outputs:
                y.fill_(float("nan"))
            ys = chain()
            torch.cuda.synchronize()
            assert chain.error_word() == 0
            inp = x
            for i, ((kind, c), y) in enumerate(zip(links, ys)):
                assert torch.isfinite(y.float()).all(), (it, i)
                full = VQ.verify_matmul(inp, c.w, c.scales, c.biases, group_size=64, bits=4)
                if kind == "plain":
                    assert torch.equal(y, full), (it, rep, i, kind)
                else:  # (the joined pair splits K like one matrix of its own: same split here and there)
                    half = c.N // 2
                    want = silu_ops(full[:, :half]) * full[:, half:]
                    assert torch.equal(y, want), (it, rep, i, kind)
                inp = y
    _workspace_is_clean(torch.device(DEV))
