"""Shapes drawn at random through the streaming M=16 qmm and the chained kernel's joint split.

The split of a launch (how many workgroups, which row blocks two of them share, who adds the
partial tiles) follows from K and N, so the shapes of the stacks exercise a handful of splits;
these draws exercise the rest: K any multiple of 512 up to 18 432, N any multiple of 16 up to
20 800, both activation types, a new shape after every launch and earlier ones again without a
wait in between.  Every result is checked against the oracle's C restatement of the reference
arithmetic (north-star bar of tests/test_gpu_qmm.py) and must repeat bit for bit; afterwards the
error word is clear and the partial-tile workspace is back at zero.
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
