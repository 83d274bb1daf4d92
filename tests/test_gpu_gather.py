"""Gathered per-expert qmm (MoE-shaped verify step) against the closed-form oracle.
The reference has no such operator (parity unpinned beyond the closed form)."""
import numpy as np
import pytest
import torch

import dflash_mlx_amd._native as nat
from dflash_mlx_amd.verify_qmm import gather_qmm
from dflash_mlx_amd.workloads import make_moe_case, seed_for
from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _check(case, y):
    xf = case.x.float().numpy()
    exact = O.qmm_gather_exact(xf, case.expert_ids.numpy(), case.w.numpy().view(np.uint32),
                               case.scales.float().numpy(), case.biases.float().numpy(), case.group_size)
    yv = y.float().cpu().numpy().astype(np.float64)
    err = np.abs(yv - exact)
    assert np.all(err <= 2e-2 * np.max(np.abs(exact), axis=1, keepdims=True))
    assert np.linalg.norm(yv - exact) / np.linalg.norm(exact) <= 5e-3


@pytest.mark.parametrize("K,N", [(2048, 512), (512, 2048)])
def test_config4_expert_shapes(native_lib, K, N):
    """16 tokens x top-8 of 256 experts: gate/up 2048->512 and down 512->2048."""
    case = make_moe_case(K, N, seed_for(4, K), experts=256)
    d = case.to(DEV)
    y = gather_qmm(d.x, d.w, d.scales, d.biases, d.expert_ids, group_size=64)
    torch.cuda.synchronize()
    assert y.shape == (128, N)
    _check(case, y)
    # deterministic
    assert torch.equal(y, gather_qmm(d.x, d.w, d.scales, d.biases, d.expert_ids, group_size=64))


def test_more_than_sixteen_rows_per_expert_and_unused_experts(native_lib):
    case = make_moe_case(256, 48, 77, experts=5, tokens=50, top_k=2, group_size=32)
    case.expert_ids = torch.tensor(([0] * 37 + [3] * 40 + [4] * 23), dtype=torch.int32)[torch.randperm(
        100, generator=torch.Generator().manual_seed(1))]
    d = case.to(DEV)
    y = gather_qmm(d.x, d.w, d.scales, d.biases, d.expert_ids, group_size=32)
    _check(case, y)
    # every row equals the plain M=1 product with its expert (row independence)
    one = gather_qmm(d.x[7:8], d.w, d.scales, d.biases, d.expert_ids[7:8], group_size=32)
    assert torch.equal(one[0], y[7])


def test_argument_checks(native_lib):
    L = native_lib
    assert L.dflash_qmm_m16_gather(None, None, None, None, None, None, 1, 64, 32, 2, 64, 0, 0, None) == -1
    import ctypes
    one = ctypes.c_void_p(256)
    assert L.dflash_qmm_m16_gather(one, one, one, one, one, one, 4096, 64, 32, 2, 64, 0, 0, None) == -2
    assert b"at most" in L.dflash_last_error()
    with pytest.raises(nat.NativeLibraryError):
        c = make_moe_case(64, 32, 1, experts=2, tokens=2, top_k=1)
        gather_qmm(c.x, c.w, c.scales, c.biases, c.expert_ids)
