"""Gathered per-expert qmm (MoE-shaped verify step) against the closed-form oracle.
The reference has no such operator (parity unpinned beyond the closed form)."""
import numpy as np
import pytest
import torch

import dflash_mlx_amd._native as nat
from dflash_mlx_amd.verify_qmm import (append_shared_expert, gather_qmm, join_expert_projections,
                                       shared_expert_rows, verify_matmul)
from dflash_mlx_amd.workloads import MoeCase, make_moe_case, make_qmm_case, seed_for
from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True, params=["auto", "tile"])
def kernel_mode(request, monkeypatch):
    """Every test runs once with the streaming kernel where it applies (auto: group 64,
    K % 512 == 0, at most 256 rows) and once with the per-(columns, expert) kernel forced."""
    monkeypatch.setenv("DFLASH_QMM_KERNEL", request.param)
    return request.param


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


def test_gate_and_up_of_the_experts_in_one_launch(native_lib):
    """Two projections that read the same rows, laid end to end per expert: the joint launch gives
    each of them its own product (to the same bar; the K split of the streaming kernel depends on
    the row count, so single output roundings may differ from the separate launches)."""
    gate = make_moe_case(1024, 384, seed_for(4, 31), experts=24)
    up = make_moe_case(1024, 256, seed_for(4, 32), experts=24)
    up.x, up.expert_ids = gate.x, gate.expert_ids
    g, u = gate.to(DEV), up.to(DEV)
    (w, sc, bi), bounds = join_expert_projections((g.w, g.scales, g.biases), (u.w, u.scales, u.biases))
    assert bounds == [(0, 384), (384, 640)] and w.shape == (24, 640, 128)
    y = gather_qmm(g.x, w, sc, bi, g.expert_ids, group_size=64)
    torch.cuda.synchronize()
    _check(gate, y[:, :384])
    _check(up, y[:, 384:])
    sep = torch.cat([gather_qmm(c.x, c.w, c.scales, c.biases, c.expert_ids, group_size=64) for c in (g, u)], dim=-1)
    close = (y.float() - sep.float()).abs() <= 2 ** -7 * sep.float().abs().amax(dim=-1, keepdim=True)
    assert bool(close.all())
    with pytest.raises(ValueError):
        join_expert_projections((g.w, g.scales, g.biases))


@pytest.mark.parametrize("K,N", [(2048, 512), (512, 2048)])
def test_shared_expert_in_the_gathered_launch(native_lib, K, N):
    """config[4] with the shared expert stored as expert 256: one launch over 128 routed pairs and
    16 shared rows gives both products, each to the bar of the closed form, and the shared rows
    also agree with the dense call on the same weights."""
    routed = make_moe_case(K, N, seed_for(4, K + 1), experts=256)
    shared = make_qmm_case(K, N, seed_for(4, K + 2))
    (w, sc, bi), sid = append_shared_expert((routed.w, routed.scales, routed.biases),
                                            (shared.w, shared.scales, shared.biases))
    assert sid == 256 and w.shape == (257, N, K // 8)
    x, ids = shared_expert_rows(routed.x, routed.expert_ids, shared.x, sid)
    assert x.shape == (144, K) and ids.dtype == torch.int32 and bool((ids[128:] == 256).all())
    both = MoeCase(x, ids, w, sc, bi, 64)
    d = both.to(DEV)
    y = gather_qmm(d.x, d.w, d.scales, d.biases, d.expert_ids, group_size=64)
    torch.cuda.synchronize()
    assert y.shape == (144, N)
    _check(both, y)
    dense = verify_matmul(d.x[128:], d.w[256], d.scales[256], d.biases[256])
    close = (y[128:].float() - dense.float()).abs() <= 2 ** -7 * dense.float().abs().amax(dim=-1, keepdim=True)
    assert bool(close.all())
    assert torch.equal(y, gather_qmm(d.x, d.w, d.scales, d.biases, d.expert_ids, group_size=64))
    with pytest.raises(ValueError):
        append_shared_expert((routed.w, routed.scales, routed.biases), (shared.w[:16], shared.scales, shared.biases))


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


@pytest.mark.parametrize("K,N,E,rows", [
    (1024, 272, 5, (37, 0, 0, 40, 23)),      # > 16 rows per expert, ragged last row block, CHUNK 4
    (1536, 128, 7, (1, 16, 17, 0, 33, 15, 2)),  # K a multiple of 512 only: CHUNK 2
    (512, 640, 3, (250, 1, 5)),              # 256 rows, nearly all on one expert
    (2048, 16, 300, None),                   # one row block of 16 columns, many experts
])
def test_streamed_shapes_and_row_tables(native_lib, K, N, E, rows):
    g = torch.Generator().manual_seed(K + N)
    if rows is None:
        ids = torch.randint(0, E, (200,), generator=g, dtype=torch.int32)
    else:
        ids = torch.cat([torch.full((n,), e, dtype=torch.int32) for e, n in enumerate(rows)])
        ids = ids[torch.randperm(ids.numel(), generator=g)]
    case = make_moe_case(K, N, 5 + K, experts=E, tokens=ids.numel(), top_k=1)
    case.expert_ids = ids
    d = case.to(DEV)
    y = gather_qmm(d.x, d.w, d.scales, d.biases, d.expert_ids, group_size=64)
    _check(case, y)
    assert torch.equal(y, gather_qmm(d.x, d.w, d.scales, d.biases, d.expert_ids, group_size=64))
    # a row's result does not depend on which other rows share the call
    j = ids.numel() // 2
    one = gather_qmm(d.x[j:j + 1], d.w, d.scales, d.biases, d.expert_ids[j:j + 1], group_size=64)
    assert torch.equal(one[0], y[j])


def test_rows_with_invalid_expert_ids_give_zeros(native_lib, kernel_mode):
    """Straight through the C ABI, so that y can be pre-filled."""
    import ctypes
    L = native_lib
    K, N, E, P = 1024, 256, 4, 24
    case = make_moe_case(K, N, 31, experts=E, tokens=P, top_k=1)
    ids = case.expert_ids.clone()
    ids[3], ids[10], ids[23] = -1, E, 1 << 20
    case.expert_ids = ids
    d = case.to(DEV)
    y = torch.full((P, N), 7.0, dtype=torch.bfloat16, device=DEV)
    need = 0 if kernel_mode == "tile" else L.dflash_qmm_m16_gather_workspace_bytes(P, K, N, E, 64)
    assert (need > 0) == (kernel_mode == "auto")
    ws = torch.zeros(max(need, 16), dtype=torch.uint8, device=DEV)
    for _ in range(2):  # the workspace is handed back reusable
        rc = L.dflash_qmm_m16_gather(d.x.data_ptr(), d.expert_ids.data_ptr(), d.w.data_ptr(),
                                     d.scales.data_ptr(), d.biases.data_ptr(), y.data_ptr(),
                                     ws.data_ptr() if need else None, need, P, K, N, E, 64, 0, 0, None)
        assert rc == 0, L.dflash_last_error()
        torch.cuda.synchronize()
    bad = [3, 10, 23]
    assert torch.all(y[bad] == 0.0)
    good = [i for i in range(P) if i not in bad]
    sub = make_moe_case(K, N, 31, experts=E, tokens=P, top_k=1)
    exact = O.qmm_gather_exact(sub.x.float().numpy()[good], ids.numpy()[good], sub.w.numpy().view(np.uint32),
                               sub.scales.float().numpy(), sub.biases.float().numpy(), 64)
    got = y[good].float().cpu().numpy()
    assert np.linalg.norm(got - exact) / np.linalg.norm(exact) <= 5e-3
    assert L.dflash_qmm_m16_gather_workspace_bytes(4096, K, N, E, 64) == 0   # too many rows to stream
    assert L.dflash_qmm_m16_gather_workspace_bytes(P, K, N, E, 32) == 0      # group size


def test_argument_checks(native_lib):
    L = native_lib
    assert L.dflash_qmm_m16_gather(None, None, None, None, None, None, None, 0, 1, 64, 32, 2, 64, 0, 0, None) == -1
    import ctypes
    one = ctypes.c_void_p(256)
    assert L.dflash_qmm_m16_gather(one, one, one, one, one, one, None, 0, 4096, 64, 32, 2, 64, 0, 0, None) == -2
    assert b"at most" in L.dflash_last_error()
    with pytest.raises(nat.NativeLibraryError):
        c = make_moe_case(64, 32, 1, experts=2, tokens=2, top_k=1)
        gather_qmm(c.x, c.w, c.scales, c.biases, c.expert_ids)
