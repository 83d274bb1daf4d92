"""Pins the qmm oracle (oracle/dflash_oracle.py, oracle/dflash_oracle_c.c) against
things it cannot have been tuned to: a literal triple loop, closed-form known
answers, algebraic invariants, and torch's own bf16 rounding."""
import numpy as np
import pytest
import torch

from oracle import dflash_oracle as O


def _case(rng, M, K, N, gs):
    x = O.round_bf16(rng.standard_normal((M, K)).astype(np.float32))
    w = rng.integers(0, 2 ** 32, size=(N, K // 8), dtype=np.uint64).astype(np.uint32)
    s = O.round_bf16((np.abs(rng.standard_normal((N, K // gs))) * 0.02 + 1e-4).astype(np.float32))
    b = O.round_bf16((-8.0 * s).astype(np.float32))
    return x, w, s, b


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(1)
    a = rng.standard_normal(200_000).astype(np.float32) * np.float32(10.0) ** rng.integers(-20, 20, 200_000).astype(np.float32)
    # exact ties and values around them
    ties = np.array([1.00390625, 1.01171875, -1.00390625, 3.0e38, 1e-40, 0.0, -0.0, np.inf, -np.inf], dtype=np.float32)
    a = np.concatenate([a, ties])
    got = O.f32_to_bf16(a)
    want = torch.from_numpy(a).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(O.bf16_to_f32(got), torch.from_numpy(a).to(torch.bfloat16).to(torch.float32).numpy())


def test_nibble_order_known_answer():
    # word 0x76543210 holds codes 0..7 at k = 0..7 (low nibble first)
    w = np.array([[0x76543210, 0xFEDCBA98]], dtype=np.uint32)
    assert O.unpack_int4(w).tolist() == [list(range(16))]
    assert np.array_equal(O.pack_int4(O.unpack_int4(w)), w)


@pytest.mark.parametrize("gs,K,N", [(64, 64, 32), (32, 96, 16), (128, 256, 8)])
def test_exact_matches_bruteforce(gs, K, N):
    rng = np.random.default_rng(gs + K)
    x, w, s, b = _case(rng, 3, K, N, gs)
    want = O.qmm_bruteforce(x, w, s, b, gs)
    got = O.qmm_exact(x, w, s, b, gs)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)


def test_all_eight_codes_cancel_bias():
    # codes == 8 everywhere and bias = -8*scale  ->  every weight is exactly 0
    rng = np.random.default_rng(2)
    x, _, s, b = _case(rng, 16, 256, 64, 64)
    w = np.full((64, 32), 0x88888888, dtype=np.uint32)
    assert np.all(O.qmm_exact(x, w, s, b, 64) == 0.0)
    assert np.all(O.qmm_kernel_semantics(x, w, s, b, 64) == 0.0)


def test_one_hot_rows_read_code_columns():
    rng = np.random.default_rng(3)
    K, N, gs = 128, 32, 64
    _, w, _, _ = _case(rng, 16, K, N, gs)
    s = np.ones((N, K // gs), dtype=np.float32)
    b = np.zeros((N, K // gs), dtype=np.float32)
    ks = rng.integers(0, K, size=16)
    x = np.zeros((16, K), dtype=np.float32)
    x[np.arange(16), ks] = 1.0
    y = O.qmm_exact(x, w, s, b, gs)
    codes = O.unpack_int4(w)
    for m in range(16):
        assert np.array_equal(y[m], codes[:, ks[m]].astype(np.float64))


def test_single_group_isolates_scale_and_bias_index():
    K, N, gs = 256, 16, 64
    rng = np.random.default_rng(4)
    _, w, _, _ = _case(rng, 1, K, N, gs)
    codes = O.unpack_int4(w).astype(np.float64)
    x = np.ones((1, K), dtype=np.float32)
    for g in range(K // gs):
        s = np.zeros((N, K // gs), dtype=np.float32)
        b = np.zeros((N, K // gs), dtype=np.float32)
        s[:, g] = 2.0
        b[:, g] = -3.0
        y = O.qmm_exact(x, w, s, b, gs)[0]
        want = 2.0 * codes[:, g * gs:(g + 1) * gs].sum(axis=1) - 3.0 * gs
        assert np.array_equal(y, want)


def test_invariants_linearity_nslice_ksplit():
    rng = np.random.default_rng(5)
    K, N, gs = 512, 96, 64
    x, w, s, b = _case(rng, 16, K, N, gs)
    x2 = O.round_bf16(rng.standard_normal((16, K)).astype(np.float32))
    y = O.qmm_exact(x, w, s, b, gs)
    y2 = O.qmm_exact(x2, w, s, b, gs)
    np.testing.assert_allclose(O.qmm_exact((2 * x - x2).astype(np.float32), w, s, b, gs), 2 * y - y2,
                               rtol=0, atol=1e-9)
    # N tiles are independent
    np.testing.assert_array_equal(O.qmm_exact(x, w[32:64], s[32:64], b[32:64], gs), y[:, 32:64])
    # K-split additivity
    half = K // 2
    ya = O.qmm_exact(x[:, :half], w[:, :half // 8], s[:, :half // gs], b[:, :half // gs], gs)
    yb = O.qmm_exact(x[:, half:], w[:, half // 8:], s[:, half // gs:], b[:, half // gs:], gs)
    np.testing.assert_allclose(ya + yb, y, rtol=0, atol=1e-9)
    # kernel flavour: pipe == mma2big up to fp32 re-association
    k1 = O.qmm_kernel_semantics(x, w, s, b, gs, k_parts=1)
    k8 = O.qmm_kernel_semantics(x, w, s, b, gs, k_parts=8)
    assert np.max(np.abs(k1 - k8)) <= 2 ** -7 * np.max(np.abs(k1))


def test_library_route_torch_dequant_matmul():
    """Dequantise with independent torch code and use torch.matmul in float64."""
    rng = np.random.default_rng(6)
    K, N, gs = 1024, 128, 64
    x, w, s, b = _case(rng, 16, K, N, gs)
    wt = torch.from_numpy(w.astype(np.int64))
    cols = [((wt >> (4 * i)) & 0xF) for i in range(8)]
    q = torch.stack(cols, dim=-1).reshape(N, K).double()
    sd = torch.from_numpy(s).double().repeat_interleave(gs, dim=1)
    bd = torch.from_numpy(b).double().repeat_interleave(gs, dim=1)
    want = torch.from_numpy(x).double() @ (q * sd + bd).T
    np.testing.assert_allclose(O.qmm_exact(x, w, s, b, gs), want.numpy(), rtol=1e-12, atol=1e-12)


def test_kernel_semantics_close_to_exact():
    rng = np.random.default_rng(7)
    K, N, gs = 2048, 64, 64
    x, w, s, b = _case(rng, 16, K, N, gs)
    exact = O.qmm_exact(x, w, s, b, gs)
    kern = O.qmm_kernel_semantics(x, w, s, b, gs).astype(np.float64)
    rel_l2 = np.linalg.norm(kern - exact) / np.linalg.norm(exact)
    assert rel_l2 < 5e-3


@pytest.mark.parametrize("flavour,k_parts", [(0, 1), (1, 1), (1, 8)])
def test_c_restatement_matches_numpy(c_oracle, flavour, k_parts):
    rng = np.random.default_rng(8)
    K, N, gs = 1024, 96, 64
    x, w, s, b = _case(rng, 16, K, N, gs)
    y32, y16 = c_oracle.qmm_m16(O.f32_to_bf16(x), w, O.f32_to_bf16(s), O.f32_to_bf16(b), gs,
                                flavour=flavour, k_parts=k_parts)
    if flavour == 0:
        want = O.qmm_exact(x, w, s, b, gs)
        np.testing.assert_allclose(y32, want, rtol=2e-7, atol=1e-6)
    else:
        want = O.qmm_kernel_semantics(x, w, s, b, gs, k_parts=k_parts)
        # same arithmetic, different fp32 summation order inside a slice
        assert np.max(np.abs(O.bf16_to_f32(y16) - want)) <= 2 ** -7 * np.max(np.abs(want))
    assert np.array_equal(y16, O.f32_to_bf16(y32))


def test_gather_exact_selects_expert():
    rng = np.random.default_rng(9)
    K, N, gs, E = 128, 32, 64, 4
    cases = [_case(rng, 1, K, N, gs) for _ in range(E)]
    w = np.stack([c[1] for c in cases]); s = np.stack([c[2] for c in cases]); b = np.stack([c[3] for c in cases])
    x = O.round_bf16(rng.standard_normal((6, K)).astype(np.float32))
    ids = np.array([3, 0, 0, 2, 1, 3])
    y = O.qmm_gather_exact(x, ids, w, s, b, gs)
    for p, e in enumerate(ids):
        want = O.qmm_bruteforce(x[p:p + 1], w[e], s[e], b[e], gs)[0]
        np.testing.assert_allclose(y[p], want, rtol=1e-12, atol=1e-12)
