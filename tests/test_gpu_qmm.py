"""Parity of the gfx950 M=16 int4 qmm against the CPU oracle (exact fp64 closed form
and the reference-kernel arithmetic), through the Python surface and the raw C ABI.

Tolerances:
  north-star bar   max|y - y_exact| <= 2e-2 * max|row|   and   rel-L2 <= 5e-3   (bf16)
  reference's own  max_abs <= 8e-3 (bf16) / 4e-3 (fp16), max_abs/(max|y_ref|+1e-3) <= 2e-2
                   on x, w ~ N(0,1)/sqrt(K)   (tests/test_verify_qmm_parity.py:83-109)
"""
import ctypes

import numpy as np
import pytest
import torch

import dflash_mlx_amd._native as nat
from dflash_mlx_amd import verify_qmm as VQ
from dflash_mlx_amd.quantized import QuantizedLinear, quantize, quantized_matmul, stock_matmul
from dflash_mlx_amd.verify_linear import (VerifyQuantizedLinear, fuse_shared_input_linears,
                                          install_verify_linears)
from dflash_mlx_amd.workloads import make_qmm_case, seed_for
from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True, params=["auto", "tile"])
def kernel_mode(request, verify_env):
    """Every test runs once with the streaming kernel where it applies (auto) and once
    with the tile kernel forced."""
    verify_env.setenv("DFLASH_QMM_KERNEL", request.param)
    return request.param


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _f32(t):
    return t.detach().cpu().float().numpy()


def _oracle_exact(c_oracle, case):
    assert case.x.dtype == torch.bfloat16
    y32, _ = c_oracle.qmm_m16(_bits(case.x), case.w.cpu().numpy().view(np.uint32), _bits(case.scales),
                              _bits(case.biases), case.group_size, flavour=0)
    return y32.astype(np.float64)


def _check_north_star(y, exact):
    err = np.abs(y - exact)
    row_inf = np.max(np.abs(exact), axis=1, keepdims=True)
    assert np.all(err <= 2e-2 * row_inf + 1e-30), f"max-abs ratio {np.max(err / row_inf):.3g}"
    rel = np.linalg.norm(y - exact) / max(np.linalg.norm(exact), 1e-30)
    assert rel <= 5e-3, f"rel-L2 {rel:.3g}"
    return rel


def _run(case, variant=None, k_parts=None, monkeypatch=None):
    d = case.to(DEV)
    y = VQ.verify_matmul(d.x, d.w, d.scales, d.biases, group_size=d.group_size, bits=4)
    torch.cuda.synchronize()
    return y


def test_config0_single_call(verify_env, native_lib, c_oracle):
    """BASELINE config[0]: 16x4096x4096, group 64 (auto dispatch -> pipe x8)."""
    case = make_qmm_case(4096, 4096, seed_for(0))
    y = _f32(_run(case)).astype(np.float64)
    exact = _oracle_exact(c_oracle, case)
    rel = _check_north_star(y, exact)
    # the kernel keeps exact affine weights, so it sits at the bf16 output-rounding floor
    assert rel < 2.5e-3
    assert np.max(np.abs(y - O.round_bf16(exact.astype(np.float32)))) <= 2 ** -7 * np.max(np.abs(exact))


@pytest.mark.parametrize("K,N", [(5120, 17408), (17408, 5120), (5120, 7168), (5120, 5120), (4096, 12288),
                                 (4096, 6144), (12288, 4096),
                                 (512, 2048), (1536, 272)])  # the last two: K a multiple of 512 only
def test_real_projection_shapes(verify_env, native_lib, c_oracle, K, N):
    """27B / 9B projection shapes at full size, both dispatch branches."""
    case = make_qmm_case(K, N, seed_for(3, K % 97))
    y = _f32(_run(case)).astype(np.float64)
    _check_north_star(y, _oracle_exact(c_oracle, case))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("K,N", [(5120, 17408), (17408, 5120)])
def test_reference_tolerances_on_reference_style_data(verify_env, native_lib, dtype, K, N):
    """The reference's own acceptance test: data ~ N(0,1)/sqrt(K) quantised from floats,
    compared with the stock operator (here: the oracle's reference-kernel arithmetic)."""
    g = torch.Generator().manual_seed(K + N)
    scale = 1.0 / np.sqrt(K)
    x = (torch.randn(16, K, generator=g) * scale).to(dtype)
    w_fp = (torch.randn(N, K, generator=g) * scale).to(dtype)
    wq, s, b = quantize(w_fp, 64, 4)
    y = VQ.verify_matmul(x.to(DEV), wq.to(DEV), s.to(DEV), b.to(DEV), group_size=64, bits=4)
    name = "bf16" if dtype == torch.bfloat16 else "fp16"
    ref = O.qmm_kernel_semantics(x.float().numpy(), wq.numpy().view(np.uint32), s.float().numpy(),
                                 b.float().numpy(), 64, dtype=name,
                                 k_parts=8 if VQ._auto_variant(K, N)[0] == "mma2big_pipe" else 1)
    yv = _f32(y)
    max_abs = float(np.max(np.abs(yv - ref)))
    max_rel = max_abs / (float(np.max(np.abs(ref))) + 1e-3)
    assert max_abs <= (8e-3 if dtype == torch.bfloat16 else 4e-3), max_abs
    assert max_rel <= 2e-2, max_rel


def _reference_sweep_shapes(n=30, seed=0xDF1A):
    """The shape sweep of the reference's parity test (tests/test_verify_qmm_parity.py:43-53):
    the same generator, seed and order of draws, hence the same 30 (M, K, N)."""
    rng = np.random.default_rng(seed)
    levels = [1, 4, 8, 12, 15, 16]
    shapes = []
    for i in range(n):
        K = int(rng.integers(2, 40)) * 64
        N = int(rng.integers(1, 64)) * 8
        shapes.append((i, levels[i % len(levels)], K, N))
    return shapes


def _kernel_sweep_shapes():
    """The same draws with 16 rows and N rounded up to a multiple of 32: none of the sweep's own
    five M = 16 shapes has N % 32 == 0, so on its own it never reaches the kernel."""
    return [(100 + i, 16, K, (N + 31) // 32 * 32) for i, _, K, N in _reference_sweep_shapes()]


@pytest.mark.parametrize("i,M,K,N", _reference_sweep_shapes() + _kernel_sweep_shapes())
def test_reference_shape_sweep(verify_env, native_lib, i, M, K, N):
    """Every shape of the reference's sweep through verify_matmul on the device - M = 16 with
    N % 32 == 0 reaches the kernel, the rest the stock route, as verify_qmm.py:276-321 decides -
    held to the reference's bars (8e-3 abs, 2e-2 rel, test_verify_qmm_parity.py:103-109) on its
    data recipe (x, w ~ N(0,1)/sqrt(K), weights quantised from floats)."""
    g = torch.Generator().manual_seed(0xDF1A + i)
    scale = 1.0 / np.sqrt(K)
    x = (torch.randn(M, K, generator=g) * scale).to(torch.bfloat16)
    w_fp = (torch.randn(N, K, generator=g) * scale).to(torch.bfloat16)
    wq, s, b = quantize(w_fp, 64, 4)
    y = VQ.verify_matmul(x.to(DEV), wq.to(DEV), s.to(DEV), b.to(DEV), group_size=64, bits=4)
    assert tuple(y.shape) == (M, N) and y.dtype == torch.bfloat16
    kernel = VQ._should_use_verify(x, 64, 4, True) and N % 32 == 0
    assert kernel == (M == 16 and N % 32 == 0)
    ref = O.qmm_kernel_semantics(x.float().numpy(), wq.numpy().view(np.uint32), s.float().numpy(),
                                 b.float().numpy(), 64, dtype="bf16")
    max_abs = float(np.max(np.abs(_f32(y) - ref)))
    assert max_abs <= 8e-3, (M, K, N, max_abs)
    assert max_abs / (float(np.max(np.abs(ref))) + 1e-3) <= 2e-2
    exact = O.qmm_exact(x.float().numpy(), wq.numpy().view(np.uint32), s.float().numpy(), b.float().numpy(), 64)
    _check_north_star(_f32(y).astype(np.float64), exact)


@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("variant,kp", [("mma2big", 1), ("mma2big_pipe", 1), ("mma2big_pipe", 2),
                                        ("mma2big_pipe", 4), ("mma2big_pipe", 8)])
def test_group_sizes_and_variants(verify_env, native_lib, c_oracle, gs, variant, kp):
    verify_env.setenv("DFLASH_VERIFY_VARIANT", variant)
    verify_env.setenv("DFLASH_VERIFY_QMM_KPARTS", str(kp))
    for K, N in [(1024, 96), (256, 32), (2304, 160)]:
        case = make_qmm_case(K, N, 100 + gs + kp, group_size=gs)
        y = _f32(_run(case)).astype(np.float64)
        _check_north_star(y, _oracle_exact(c_oracle, case))


def test_fp16_activations_and_scales(verify_env, native_lib):
    for sdt in (torch.float16, torch.bfloat16):
        case = make_qmm_case(1024, 128, 7, dtype=torch.float16)
        case.scales = case.scales.to(sdt)
        case.biases = (-8.0 * case.scales.float()).to(sdt)
        y = _f32(_run(case)).astype(np.float64)
        exact = O.qmm_exact(case.x.float().numpy(), case.w.numpy().view(np.uint32),
                            case.scales.float().numpy(), case.biases.float().numpy(), 64)
        err = np.abs(y - exact)
        assert np.all(err <= 2e-3 * np.max(np.abs(exact), axis=1, keepdims=True))
        assert np.linalg.norm(y - exact) / np.linalg.norm(exact) <= 1e-3


def test_known_answers_on_device(verify_env, native_lib):
    K, N, gs = 512, 64, 64
    case = make_qmm_case(K, N, 11)
    # (1) all codes 8 with bias = -8*scale: every weight is zero
    zero = make_qmm_case(K, N, 11)
    zero.w = torch.full_like(zero.w, 0x88888888 - 2 ** 32)
    y = _f32(_run(zero))
    bound = 1e-5 * float(case.scales.float().max()) * float(case.x.float().abs().sum(dim=1).max())
    assert np.max(np.abs(y)) <= bound
    # (2) one-hot rows read single weights: y[m, n] == bf16(s*q + b) exactly
    ks = torch.randint(0, K, (16,), generator=torch.Generator().manual_seed(5))
    hot = make_qmm_case(K, N, 11)
    hot.x = torch.zeros_like(hot.x)
    hot.x[torch.arange(16), ks] = 1.0
    y = _f32(_run(hot))
    wd = O.dequant_affine(hot.w.numpy().view(np.uint32), hot.scales.float().numpy(), hot.biases.float().numpy(), gs)
    want = O.round_bf16(wd[:, ks.numpy()].T.astype(np.float32))
    assert np.array_equal(y, want)
    # (3) nibble order: codes 0..7 in every word, s=1, b=0, x = e_k  ->  y = k % 8
    seq = make_qmm_case(K, N, 11)
    seq.w = torch.full_like(seq.w, 0x76543210)
    seq.scales = torch.ones_like(seq.scales)
    seq.biases = torch.zeros_like(seq.biases)
    seq.x = hot.x
    y = _f32(_run(seq))
    assert np.array_equal(y, np.repeat((ks.numpy() % 8)[:, None], N, axis=1).astype(np.float32))


def test_deterministic_and_workspace_reuse(verify_env, native_lib, c_oracle):
    a = make_qmm_case(4096, 4096, 21).to(DEV)
    b = make_qmm_case(1024, 512, 22).to(DEV)
    ya = [VQ.verify_matmul(a.x, a.w, a.scales, a.biases) for _ in range(3)]
    yb = VQ.verify_matmul(b.x, b.w, b.scales, b.biases)
    ya.append(VQ.verify_matmul(a.x, a.w, a.scales, a.biases))
    torch.cuda.synchronize()
    for y in ya[1:]:
        assert torch.equal(y, ya[0])
    _check_north_star(_f32(yb).astype(np.float64), _oracle_exact(c_oracle, b.to("cpu")))


def test_every_kernel_hands_the_shared_workspace_back_zero_filled(verify_env, native_lib, c_oracle):
    """The streaming kernel takes a non-zero word in a partial-tile slot for a tile that has
    arrived, so every kernel that writes partial tiles puts them back to zero: the streaming
    kernel itself, the tile kernel's split-K form, the chained and the gathered form.  One
    workspace through all of them, checked after each, with the streaming kernel's result still
    right (and the same bits as with a workspace of its own) at the end."""
    verify_env.setenv("DFLASH_QMM_KERNEL", "auto")
    ws = VQ._workspace(torch.device(DEV), nat.raw_stream(torch.device(DEV)), 1)

    def clean():
        torch.cuda.synchronize()
        word = ctypes.c_uint32(7)
        assert native_lib.dflash_qmm_error(ws.data_ptr(), ctypes.byref(word), None) == 0 and word.value == 0
        return int((ws != 0).sum()) == 0

    a = make_qmm_case(5120, 7168, 31).to(DEV)       # streaming kernel, four workgroups per row block
    b = make_qmm_case(4096, 1536, 32).to(DEV)       # row blocks that straddle unit ranges
    ya = VQ.verify_matmul(a.x, a.w, a.scales, a.biases)
    yb = VQ.verify_matmul(b.x, b.w, b.scales, b.biases)
    assert clean()
    verify_env.setenv("DFLASH_QMM_KERNEL", "tile")  # split-K form of the tile kernel (K >= 8192 -> pipe x 8)
    c = make_qmm_case(8192, 512, 33).to(DEV)
    yc = VQ.verify_matmul(c.x, c.w, c.scales, c.biases)
    verify_env.setenv("DFLASH_QMM_KERNEL", "auto")
    assert clean()
    chain = VQ.QmmChain([VQ.ChainProblem(a.x, a.w, a.scales, a.biases), VQ.ChainProblem(b.x, b.w, b.scales, b.biases)])
    chained = chain()
    assert clean()
    assert torch.equal(chained[0], ya) and torch.equal(chained[1], yb)
    ya2 = VQ.verify_matmul(a.x, a.w, a.scales, a.biases)
    assert clean() and torch.equal(ya2, ya)
    _check_north_star(_f32(ya2).astype(np.float64), _oracle_exact(c_oracle, a.to("cpu")))
    _check_north_star(_f32(yc).astype(np.float64), _oracle_exact(c_oracle, c.to("cpu")))


def test_adding_workgroup_that_gives_up_says_so_and_the_launch_ends(verify_env, native_lib):
    """The wait of the streaming kernel's adding workgroups cut to two polls from the host (an
    option of the library): the launch ends like any other, the workgroups that found a tile
    missing leave the error word behind, `raise_on_device_errors` turns it into an exception and
    zero-fills the workspace - late tiles may sit in it - and the next launch, with the wait at its
    default, is right again.  5120 x 17408: 136 row blocks, each shared by two or three workgroups
    that finish microseconds apart, so some of the 136 waits are cut short in any run."""
    verify_env.setenv("DFLASH_QMM_KERNEL", "auto")
    case = make_qmm_case(5120, 17408, 41).to(DEV)
    good = VQ.verify_matmul(case.x, case.w, case.scales, case.biases)
    torch.cuda.synchronize()
    VQ.raise_on_device_errors(torch.device(DEV))                       # nothing to report
    assert native_lib.dflash_set_option(nat.OPT_QMM_SPIN_LIMIT, 1) == 0
    try:
        VQ.verify_matmul(case.x, case.w, case.scales, case.biases)
        torch.cuda.synchronize()                                       # the launch ends
    finally:
        assert native_lib.dflash_set_option(nat.OPT_QMM_SPIN_LIMIT, 0) == 0
    with pytest.raises(nat.NativeLibraryError, match="partial tiles of row block"):
        VQ.raise_on_device_errors(torch.device(DEV))
    ws = VQ._workspace(torch.device(DEV), nat.raw_stream(torch.device(DEV)), 1)
    assert int((ws != 0).sum()) == 0
    again = VQ.verify_matmul(case.x, case.w, case.scales, case.biases)
    torch.cuda.synchronize()
    VQ.raise_on_device_errors(torch.device(DEV))
    assert torch.equal(again, good)


def test_n_tiles_are_independent_full_size(verify_env, native_lib, kernel_mode):
    """Size-independent property at a full 27B shape: any N-slice of W gives the matching
    slice of the full product - the same bits with the tile kernel (fixed K split), and to
    within one output rounding with the streaming kernel, whose K split follows the even
    division of the whole matrix among workgroups and therefore changes with N."""
    case = make_qmm_case(5120, 17408, 31).to(DEV)
    full = VQ.verify_matmul(case.x, case.w, case.scales, case.biases)
    for n0, n1 in [(0, 32), (4096, 4096 + 512), (17408 - 64, 17408)]:
        part = VQ.verify_matmul(case.x, case.w[n0:n1], case.scales[n0:n1], case.biases[n0:n1])
        if kernel_mode == "tile":
            assert torch.equal(part, full[:, n0:n1])
        else:
            ref = full[:, n0:n1].float()
            assert (part.float() - ref).abs().max() <= 2 ** -7 * ref.abs().max()
            assert (part == full[:, n0:n1]).float().mean() > 0.95


def test_linearity_full_size(verify_env, native_lib):
    case = make_qmm_case(17408, 5120, 32).to(DEV)
    x2 = torch.randn_like(case.x.float()).to(torch.bfloat16)
    # 2*x and x+x2 are formed in bf16 so that every operand is exactly representable
    xs = (case.x.float() + x2.float()).to(torch.bfloat16)
    exact_sum = xs.float() - case.x.float() - x2.float()
    y1 = VQ.verify_matmul(case.x, case.w, case.scales, case.biases).float()
    y2 = VQ.verify_matmul(x2, case.w, case.scales, case.biases).float()
    ys = VQ.verify_matmul(xs, case.w, case.scales, case.biases).float()
    yr = VQ.verify_matmul(exact_sum.to(torch.bfloat16), case.w, case.scales, case.biases).float()
    resid = (ys - y1 - y2 - yr).abs().max().item()
    assert resid <= 4 * 2 ** -8 * max(y1.abs().max().item(), y2.abs().max().item())


def test_random_shapes_repeat_bit_for_bit_and_stay_close(verify_env, native_lib):
    """Shapes drawn at random (every split of the rows and of K over the workgroups comes up):
    each call gives the same bits when repeated at once and again later, after other shapes
    have used the workspace, and stays within the bf16 bar of an fp32 product on the device."""
    gen = torch.Generator(device=DEV).manual_seed(seed_for(0, 77))
    draw = torch.Generator().manual_seed(seed_for(0, 78))
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=draw))
    shifts = torch.arange(8, device=DEV, dtype=torch.int32) * 4
    earlier = []
    for i in range(48):
        K = 512 * pick(1, 34)
        N = 16 * pick(1, 1200) if i % 3 else 64 * pick(1, 300)
        dtype = torch.float16 if i % 4 == 0 else torch.bfloat16
        x = torch.randn((16, K), generator=gen, device=DEV).to(dtype)
        w = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), generator=gen, device=DEV).to(torch.int32)
        s = (torch.randn((N, K // 64), generator=gen, device=DEV).abs() * 0.02 + 1e-4).to(dtype)
        b = (-8 * s.float() + 0.01 * torch.randn((N, K // 64), generator=gen, device=DEV)).to(dtype)
        first, second = (VQ.verify_matmul(x, w, s, b, group_size=64, bits=4).clone() for _ in range(2))
        codes = ((w.unsqueeze(-1) >> shifts) & 15).reshape(N, K).float()
        dense = codes * s.float().repeat_interleave(64, 1) + b.float().repeat_interleave(64, 1)
        exact = x.float() @ dense.t()
        assert torch.equal(first, second), f"K={K} N={N} {dtype}: two calls in a row differ"
        rel = ((first.float() - exact).norm() / exact.norm()).item()
        assert rel <= 5e-3, f"K={K} N={N} {dtype}: rel-L2 {rel:.3g}"
        earlier.append((K, N, x, w, s, b, first))
        if len(earlier) == 8:
            again = [VQ.verify_matmul(e[2], e[3], e[4], e[5], group_size=64, bits=4).clone() for e in earlier]
            for e, y in zip(earlier, again):
                assert torch.equal(y, e[6]), f"K={e[0]} N={e[1]}: differs after other shapes ran"
            earlier = []


@pytest.mark.parametrize("K,N,rows", [(5120, 151936, 16), (2048, 262144, 5)])
def test_vocabulary_sized_projection(verify_env, native_lib, kernel_mode, K, N, rows):
    """An output head: more rows of W than any layer projection has (1187 and 2048 row blocks).
    16 rows through verify_matmul, fewer through the stock operator's small-M route."""
    if kernel_mode == "tile":
        pytest.skip("one kernel is enough at this size")
    gen = torch.Generator(device=DEV).manual_seed(seed_for(0, 91))
    x = torch.randn((rows, K), generator=gen, device=DEV).to(torch.bfloat16)
    w = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), generator=gen, device=DEV).to(torch.int32)
    s = (torch.randn((N, K // 64), generator=gen, device=DEV).abs() * 0.02 + 1e-4).to(torch.bfloat16)
    b = (-8 * s.float()).to(torch.bfloat16)
    run = (lambda: VQ.verify_matmul(x, w, s, b, group_size=64, bits=4)) if rows == 16 else \
        (lambda: stock_matmul(x, w, s, b, transpose=True, group_size=64, bits=4))
    y = run()
    assert y.shape == (rows, N) and torch.equal(y, run())
    shifts = torch.arange(8, device=DEV, dtype=torch.int32) * 4
    exact = torch.empty((rows, N), dtype=torch.float32, device=DEV)
    for n0 in range(0, N, 16384):
        rows_w = slice(n0, min(n0 + 16384, N))
        codes = ((w[rows_w].unsqueeze(-1) >> shifts) & 15).reshape(-1, K).float()
        dense = codes * s[rows_w].float().repeat_interleave(64, 1) + b[rows_w].float().repeat_interleave(64, 1)
        exact[:, rows_w] = x.float() @ dense.t()
    rel = ((y.float() - exact).norm() / exact.norm()).item()
    assert rel <= 5e-3, rel


def test_leading_shapes_and_stock_fallbacks_on_device(verify_env, native_lib):
    case = make_qmm_case(512, 64, 41).to(DEV)
    y = VQ.verify_matmul(case.x, case.w, case.scales, case.biases)
    for shape in [(1, 16, 512), (4, 4, 512), (2, 2, 4, 512)]:
        yr = VQ.verify_matmul(case.x.reshape(shape), case.w, case.scales, case.biases)
        assert yr.shape == (*shape[:-1], 64) and torch.equal(yr.reshape(16, 64), y)
    # M != 16 and fp32 activations use the stock operator
    x8 = case.x[:8]
    assert torch.equal(VQ.verify_matmul(x8, case.w, case.scales, case.biases),
                       quantized_matmul(x8, case.w, case.scales, case.biases))
    xf = case.x.float()
    assert torch.equal(VQ.verify_matmul(xf, case.w, case.scales, case.biases),
                       quantized_matmul(xf, case.w, case.scales, case.biases))
    verify_env.setenv("DFLASH_VERIFY_QMM", "0")
    assert torch.equal(VQ.verify_matmul(case.x, case.w, case.scales, case.biases),
                       quantized_matmul(case.x, case.w, case.scales, case.biases))


def test_verify_linear_on_device(verify_env, native_lib):
    """tests/test_verify_linear_parity.py:50-72 - M != 16 identical to stock, M == 16
    identical to a direct verify_matmul call."""
    torch.manual_seed(0)
    lin = torch.nn.Linear(512, 1024, bias=False)
    with torch.no_grad():
        lin.weight.mul_(0.1 / lin.weight.std())
    ql = QuantizedLinear.from_linear(lin.to(torch.bfloat16), 64, 4).to(DEV)
    v = VerifyQuantizedLinear.from_quantized(ql)
    for M in (1, 8, 32):
        x = (torch.randn(M, 512, device=DEV) * 0.5).to(torch.bfloat16)
        assert torch.equal(ql(x), v(x))
    x = (torch.randn(16, 512, device=DEV) * 0.5).to(torch.bfloat16)
    direct = VQ.verify_matmul(x, ql.weight, ql.scales, ql.biases, transpose=True, group_size=64, bits=4)
    assert torch.equal(direct, v(x))
    stock = ql(x).float()
    assert (direct.float() - stock).abs().max() <= 2e-2 * stock.abs().max()
    # a module moved after construction still dispatches on its current buffers
    v2 = VerifyQuantizedLinear.from_quantized(QuantizedLinear.from_linear(lin.to(torch.bfloat16), 64, 4)).to(DEV)
    assert torch.equal(v2(x), direct)


def test_shared_input_projections_in_one_launch(verify_env, native_lib, c_oracle, monkeypatch):
    """gate/up of an MLP joined into one launch: every member's output meets the bar against
    the exact product of its own rows, equals the columns of a direct call on the joint matrix,
    and M != 16 still takes the stock operator on the member's rows."""
    import dflash_mlx_amd.verify_linear as VL

    K = 1024
    cases = {"gate_proj": make_qmm_case(K, 1536, seed_for(0, 71)), "up_proj": make_qmm_case(K, 2048 + 32, seed_for(0, 72))}
    mlp = torch.nn.Module()
    for name, c in cases.items():
        setattr(mlp, name, QuantizedLinear(c.w.clone(), c.scales.clone(), c.biases.clone(), group_size=64, bits=4))
    model = torch.nn.Module()
    model.mlp = mlp.to(DEV)
    assert install_verify_linears(model) == 2 and fuse_shared_input_linears(model) == 1
    launches = []
    direct = VL.verify_matmul
    monkeypatch.setattr(VL, "verify_matmul", lambda x, w, *a, **k: (launches.append(int(w.shape[0])), direct(x, w, *a, **k))[1])
    x = cases["gate_proj"].x.to(DEV)
    out = dict(zip(cases, VL.shared_input_outputs(model.mlp, tuple(cases), x)))
    torch.cuda.synchronize()
    assert launches == [1536 + 2080]
    group = model.mlp.gate_proj._shared_input[0]
    # a member asked on its own answers from its rows, with a launch of its own
    alone = model.mlp.up_proj(x)
    assert launches == [1536 + 2080, 2080]
    assert torch.equal(alone, VQ.verify_matmul(x, group.weight[1536:], group.scales[1536:], group.biases[1536:],
                                               group_size=64, bits=4))
    del launches[1:]
    joint = VQ.verify_matmul(x, group.weight, group.scales, group.biases, group_size=64, bits=4)
    assert torch.equal(torch.cat([out["gate_proj"], out["up_proj"]], dim=-1), joint)
    for name, c in cases.items():
        exact, _ = c_oracle.qmm_m16(_bits(x), c.w.numpy().view(np.uint32), _bits(c.scales), _bits(c.biases), 64, flavour=0)
        _check_north_star(_f32(out[name]).astype(np.float64), exact.astype(np.float64))
    x3 = (torch.randn(3, K, device=DEV)).to(torch.bfloat16)
    c = cases["up_proj"].to(DEV)
    assert torch.equal(model.mlp.up_proj(x3), stock_matmul(x3, c.w, c.scales, c.biases))
    assert launches == [1536 + 2080]


def test_input_projections_of_a_linear_attention_layer_in_one_launch(verify_env, native_lib, c_oracle, monkeypatch):
    """qkv, z and the two 48-row gates (behind their pad-to-16 wrappers) read the same input: a
    16-token block takes one launch for the four of them, a shorter block (padded by the wrappers
    only) goes member by member, and every result meets the bar against its own exact product."""
    import dflash_mlx_amd.verify_linear as VL
    from dflash_mlx_amd.gdn_layer import _install_exact_small_proj_hooks

    K = 1024
    cases = {"in_proj_qkv": make_qmm_case(K, 1024, seed_for(0, 95)), "in_proj_z": make_qmm_case(K, 512, seed_for(0, 96)),
             "in_proj_b": make_qmm_case(K, 48, seed_for(0, 97)), "in_proj_a": make_qmm_case(K, 48, seed_for(0, 98))}
    la = torch.nn.Module()
    for name, c in cases.items():
        setattr(la, name, QuantizedLinear(c.w.clone(), c.scales.clone(), c.biases.clone(), group_size=64, bits=4))
    model = torch.nn.Module()
    model.linear_attn = la.to(DEV)
    assert install_verify_linears(model) == 2
    _install_exact_small_proj_hooks(model.linear_attn)
    assert fuse_shared_input_linears(model) == 1
    launches = []
    direct = VL.verify_matmul
    monkeypatch.setattr(VL, "verify_matmul", lambda x, w, *a, **k: (launches.append(int(w.shape[0])), direct(x, w, *a, **k))[1])
    x = cases["in_proj_qkv"].x.to(DEV).reshape(1, 16, K)
    out = dict(zip(cases, VL.shared_input_outputs(model.linear_attn, tuple(cases), x)))
    torch.cuda.synchronize()
    assert launches == [1024 + 512 + 48 + 48]
    for name, c in cases.items():
        exact, _ = c_oracle.qmm_m16(_bits(x.reshape(16, K)), c.w.numpy().view(np.uint32), _bits(c.scales), _bits(c.biases), 64,
                                    flavour=0)
        assert out[name].shape == (1, 16, c.N)
        _check_north_star(_f32(out[name].reshape(16, c.N)).astype(np.float64), exact.astype(np.float64))
    # a 3-token block: the wrappers pad the gates' input to 16 (a tensor of their own each), qkv and z see 3 rows
    x3 = x[:, :3]
    short = {n: getattr(model.linear_attn, n)(x3) for n in cases}
    torch.cuda.synchronize()
    for name, c in cases.items():
        assert short[name].shape == (1, 3, c.N)
        ref = out[name][:, :3].float()
        assert (short[name].float() - ref).abs().max() <= 2 ** -6 * ref.abs().max()


def test_stock_operator_takes_the_kernel_for_few_rows(verify_env, native_lib, c_oracle):
    """Outside the verify switch a module with at most 16 rows of device activations runs the
    M=16 kernel on zero-padded rows: a row's result does not depend on what shares its block, a
    48-row projection (which the Python gate of verify_matmul does not admit) is served, and
    DFLASH_STOCK_KERNEL=0 or more than 16 rows give the array-op form."""
    case = make_qmm_case(1024, 48, seed_for(0, 91))
    d = case.to(DEV)
    full = stock_matmul(d.x, d.w, d.scales, d.biases)
    exact, _ = c_oracle.qmm_m16(_bits(case.x), case.w.numpy().view(np.uint32), _bits(case.scales), _bits(case.biases), 64,
                                flavour=0)
    _check_north_star(_f32(full).astype(np.float64), exact.astype(np.float64))
    for rows in (slice(0, 1), slice(5, 6), slice(3, 12)):
        part = stock_matmul(d.x[rows], d.w, d.scales, d.biases)
        assert torch.equal(part, full[rows])
    assert torch.equal(stock_matmul(d.x[:4].reshape(2, 2, 1024), d.w, d.scales, d.biases), full[:4].reshape(2, 2, 48))
    ql = QuantizedLinear(d.w, d.scales, d.biases, group_size=64, bits=4)
    assert torch.equal(ql(d.x[2:3]), full[2:3])
    # the array-op form: asked for, or too many rows
    x20 = torch.cat([d.x, d.x[:4]])
    assert torch.equal(stock_matmul(x20, d.w, d.scales, d.biases), quantized_matmul(x20, d.w, d.scales, d.biases))
    verify_env.setenv("DFLASH_STOCK_KERNEL", "0")
    assert torch.equal(stock_matmul(d.x[:1], d.w, d.scales, d.biases), quantized_matmul(d.x[:1], d.w, d.scales, d.biases))
    # and verify_matmul's own fallback stays the array-op form (the reference's A/B switch)
    verify_env.delenv("DFLASH_STOCK_KERNEL")
    verify_env.setenv("DFLASH_VERIFY_QMM", "0")
    big = make_qmm_case(512, 64, 41).to(DEV)
    assert torch.equal(VQ.verify_matmul(big.x, big.w, big.scales, big.biases),
                       quantized_matmul(big.x, big.w, big.scales, big.biases))


def test_c_abi_direct_n16_and_errors(native_lib):
    """N % 32 != 0 is outside the Python gate but inside the C ABI contract (N % 16)."""
    L = native_lib
    case = make_qmm_case(1024, 48, 51).to(DEV)
    y = torch.empty((16, 48), dtype=torch.bfloat16, device=DEV)
    ws = torch.zeros(L.dflash_qmm_m16_workspace_bytes(1024, 48, 64, 1, 4, nat.QMM_KERNEL_AUTO),
                     dtype=torch.uint8, device=DEV)
    for variant, kp, kernel in ((0, 1, nat.QMM_KERNEL_TILE), (1, 4, nat.QMM_KERNEL_TILE),
                                (0, 1, nat.QMM_KERNEL_STREAM), (1, 4, nat.QMM_KERNEL_AUTO)):
        y.zero_()
        rc = L.dflash_qmm_m16(case.x.data_ptr(), case.w.data_ptr(), case.scales.data_ptr(),
                              case.biases.data_ptr(), y.data_ptr(), ws.data_ptr(), ws.numel(),
                              1024, 48, 64, nat.BF16, nat.BF16, variant, kp, kernel, None)
        assert rc == 0, L.dflash_last_error()
        torch.cuda.synchronize()
        exact = O.qmm_exact(case.x.float().cpu().numpy(), case.w.cpu().numpy().view(np.uint32),
                            case.scales.float().cpu().numpy(), case.biases.float().cpu().numpy(), 64)
        _check_north_star(_f32(y).astype(np.float64), exact)
    assert int(ws[:65536].view(torch.int32).abs().sum()) == 0   # counter block handed back zeroed
