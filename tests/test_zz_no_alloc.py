"""dflash_qmm_m16_static, the entry point that allocates nothing: its workspace is an array
inside the library's device image.  Called through the C ABI and compared bit for bit with
dflash_qmm_m16 (caller's workspace) on calls in a row, each smaller than the one before or
of another kernel, so that what one call leaves in the array is what the next one finds."""
import ctypes

import numpy as np
import pytest
import torch

import dflash_mlx_amd._native as nat
from dflash_mlx_amd.workloads import make_qmm_case

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(lib, case, K, N, gs, variant, k_parts, kernel, ws):
    d = case.to("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    y_ref = torch.full((16, N), float("nan"), dtype=torch.bfloat16, device="cuda:0")
    y_new = torch.full((16, N), float("nan"), dtype=torch.bfloat16, device="cuda:0")
    rc = lib.dflash_qmm_m16(_ptr(d.x), _ptr(d.w), _ptr(d.scales), _ptr(d.biases), _ptr(y_ref), _ptr(ws),
                            ws.numel(), K, N, gs, nat.BF16, nat.BF16, variant, k_parts, kernel, stream)
    nat.check(rc, "dflash_qmm_m16")
    rc = lib.dflash_qmm_m16_static(_ptr(d.x), _ptr(d.w), _ptr(d.scales), _ptr(d.biases), _ptr(y_new),
                                   K, N, gs, nat.BF16, nat.BF16, variant, k_parts, kernel, stream)
    nat.check(rc, "dflash_qmm_m16_static")
    torch.cuda.synchronize()
    return y_ref, y_new


def test_static_scratch_matches_workspace_form_on_calls_in_a_row(native_lib):
    lib = native_lib
    ws = torch.zeros(nat.QMM_STATIC_SCRATCH_BYTES, dtype=torch.uint8, device="cuda:0")
    # (K, N, group, variant, k_parts, kernel): streaming kernel with shared row blocks, a smaller
    # one, the tile kernel's split-K form (other layout of partial tiles), streaming again
    calls = [
        (5120, 7168, 64, nat.QMM_MMA2BIG_PIPE, 8, nat.QMM_KERNEL_AUTO),
        (1024, 512, 64, nat.QMM_MMA2BIG_PIPE, 8, nat.QMM_KERNEL_AUTO),
        (2048, 256, 32, nat.QMM_MMA2BIG_PIPE, 8, nat.QMM_KERNEL_AUTO),
        (1024, 4096, 64, nat.QMM_MMA2BIG_PIPE, 8, nat.QMM_KERNEL_TILE),
        (4096, 4096, 64, nat.QMM_MMA2BIG_PIPE, 8, nat.QMM_KERNEL_STREAM),
        (512, 128, 64, nat.QMM_MMA2BIG, 1, nat.QMM_KERNEL_AUTO),
    ]
    for i, (K, N, gs, variant, k_parts, kernel) in enumerate(calls):
        print(f"static scratch call {i}: K={K} N={N} gs={gs} variant={variant} kernel={kernel}", flush=True)
        case = make_qmm_case(K, N, 4100 + i, group_size=gs)
        y_ref, y_new = _both(lib, case, K, N, gs, variant, k_parts, kernel, ws)
        assert torch.isfinite(y_new.float()).all()
        assert torch.equal(y_ref.view(torch.int16), y_new.view(torch.int16)), (K, N, gs)
        # and the product itself is right, not merely the same
        from oracle import dflash_oracle as O

        if K * N <= 1024 * 4096:
            exact = O.qmm_exact(case.x.float().numpy(), case.w.numpy().view(np.uint32),
                                case.scales.float().numpy(), case.biases.float().numpy(), gs)
            err = np.abs(y_new.float().cpu().numpy() - exact)
            assert (err <= 2e-2 * np.abs(exact).max(axis=1, keepdims=True)).all()


def test_static_scratch_rejects_what_does_not_fit(native_lib):
    lib = native_lib
    one = ctypes.c_void_p(256)  # never dereferenced: the size check comes first
    # tile kernel, 8 K slices of 16 x 32768 fp32: 16.8 MB of partial tiles
    rc = lib.dflash_qmm_m16_static(one, one, one, one, one, 4096, 32768, 64, nat.BF16, nat.BF16,
                                   nat.QMM_MMA2BIG_PIPE, 8, nat.QMM_KERNEL_TILE, None)
    assert rc == -3
    assert b"scratch" in lib.dflash_last_error()


def test_static_scratch_under_stream_capture(native_lib):
    """The entry point enqueues nothing but the product's kernel, so it can be captured - also as
    the first call of a process - and replayed; every replay equals the eager result."""
    lib = native_lib
    K, N = 5120, 5120
    d = make_qmm_case(K, N, 4200).to("cuda:0")
    ws = torch.zeros(nat.QMM_STATIC_SCRATCH_BYTES, dtype=torch.uint8, device="cuda:0")
    y_ref = torch.empty((16, N), dtype=torch.bfloat16, device="cuda:0")
    y_cap = torch.empty((16, N), dtype=torch.bfloat16, device="cuda:0")
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.dflash_qmm_m16_static(_ptr(d.x), _ptr(d.w), _ptr(d.scales), _ptr(d.biases), _ptr(y_cap), K, N, 64,
                                           nat.BF16, nat.BF16, nat.QMM_MMA2BIG_PIPE, 8, nat.QMM_KERNEL_AUTO,
                                           ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
            nat.check(rc, "dflash_qmm_m16_static under capture")
    torch.cuda.current_stream().wait_stream(side)
    rc = lib.dflash_qmm_m16(_ptr(d.x), _ptr(d.w), _ptr(d.scales), _ptr(d.biases), _ptr(y_ref), _ptr(ws), ws.numel(),
                            K, N, 64, nat.BF16, nat.BF16, nat.QMM_MMA2BIG_PIPE, 8, nat.QMM_KERNEL_AUTO,
                            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    nat.check(rc, "dflash_qmm_m16")
    torch.cuda.synchronize()
    for replay in range(3):
        y_cap.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_cap.view(torch.int16), y_ref.view(torch.int16)), replay
