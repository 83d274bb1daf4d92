"""Parity of the gfx950 GatedDeltaNet forward-with-tape kernel against the CPU oracle
(fp64 restatement of dflash_mlx/kernels.py:131-173), and its contract with the replay:
the tape it records, replayed for any prefix, gives the state the forward had there.

Bars: fp32 state and fp32 tape rel-L2 <= 2e-5; y (rounded to the input dtype) within one
rounding of the input dtype of the exact value; low-precision states compared against the
oracle run with the same per-step rounding."""
import numpy as np
import pytest
import torch

import dflash_mlx_amd._native as nat
from dflash_mlx_amd.gdn_layer import gated_norm
from dflash_mlx_amd.kernels import (_gated_delta_ops_with_tape, fused_output_norm_applies,
                                    gated_delta_kernel_with_tape, tape_replay_kernel)
from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(B=2, T=16, Hk=4, Hv=8, Dk=128, Dv=128, seed=0, g_per_dk=False, dtype=torch.bfloat16,
          state_dtype=torch.float32):
    g = torch.Generator().manual_seed(0xDF1A + seed)
    q = torch.randn((B, T, Hk, Dk), generator=g)
    k = torch.randn((B, T, Hk, Dk), generator=g)
    q = (q / q.norm(dim=-1, keepdim=True) * Dk ** -0.5).to(dtype)
    k = (k / k.norm(dim=-1, keepdim=True)).to(dtype)
    v = torch.randn((B, T, Hv, Dv), generator=g).to(dtype)
    gshape = (B, T, Hv, Dk) if g_per_dk else (B, T, Hv)
    gate = torch.exp(-torch.nn.functional.softplus(torch.randn(gshape, generator=g)))
    beta = torch.sigmoid(torch.randn((B, T, Hv), generator=g)).to(dtype)
    state = (torch.randn((B, Hv, Dv, Dk), generator=g) * 0.1).to(state_dtype)
    return q, k, v, gate, beta, state


def _f64(t):
    return t.detach().cpu().to(torch.float64).numpy()


def _rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def _run(args, mask=None):
    dev = [t.to(DEV) for t in args]
    y, s, tape = gated_delta_kernel_with_tape(*dev, mask=None if mask is None else mask.to(DEV))
    torch.cuda.synchronize()
    return y, s, tape


@pytest.mark.parametrize("g_per_dk", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_against_fp64_oracle(native_lib, g_per_dk, dtype):
    args = _case(seed=1 + int(g_per_dk), g_per_dk=g_per_dk, dtype=dtype)
    y, s, tape = _run(args)
    assert y.dtype == dtype and s.dtype == torch.float32 and tape.dtype == torch.float32
    yo, so, to = O.gated_delta_ops_with_tape(*[_f64(t) for t in args])
    assert _rel(_f64(s), so) <= 2e-5
    assert _rel(_f64(tape), to) <= 2e-5
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -20}[dtype]
    assert np.all(np.abs(_f64(y) - yo) <= eps * np.abs(yo) + 2e-5 * np.abs(yo).max())


def test_config2_shape_all_heads(native_lib):
    """32 value heads of 128 x 128 with 16 key heads, 16 steps: the GDN layer shape of config[2]."""
    args = _case(B=3, Hk=16, Hv=32, seed=7)
    y, s, tape = _run(args)
    yo, so, to = O.gated_delta_ops_with_tape(*[_f64(t) for t in args])
    assert _rel(_f64(s), so) <= 2e-5 and _rel(_f64(tape), to) <= 2e-5 and _rel(_f64(y), yo) <= 4e-3


def test_mask_skips_steps(native_lib):
    args = _case(seed=3)
    mask = torch.tensor([[1, 1, 0, 1, 0, 0, 1, 1, 1, 0, 1, 1, 1, 1, 0, 1],
                         [0, 0, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 0]], dtype=torch.bool)
    y, s, tape = _run(args, mask)
    yo, so, to = O.gated_delta_ops_with_tape(*[_f64(t) for t in args], mask=mask.numpy())
    assert _rel(_f64(s), so) <= 2e-5 and _rel(_f64(tape), to) <= 2e-5
    off = ~mask
    assert torch.all(tape.cpu()[off] == 0) and torch.all(y.cpu()[off] == 0)


def test_recorded_tape_replays_to_every_prefix_state(native_lib):
    """The contract between the two kernels (dflash_mlx/recurrent_rollback_cache.py:160-167)."""
    q, k, v, gate, beta, state = _case(seed=5)
    y, s_full, tape = _run((q, k, v, gate, beta, state))
    kd, gd, sd = k.to(DEV), gate.to(DEV), state.to(DEV)
    for a in (0, 1, 7, 16):
        prefix = [t[:, :a] for t in (q, k, v, gate, beta)]
        if a == 0:
            want = sd
        else:
            _, want, _ = _run(prefix + [state])
        got = tape_replay_kernel(tape[:, :a], kd[:, :a], gd[:, :a], sd) if a else sd
        assert _rel(_f64(got), _f64(want)) <= 2e-5
    assert _rel(_f64(tape_replay_kernel(tape, kd, gd, sd)), _f64(s_full)) <= 2e-5


@pytest.mark.parametrize("state_dtype", [torch.bfloat16, torch.float16])
def test_low_precision_state_is_rounded_after_every_step(native_lib, state_dtype):
    """kernels.py:96-98: the state goes through its storage type after every step."""
    args = _case(B=1, Hk=2, Hv=2, seed=9, state_dtype=state_dtype)
    y, s, tape = _run(args)
    assert s.dtype == state_dtype
    # the same recurrence on the host, fp32 arithmetic, rounding through the state dtype per step
    q, k, v, gate, beta, state = args
    S = state.float()
    tapes = []
    for t in range(q.shape[1]):
        _, S, tp = _gated_delta_ops_with_tape(q[:, t:t + 1].float(), k[:, t:t + 1].float(), v[:, t:t + 1].float(),
                                              gate[:, t:t + 1], beta[:, t:t + 1].float(), S)
        S = S.to(state_dtype).float()
        tapes.append(tp)
    assert _rel(_f64(s), _f64(S)) <= 2e-3            # one unit of the state dtype here and there
    assert _rel(_f64(tape), _f64(torch.cat(tapes, dim=1))) <= 2e-3


@pytest.mark.parametrize("shape", [dict(Dk=64, Dv=64), dict(Dk=96, Dv=32, Hk=2, Hv=2), dict(Dk=128, Dv=64),
                                   dict(T=3), dict(T=40, Hk=1, Hv=2, B=1)])
def test_other_shapes(native_lib, shape):
    args = _case(seed=11, **shape)
    y, s, tape = _run(args)
    yo, so, to = O.gated_delta_ops_with_tape(*[_f64(t) for t in args])
    assert _rel(_f64(s), so) <= 2e-5 and _rel(_f64(tape), to) <= 2e-5 and _rel(_f64(y), yo) <= 4e-3


@pytest.mark.parametrize("T", [1, 2, 7, 15, 16])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_closed_form_block_lengths(native_lib, T, dtype):
    """Scalar gate, fp32 state, 128 x 128 heads, T <= 16: the block kernel on the matrix cores,
    every block length with a ragged mask, against the fp64 oracle."""
    args = _case(B=2, T=T, Hk=2, Hv=4, seed=20 + T, dtype=dtype)
    mask = torch.ones((2, T), dtype=torch.bool)
    mask[1, T // 2] = False
    y, s, tape = _run(args, mask)
    yo, so, to = O.gated_delta_ops_with_tape(*[_f64(t) for t in args], mask=mask.numpy())
    assert _rel(_f64(s), so) <= 2e-5 and _rel(_f64(tape), to) <= 2e-5
    eps = {torch.bfloat16: 2.0 ** -8, torch.float32: 2.0 ** -20}[dtype]
    assert np.all(np.abs(_f64(y) - yo) <= eps * np.abs(yo) + 2e-5 * np.abs(yo).max())


def test_closed_form_with_vanishing_gates(native_lib):
    """Gates near 1e-4 per step: the running product leaves the fp32 range after a few steps,
    the ratios c_t / c_s between neighbouring steps do not.  Also gates of exactly 0 and 1."""
    q, k, v, gate, beta, state = _case(B=2, Hk=2, Hv=4, seed=31)
    gate = gate * 1e-4
    gate[0, 3, 1] = 0.0
    gate[1, :, 2] = 1.0
    args = (q, k, v, gate, beta, state)
    y, s, tape = _run(args)
    yo, so, to = O.gated_delta_ops_with_tape(*[_f64(t) for t in args])
    assert np.all(np.isfinite(_f64(s))) and np.all(np.isfinite(_f64(tape)))
    assert _rel(_f64(s), so) <= 2e-5 and _rel(_f64(tape), to) <= 2e-5 and _rel(_f64(y), yo) <= 4e-3


def test_closed_form_equals_the_sequential_kernel(native_lib, monkeypatch):
    """The two kernels for the same shape differ only in the order of fp32 additions."""
    args = _case(B=2, Hk=4, Hv=8, seed=33)
    mask = torch.ones((2, 16), dtype=torch.bool)
    mask[0, 5:8] = False
    block = _run(args, mask)
    assert native_lib.dflash_set_option(nat.OPT_GDN_STEP_BY_STEP, 1) == 0
    try:
        steps = _run(args, mask)
    finally:
        native_lib.dflash_set_option(nat.OPT_GDN_STEP_BY_STEP, 0)
    for a, b in zip(block, steps):
        assert _rel(_f64(a), _f64(b)) <= 2e-5
    assert _rel(_f64(block[2]), _f64(steps[2])) > 0     # two different kernels did run


@pytest.mark.parametrize("spread", ["even", "wide"])
def test_bf16_arrays_take_the_16_bit_matrix_cores_without_losing_a_bit(native_lib, spread):
    """With bf16 q and k the block kernel multiplies the fp32 state (cut exactly into three bf16
    pieces) on the bf16 matrix cores; with fp16 arrays it keeps the fp32 matrix cores.  The same
    numbers handed over either way must come back equally close to the fp64 result: 5e-7, forty
    times below the bar of the other tests, and far below the 2^-9 a state piece left out or
    rounded instead of cut would cost.  `wide`: state entries from 1e-12 to 1e+3 in one head."""
    q, k, v, gate, beta, state = _case(seed=21, dtype=torch.bfloat16)
    q, k, v, beta = [(t.float().clamp(-4, 4)) for t in (q, k, v, beta)]
    tiny = q.abs() < 2.0 ** -10                      # fp16 would hold these with fewer bits than bf16
    q = torch.where(tiny, torch.zeros_like(q), q)
    k = torch.where(k.abs() < 2.0 ** -10, torch.zeros_like(k), k)
    v = torch.where(v.abs() < 2.0 ** -10, torch.zeros_like(v), v)
    if spread == "wide":
        g = torch.Generator().manual_seed(77)
        state = state * torch.pow(10.0, torch.randint(-11, 5, state.shape, generator=g).float())
    got = {}
    for dt in (torch.bfloat16, torch.float16):
        args = [q.to(dt), k.to(dt), v.to(dt), gate, beta.to(dt), state]
        for a, b in zip(args[:3], (q, k, v)):
            assert torch.equal(a.float(), b)         # the same numbers in both dtypes
        ref = O.gated_delta_ops_with_tape(*[_f64(t) for t in args])
        y, s, tape = _run(args)
        assert _rel(_f64(s), ref[1]) <= 5e-7 and _rel(_f64(tape), ref[2]) <= 5e-7, (dt, spread)
        got[dt] = (s, tape)
    assert _rel(_f64(got[torch.bfloat16][0]), _f64(got[torch.float16][0])) <= 5e-7
    assert _rel(_f64(got[torch.bfloat16][1]), _f64(got[torch.float16][1])) <= 5e-7
    # Element by element: the two routes add the same exact products in another order, so a state
    # entry may differ by the roundings of its partial sums, never by more.  An entry is a sum of
    # T + 1 terms, each with a rounding of its own and the roundings of the delta it is made from:
    #   S_T = c_T S_0 + sum_t (c_T / c_t) delta_t (x) k_t,   c_t = g_1 .. g_t
    # Bar: 8 units in the last place of fp32 at the size of the entry's terms (not at the size of
    # the entry itself, which cancellation can make much smaller); 2.5 units are seen.  The third
    # bf16 piece of a state entry left out would cost 2^-16 of a term, sixteen times the bar.
    g64, k64, tape64, s064 = _f64(gate), _f64(k), ref[2], _f64(state)
    B, T, Hv = g64.shape
    rep = Hv // k64.shape[2]
    c = np.cumprod(g64, axis=1)                                   # [B, T, Hv]
    size = np.abs(c[:, -1][:, :, None, None] * s064)
    for t in range(T):
        w = (c[:, -1] / c[:, t])[:, :, None, None]
        size += np.abs(w * tape64[:, t][:, :, :, None] * np.repeat(k64[:, t], rep, axis=1)[:, :, None, :])
    diff = np.abs(_f64(got[torch.bfloat16][0]) - _f64(got[torch.float16][0]))
    assert np.all(diff <= 2.0 ** -20 * size), float((diff / (2.0 ** -23 * size + 1e-300)).max())


def test_errors_and_host_tensors(native_lib):
    q, k, v, gate, beta, state = _case(B=1, T=2, Hk=3, Hv=4, Dk=32, Dv=8)
    with pytest.raises(ValueError, match="Cannot align"):
        gated_delta_kernel_with_tape(q, k, v, gate, beta, state)
    q, k, v, gate, beta, state = _case(B=1, T=2, Hk=2, Hv=4, Dk=32, Dv=8)
    with pytest.raises(ValueError, match="Unsupported gating shape"):
        gated_delta_kernel_with_tape(q, k, v, gate[..., 0], beta, state)
    # host tensors: the array ops, as in the reference without its kernel
    y, s, tape = gated_delta_kernel_with_tape(q.float(), k.float(), v.float(), gate, beta.float(), state)
    yo, so, to = O.gated_delta_ops_with_tape(*[_f64(t) for t in (q, k, v, gate, beta, state)])
    assert _rel(_f64(s), so) <= 1e-5 and _rel(_f64(tape), to) <= 1e-5 and _rel(_f64(y), yo) <= 1e-5
    # the C entry point refuses aliasing and null pointers
    L = native_lib
    assert L.dflash_gdn_forward_tape(None, None, None, None, None, None, None, None, None, None,
                                     1, 1, 1, 1, 32, 8, 0, 2, 0, 2, 0, None) == -1


@pytest.mark.parametrize("accepted", [0, 5, 14])
def test_speculative_cycle_through_the_rollback_cache(native_lib, accepted):
    """One verify cycle of a GatedDeltaNet layer on the device (runtime.py:411-442, 878-907):
    arm, run the block with the tape recorded, roll back to `accepted` drafted tokens - the
    cache must hold what a run over only the committed accepted+1 tokens leaves."""
    from dflash_mlx_amd.recurrent_rollback_cache import RecurrentRollbackCache
    q, k, v, gate, beta, state = [t.to(DEV) for t in _case(B=1, Hk=4, Hv=8, seed=21)]
    C = 64
    gen = torch.Generator().manual_seed(5)
    conv0 = torch.randn((1, 3, C), generator=gen).to(torch.bfloat16).to(DEV)
    qkv = torch.randn((1, 16, C), generator=gen).to(torch.bfloat16).to(DEV)
    cache = RecurrentRollbackCache(size=2, conv_kernel_size=4)
    cache[0], cache[1] = conv0, state
    cache.arm_rollback()
    y, s_block, tape = gated_delta_kernel_with_tape(q, k, v, gate, beta, cache[1])
    cache.record_tape(tape=tape, k=k, g=gate, qkv=qkv)
    cache[0], cache[1] = qkv[:, -3:].clone(), s_block          # what the layer leaves after 16 tokens
    cache.rollback(accepted)
    torch.cuda.synchronize()
    n = accepted + 1
    y_n, s_n, _ = gated_delta_kernel_with_tape(q[:, :n], k[:, :n], v[:, :n], gate[:, :n], beta[:, :n], state)
    assert _rel(_f64(cache[1]), _f64(s_n)) <= 2e-5
    assert torch.equal(y[:, :n], y_n)                             # outputs of the kept tokens are the block's
    want_conv = torch.cat([conv0, qkv], dim=1)[:, n:n + 3]
    assert torch.equal(cache[0], want_conv)
    assert not cache._armed and cache._tape is None


@pytest.mark.parametrize("dtype,wdtype,state_dtype,T", [(torch.bfloat16, torch.bfloat16, torch.float32, 16),
                                                        (torch.float16, torch.float32, torch.float32, 16),
                                                        (torch.float32, torch.float32, torch.float32, 16),
                                                        (torch.bfloat16, torch.bfloat16, torch.float32, 5),
                                                        (torch.bfloat16, torch.bfloat16, torch.bfloat16, 16)])
def test_output_norm_in_the_same_launch(native_lib, dtype, wdtype, state_dtype, T):
    """silu(z) * rms_norm(y, weight) computed by the recurrence's launch: state and tape are those
    of the plain call bit for bit, and the output is the norm operator applied to the plain
    call's y - up to one rounding of the array dtype where the two add the squares in a different
    order (block kernel), exactly where the entry point runs the two kernels itself (bf16 state)."""
    args = [t.to(DEV) for t in _case(B=2, T=T, Hk=2, Hv=4, seed=40 + T, dtype=dtype, state_dtype=state_dtype)]
    g = torch.Generator().manual_seed(7)
    z = torch.randn((2, T, 4, 128), generator=g).to(dtype).to(DEV)
    weight = (1 + 0.2 * torch.randn(128, generator=g)).to(wdtype).to(DEV)
    mask = torch.ones((2, T), dtype=torch.bool)
    mask[1, T // 2] = False
    for m in (None, mask.to(DEV)):
        assert fused_output_norm_applies(args[0], args[2], args[5], z, weight)
        y, s_plain, tape_plain = gated_delta_kernel_with_tape(*args, mask=m)
        out, s_fused, tape_fused = gated_delta_kernel_with_tape(*args, mask=m, output_norm=(z, weight, 1e-6))
        torch.cuda.synchronize()
        assert torch.equal(s_plain, s_fused) and torch.equal(tape_plain, tape_fused)
        want = gated_norm(y, z, weight, 1e-6)
        if state_dtype != torch.float32:
            assert torch.equal(out, want)
        else:
            ulp = {torch.bfloat16: 2 ** -7, torch.float16: 2 ** -10, torch.float32: 2 ** -22}[dtype]
            w64, o64 = want.double(), out.double()
            assert bool(((o64 - w64).abs() <= 2 * ulp * w64.abs() + 1e-6).all())
            assert float((o64 - w64).norm() / w64.norm()) <= ulp / 4
        if m is not None:
            assert float(out[1, T // 2].abs().max()) == 0.0   # a masked step's output is zero, normed or not
    # a z of another shape is not taken
    assert not fused_output_norm_applies(args[0], args[2], args[5], z[..., :64], weight)
    with pytest.raises(ValueError):
        gated_delta_kernel_with_tape(*args, output_norm=(z[..., :64], weight, 1e-6))
