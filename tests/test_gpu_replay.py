"""Parity of the gfx950 tape-replay kernel and the rollback cache against the CPU oracle.

Bar: replayed fp32 state rel-L2 <= 1e-5 against the fp64 array-op restatement of
dflash_mlx/kernels.py:328-358; conv-window rebuild, KV trim and accepted-length
indexing bit-exact."""
import numpy as np
import pytest
import torch

from dflash_mlx_amd import runtime as R
from dflash_mlx_amd.cache import KVCache
from dflash_mlx_amd.kernels import _tape_replay_ops, replay_launch, tape_replay_kernel
from dflash_mlx_amd.recurrent_rollback_cache import (RecurrentRollbackCache, RollbackArena,
                                                     conv_state_rebuild)
from dflash_mlx_amd.workloads import make_replay_case
from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-5


def _rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64); b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def _np(t):
    return t.detach().cpu().float().numpy()


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _oracle_slots(case, steps, mask=None):
    """fp64 array-op replay per slot with its own step count."""
    L, B = case.state.shape[:2]
    S = L * B
    tape = _np(case.tape).reshape(S, *case.tape.shape[2:])
    k = _np(case.k).reshape(S, *case.k.shape[2:])
    g = _np(case.g).reshape(S, *case.g.shape[2:])
    st = _np(case.state).reshape(S, *case.state.shape[2:])
    out = np.empty(st.shape, dtype=np.float64)
    for s in range(S):
        a = int(steps[s])
        m = None if mask is None else mask[s:s + 1, :a]
        out[s] = O.tape_replay_ops(tape[s:s + 1, :a], k[s:s + 1, :a], g[s:s + 1, :a], st[s:s + 1], m)[0]
    return out.reshape(case.state.shape)


def _launch(case, steps, *, mask=None, exact=False):
    d = case.to(DEV)
    out = torch.empty_like(d.state)
    S = d.state.shape[0] * d.state.shape[1]
    m = None if mask is None else torch.from_numpy(mask.astype(np.uint8)).to(DEV)
    replay_launch(d.tape, d.k, d.g, d.state, out, steps=steps if isinstance(steps, int) else steps.to(DEV),
                  T_alloc=d.tape.shape[2], mask=m, slots=S, exact_order=exact)
    torch.cuda.synchronize()
    return out


def test_config2_full_size_against_c_oracle(native_lib, c_oracle):
    """BASELINE config[2]: 48 layers x 32 heads, 128x128 fp32 state, 16 recorded steps;
    every accepted length 0..16 appears among the slots."""
    case = make_replay_case(48, steps=16)
    steps = torch.arange(48, dtype=torch.int32) % 17
    out = _launch(case, steps)
    S = 48
    want = c_oracle.tape_replay(_bits(case.tape).reshape(S, 16, 32, 128), _bits(case.k).reshape(S, 16, 32, 128),
                                _np(case.g).reshape(S, 16, 32), _np(case.state).reshape(S, 32, 128, 128),
                                steps=steps.numpy())
    got = _np(out).reshape(S, 32, 128, 128)
    for s in range(S):
        assert _rel_l2(got[s], want[s]) <= TOL, (s, int(steps[s]))
    # zero accepted steps is a bit-exact copy
    assert np.array_equal(got[0], _np(case.state).reshape(S, 32, 128, 128)[0])
    assert np.array_equal(got[17], _np(case.state).reshape(S, 32, 128, 128)[17])


@pytest.mark.parametrize("exact", [False, True])
@pytest.mark.parametrize("g_per_dk", [False, True])
def test_fp64_oracle_all_step_counts(native_lib, exact, g_per_dk):
    case = make_replay_case(17, Hk=4, Hv=8, steps=16, g_per_dk=g_per_dk, seed=77)
    steps = torch.arange(17, dtype=torch.int32)
    out = _np(_launch(case, steps, exact=exact))
    want = _oracle_slots(case, steps.numpy())
    for s in range(17):
        assert _rel_l2(out[s], want[s]) <= TOL, s


def test_host_step_count_and_mask(native_lib):
    case = make_replay_case(3, batch=2, Hk=2, Hv=4, steps=16, seed=78)
    rng = np.random.default_rng(3)
    mask = rng.integers(0, 2, (6, 16)).astype(bool)
    for exact in (False, True):
        for a in (0, 1, 9, 16):
            out = _np(_launch(case, a, mask=mask, exact=exact))
            want = _oracle_slots(case, np.full(6, a), mask)
            assert _rel_l2(out, want) <= TOL
    # step counts outside [0, T] are clamped
    assert torch.equal(_launch(case, 99), _launch(case, 16))
    assert torch.equal(_launch(case, -3), case.state.to(DEV))


def test_closed_forms_on_device(native_lib):
    case = make_replay_case(2, Hk=2, Hv=2, steps=16, seed=79)
    zero = make_replay_case(2, Hk=2, Hv=2, steps=16, seed=79)
    zero.tape = torch.zeros_like(zero.tape)
    out = _np(_launch(zero, 16)).astype(np.float64)
    G = np.prod(_np(case.g).astype(np.float64), axis=2)            # [L,B,Hv]
    want = _np(case.state).astype(np.float64) * G[..., None, None]
    assert _rel_l2(out, want) <= 1e-6
    one = make_replay_case(2, Hk=2, Hv=2, steps=16, seed=79)
    one.g = torch.ones_like(one.g)
    out = _np(_launch(one, 1)).astype(np.float64)
    want = _np(case.state).astype(np.float64) + np.einsum("lbhv,lbhk->lbhvk", _np(case.tape)[:, :, 0], _np(case.k)[:, :, 0])
    assert _rel_l2(out, want) <= 1e-6


@pytest.mark.parametrize("shape", [dict(Hk=2, Hv=4, Dk=64, Dv=32), dict(Hk=1, Hv=3, Dk=96, Dv=40),
                                   dict(Hk=2, Hv=2, Dk=256, Dv=16), dict(Hk=4, Hv=4, Dk=128, Dv=128, T=8)])
def test_generic_shapes(native_lib, shape):
    T = shape.pop("T", 16)
    case = make_replay_case(3, T=T, steps=T, seed=80, **shape)
    steps = torch.tensor([0, T // 2, T], dtype=torch.int32)
    for exact in (False, True):
        out = _np(_launch(case, steps, exact=exact))
        assert _rel_l2(out, _oracle_slots(case, steps.numpy())) <= TOL


def test_fp32_tape_and_bf16_gate(native_lib):
    case = make_replay_case(2, Hk=2, Hv=2, steps=16, seed=81, tape_dtype=torch.float32)
    out = _np(_launch(case, 16))
    assert _rel_l2(out, _oracle_slots(case, np.full(2, 16))) <= TOL
    case.g = case.g.to(torch.bfloat16)
    out = _np(_launch(case, 16))
    assert _rel_l2(out, _oracle_slots(case, np.full(2, 16))) <= TOL


@pytest.mark.parametrize("g_per_dk", [False, True])
@pytest.mark.parametrize("tape_dt,k_dt,g_dt", [(torch.bfloat16, torch.bfloat16, torch.float32),
                                               (torch.float16, torch.float16, torch.float16),
                                               (torch.float32, torch.bfloat16, torch.bfloat16),
                                               (torch.bfloat16, torch.float32, torch.float32),
                                               (torch.float32, torch.float32, torch.float32)])
def test_matrix_core_kernel_dtypes_masks_and_short_tapes(native_lib, tape_dt, k_dt, g_dt, g_per_dk):
    """The 128 x 128 kernel fetches the tape as raw 16-byte pieces and sorts out dtype, mask and
    accepted length afterwards: every combination of 2- and 4-byte tape, k and gate, per-head
    and per-element gates, with a mask, per-slot lengths and a tape of fewer than 16 steps."""
    for T in (16, 5):
        case = make_replay_case(3, batch=2, T=T, Hk=2, Hv=4, steps=T, g_per_dk=g_per_dk, seed=90 + T, tape_dtype=tape_dt)
        case.k = case.k.to(k_dt)
        case.g = case.g.to(g_dt)
        rng = np.random.default_rng(T)
        mask = rng.integers(0, 4, (6, T)) > 0
        steps = torch.tensor([0, 1, T // 2, T - 1, T, T], dtype=torch.int32)
        for m in (None, mask):
            out = _np(_launch(case, steps, mask=m))
            want = _oracle_slots(case, steps.numpy(), m)
            for s in range(6):
                assert _rel_l2(out.reshape(6, -1)[s], want.reshape(6, -1)[s]) <= TOL, (T, s, m is not None)


@pytest.mark.parametrize("name,dt", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_low_precision_state_rounds_every_step(native_lib, name, dt):
    """kernels.py:281-283: a bf16/fp16 state is rounded after every step."""
    case = make_replay_case(2, Hk=2, Hv=2, Dk=64, Dv=16, steps=16, seed=82)
    case.state = case.state.to(dt)
    out = _launch(case, 16)
    assert out.dtype == dt
    want = O.tape_replay_kernel_semantics(_np(case.tape).reshape(2, 16, 2, 16), _np(case.k).reshape(2, 16, 2, 64),
                                          _np(case.g).reshape(2, 16, 2), _np(case.state).reshape(2, 2, 16, 64),
                                          state_dtype=name)
    got = _np(out).reshape(2, 2, 16, 64)
    ulp = 2.0 ** (-8 if name == "bf16" else -11)
    # identical arithmetic up to fused multiply-add contraction: at most one ulp apart, rarely
    assert np.max(np.abs(got - want)) <= ulp * np.max(np.abs(want))
    assert np.mean(got == want) > 0.98


def test_functional_form_and_prefix_slices(native_lib):
    """tape_replay_kernel(tape[:, :a], k[:, :a], g[:, :a], state): the slices are
    non-contiguous for B > 1 and are consumed without a copy."""
    case = make_replay_case(1, batch=3, Hk=2, Hv=4, steps=16, seed=83).to(DEV)
    tape, k, g, st = case.tape[0], case.k[0], case.g[0], case.state[0]
    for a in (1, 5, 16):
        got = tape_replay_kernel(tape[:, :a], k[:, :a], g[:, :a], st)
        want = _tape_replay_ops(tape[:, :a].double(), k[:, :a].double(), g[:, :a].double(), st.double())
        assert got.dtype == st.dtype and got.data_ptr() != st.data_ptr()
        assert _rel_l2(_np(got), want.cpu().numpy()) <= TOL
        # the step count instead of the three views: the same launch, the same bits
        assert torch.equal(tape_replay_kernel(tape, k, g, st, steps=a), got)
    assert torch.equal(tape_replay_kernel(tape, k, g, st, steps=0), st)
    assert torch.equal(tape_replay_kernel(tape, k, g, st, steps=99), tape_replay_kernel(tape, k, g, st))
    mask = torch.rand(3, 16, device=DEV) > 0.4
    got = tape_replay_kernel(tape, k, g, st, mask)
    want = _tape_replay_ops(tape.double(), k.double(), g.double(), st.double(), mask)
    assert _rel_l2(_np(got), want.cpu().numpy()) <= TOL
    assert torch.equal(tape_replay_kernel(tape, k, g, st, mask, steps=7), tape_replay_kernel(tape[:, :7], k[:, :7], g[:, :7], st, mask[:, :7]))
    # Dk not a multiple of 32 takes the array-op route, as in the reference (kernels.py:374-375)
    odd = make_replay_case(1, batch=2, Hk=2, Hv=2, Dk=48, Dv=8, steps=4, T=4, seed=84).to(DEV)
    got = tape_replay_kernel(odd.tape[0], odd.k[0], odd.g[0], odd.state[0])
    assert torch.equal(got, _tape_replay_ops(odd.tape[0], odd.k[0], odd.g[0], odd.state[0]))
    with pytest.raises(ValueError):
        tape_replay_kernel(tape[:, :, :3], k, g[:, :, :3], st[:, :3])


def test_conv_rebuild_kernel_bit_exact(native_lib):
    rng = np.random.default_rng(5)
    for C, dt in ((10240, torch.bfloat16), (6, torch.float32), (7, torch.bfloat16)):
        qkv = torch.from_numpy(rng.standard_normal((4, 16, C)).astype(np.float32)).to(dt)
        prev = torch.from_numpy(rng.standard_normal((4, 3, C)).astype(np.float32)).to(dt)
        for p in (prev, None):
            for steps in (0, 1, 2, 3, 7, 16):
                got = conv_state_rebuild(None if p is None else p.to(DEV), qkv.to(DEV), steps, 3)
                want = O.rebuild_conv_state(None if p is None else p.float().numpy(), qkv.float().numpy(), steps, 4)
                assert np.array_equal(got.cpu().float().numpy(), want)
    st = torch.tensor([0, 3, 9, 16], dtype=torch.int32, device=DEV)
    got = conv_state_rebuild(prev.to(DEV), qkv.to(DEV), st, 3)
    for s in range(4):
        want = O.rebuild_conv_state(prev[s:s + 1].float().numpy(), qkv[s:s + 1].float().numpy(), int(st[s]), 4)
        assert np.array_equal(got[s:s + 1].cpu().float().numpy(), want)


def _gdn_cycle_inputs(seed, L=4, B=1, T=16, Hk=4, Hv=8, Dk=128, Dv=128, C=96):
    case = make_replay_case(L, batch=B, T=T, Hk=Hk, Hv=Hv, Dk=Dk, Dv=Dv, steps=T, seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    qkv = torch.randn((L, B, T, C), generator=g).to(torch.bfloat16)
    conv0 = torch.randn((L, B, 3, C), generator=g).to(torch.bfloat16)
    return case, qkv, conv0


def test_rollback_cache_on_device_matches_oracle_model(native_lib):
    case, qkv, conv0 = _gdn_cycle_inputs(90, L=1)
    for acc in (0, 7, 14):
        model = O.RollbackCacheModel()
        model.cache = [conv0[0].float().numpy(), _np(case.state[0]).astype(np.float64)]
        cache = RecurrentRollbackCache(size=2, conv_kernel_size=4)
        cache[0], cache[1] = conv0[0].to(DEV), case.state[0].to(DEV)
        model.arm_rollback(); cache.arm_rollback(prefix_len=123)
        snap_ptr = cache[1].data_ptr()
        # the verify forward leaves some other state / conv window behind
        cache[1] = torch.randn_like(cache[1]); cache[0] = torch.randn_like(cache[0].float()).to(torch.bfloat16)
        model.record_tape(tape=_np(case.tape[0]).astype(np.float64), k=_np(case.k[0]).astype(np.float64),
                          g=_np(case.g[0]).astype(np.float64), qkv=qkv[0].float().numpy())
        cache.record_tape(tape=case.tape[0].to(DEV), k=case.k[0].to(DEV), g=case.g[0].to(DEV), qkv=qkv[0].to(DEV))
        model.rollback(acc); cache.rollback(acc)
        torch.cuda.synchronize()
        assert _rel_l2(_np(cache[1]), model.cache[1]) <= TOL
        assert cache[1].data_ptr() != snap_ptr               # snapshot tensor left untouched
        assert np.array_equal(cache[0].cpu().float().numpy(), model.cache[0])
        assert cache._snapshot is None and cache._tape is None and not cache._armed


@pytest.mark.parametrize("batch,with_window", [(1, True), (3, True), (2, False)])
def test_rollback_in_one_library_call_equals_the_two_wrappers(native_lib, monkeypatch, batch, with_window):
    """``rollback`` of a cache outside an arena makes one ``dflash_rollback_layer`` call; with that
    path switched off it goes through ``tape_replay_kernel`` and ``conv_state_rebuild``.  Same
    state and conv window bit for bit, for every accepted length, several batch rows and a cache
    that had no conv window when it was armed."""
    case, qkv, conv0 = _gdn_cycle_inputs(91, L=1, B=batch)
    used = []
    real = RecurrentRollbackCache._rollback_in_one_call

    def run(acc, one_call):
        cache = RecurrentRollbackCache(size=2, conv_kernel_size=4)
        cache[0], cache[1] = (conv0[0].to(DEV) if with_window else None), case.state[0].to(DEV)
        cache.arm_rollback(prefix_len=7)
        cache.record_tape(tape=case.tape[0].to(DEV), k=case.k[0].to(DEV), g=case.g[0].to(DEV), qkv=qkv[0].to(DEV))
        monkeypatch.setattr(RecurrentRollbackCache, "_rollback_in_one_call",
                            (lambda self, n: used.append(n) or real(self, n)) if one_call else (lambda self, n: False))
        cache.rollback(acc)
        torch.cuda.synchronize()
        return cache[0], cache[1]

    for acc in (0, 1, 6, 14, 15):
        used.clear()
        conv_a, state_a = run(acc, True)
        assert used == [acc + 1]
        conv_b, state_b = run(acc, False)
        assert torch.equal(state_a, state_b) and torch.equal(conv_a, conv_b)
        assert state_a.data_ptr() != state_b.data_ptr()


def test_rollback_outside_the_one_call_case_takes_the_wrappers(native_lib):
    """Per-element gates are not what the one-call path takes: it declines, and the result is
    the oracle model's all the same."""
    case = make_replay_case(1, batch=1, T=8, Hk=2, Hv=4, Dk=128, Dv=128, steps=8, seed=93, g_per_dk=True)
    g = torch.Generator().manual_seed(94)
    qkv = torch.randn((1, 8, 64), generator=g).to(torch.bfloat16)
    conv0 = torch.randn((1, 3, 64), generator=g).to(torch.bfloat16)
    model = O.RollbackCacheModel()
    model.cache = [conv0.float().numpy(), _np(case.state[0]).astype(np.float64)]
    cache = RecurrentRollbackCache(size=2, conv_kernel_size=4)
    cache[0], cache[1] = conv0.to(DEV), case.state[0].to(DEV)
    model.arm_rollback(); cache.arm_rollback()
    model.record_tape(tape=_np(case.tape[0]).astype(np.float64), k=_np(case.k[0]).astype(np.float64),
                      g=_np(case.g[0]).astype(np.float64), qkv=qkv.float().numpy())
    cache.record_tape(tape=case.tape[0].to(DEV), k=case.k[0].to(DEV), g=case.g[0].to(DEV), qkv=qkv.to(DEV))
    assert cache._rollback_in_one_call(4) is False and cache._tape is not None
    model.rollback(3); cache.rollback(3)
    torch.cuda.synchronize()
    assert _rel_l2(_np(cache[1]), model.cache[1]) <= TOL
    assert np.array_equal(cache[0].cpu().float().numpy(), model.cache[0])


def test_arena_batched_rollback_equals_per_layer(native_lib):
    L, B, T, Hk, Hv, Dk, Dv, C = 4, 1, 16, 4, 8, 128, 128, 96
    case, qkv, conv0 = _gdn_cycle_inputs(91, L=L, C=C)

    def run(batched, acc, device_steps=False):
        arena = RollbackArena(L, batch=B, max_steps=T, Hk=Hk, Hv=Hv, Dk=Dk, Dv=Dv, conv_dim=C, device=DEV)
        caches = R.make_target_cache([True, True, False, True, True, False], arena=arena)
        gdn = [c for c in caches if hasattr(c, "rollback")]
        for l, c in enumerate(gdn):
            c[1].copy_(case.state[l].to(DEV)); c[0].copy_(conv0[l].to(DEV))
        for c in caches:
            if isinstance(c, KVCache):
                c.offset = 4096 + 16
        R._arm_target_rollback_with_prefix(caches, prefix_len=4096)
        for l, c in enumerate(gdn):       # "verify forward": new state into the other half + tape
            nxt = arena.next_state(l); nxt.normal_()
            nconv = arena.next_conv(l); nconv.copy_(qkv[l, :, -3:].to(DEV))
            c[1], c[0] = nxt, nconv
            c.record_tape(tape=case.tape[l].to(DEV), k=case.k[l].to(DEV), g=case.g[l].to(DEV), qkv=qkv[l].to(DEV))
        if device_steps:
            arena.rollback_all(torch.tensor(acc, dtype=torch.int32, device=DEV))
            for c in caches:
                if isinstance(c, KVCache):
                    c.trim(c.offset - (4096 + acc + 1))
        elif batched:
            ns = R._restore_target_cache_after_acceptance(caches, target_len=4096 + acc + 1,
                                                          acceptance_length=acc, drafted_tokens=15)
            assert ns >= 0
        else:
            for c in caches:
                if hasattr(c, "rollback"):
                    c.rollback(acc)
                else:
                    c.trim(c.offset - (4096 + acc + 1))
        torch.cuda.synchronize()
        return ([c[1].clone() for c in gdn], [c[0].clone() for c in gdn],
                [c.offset for c in caches if isinstance(c, KVCache)])

    for acc in (0, 6, 14):
        s_b, c_b, o_b = run(True, acc)
        s_l, c_l, o_l = run(False, acc)
        s_d, c_d, o_d = run(True, acc, device_steps=True)
        assert o_b == o_l == o_d == [4096 + acc + 1] * 2
        for l in range(L):
            assert torch.equal(s_b[l], s_l[l]) and torch.equal(c_b[l], c_l[l])
            assert torch.equal(s_d[l], s_l[l]) and torch.equal(c_d[l], c_l[l])
            want = O.tape_replay_ops(_np(case.tape[l])[:, :acc + 1], _np(case.k[l])[:, :acc + 1],
                                     _np(case.g[l])[:, :acc + 1], _np(case.state[l]))
            assert _rel_l2(_np(s_b[l]), want) <= TOL
            wconv = O.rebuild_conv_state(conv0[l].float().numpy(), qkv[l].float().numpy(), acc + 1, 4)
            assert np.array_equal(c_b[l].cpu().float().numpy(), wconv)
    # everything accepted: the forward's state is kept, transients dropped
    s_f, _, o_f = run(True, 15)
    assert o_f == [4096 + 16] * 2


def test_mask_with_prefix_slices_of_a_longer_tape_and_several_batch_rows(native_lib):
    """tape[:, :a] of a 16-step recording is read in place (row count 16 per slot); the mask
    has `a` columns.  Every batch row must see its own mask row."""
    case = make_replay_case(1, batch=3, T=16, Hk=2, Hv=4, steps=16, seed=171, tape_dtype=torch.float32)
    d = case.to(DEV)
    rng = np.random.default_rng(172)
    for a in (1, 5, 11, 16):
        mask = rng.random((3, a)) < 0.6
        mask[1] = True
        m = torch.from_numpy(mask).to(DEV)
        tape, k, g = d.tape[0][:, :a], d.k[0][:, :a], d.g[0][:, :a]
        assert a == 16 or not tape.is_contiguous()
        got = tape_replay_kernel(tape, k, g, d.state[0], m)
        want = _tape_replay_ops(tape, k, g, d.state[0], m)
        torch.cuda.synchronize()
        assert _rel_l2(_np(got), _np(want)) <= TOL, a
        exact = O.tape_replay_ops(_np(case.tape[0])[:, :a], _np(case.k[0])[:, :a], _np(case.g[0])[:, :a],
                                  _np(case.state[0]), mask)
        assert _rel_l2(_np(got), exact) <= TOL, a


def test_arena_takes_per_batch_row_acceptance_and_other_tape_dtypes(native_lib):
    """One accepted count per batch row on the device is spread over the layers
    (slot = layer * B + row); a bf16 tape handed to an fp32 arena is converted."""
    L, B, T, Hk, Hv, Dk, Dv, C = 3, 2, 16, 2, 4, 128, 128, 64
    case = make_replay_case(L, batch=B, T=T, Hk=Hk, Hv=Hv, steps=T, seed=173)      # bf16 tape
    gen = torch.Generator().manual_seed(174)
    qkv = torch.randn((L, B, T, C), generator=gen).to(torch.bfloat16)
    arena = RollbackArena(L, batch=B, max_steps=T, Hk=Hk, Hv=Hv, Dk=Dk, Dv=Dv, conv_dim=C, device=DEV)
    assert arena.tape.dtype == torch.float32
    caches = arena.caches()
    for l, c in enumerate(caches):
        c[1].copy_(case.state[l].to(DEV))
    arena.arm_all(prefix_len=5)
    for l, c in enumerate(caches):
        c[1], c[0] = arena.next_state(l).normal_(), arena.next_conv(l).zero_()
        c.record_tape(tape=case.tape[l].to(DEV), k=case.k[l].to(DEV), g=case.g[l].to(DEV), qkv=qkv[l].to(DEV))
    acc = torch.tensor([3, 12], dtype=torch.int32, device=DEV)
    arena.rollback_all(acc)
    torch.cuda.synchronize()
    for l, c in enumerate(caches):
        for b, a in enumerate((4, 13)):
            want = O.tape_replay_ops(_np(case.tape[l])[b:b + 1, :a], _np(case.k[l])[b:b + 1, :a],
                                     _np(case.g[l])[b:b + 1, :a], _np(case.state[l])[b:b + 1])
            assert _rel_l2(_np(c[1][b:b + 1]), want) <= TOL, (l, b)
    with pytest.raises(ValueError):
        arena.arm_all()
        for l, c in enumerate(caches):
            c.record_tape(tape=case.tape[l].to(DEV), k=case.k[l].to(DEV), g=case.g[l].to(DEV), qkv=qkv[l].to(DEV))
        arena.rollback_all(torch.zeros(5, dtype=torch.int32, device=DEV))
