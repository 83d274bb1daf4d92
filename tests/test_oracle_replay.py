"""Pins the replay / rollback / index oracle: forward-vs-replay consistency between two
independently written routines, closed forms, and exhaustive brute force for the
pure-index functions."""
import itertools

import numpy as np
import pytest

from oracle import dflash_oracle as O


def _gdn_case(rng, B=2, T=6, Hk=2, Hv=4, Dk=8, Dv=5, g_per_dk=False):
    q = rng.standard_normal((B, T, Hk, Dk))
    k = rng.standard_normal((B, T, Hk, Dk))
    k /= np.linalg.norm(k, axis=-1, keepdims=True)
    v = rng.standard_normal((B, T, Hv, Dv))
    gshape = (B, T, Hv, Dk) if g_per_dk else (B, T, Hv)
    g = np.exp(-np.log1p(np.exp(rng.standard_normal(gshape))))
    beta = 1.0 / (1.0 + np.exp(-rng.standard_normal((B, T, Hv))))
    S0 = rng.standard_normal((B, Hv, Dv, Dk)) * 0.1
    return q, k, v, g, beta, S0


@pytest.mark.parametrize("g_per_dk", [False, True])
def test_replay_reproduces_forward_prefix_states(g_per_dk):
    """replay(tape[:a]) from S0 must equal the forward's state after a steps, for all a."""
    rng = np.random.default_rng(10 + g_per_dk)
    q, k, v, g, beta, S0 = _gdn_case(rng, g_per_dk=g_per_dk)
    T = k.shape[1]
    _, S_T, tape = O.gated_delta_ops_with_tape(q, k, v, g, beta, S0)
    for a in range(T + 1):
        _, S_a, _ = O.gated_delta_ops_with_tape(q[:, :a], k[:, :a], v[:, :a], g[:, :a], beta[:, :a], S0) \
            if a > 0 else (None, S0, None)
        got = O.tape_replay_ops(tape[:, :a], k[:, :a], g[:, :a], S0)
        np.testing.assert_allclose(got, S_a, rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(O.tape_replay_ops(tape, k, g, S0), S_T, rtol=1e-12, atol=1e-13)


def test_forward_delta_rule_textbook_single_step():
    """One step from a zero state with g=1, beta=1: S = v (x) k, y = (k.q) v."""
    rng = np.random.default_rng(12)
    q, k, v, g, beta, S0 = _gdn_case(rng, B=1, T=1, Hk=1, Hv=1, Dk=4, Dv=3)
    g[:] = 1.0
    beta[:] = 1.0
    y, S, tape = O.gated_delta_ops_with_tape(q, k, v, g, beta, np.zeros_like(S0))
    np.testing.assert_allclose(S[0, 0], np.outer(v[0, 0, 0], k[0, 0, 0]), atol=1e-14)
    np.testing.assert_allclose(tape[0, 0, 0], v[0, 0, 0], atol=1e-14)
    np.testing.assert_allclose(y[0, 0, 0], v[0, 0, 0] * np.dot(k[0, 0, 0], q[0, 0, 0]), atol=1e-14)


def test_replay_closed_forms():
    rng = np.random.default_rng(13)
    B, T, Hk, Hv, Dk, Dv = 2, 5, 2, 4, 8, 6
    tape = rng.standard_normal((B, T, Hv, Dv)) * 0.05
    k = rng.standard_normal((B, T, Hk, Dk))
    g = rng.uniform(0.2, 1.0, (B, T, Hv))
    S0 = rng.standard_normal((B, Hv, Dv, Dk))
    # zero steps -> identity
    np.testing.assert_array_equal(O.tape_replay_ops(tape[:, :0], k[:, :0], g[:, :0], S0), S0)
    # delta == 0 -> pure decay by prod(g)
    got = O.tape_replay_ops(np.zeros_like(tape), k, g, S0)
    np.testing.assert_allclose(got, S0 * np.prod(g, axis=1)[:, :, None, None], rtol=1e-13)
    # g == 1, one step -> rank-1 update with the repeated k head
    got = O.tape_replay_ops(tape[:, :1], k[:, :1], np.ones_like(g[:, :1]), S0)
    for b in range(B):
        for hv in range(Hv):
            want = S0[b, hv] + np.outer(tape[b, 0, hv], k[b, 0, hv // (Hv // Hk)])
            np.testing.assert_allclose(got[b, hv], want, rtol=1e-13, atol=1e-14)
    # unrolled sum, all prefix lengths
    for a in range(T + 1):
        np.testing.assert_allclose(O.tape_replay_ops(tape[:, :a], k[:, :a], g[:, :a], S0),
                                   O.tape_replay_unrolled(tape, k, g, S0, a), rtol=1e-12, atol=1e-13)


def test_mask_equals_skipping_and_hk_repeat():
    rng = np.random.default_rng(14)
    B, T, Hk, Hv, Dk, Dv = 2, 6, 2, 4, 8, 4
    tape = rng.standard_normal((B, T, Hv, Dv))
    k = rng.standard_normal((B, T, Hk, Dk))
    g = rng.uniform(0.2, 1.0, (B, T, Hv))
    S0 = rng.standard_normal((B, Hv, Dv, Dk))
    mask = rng.integers(0, 2, (B, T)).astype(bool)
    got = O.tape_replay_ops(tape, k, g, S0, mask)
    for b in range(B):
        keep = np.nonzero(mask[b])[0]
        want = O.tape_replay_ops(tape[b:b + 1, keep], k[b:b + 1, keep], g[b:b + 1, keep], S0[b:b + 1])
        np.testing.assert_allclose(got[b:b + 1], want, rtol=1e-13)
    # Hk < Hv is the same as repeating k heads
    np.testing.assert_array_equal(O.tape_replay_ops(tape, k, g, S0),
                                  O.tape_replay_ops(tape, np.repeat(k, Hv // Hk, axis=2), g, S0))
    with pytest.raises(ValueError):
        O.tape_replay_ops(tape[:, :, :3], k, g[:, :, :3], S0[:, :3])
    with pytest.raises(ValueError):
        O.tape_replay_ops(tape, k, g[:, :, 0], S0)


def test_kernel_semantics_fp32_and_bf16_state():
    rng = np.random.default_rng(15)
    B, T, Hk, Hv, Dk, Dv = 1, 8, 2, 2, 32, 8
    tape = O.round_bf16((rng.standard_normal((B, T, Hv, Dv)) * 0.05).astype(np.float32))
    k = O.round_bf16(rng.standard_normal((B, T, Hk, Dk)).astype(np.float32))
    g = rng.uniform(0.2, 1.0, (B, T, Hv)).astype(np.float32)
    S0 = (rng.standard_normal((B, Hv, Dv, Dk)) * 0.1).astype(np.float32)
    f32 = O.tape_replay_kernel_semantics(tape, k, g, S0)
    ref = O.tape_replay_ops(tape, k, g, S0)
    assert np.linalg.norm(f32 - ref) / np.linalg.norm(ref) < 1e-6
    # bf16 state: every step rounds; result is representable in bf16 and near the fp64 answer
    S0b = O.round_bf16(S0)
    b16 = O.tape_replay_kernel_semantics(tape, k, g, S0b, state_dtype="bf16")
    assert np.array_equal(b16, O.round_bf16(b16))
    refb = O.tape_replay_ops(tape, k, g, S0b)
    assert np.linalg.norm(b16 - refb) / np.linalg.norm(refb) < 2e-2


def test_c_replay_matches_numpy(c_oracle):
    rng = np.random.default_rng(16)
    S, T, Hk, Hv, Dk, Dv = 3, 7, 2, 4, 32, 16
    tape = (rng.standard_normal((S, T, Hv, Dv)) * 0.05).astype(np.float32)
    k = rng.standard_normal((S, T, Hk, Dk)).astype(np.float32)
    tape_b, k_b = O.f32_to_bf16(tape), O.f32_to_bf16(k)
    tape_r, k_r = O.bf16_to_f32(tape_b), O.bf16_to_f32(k_b)
    S0 = (rng.standard_normal((S, Hv, Dv, Dk)) * 0.1).astype(np.float32)
    steps = np.array([0, 4, 7], dtype=np.int32)
    mask = rng.integers(0, 2, (S, T)).astype(np.uint8)
    for g in (rng.uniform(0.2, 1, (S, T, Hv)).astype(np.float32),
              rng.uniform(0.2, 1, (S, T, Hv, Dk)).astype(np.float32)):
        for m in (None, mask):
            got = c_oracle.tape_replay(tape_b, k_b, g, S0, steps=steps, mask=m)
            for s in range(S):
                a = int(steps[s])
                mm = None if m is None else m[s:s + 1, :a].astype(bool)
                want = O.tape_replay_ops(tape_r[s:s + 1, :a], k_r[s:s + 1, :a], g[s:s + 1, :a], S0[s:s + 1], mm)
                np.testing.assert_allclose(got[s:s + 1], want, rtol=2e-6, atol=1e-7)
    # fp32 tape path
    got = c_oracle.tape_replay(tape, k_b, g[..., 0] if g.ndim == 4 else g, S0)
    want = O.tape_replay_ops(tape, k_r, g[..., 0] if g.ndim == 4 else g, S0)
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)


def test_conv_rebuild_bruteforce():
    """All steps in 1..T, with and without a snapshot, against explicit row picking."""
    rng = np.random.default_rng(17)
    B, T, C, ksz = 2, 16, 5, 4
    keep = ksz - 1
    qkv = rng.standard_normal((B, T, C)).astype(np.float32)
    snap = rng.standard_normal((B, keep, C)).astype(np.float32)
    for prefix in (snap, None):
        for steps in range(0, T + 1):
            got = O.rebuild_conv_state(prefix, qkv, steps, ksz)
            assert got.shape == (B, keep, C)
            for j in range(keep):
                src = steps + j
                if src < keep:
                    want = prefix[:, src] if prefix is not None else np.zeros((B, C), np.float32)
                else:
                    want = qkv[:, src - keep]
                np.testing.assert_array_equal(got[:, j], want)
    # after accepting all T steps the window is the last `keep` recorded rows
    np.testing.assert_array_equal(O.rebuild_conv_state(snap, qkv, T, ksz), qkv[:, -keep:])
    assert O.rebuild_conv_state(snap, qkv, 3, 1) is None


def test_acceptance_length_exhaustive():
    for n in range(0, 8):
        for pattern in itertools.product([0, 1], repeat=n):
            drafted = list(range(10, 10 + n))
            posterior = [d if p else d + 100 for d, p in zip(drafted, pattern)]
            assert O.match_acceptance_length(drafted, posterior) == O.match_acceptance_length_loop(drafted, posterior)
    assert O.match_acceptance_length([], []) == 0
    # length 15 block: every prefix length
    d = list(range(15))
    for a in range(16):
        p = list(d)
        if a < 15:
            p[a] = -1
        assert O.match_acceptance_length(d, p) == a


def test_commit_cycle_and_trim_indexing():
    verify_ids = [7] + list(range(100, 115))          # staged first + 15 drafts
    for acc in range(16):
        posterior = list(range(100, 115)) + [999]      # target agrees with every draft ...
        if acc < 15:
            posterior[acc] = 555                       # ... until position acc
        out = O.commit_cycle(4096, verify_ids, posterior)
        assert out["acceptance_len"] == acc
        assert out["commit_count"] == acc + 1
        assert out["committed"] == verify_ids[:acc + 1]
        assert out["staged_next"] == posterior[acc]
        assert out["new_start"] == 4096 + acc + 1
        # KV cache wrote 16 rows during verify; trim back to the committed length
        new_off, trimmed = O.kv_trim(4096 + 16, (4096 + 16) - out["new_start"])
        assert (new_off, trimmed) == (4096 + acc + 1, 15 - acc)
    assert O.kv_trim(5, 9) == (0, 5)
    assert O.kv_trim(5, 0) == (5, 0)


def test_restore_plan():
    kinds = ["gdn", "gdn", "gdn", "kv"] * 2
    offs = [0, 0, 0, 4112] * 2
    plan = O.restore_plan(kinds, offs, target_len=4100, acceptance_length=3, drafted_tokens=15)
    assert plan == [("rollback", 3)] * 3 + [("trim", 12)] + [("rollback", 3)] * 3 + [("trim", 12)]
    plan = O.restore_plan(kinds, offs, target_len=4112, acceptance_length=15, drafted_tokens=15)
    assert plan == [("clear",)] * 3 + [("none",)] + [("clear",)] * 3 + [("none",)]


def test_rollback_model_state_machine():
    rng = np.random.default_rng(18)
    B, T, Hk, Hv, Dk, Dv, C = 1, 16, 2, 2, 8, 4, 6
    q, k, v, g, beta, S0 = _gdn_case(rng, B=B, T=T, Hk=Hk, Hv=Hv, Dk=Dk, Dv=Dv)
    conv0 = rng.standard_normal((B, 3, C))
    qkv = rng.standard_normal((B, T, C))
    m = O.RollbackCacheModel()
    m.cache = [conv0, S0]
    m.rollback(3)                       # un-armed: no-op apart from clearing
    assert m.cache[1] is S0
    m.arm_rollback()
    _, S_T, tape = O.gated_delta_ops_with_tape(q, k, v, g, beta, S0)
    m.cache = [qkv[:, -3:], S_T]
    m.record_tape(tape=tape, k=k, g=g, qkv=qkv)
    m.rollback(4)                       # 4 drafts accepted -> 5 steps committed
    _, S_5, _ = O.gated_delta_ops_with_tape(q[:, :5], k[:, :5], v[:, :5], g[:, :5], beta[:, :5], S0)
    np.testing.assert_allclose(m.cache[1], S_5, rtol=1e-12, atol=1e-13)
    np.testing.assert_array_equal(m.cache[0], np.concatenate([conv0, qkv], axis=1)[:, 5:8])
    assert m._snapshot is None and m._tape is None and not m._armed
