"""Host-side gate / dispatch / module-swap / rollback bookkeeping, all on CPU tensors.
Modelled on the reference's tests/test_verify_linear_parity.py and the gate cases of
tests/test_verify_qmm_parity.py; expected values come from the oracle's restatement."""
import itertools

import numpy as np
import pytest
import torch

from dflash_mlx_amd.gdn_layer import silu_ops
import torch.nn as nn

import dflash_mlx_amd._native as nat
from dflash_mlx_amd import runtime as R
from dflash_mlx_amd import verify_qmm as VQ
from dflash_mlx_amd.cache import KVCache
from dflash_mlx_amd.quantized import (QuantizedLinear, dequantize, pack_codes, quantize,
                                      quantized_matmul, unpack_codes)
from dflash_mlx_amd.recurrent_rollback_cache import RecurrentRollbackCache
from dflash_mlx_amd.verify_linear import (VerifyQuantizedLinear, install_verify_linears,
                                          is_verify_eligible, uninstall_verify_linears,
                                          fuse_shared_input_linears)
from dflash_mlx_amd.workloads import make_qmm_case
from oracle import dflash_oracle as O


def _mk_linear(i, o, bias=False):
    lin = nn.Linear(i, o, bias=bias)
    with torch.no_grad():
        lin.weight.copy_(torch.randn(o, i) * 0.1)
    return lin.to(torch.bfloat16)


@pytest.fixture(scope="module")
def small_ql():
    torch.manual_seed(0)
    return QuantizedLinear.from_linear(_mk_linear(512, 1024), group_size=64, bits=4)


def test_auto_variant_table():
    shapes = {(4096, 4096): ("mma2big_pipe", 8), (4096, 6144): ("mma2big_pipe", 8),
              (4096, 12288): ("mma2big", 1), (12288, 4096): ("mma2big_pipe", 8),
              (5120, 7168): ("mma2big_pipe", 8), (5120, 5120): ("mma2big_pipe", 8),
              (5120, 17408): ("mma2big", 1), (17408, 5120): ("mma2big_pipe", 8),
              (2048, 512): ("mma2big_pipe", 8), (512, 2048): ("mma2big_pipe", 8)}
    for (K, N), want in shapes.items():
        assert VQ._auto_variant(K, N) == want == O.auto_variant(K, N)
    for K, N in itertools.product([64, 8191, 8192, 8193], [32, 8192, 8193, 20000]):
        assert VQ._auto_variant(K, N) == O.auto_variant(K, N)


def test_gate_matches_restatement(monkeypatch):
    names = {torch.bfloat16: "bf16", torch.float16: "fp16", torch.float32: "fp32"}
    for flag in ("", "0", "1", "true"):
        monkeypatch.setenv("DFLASH_VERIFY_QMM", flag)
        for shape, dt, gs, bits, tr in itertools.product(
                [(16, 64), (1, 16, 64), (4, 4, 64), (2, 2, 4, 64), (15, 64), (32, 64), (64,)],
                names, [32, 64, 128, 16], [4, 8], [True, False]):
            x = torch.zeros(shape, dtype=dt)
            assert VQ._should_use_verify(x, gs, bits, tr) == O.should_use_verify(
                flag, shape, names[dt], gs, bits, tr)


def test_disabled_flag_is_exactly_stock(monkeypatch):
    monkeypatch.delenv("DFLASH_VERIFY_QMM", raising=False)
    c = make_qmm_case(512, 64, 1)
    y = VQ.verify_matmul(c.x, c.w, c.scales, c.biases, group_size=64, bits=4)
    ref = quantized_matmul(c.x, c.w, c.scales, c.biases, group_size=64, bits=4)
    assert torch.equal(y, ref)


def test_divisibility_guard_falls_back_to_stock(verify_env):
    # N % 32 != 0 -> stock even with the flag on (CPU tensors would otherwise raise)
    c = make_qmm_case(512, 48, 2)
    y = VQ.verify_matmul(c.x, c.w, c.scales, c.biases)
    assert torch.equal(y, quantized_matmul(c.x, c.w, c.scales, c.biases))
    # pipe with K % (32*k_parts) != 0 -> stock
    verify_env.setenv("DFLASH_VERIFY_VARIANT", "mma2big_pipe")
    verify_env.setenv("DFLASH_VERIFY_QMM_KPARTS", "3")
    c = make_qmm_case(512, 64, 3)
    assert torch.equal(VQ.verify_matmul(c.x, c.w, c.scales, c.biases),
                       quantized_matmul(c.x, c.w, c.scales, c.biases))
    for K, N, var, kp in [(512, 48, "auto", "4"), (512, 64, "mma2big_pipe", "3"),
                          (96, 64, "mma2big", "4"), (96, 64, "mma2big_pipe", "2")]:
        want = O.dispatch_variant(K, N, var, kp)
        assert want[0] in ("stock", "mma2big", "mma2big_pipe")


def test_eligible_call_on_host_tensors_fails_loudly(verify_env):
    c = make_qmm_case(512, 64, 4)
    with pytest.raises(nat.NativeLibraryError):
        VQ.verify_matmul(c.x, c.w, c.scales, c.biases)


def test_verify_qmm_takes_group_size_and_bits_positionally(verify_env):
    """verify_qmm(x, w_packed, scales, biases, group_size, bits): the spelling of the hot path's
    name; ineligible calls (4 rows here) go to the stock operator like verify_matmul's."""
    c = make_qmm_case(256, 32, 6, M=4)
    want = VQ.verify_matmul(c.x, c.w, c.scales, c.biases, group_size=64, bits=4)
    assert torch.equal(VQ.verify_qmm(c.x, c.w, c.scales, c.biases, 64, 4), want)
    assert torch.equal(VQ.verify_qmm(c.x, c.w, c.scales, c.biases, group_size=64, bits=4), want)
    with pytest.raises(nat.NativeLibraryError):          # 16 rows: the kernel path, as for verify_matmul
        c16 = make_qmm_case(256, 32, 6)
        VQ.verify_qmm(c16.x, c16.w, c16.scales, c16.biases, 64, 4)


def test_stock_dequant_matches_oracle():
    c = make_qmm_case(256, 32, 5)
    w_np = c.w.numpy().view(np.uint32)
    want = O.dequant_affine(w_np, c.scales.float().numpy(), c.biases.float().numpy(), 64)
    got = dequantize(c.w, c.scales, c.biases, 64, 4, dtype=torch.float32).double().numpy()
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-7)
    assert np.array_equal(unpack_codes(c.w).numpy(), O.unpack_int4(w_np))
    assert torch.equal(pack_codes(unpack_codes(c.w)), c.w)


def test_quantize_roundtrip_is_well_formed():
    torch.manual_seed(1)
    w = (torch.randn(64, 256) * 0.1).to(torch.bfloat16)
    q, s, b = quantize(w, 64, 4)
    assert q.shape == (64, 32) and s.shape == b.shape == (64, 4)
    wd = dequantize(q, s, b, 64, 4, dtype=torch.float32)
    step = s.float().abs().repeat_interleave(64, dim=1)
    assert torch.all((wd - w.float()).abs() <= 1.0 * step + 1e-3)  # half a step + edge snapping


def test_eligibility(small_ql, verify_env):
    assert is_verify_eligible(small_ql)
    assert not is_verify_eligible(nn.Linear(8, 8))
    big = QuantizedLinear(torch.zeros((150_000, 64), dtype=torch.int32),
                          torch.zeros((150_000, 8), dtype=torch.bfloat16),
                          torch.zeros((150_000, 8), dtype=torch.bfloat16))
    assert not is_verify_eligible(big)
    verify_env.setenv("DFLASH_VERIFY_MAX_N", "1000")
    assert not is_verify_eligible(small_ql)      # N=1024 >= 1000
    verify_env.setenv("DFLASH_VERIFY_MAX_N", "garbage")
    assert is_verify_eligible(small_ql)          # unparsable -> default
    odd = QuantizedLinear(torch.zeros((48, 64), dtype=torch.int32), torch.zeros((48, 8), dtype=torch.bfloat16),
                          torch.zeros((48, 8), dtype=torch.bfloat16))
    assert not is_verify_eligible(odd)           # N % 32
    eight = QuantizedLinear(small_ql.weight, small_ql.scales, small_ql.biases, bits=8)
    assert not is_verify_eligible(eight)
    verify_env.setenv("DFLASH_VERIFY_INCLUDE", "mlp, attn_o")
    assert is_verify_eligible(small_ql, path="model.layers.3.mlp.down_proj")
    assert is_verify_eligible(small_ql, path="model.layers.3.self_attn.o_proj")
    assert not is_verify_eligible(small_ql, path="model.layers.3.self_attn.q_proj")
    assert not is_verify_eligible(small_ql, path="model.layers.3.linear_attn.in_proj_qkv")
    assert not is_verify_eligible(small_ql, path="lm_head")
    verify_env.setenv("DFLASH_VERIFY_INCLUDE", "gdn")
    assert is_verify_eligible(small_ql, path="model.layers.3.linear_attn.out_proj")


@pytest.mark.parametrize("M", [1, 8, 32])
def test_parity_non_verify(small_ql, verify_env, M):
    """M != 16 stays on the stock operator: bit-identical to QuantizedLinear."""
    verify = VerifyQuantizedLinear.from_quantized(small_ql)
    assert verify.weight is small_ql.weight and verify.scales is small_ql.scales
    x = (torch.randn(M, 512) * 0.5).to(torch.bfloat16)
    assert torch.equal(small_ql(x), verify(x))


def test_additive_bias_kept(verify_env):
    torch.manual_seed(3)
    lin = nn.Linear(128, 64, bias=True).to(torch.bfloat16)
    ql = QuantizedLinear.from_linear(lin, 64, 4)
    v = VerifyQuantizedLinear.from_quantized(ql)
    x = torch.randn(4, 128).to(torch.bfloat16)
    assert torch.equal(v(x), ql(x))
    assert torch.equal(ql(x), quantized_matmul(x, ql.weight, ql.scales, ql.biases) + ql.bias)


def test_swap_and_unswap(verify_env):
    class Tiny(nn.Module):
        def __init__(self):
            super().__init__()
            self.proj_a = QuantizedLinear.from_linear(_mk_linear(512, 1024), 64, 4)
            self.inner = nn.ModuleDict({"proj_b": QuantizedLinear.from_linear(_mk_linear(512, 1024), 64, 4)})
            self.proj_bad = QuantizedLinear(torch.zeros((150_000, 64), dtype=torch.int32),
                                            torch.zeros((150_000, 8), dtype=torch.bfloat16),
                                            torch.zeros((150_000, 8), dtype=torch.bfloat16))

    m = Tiny()
    wa = m.proj_a.weight
    assert install_verify_linears(m) == 2
    assert isinstance(m.proj_a, VerifyQuantizedLinear) and isinstance(m.inner["proj_b"], VerifyQuantizedLinear)
    assert not isinstance(m.proj_bad, VerifyQuantizedLinear)
    assert m.proj_a.weight is wa
    assert install_verify_linears(m) == 0          # idempotent
    assert uninstall_verify_linears(m) == 2
    assert type(m.proj_a) is QuantizedLinear and m.proj_a.weight is wa
    assert install_verify_linears(m, predicate=lambda path, mod: path == "proj_a") == 1


def test_verify_enabled_for(monkeypatch):
    cfgs = [{}, {"num_hidden_layers": 39}, {"num_hidden_layers": 40}, {"num_experts": 256, "num_hidden_layers": 4},
            {"text_config": {"num_hidden_layers": 64}}, {"text_config": {"num_experts": None, "num_hidden_layers": None}},
            {"num_hidden_layers": "x"}, None]
    for ov in ("", "1", "0", " 1 ", "yes"):
        monkeypatch.setenv("DFLASH_VERIFY_LINEAR", ov)
        for cfg in cfgs:
            assert R._verify_enabled_for(cfg) == O.verify_enabled_for(cfg, ov)
    monkeypatch.delenv("DFLASH_VERIFY_LINEAR")
    assert R._verify_enabled_for({"num_hidden_layers": 64}) and not R._verify_enabled_for({"num_hidden_layers": 32})


def test_enable_verify_linears_sets_default_flag(monkeypatch):
    monkeypatch.delenv("DFLASH_VERIFY_QMM", raising=False)
    monkeypatch.delenv("DFLASH_VERIFY_LINEAR", raising=False)
    m = nn.Sequential(QuantizedLinear.from_linear(_mk_linear(64, 32), 64, 4))
    meta = {}
    assert R.enable_verify_linears(m, {"num_hidden_layers": 12}, meta) == 0 and "verify_linear_swapped" not in meta
    import os
    assert "DFLASH_VERIFY_QMM" not in os.environ
    assert R.enable_verify_linears(m, {"num_hidden_layers": 64}, meta) == 1 and meta["verify_linear_swapped"] == 1
    assert os.environ["DFLASH_VERIFY_QMM"] == "1"
    monkeypatch.setenv("DFLASH_VERIFY_QMM", "0")
    R.enable_verify_linears(nn.Sequential(), {"num_experts": 8})
    assert os.environ["DFLASH_VERIFY_QMM"] == "0"     # explicit user choice survives


def test_acceptance_length_matches_loop():
    rng = np.random.default_rng(0)
    for n in (0, 1, 5, 15):
        for _ in range(20):
            d = rng.integers(0, 3, n)
            p = rng.integers(0, 3, n)
            got = int(R._match_acceptance_length(torch.from_numpy(d), torch.from_numpy(p)))
            assert got == O.match_acceptance_length_loop(d, p)


def test_kv_trim_matches_restatement():
    for off, n in itertools.product([0, 5, 4112], [0, 3, 16, 5000]):
        c = KVCache()
        c.offset = off
        assert c.trim(n) == O.kv_trim(off, n)[1] and c.offset == O.kv_trim(off, n)[0]
    c = KVCache()
    k = torch.arange(2 * 3 * 20 * 4, dtype=torch.float32).reshape(2, 3, 20, 4)
    kk, vv = c.update_and_fetch(k, -k)
    assert c.offset == 20 and torch.equal(kk, k) and torch.equal(vv, -k)
    c.trim(5)
    kk, _ = c.update_and_fetch(k[:, :, :2] + 1000, k[:, :, :2])
    assert c.offset == 17 and torch.equal(kk[:, :, :15], k[:, :, :15]) and torch.equal(kk[:, :, 15:], k[:, :, :2] + 1000)


class _FakeGdn:
    def __init__(self):
        self.calls = []

    def rollback(self, n):
        self.calls.append(("rollback", n))

    def clear_transients(self):
        self.calls.append(("clear",))


def test_restore_follows_plan():
    for acc, drafted, target in [(3, 15, 4100), (15, 15, 4112), (0, 15, 4097), (2, 0, 50)]:
        kinds = ["gdn", "gdn", "gdn", "kv"] * 3
        caches, offs = [], []
        for kd in kinds:
            if kd == "gdn":
                caches.append(_FakeGdn()); offs.append(0)
            else:
                c = KVCache(); c.offset = 4112; caches.append(c); offs.append(4112)
        plan = O.restore_plan(kinds, offs, target_len=target, acceptance_length=acc, drafted_tokens=drafted)
        ns = R._restore_target_cache_after_acceptance(caches, target_len=target, acceptance_length=acc,
                                                      drafted_tokens=drafted)
        assert isinstance(ns, int) and ns >= 0
        for c, step in zip(caches, plan):
            if step[0] in ("rollback", "clear"):
                assert c.calls == [step]
            elif step[0] == "trim":
                assert c.offset == 4112 - step[1] == target
            else:
                assert c.offset == 4112


def test_rollback_cache_state_machine_on_host():
    """CPU tensors take the array-op replay (as the reference does without its GPU)."""
    rng = np.random.default_rng(18)
    B, T, Hk, Hv, Dk, Dv, C = 2, 16, 2, 4, 8, 4, 6
    k = rng.standard_normal((B, T, Hk, Dk)); v = rng.standard_normal((B, T, Hv, Dv))
    q = rng.standard_normal((B, T, Hk, Dk))
    g = rng.uniform(0.2, 1, (B, T, Hv)); beta = rng.uniform(0, 1, (B, T, Hv))
    S0 = rng.standard_normal((B, Hv, Dv, Dk)) * 0.1
    conv0 = rng.standard_normal((B, 3, C)); qkv = rng.standard_normal((B, T, C))
    _, S_T, tape = O.gated_delta_ops_with_tape(q, k, v, g, beta, S0)
    t = torch.from_numpy
    for acc in (0, 4, 14):
        model = O.RollbackCacheModel()
        model.cache = [conv0, S0]
        cache = RecurrentRollbackCache(size=2, conv_kernel_size=4)
        cache[0], cache[1] = t(conv0), t(S0)
        cache.rollback(acc)                      # un-armed: no-op
        assert cache[1] is not None and not cache._armed
        cache[0], cache[1] = t(conv0), t(S0)
        for c in (model, cache):
            c.arm_rollback()
        assert cache._armed and cache._snapshot is not None
        model.cache = [qkv[:, -3:], S_T]
        cache[0], cache[1] = t(qkv[:, -3:].copy()), t(S_T)
        model.record_tape(tape=tape, k=k, g=g, qkv=qkv)
        cache.record_tape(tape=t(tape), k=t(k), g=t(g), qkv=t(qkv))
        model.rollback(acc); cache.rollback(acc)
        np.testing.assert_allclose(cache[1].numpy(), model.cache[1], rtol=1e-12, atol=1e-13)
        np.testing.assert_array_equal(cache[0].numpy(), model.cache[0])
        assert cache._snapshot is None and cache._tape is None and not cache._armed
    with pytest.raises(ValueError):
        from dflash_mlx_amd.kernels import _tape_replay_ops
        _tape_replay_ops(t(tape)[:, :, :3], t(k), t(g)[:, :, :3], t(S0)[:, :3])


def test_rollback_cache_batch_protocol():
    """filter / extend / extract / prepare / finalize / advance / make_mask / empty, as the batched
    generation loops of mlx-lm use them on the reference class
    (dflash_mlx/recurrent_rollback_cache.py:18-19, 46-94)."""
    conv = torch.arange(4 * 3 * 5, dtype=torch.float32).reshape(4, 3, 5)
    state = torch.arange(4 * 2 * 3 * 8, dtype=torch.float32).reshape(4, 2, 3, 8)
    cache = RecurrentRollbackCache(size=2, conv_kernel_size=4)
    assert cache.empty() and cache.lengths is None and cache.left_padding is None
    assert cache.make_mask(5) is None
    cache[0], cache[1] = conv.clone(), state.clone()
    assert not cache.empty()

    # lengths of a right-padded block: true where a row still has tokens
    cache.prepare(lengths=[3, 5, 0, 2])
    assert torch.equal(cache.make_mask(4), torch.tensor([[1, 1, 1, 0], [1, 1, 1, 1], [0, 0, 0, 0], [1, 1, 0, 0]]).bool())
    cache.advance(2)
    assert cache.lengths.tolist() == [1, 3, -2, 0]
    assert torch.equal(cache.make_mask(2), torch.tensor([[1, 0], [1, 1], [0, 0], [0, 0]]).bool())
    # left padding wins over lengths: true from the first real token on
    cache.left_padding = torch.tensor([0, 2, 1, 4])
    assert torch.equal(cache.make_mask(3), torch.tensor([[1, 1, 1], [0, 0, 1], [0, 1, 1], [0, 0, 0]]).bool())
    cache.advance(1)
    assert cache.left_padding.tolist() == [-1, 1, 0, 3] and cache.lengths.tolist() == [0, 2, -3, -1]

    # a change of the batch drops what a rollback would need, and keeps rows in the order asked for
    cache.arm_rollback()
    cache.record_tape(tape=torch.zeros(4, 2, 2, 3), k=torch.zeros(4, 2, 1, 8), g=torch.ones(4, 2, 2), qkv=torch.zeros(4, 2, 5))
    cache.filter(torch.tensor([2, 0]))
    assert cache._snapshot is None and cache._tape is None and not cache._armed
    assert torch.equal(cache[0], conv[[2, 0]]) and torch.equal(cache[1], state[[2, 0]])
    assert cache.lengths.tolist() == [-3, 0] and cache.left_padding.tolist() == [0, -1]
    cache.rollback(0)   # nothing armed any more: a no-op
    assert torch.equal(cache[1], state[[2, 0]])

    one = cache.extract(1)
    assert isinstance(one, RecurrentRollbackCache) and one.conv_kernel_size == 4
    assert torch.equal(one[0], conv[0:1]) and torch.equal(one[1], state[0:1]) and one.lengths is None

    other = RecurrentRollbackCache(size=2, conv_kernel_size=4)
    other[0], other[1] = conv[3:4].clone(), state[3:4].clone()
    cache.extend(other)
    assert torch.equal(cache[0], conv[[2, 0, 3]]) and torch.equal(cache[1], state[[2, 0, 3]])
    fresh = RecurrentRollbackCache(size=2)
    fresh.extend(other)   # an empty cache takes the other's rows
    assert torch.equal(fresh[1], state[3:4])
    with pytest.raises(ValueError):
        cache.extend(RecurrentRollbackCache(size=3))

    cache.arm_rollback()
    cache.finalize()
    assert cache.lengths is None and cache.left_padding is None and cache._snapshot is None and not cache._armed
    cache.prepare(lengths=None)
    assert cache.lengths is None

    # a cache that is a view into an arena stands on its own tensors after the batch changed
    from dflash_mlx_amd.recurrent_rollback_cache import RollbackArena
    arena = RollbackArena(2, batch=3, max_steps=4, Hk=1, Hv=2, Dk=32, Dv=4, conv_dim=6, device="cpu")
    view = arena.caches()[1]
    assert view._arena is arena
    view.filter(torch.tensor([1]))
    assert view._arena is None and view[1].shape[0] == 1 and view[1].data_ptr() != arena.state[0, 1].data_ptr()


@pytest.mark.parametrize("g_per_dk", [False, True])
def test_array_op_forms_match_the_oracle(g_per_dk):
    """The torch array-op forms of forward-with-tape and replay (what host tensors and
    uncovered shapes take) against the NumPy oracle, with a mask and Hk < Hv."""
    from dflash_mlx_amd.kernels import (_gated_delta_ops_with_tape, _tape_replay_ops,
                                        gated_delta_kernel_with_tape)
    rng = np.random.default_rng(31 + int(g_per_dk))
    B, T, Hk, Hv, Dk, Dv = 2, 7, 2, 6, 8, 5
    q = rng.standard_normal((B, T, Hk, Dk)); k = rng.standard_normal((B, T, Hk, Dk))
    v = rng.standard_normal((B, T, Hv, Dv))
    g = rng.uniform(0.2, 1, (B, T, Hv, Dk) if g_per_dk else (B, T, Hv))
    beta = rng.uniform(0, 1, (B, T, Hv)); S0 = rng.standard_normal((B, Hv, Dv, Dk)) * 0.1
    mask = rng.uniform(size=(B, T)) > 0.3
    t = torch.from_numpy
    for m in (None, mask):
        yo, so, to = O.gated_delta_ops_with_tape(q, k, v, g, beta, S0, mask=m)
        tm = None if m is None else t(m)
        y, s, tape = _gated_delta_ops_with_tape(t(q), t(k), t(v), t(g), t(beta), t(S0), tm)
        np.testing.assert_allclose(y.numpy(), yo, rtol=1e-12, atol=1e-13)
        np.testing.assert_allclose(s.numpy(), so, rtol=1e-12, atol=1e-13)
        np.testing.assert_allclose(tape.numpy(), to, rtol=1e-6, atol=1e-7)   # the tape is fp32
        y2, s2, _ = gated_delta_kernel_with_tape(t(q), t(k), t(v), t(g), t(beta), t(S0), tm)  # host tensors
        assert torch.equal(y2, y) and torch.equal(s2, s)
        ro = O.tape_replay_ops(to, k, g, S0, mask=m)
        r = _tape_replay_ops(t(to), t(k), t(g), t(S0), tm)
        np.testing.assert_allclose(r.numpy(), ro, rtol=1e-12, atol=1e-13)
        np.testing.assert_allclose(r.numpy(), so, rtol=1e-9, atol=1e-10)     # replay of the full tape


class _SharedInputToy(nn.Module):
    def __init__(self):
        super().__init__()
        self.mlp = nn.Module()
        self.mlp.gate_proj = QuantizedLinear.from_linear(_mk_linear(512, 256), 64, 4)
        self.mlp.up_proj = QuantizedLinear.from_linear(_mk_linear(512, 384), 64, 4)
        self.mlp.down_proj = QuantizedLinear.from_linear(_mk_linear(384, 512), 64, 4)
        self.attn = nn.Module()
        self.attn.q_proj = QuantizedLinear.from_linear(_mk_linear(512, 256), 64, 4)
        self.attn.k_proj = QuantizedLinear.from_linear(_mk_linear(512, 64), 64, 4)
        self.attn.v_proj = QuantizedLinear.from_linear(_mk_linear(512, 64, bias=True), 64, 4)   # adds a bias: stays out
        self.odd = nn.Module()
        self.odd.gate_proj = QuantizedLinear.from_linear(_mk_linear(384, 256), 64, 4)     # K % 512 != 0: not joined
        self.odd.up_proj = QuantizedLinear.from_linear(_mk_linear(384, 256), 64, 4)


def test_fuse_shared_input_groups_keep_every_result(monkeypatch):
    """Joined projections: the modules keep their values (as views of one storage), the stock
    path is untouched, and with the verify gate open a parent that asks for all members at once
    (``shared_input_outputs``) gets them from one product."""
    import dflash_mlx_amd.verify_linear as VL

    monkeypatch.delenv("DFLASH_VERIFY_QMM", raising=False)
    m = _SharedInputToy()
    assert install_verify_linears(m) == 8
    before = {k: v.clone() for k, v in m.state_dict().items()}
    x = torch.randn(16, 512).to(torch.bfloat16)
    stock = {n: getattr(m.mlp, n)(x) for n in ("gate_proj", "up_proj")}
    assert fuse_shared_input_linears(m) == 2            # gate/up of mlp, q/k of attn
    assert fuse_shared_input_linears(m) == 0            # idempotent
    after = m.state_dict()
    assert before.keys() == after.keys() and all(torch.equal(before[k], after[k]) for k in before)
    group = m.mlp.gate_proj._shared_input[0]
    assert m.mlp.up_proj._shared_input == (group, 1) and group.bounds == [(0, 256), (256, 640)]
    assert m.mlp.up_proj.weight.data_ptr() == group.weight[256:].data_ptr()
    assert m.attn.v_proj._shared_input is None and m.odd.gate_proj._shared_input is None
    assert m.attn.q_proj._shared_input[0].bounds == [(0, 256), (256, 320)]
    # gate closed (no DFLASH_VERIFY_QMM): every member runs the stock operator on its own rows
    for n in ("gate_proj", "up_proj"):
        assert torch.equal(getattr(m.mlp, n)(x), stock[n])
    x5 = torch.randn(5, 512).to(torch.bfloat16)
    assert torch.equal(m.mlp.up_proj(x5), quantized_matmul(x5, before["mlp.up_proj.weight"], before["mlp.up_proj.scales"],
                                                           before["mlp.up_proj.biases"]))

    # gate open, device product replaced by the stock operator: count the products and their rows
    calls = []

    def product(x, w, s, b, **kw):
        calls.append(int(w.shape[0]))
        return quantized_matmul(x, w, s, b, **kw)

    monkeypatch.setattr(VL, "verify_matmul", product)
    monkeypatch.setattr(VL, "_should_use_verify", lambda x, gs, bits, tr: True)
    full = quantized_matmul(x, group.weight, group.scales, group.biases)
    # the parent asks for both at once: one product over the joint rows
    g1, u1 = VL.shared_input_outputs(m.mlp, ("gate_proj", "up_proj"), x)
    assert calls == [640] and torch.equal(g1, full[:, :256]) and torch.equal(u1, full[:, 256:])
    # a member on its own answers from its rows with a product of its own; nothing is remembered
    assert torch.equal(m.mlp.up_proj(x), quantized_matmul(x, group.weight[256:], group.scales[256:], group.biases[256:]))
    assert calls == [640, 384]
    x.add_(1.0)   # (an input changed in place is just an input)
    g2, u2 = VL.shared_input_outputs(m.mlp, ("gate_proj", "up_proj"), x)
    full2 = quantized_matmul(x, group.weight, group.scales, group.biases)
    assert calls == [640, 384, 640] and torch.equal(g2, full2[:, :256]) and torch.equal(u2, full2[:, 256:])
    # names that are only partly joined: q and k by their launch, v (adds a bias) by itself
    q, k, v = VL.shared_input_outputs(m.attn, ("q_proj", "k_proj", "v_proj"), x)
    assert calls[3:] == [320, 64] and q.shape == (16, 256) and k.shape == (16, 64)
    assert torch.equal(v, m.attn.v_proj(x))
    # a parent without groups, and an input that is not a verify block: every member by itself
    del calls[:]
    og, ou = VL.shared_input_outputs(m.odd, ("gate_proj", "up_proj"), torch.randn(16, 384).to(torch.bfloat16))
    assert calls == [256, 256] and og.shape == ou.shape == (16, 256)
    g5, u5 = VL.shared_input_outputs(m.mlp, ("gate_proj", "up_proj"), x5)
    assert calls == [256, 256] and torch.equal(u5, m.mlp.up_proj(x5))
    # moving the module gives it buffers of its own: it leaves the group
    m.mlp.up_proj._apply(lambda t: t.clone())
    assert m.mlp.up_proj._shared_input is None
    del calls[:]
    g6, u6 = VL.shared_input_outputs(m.mlp, ("gate_proj", "up_proj"), x)
    assert calls == [256, 384] and torch.equal(g6, g2) and torch.equal(u6, u2)
    assert uninstall_verify_linears(m) == 8


def test_silu_gate_up_on_the_host_is_the_array_operators(monkeypatch):
    """No device, or no group: the hidden activation of a gated MLP from its two projections."""
    import dflash_mlx_amd.verify_linear as VL

    monkeypatch.delenv("DFLASH_VERIFY_QMM", raising=False)
    m = _SharedInputToy()
    install_verify_linears(m)
    x = torch.randn(16, 512).to(torch.bfloat16)
    m.mlp.up_proj = VerifyQuantizedLinear.from_quantized(QuantizedLinear.from_linear(_mk_linear(512, 256), 64, 4))
    want = silu_ops(m.mlp.gate_proj(x)) * m.mlp.up_proj(x)
    assert torch.equal(VL.silu_gate_up(m.mlp, x), want)
    assert fuse_shared_input_linears(m) >= 1
    group = m.mlp.gate_proj._shared_input[0]
    assert group.bounds == [(0, 256), (256, 512)] and not group.silu_mul_ready(x)      # host tensor
    assert torch.equal(VL.silu_gate_up(m.mlp, x), want)
    assert torch.equal(VL.silu_gate_up(m.odd, torch.ones(3, 384).to(torch.bfloat16)),
                       silu_ops(m.odd.gate_proj(torch.ones(3, 384).to(torch.bfloat16))) *
                       m.odd.up_proj(torch.ones(3, 384).to(torch.bfloat16)))


def test_fuse_shared_input_switch(monkeypatch):
    m = _SharedInputToy()
    install_verify_linears(m)
    monkeypatch.setenv("DFLASH_VERIFY_FUSE_SHARED_INPUT", "0")
    assert fuse_shared_input_linears(m) == 0 and m.mlp.gate_proj._shared_input is None


def test_narrow_projections_join_a_shared_input_group(monkeypatch):
    """The 48-row gates of a linear-attention layer are kept out of the swap by the N % 32 rule,
    but join the group of the layer's input projections (behind their pad-to-16 wrappers too);
    without a group they stay what they were."""
    import dflash_mlx_amd.verify_linear as VL
    from dflash_mlx_amd.gdn_layer import _install_exact_small_proj_hooks

    monkeypatch.delenv("DFLASH_VERIFY_QMM", raising=False)

    def layer():
        la = nn.Module()
        la.in_proj_qkv = QuantizedLinear.from_linear(_mk_linear(512, 256), 64, 4)
        la.in_proj_z = QuantizedLinear.from_linear(_mk_linear(512, 128), 64, 4)
        la.in_proj_b = QuantizedLinear.from_linear(_mk_linear(512, 48), 64, 4)
        la.in_proj_a = QuantizedLinear.from_linear(_mk_linear(512, 48), 64, 4)
        m = nn.Module()
        m.linear_attn = la
        return m

    for wrap_first in (False, True):
        m = layer()
        x = torch.randn(16, 512).to(torch.bfloat16)
        want = {n: getattr(m.linear_attn, n)(x) for n in ("in_proj_qkv", "in_proj_z", "in_proj_b", "in_proj_a")}
        assert install_verify_linears(m) == 2                       # qkv and z only
        if wrap_first:
            _install_exact_small_proj_hooks(m.linear_attn)
        assert fuse_shared_input_linears(m) == 1
        if not wrap_first:
            _install_exact_small_proj_hooks(m.linear_attn)
        inner = m.linear_attn.in_proj_a.linear
        assert isinstance(inner, VerifyQuantizedLinear) and inner._shared_input[0].bounds == [
            (0, 256), (256, 384), (384, 432), (432, 480)] and inner._shared_input[1] == 3
        for n, w in want.items():
            assert torch.equal(getattr(m.linear_attn, n)(x), w)
        group = inner._shared_input[0]
        assert m.linear_attn._dflash_fused == (group,) and group.names == ("in_proj_qkv", "in_proj_z", "in_proj_b", "in_proj_a")
        # behind the wrappers a block of 16 is passed through as it is: the joint launch applies
        monkeypatch.setattr(VL, "_should_use_verify", lambda x, gs, bits, tr: True)
        x3 = x.reshape(1, 16, 512)
        assert group.applies(m.linear_attn, x3) and not group.applies(m.linear_attn, x3[:, :5])
        monkeypatch.undo()
        monkeypatch.delenv("DFLASH_VERIFY_QMM", raising=False)
    # 256 + 48 rows are not a multiple of 32: no group, and the narrow projection is left alone
    m = layer()
    del m.linear_attn.in_proj_z, m.linear_attn.in_proj_a
    install_verify_linears(m)
    assert fuse_shared_input_linears(m) == 0 and type(m.linear_attn.in_proj_b) is QuantizedLinear
