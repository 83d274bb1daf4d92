"""End to end on the device: the small hybrid model in bf16 with its 4-bit projections swapped
to the verify kernel, GatedDeltaNet layers on the fused glue and recurrence kernels, rollback by
tape replay, conv rebuild and KV trim - driven by the speculative cycle.

Every committed token comes out of a 16-row verify forward, whatever the draft proposed, so
runs with different drafts must agree token for token.  Against plain token-by-token decoding
(1-row forwards through the stock matmul) bf16 rounding differs, so there the sequences may
part ways only where the two best logits are nearly tied."""
import pytest
import torch

from dflash_mlx_amd.generate import generate_greedy, generate_speculative
from dflash_mlx_amd.runtime import make_target_cache
from dflash_mlx_amd.verify_linear import (VerifyQuantizedLinear, fuse_shared_input_linears,
                                          install_verify_linears)
from _toy_lm import ToyHybridLM, drafts

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _model(seed, join_shared_input=False):
    model = ToyHybridLM(seed=seed, hidden=512, Hk=2, Hv=4, D=128, dtype=torch.bfloat16).to(DEV)
    swapped = install_verify_linears(model)
    assert swapped == sum(isinstance(m, VerifyQuantizedLinear) for m in model.modules()) > 0
    if join_shared_input:
        # gate/up of every MLP, q/k/v of every attention layer, qkv/z of every linear-attention layer
        assert fuse_shared_input_linears(model) == 2 * len(model.layers)
    return model.install_hooks()


def _cache(model, fp32_state):
    cache = make_target_cache(model.pattern)
    if fp32_state:
        for layer, c in zip(model.layers, cache):
            if layer.is_linear:
                la = layer.linear_attn
                c[1] = torch.zeros((1, la.num_v_heads, la.head_v_dim, la.head_k_dim), dtype=torch.float32, device=DEV)
    return cache


def _same_or_parting_at_a_near_tie(model, prompt, a, b, fp32_state):
    """Two token sequences are equal, or where they first differ the plain path's two best
    logits are within 5 % of the logits' spread and are exactly those two tokens."""
    n = min(a.shape[0], b.shape[0])
    diverged = (a[:n] != b[:n]).nonzero()
    if not diverged.numel():
        return True
    at = int(diverged[0])
    with torch.no_grad():
        logits = model(torch.cat([prompt, a[:at]])[None], _cache(model, fp32_state))[0, -1]
    top = torch.topk(logits, 2)
    assert float(top.values[0] - top.values[1]) < 0.05 * float(logits.std()), (at, top.values)
    assert {int(a[at]), int(b[at])} == set(top.indices.tolist())
    return False


@pytest.mark.parametrize("fp32_state,join_shared_input", [(True, False), (False, False), (True, True)])
def test_speculative_decoding_on_the_device(native_lib, monkeypatch, fp32_state, join_shared_input):
    monkeypatch.setenv("DFLASH_VERIFY_QMM", "1")
    model = _model(11, join_shared_input)
    target = lambda ids, cache: model(ids, cache)
    prompt = torch.randint(0, 384, (11,), generator=torch.Generator().manual_seed(5)).to(DEV)
    n_new = 64
    greedy = generate_greedy(target, _cache(model, fp32_state), prompt, n_new)

    # a draft that is never right: every committed token is the target's own
    histories = {"random": [], "perfect": [], "partly": []}
    spec = generate_speculative(target, drafts(greedy.cpu(), 384, seed=3)["random"], _cache(model, fp32_state),
                                prompt, n_new, block_tokens=16, acceptance_history=histories["random"])
    assert max(histories["random"]) <= 2
    # drafts that know that sequence: whole blocks are accepted, and nothing changes
    runs = {}
    for kind in ("perfect", "partly"):
        runs[kind] = generate_speculative(target, drafts(spec.cpu(), 384, seed=3)[kind], _cache(model, fp32_state),
                                          prompt, n_new, block_tokens=16, acceptance_history=histories[kind])
    torch.cuda.synchronize()
    if fp32_state:
        # an fp32 state is the same to ~1e-7 however the blocks fall: no token moves
        assert torch.equal(runs["perfect"], spec) and torch.equal(runs["partly"], spec)
        assert histories["perfect"][:3] == [15, 15, 15] and len(histories["perfect"]) == 4
    else:
        # a bf16 state is rounded after every step, by the forward and by the replay: block
        # boundaries move single roundings, which may decide a near-tie
        for kind in ("perfect", "partly"):
            _same_or_parting_at_a_near_tie(model, prompt, runs[kind], spec, fp32_state)
    assert 0 < sum(histories["partly"]) < n_new
    # against 1-row decoding through the stock matmul
    _same_or_parting_at_a_near_tie(model, prompt, spec, greedy, fp32_state)


def test_long_prompt_takes_the_attention_kernel(native_lib, monkeypatch):
    """1100 cached positions: every 16-token verify block of the attention layer goes through the
    16-query kernel (shorter tail blocks and the prefill through the general attention)."""
    from dflash_mlx_amd import attention_layer as A
    from dflash_mlx_amd import kernels as K

    monkeypatch.setenv("DFLASH_VERIFY_QMM", "1")
    model = _model(13)
    seen = []
    real = K.batched_sdpa_2pass_exact
    monkeypatch.setattr(A, "batched_sdpa_2pass_exact", lambda **kw: seen.append(int(kw["keys"].shape[2])) or real(**kw))
    target = lambda ids, cache: model(ids, cache)
    prompt = torch.randint(0, 384, (1100,), generator=torch.Generator().manual_seed(8)).to(DEV)
    n_new = 40
    greedy = generate_greedy(target, _cache(model, True), prompt, n_new)
    seen.clear()
    history = []
    spec = generate_speculative(target, drafts(greedy.cpu(), 384, seed=4)["partly"], _cache(model, True), prompt, n_new,
                                block_tokens=16, acceptance_history=history)
    torch.cuda.synchronize()
    assert len(seen) >= 2 and all(n >= 1116 for n in seen)
    _same_or_parting_at_a_near_tie(model, prompt, spec, greedy, True)


def test_device_tokens_against_the_host_run_of_the_same_model(native_lib, monkeypatch):
    """The same weights, prompt and drafts decoded on the host (array operators, stock matmul:
    the path tests/test_generate_loop.py holds to exact greedy parity) and on the device (verify
    kernels, fused glue, tape replay).  bf16 activations are rounded in different places, so the
    two token sequences must be equal or part at a near-tie of the HOST model's two best logits."""
    monkeypatch.setenv("DFLASH_VERIFY_QMM", "1")
    host = ToyHybridLM(seed=11, hidden=512, Hk=2, Hv=4, D=128, dtype=torch.bfloat16).install_hooks()
    dev = _model(11)
    prompt = torch.randint(0, 384, (11,), generator=torch.Generator().manual_seed(5))
    n_new = 48

    def host_cache():
        cache = make_target_cache(host.pattern)
        for layer, c in zip(host.layers, cache):
            if layer.is_linear:
                la = layer.linear_attn
                c[1] = torch.zeros((1, la.num_v_heads, la.head_v_dim, la.head_k_dim), dtype=torch.float32)
        return cache

    host_target = lambda ids, cache: host(ids, cache)
    host_greedy = generate_greedy(host_target, host_cache(), prompt, n_new)
    host_spec = generate_speculative(host_target, drafts(host_greedy, 384, seed=3)["partly"], host_cache(), prompt,
                                     n_new, block_tokens=16)
    assert torch.equal(host_spec, host_greedy)          # the host path's own guarantee
    history = []
    dev_spec = generate_speculative(lambda ids, cache: dev(ids, cache), drafts(host_greedy, 384, seed=3)["partly"],
                                    _cache(dev, True), prompt.to(DEV), n_new, block_tokens=16,
                                    acceptance_history=history)
    torch.cuda.synchronize()
    assert sum(history) > 0                               # drafts were accepted: rollbacks of every length ran
    a, b = dev_spec.cpu(), host_spec
    n = min(a.shape[0], b.shape[0])
    diverged = (a[:n] != b[:n]).nonzero()
    if diverged.numel():
        at = int(diverged[0])
        with torch.no_grad():
            logits = host(torch.cat([prompt, b[:at]])[None], host_cache())[0, -1].float()
        top = torch.topk(logits, 2)
        assert float(top.values[0] - top.values[1]) < 0.05 * float(logits.std()), (at, top.values)
        assert {int(a[at]), int(b[at])} == set(top.indices.tolist())


def test_speculative_decoding_with_the_mlp_activation_in_the_projection_launch(native_lib, monkeypatch):
    """hidden = 1024: gate/up of every MLP are joined and their silu * up comes out of one chained
    launch with the epilogue (verify_linear.silu_gate_up); drafts of any quality commit the same
    tokens, and plain decoding agrees up to near-ties."""
    from dflash_mlx_amd import verify_qmm as VQ

    monkeypatch.setenv("DFLASH_VERIFY_QMM", "1")
    model = ToyHybridLM(seed=17, hidden=1024, Hk=2, Hv=4, D=128, dtype=torch.bfloat16).to(DEV)
    assert install_verify_linears(model) > 0 and fuse_shared_input_linears(model) == 2 * len(model.layers)
    model.install_hooks()
    chained = []
    real = VQ.QmmChain.__call__
    monkeypatch.setattr(VQ.QmmChain, "__call__", lambda self: (chained.append(1), real(self))[1])
    target = lambda ids, cache: model(ids, cache)
    prompt = torch.randint(0, 384, (9,), generator=torch.Generator().manual_seed(6)).to(DEV)
    n_new = 48
    greedy = generate_greedy(target, _cache(model, True), prompt, n_new)
    assert not chained                                   # one-token steps: no verify block
    spec = generate_speculative(target, drafts(greedy.cpu(), 384, seed=3)["random"], _cache(model, True), prompt, n_new,
                                block_tokens=16)
    blocks = len(chained) // len(model.layers)
    assert blocks >= n_new // 2 and len(chained) == blocks * len(model.layers)   # every MLP of every verify block
    again = generate_speculative(target, drafts(spec.cpu(), 384, seed=3)["perfect"], _cache(model, True), prompt, n_new,
                                 block_tokens=16)
    torch.cuda.synchronize()
    # block boundaries fall differently in the two runs: the fp32 states agree to ~1e-7, which a
    # bf16 rounding further down may turn into the decision of a near-tie
    _same_or_parting_at_a_near_tie(model, prompt, again, spec, True)
    _same_or_parting_at_a_near_tie(model, prompt, spec, greedy, True)

