"""End to end on the host: an MLX-format checkpoint is written, read back and placed into a
small hybrid model; the speculative cycle (dflash_mlx/runtime.py:1290-1458) with rollback over
GatedDeltaNet and attention caches must commit exactly the target's own greedy tokens, whatever
the draft proposes."""
import os

import pytest
import torch

from dflash_mlx_amd import loader
from dflash_mlx_amd.generate import generate_greedy, generate_speculative
from dflash_mlx_amd.quantized import QuantizedLinear
from dflash_mlx_amd.runtime import make_target_cache
from _toy_lm import ToyHybridLM, drafts


def _named_qlinears(model):
    return {name: m for name, m in model.named_modules() if isinstance(m, QuantizedLinear)}


def test_checkpoint_round_trip(tmp_path):
    model = ToyHybridLM(seed=1, dtype=torch.bfloat16)
    linears = _named_qlinears(model)
    assert len(linears) == 3 * 8 + 1 * 7
    ckpt = os.path.join(tmp_path, "ckpt")
    loader.save_quantized_linears(ckpt, linears, extra={"embed.weight": model.embed.weight})
    assert loader.read_quantization(os.path.join(ckpt, "config.json")) == (64, 4)
    tensors = loader.load_tensors(ckpt)
    assert tensors["layers.0.mlp.gate_proj.weight"].dtype in (torch.uint32, torch.int32)
    assert tuple(tensors["layers.0.mlp.gate_proj.weight"].shape) == (512, 256 // 8)
    assert tuple(tensors["layers.0.mlp.gate_proj.scales"].shape) == (512, 256 // 64)
    read = loader.load_quantized_linears(ckpt)
    assert set(read) == set(linears)
    for name, ql in linears.items():
        assert torch.equal(read[name].weight, ql.weight) and torch.equal(read[name].scales, ql.scales)
        assert torch.equal(read[name].biases, ql.biases) and read[name].group_size == 64 and read[name].bits == 4

    blank = ToyHybridLM(seed=2, dtype=torch.bfloat16)
    assert loader.assign_quantized_linears(blank, read) == len(linears)
    blank.embed.weight.data = tensors["embed.weight"]
    blank.lm_head.weight.data, blank.norm.weight.data = model.lm_head.weight.data, model.norm.weight.data
    for a, b in zip(model.layers, blank.layers):      # what the checkpoint does not hold
        if a.is_linear:
            for n in ("A_log", "dt_bias"):
                getattr(b.linear_attn, n).data = getattr(a.linear_attn, n).data
            b.linear_attn.conv1d.weight.data = a.linear_attn.conv1d.weight.data
        else:
            b.self_attn.q_norm.weight.data = a.self_attn.q_norm.weight.data
            b.self_attn.k_norm.weight.data = a.self_attn.k_norm.weight.data
    ids = torch.randint(0, 384, (1, 9))
    cache = lambda m: make_target_cache(m.pattern)
    assert torch.equal(model(ids, cache(model)), blank(ids, cache(blank)))


def test_loader_rejects_malformed_triples(tmp_path):
    good = QuantizedLinear(torch.zeros((32, 8), dtype=torch.int32), torch.ones((32, 1), dtype=torch.bfloat16),
                           torch.zeros((32, 1), dtype=torch.bfloat16))
    t = {"a.weight": good.weight, "a.scales": good.scales}
    with pytest.raises(KeyError):
        loader.quantized_linears(t)
    t["a.biases"] = torch.zeros((32, 2), dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        loader.quantized_linears(t)
    t["a.biases"] = good.biases
    assert set(loader.quantized_linears(t)) == {"a"}
    with pytest.raises(KeyError):
        loader.assign_quantized_linears(torch.nn.Linear(2, 2), loader.quantized_linears(t))
    assert loader.assign_quantized_linears(torch.nn.Linear(2, 2), loader.quantized_linears(t), strict=False) == 0
    with pytest.raises(FileNotFoundError):
        loader.load_tensors(str(tmp_path))


@pytest.mark.parametrize("kind", ["perfect", "random", "partly"])
@pytest.mark.parametrize("exact_attention_over", [None, 4])
def test_speculative_cycle_commits_the_targets_greedy_tokens(kind, exact_attention_over):
    # exact_attention_over = 4: the attention layers take their query-by-query path in every verify block
    model = ToyHybridLM(seed=3).install_hooks(exact_attention_over=exact_attention_over)
    target = lambda ids, cache: model(ids, cache)
    prompt = torch.randint(0, 384, (11,), generator=torch.Generator().manual_seed(5))
    n_new = 45
    reference = generate_greedy(target, make_target_cache(model.pattern), prompt, n_new)
    history = []
    out = generate_speculative(target, drafts(reference, 384, seed=7)[kind], make_target_cache(model.pattern),
                               prompt, n_new, block_tokens=16, acceptance_history=history)
    assert torch.equal(out, reference)
    if kind == "perfect":
        assert history[0] == 15 and sum(history) + len(history) >= n_new
    if kind == "random":
        assert max(history) <= 2
    if kind == "partly":
        assert 0 < sum(history) < n_new


def test_stop_token_ends_the_loop_after_the_committing_cycle():
    model = ToyHybridLM(seed=4).install_hooks()
    target = lambda ids, cache: model(ids, cache)
    prompt = torch.randint(0, 384, (6,), generator=torch.Generator().manual_seed(6))
    reference = generate_greedy(target, make_target_cache(model.pattern), prompt, 40)
    stop = int(reference[20])
    out = generate_speculative(target, drafts(reference, 384)["perfect"], make_target_cache(model.pattern),
                               prompt, 40, block_tokens=8, stop_token_ids=[stop])
    assert stop in out.tolist() and torch.equal(out, reference[:out.shape[0]]) and out.shape[0] < 40
