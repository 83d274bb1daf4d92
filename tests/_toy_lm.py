"""A small hybrid language model for the end-to-end tests: GatedDeltaNet mixers (the
package's layer) and full-attention mixers over ``KVCache``, every projection an MLX-format
4-bit ``QuantizedLinear``, random weights.  Test infrastructure only."""
import torch
import torch.nn as nn

from dflash_mlx_amd import gdn_layer as G
from dflash_mlx_amd.quantized import QuantizedLinear
from dflash_mlx_amd.verify_linear import silu_gate_up


def _qlinear(n_in, n_out, gen, dtype, scale=1.0):
    lin = nn.Linear(n_in, n_out, bias=False)
    lin.weight.data = torch.randn((n_out, n_in), generator=gen) * (scale * n_in ** -0.5)
    return QuantizedLinear.from_linear(lin.to(dtype))


class RMSNorm(nn.Module):
    def __init__(self, dim, dtype):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim, dtype=dtype), requires_grad=False)

    def forward(self, x):
        return G.rms_norm_ops(x, self.weight, 1e-6)


def _attention(hidden, heads, kv_heads, head_dim, gen, dtype):
    """The package's gated attention layer over 4-bit projections."""
    from dflash_mlx_amd.attention_layer import GatedAttention

    attn = GatedAttention(num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
                          q_proj=_qlinear(hidden, 2 * heads * head_dim, gen, dtype),
                          k_proj=_qlinear(hidden, kv_heads * head_dim, gen, dtype),
                          v_proj=_qlinear(hidden, kv_heads * head_dim, gen, dtype),
                          o_proj=_qlinear(heads * head_dim, hidden, gen, dtype), dtype=dtype)
    attn.q_norm.weight.data = (1 + 0.1 * torch.randn(head_dim, generator=gen)).to(dtype)
    attn.k_norm.weight.data = (1 + 0.1 * torch.randn(head_dim, generator=gen)).to(dtype)
    return attn


class MLP(nn.Module):
    def __init__(self, hidden, inner, gen, dtype):
        super().__init__()
        self.gate_proj = _qlinear(hidden, inner, gen, dtype)
        self.up_proj = _qlinear(hidden, inner, gen, dtype)
        self.down_proj = _qlinear(inner, hidden, gen, dtype)

    def forward(self, x):
        return self.down_proj(silu_gate_up(self, x))


class Block(nn.Module):
    def __init__(self, hidden, is_linear, gen, dtype, Hk, Hv, D):
        super().__init__()
        self.is_linear = is_linear
        self.input_layernorm, self.post_attention_layernorm = RMSNorm(hidden, dtype), RMSNorm(hidden, dtype)
        if is_linear:
            C = 2 * Hk * D + Hv * D
            self.linear_attn = G.GatedDeltaNet(
                hidden, num_k_heads=Hk, num_v_heads=Hv, head_k_dim=D, head_v_dim=D,
                in_proj_qkv=_qlinear(hidden, C, gen, dtype, 2.0), in_proj_z=_qlinear(hidden, Hv * D, gen, dtype),
                in_proj_b=_qlinear(hidden, 32, gen, dtype), in_proj_a=_qlinear(hidden, 32, gen, dtype),
                out_proj=_qlinear(Hv * D, hidden, gen, dtype), dtype=dtype)
            la = self.linear_attn
            la.in_proj_b, la.in_proj_a = _Slice(la.in_proj_b, Hv), _Slice(la.in_proj_a, Hv)
            la.conv1d.weight.data = (torch.randn((C, 4, 1), generator=gen) * 0.5).to(dtype)
            la.A_log.data = torch.log(torch.rand(Hv, generator=gen) * 2 + 0.2).to(dtype)
            la.dt_bias.data = (torch.randn(Hv, generator=gen) * 0.3).to(dtype)
        else:
            self.self_attn = _attention(hidden, Hv, max(1, Hv // 2), D, gen, dtype)
        self.mlp = MLP(hidden, 2 * hidden, gen, dtype)

    def forward(self, x, cache):
        if self.is_linear:
            mixed = self.linear_attn(self.input_layernorm(x), mask=None, cache=cache)
        else:
            mixed = self.self_attn(self.input_layernorm(x), mask="causal", cache=cache)
        x = x + mixed.to(x.dtype)
        return x + self.mlp(self.post_attention_layernorm(x))


class _Slice(nn.Module):
    """The first ``n`` outputs of a projection (keeps N a multiple of 32 for the 4-bit format)."""

    def __init__(self, inner, n):
        super().__init__()
        self.inner, self.n = inner, n

    def forward(self, x):
        return self.inner(x)[..., :self.n]


class ToyHybridLM(nn.Module):
    def __init__(self, *, vocab=384, hidden=256, pattern=(True, True, False, True), Hk=2, Hv=4, D=64,
                 dtype=torch.float32, seed=0):
        super().__init__()
        gen = torch.Generator().manual_seed(0xDF1A + seed)
        self.pattern = tuple(pattern)
        self.embed = nn.Embedding(vocab, hidden)
        self.embed.weight.data = torch.randn((vocab, hidden), generator=gen).to(dtype)
        self.layers = nn.ModuleList(Block(hidden, lin, gen, dtype, Hk, Hv, D) for lin in pattern)
        self.norm = RMSNorm(hidden, dtype)
        self.lm_head = nn.Linear(hidden, vocab, bias=False)
        self.lm_head.weight.data = (torch.randn((vocab, hidden), generator=gen) * hidden ** -0.5 * 4).to(dtype)

    def forward(self, ids, cache):
        x = self.embed(ids)
        for layer, c in zip(self.layers, cache):
            x = layer(x, c)
        return self.lm_head(self.norm(x)).float()

    def install_hooks(self, *, exact_attention_over=None):
        """The reference's per-layer hooks (dflash_mlx/runtime.py:620-652); the exact attention
        path starts at ``exact_attention_over`` cached positions (1024 if None)."""
        from dflash_mlx_amd.attention_layer import configure_full_attention_split

        for layer in self.layers:
            if layer.is_linear:
                G._install_exact_small_proj_hooks(layer.linear_attn)
                G._install_speculative_linear_cache_hook(layer.linear_attn)
        configure_full_attention_split(self.layers, enabled=True)
        if exact_attention_over is not None:
            for layer in self.layers:
                if not layer.is_linear:
                    layer.self_attn._dflash_split_sdpa_exact_kv_threshold = int(exact_attention_over)
        return self


def drafts(reference, vocab, seed=0):
    """Draft functions keyed by name: perfect (the reference continuation), random, and one
    that is right for the first few tokens of every block."""
    gen = torch.Generator().manual_seed(seed)

    def perfect(staged_first, block_len, committed):
        n = int(committed.shape[0])
        d = reference[n + 1:n + block_len]
        pad = block_len - 1 - int(d.shape[0])
        return torch.cat([d, d.new_zeros(pad)]).to(staged_first.device) if pad > 0 else d.to(staged_first.device)

    def random(staged_first, block_len, committed):
        return torch.randint(0, vocab, (block_len - 1,), generator=gen).to(staged_first.device)

    def partly(staged_first, block_len, committed):
        d = perfect(staged_first, block_len, committed).clone()
        right = int(torch.randint(0, block_len, (1,), generator=gen))
        if right < block_len - 1:
            d[right] = (d[right] + 1) % vocab
        return d

    return dict(perfect=perfect, random=random, partly=partly)
