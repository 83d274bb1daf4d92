"""A small hybrid language model for the end-to-end tests: GatedDeltaNet mixers (the
package's layer) and full-attention mixers over ``KVCache``, every projection an MLX-format
4-bit ``QuantizedLinear``, random weights.  Test infrastructure only."""
import torch
import torch.nn as nn

from dflash_mlx_amd import gdn_layer as G
from dflash_mlx_amd.cache import KVCache
from dflash_mlx_amd.quantized import QuantizedLinear


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


class Attention(nn.Module):
    def __init__(self, hidden, heads, head_dim, gen, dtype):
        super().__init__()
        self.heads, self.head_dim = heads, head_dim
        self.q_proj = _qlinear(hidden, heads * head_dim, gen, dtype)
        self.k_proj = _qlinear(hidden, heads * head_dim, gen, dtype)
        self.v_proj = _qlinear(hidden, heads * head_dim, gen, dtype)
        self.o_proj = _qlinear(heads * head_dim, hidden, gen, dtype)

    def forward(self, x, mask=None, cache=None):
        B, S, _ = x.shape
        split = lambda t: t.reshape(B, S, self.heads, self.head_dim).transpose(1, 2)
        q, k, v = split(self.q_proj(x)), split(self.k_proj(x)), split(self.v_proj(x))
        past = cache.offset if cache is not None else 0
        if cache is not None:
            k, v = cache.update_and_fetch(k, v)
        T = k.shape[2]
        pos_q = torch.arange(past, past + S, device=x.device)[:, None]
        allowed = torch.arange(T, device=x.device)[None, :] <= pos_q
        scores = (q.float() @ k.float().transpose(-1, -2)) * self.head_dim ** -0.5
        scores = scores.masked_fill(~allowed, float("-inf"))
        out = (torch.softmax(scores, dim=-1) @ v.float()).to(x.dtype)
        return self.o_proj(out.transpose(1, 2).reshape(B, S, -1))


class MLP(nn.Module):
    def __init__(self, hidden, inner, gen, dtype):
        super().__init__()
        self.gate_proj = _qlinear(hidden, inner, gen, dtype)
        self.up_proj = _qlinear(hidden, inner, gen, dtype)
        self.down_proj = _qlinear(inner, hidden, gen, dtype)

    def forward(self, x):
        return self.down_proj(G.silu_ops(self.gate_proj(x)) * self.up_proj(x))


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
            self.self_attn = Attention(hidden, Hv, D, gen, dtype)
        self.mlp = MLP(hidden, 2 * hidden, gen, dtype)

    def forward(self, x, cache):
        mixer = self.linear_attn if self.is_linear else self.self_attn
        x = x + mixer(self.input_layernorm(x), mask=None, cache=cache).to(x.dtype)
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

    def install_hooks(self):
        for layer in self.layers:
            if layer.is_linear:
                G._install_exact_small_proj_hooks(layer.linear_attn)
                G._install_speculative_linear_cache_hook(layer.linear_attn)
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
