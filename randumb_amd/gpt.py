"""GPT-2-small-shaped model whose linears are random-backed, for the end-to-end step-time configuration.

Mirrors the reference's RT_* classes (modded-nanogpt/gpt_models.py:186-257: RT_norm, RT_CastedLinear,
RT_CausalSelfAttention, RT_MLP, RT_Block) with the deviations the benchmark configuration states: the four linears of a
block are qkv (d -> 3d), proj (d -> d), fc (d -> 4d) and mlp-proj (4d -> d), all in matrix-coef form with coefficient
dimension k and seeds taken in layer order from one generator (0..47 for 12 layers); attention is plain causal
scaled-dot-product attention (the reference's FlexAttention document mask needs a tracing compiler); the token embedding
and the language-model head are ordinary dense layers unless the configuration asks for the reference's random-backed ones
(modded-nanogpt/gpt_models.py:303, 310).  Everything that is not a random-backed linear is stock PyTorch: this file
wires layers, the kernels are reached through SillyLinear.
"""
from dataclasses import dataclass
from typing import Generator

import torch
import torch.nn.functional as F
from torch import nn

from .SillyLayers import SillyEmbedding, SillyLinear


def RT_norm(x: torch.Tensor) -> torch.Tensor:
    return F.rms_norm(x, (x.size(-1),))


class Rotary(nn.Module):
    """Rotary position embedding over (batch, time, head, head_dim), as gpt_models.py:29-49."""

    def __init__(self, dim: int, base: float = 10000.0):
        super().__init__()
        self.register_buffer("inv_freq", (1.0 / base) ** (torch.arange(0, dim, 2) / dim), persistent=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        t = torch.arange(x.shape[1], device=x.device)
        freqs = torch.outer(t, self.inv_freq.to(x.device))
        cos, sin = freqs.cos()[None, :, None, :], freqs.sin()[None, :, None, :]
        x1, x2 = x.float().chunk(2, dim=3)
        return torch.cat((x1 * cos + x2 * sin, x2 * cos - x1 * sin), 3).type_as(x)


@dataclass
class RT_GPTConfig:
    int_dim_gen: Generator
    seed_gen: Generator
    vocab_size: int = 50304
    n_layer: int = 12
    n_head: int = 12
    n_embd: int = 768
    # True: the token embedding and the output head are random-backed too, as in the reference's model
    # (modded-nanogpt/gpt_models.py:303, 310); they then draw the first and the last (k, seed) of the generators
    random_embedding_and_head: bool = False


class RT_CastedLinear(SillyLinear):
    """Bias-free random-backed linear in matrix-coef form; the fused kernels run in the activations' dtype."""

    def __init__(self, in_features: int, out_features: int, config: RT_GPTConfig):
        k, seed = next(config.int_dim_gen), next(config.seed_gen)
        super().__init__(in_features, out_features, [k, k], [seed, seed], bias=False, matrix_coef=True)
        std = 0.02
        with torch.no_grad():   # C ~ N(0, 3*std^2/k): the weight then has standard deviation ~std
            self.weight_coef.normal_(0.0, (3.0 * std * std / k) ** 0.5)
            self.weight_scale_bias.zero_()


class RT_CausalSelfAttention(nn.Module):
    def __init__(self, dim: int, n_head: int, config: RT_GPTConfig):
        super().__init__()
        assert dim % n_head == 0
        self.n_head = n_head
        self.c_qkv = RT_CastedLinear(dim, 3 * dim, config)
        self.rotary = Rotary(dim // n_head)
        self.c_proj = RT_CastedLinear(dim, dim, config)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        B, T, D = x.shape
        q, k, v = self.c_qkv(x).view(B, T, 3, self.n_head, D // self.n_head).unbind(2)
        q, k = RT_norm(q), RT_norm(k)
        q, k = self.rotary(q), self.rotary(k)
        y = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True)
        return self.c_proj(y.transpose(1, 2).reshape(B, T, D))


class RT_MLP(nn.Module):
    def __init__(self, dim: int, config: RT_GPTConfig):
        super().__init__()
        self.c_fc = RT_CastedLinear(dim, 4 * dim, config)
        self.c_proj = RT_CastedLinear(4 * dim, dim, config)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.c_proj(F.relu(self.c_fc(x)).square())


class RT_Block(nn.Module):
    def __init__(self, config: RT_GPTConfig):
        super().__init__()
        self.attn = RT_CausalSelfAttention(config.n_embd, config.n_head, config)
        self.mlp = RT_MLP(config.n_embd, config)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        x = x + self.attn(RT_norm(x))
        return x + self.mlp(RT_norm(x))


class RT_GPT(nn.Module):
    """Seeds are drawn qkv, proj, fc, mlp-proj per block, block after block."""

    def __init__(self, config: RT_GPTConfig):
        super().__init__()
        if config.random_embedding_and_head:
            self.wte = SillyEmbedding(config.vocab_size, config.n_embd, config.int_dim_gen, config.seed_gen)
        else:
            self.wte = nn.Embedding(config.vocab_size, config.n_embd)
        self.h = nn.ModuleList([RT_Block(config) for _ in range(config.n_layer)])
        if config.random_embedding_and_head:
            self.lm_head = RT_CastedLinear(config.n_embd, config.vocab_size, config)
        else:
            self.lm_head = nn.Linear(config.n_embd, config.vocab_size, bias=False)

    def forward(self, idx: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
        x = self.wte(idx)
        x = RT_norm(x.to(self.h[0].mlp.c_fc.weight_coef.dtype))
        for block in self.h:
            x = block(x)
        logits = self.lm_head(RT_norm(x)).float()
        return F.cross_entropy(logits.view(-1, logits.size(-1)), target.view(-1))
