"""A Llama-3 style decoder, used only to give the planner benchmark graphs their shape
(it is traced on fake tensors; no weights are ever materialised).

Architecture: token embedding, N pre-norm blocks of grouped-query attention with rotary
embeddings (complex formulation) and a SwiGLU feed-forward, final RMSNorm and an output
projection.  The configurations follow the public Llama-3 model cards, as the reference's
planning example selects them (examples/example_llama3.py:56-80).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F
from torch import nn


@dataclass
class LlamaConfig:
    dim: int = 4096
    n_layers: int = 32
    n_heads: int = 32
    n_kv_heads: int = 8
    vocab_size: int = 128256
    ffn_dim_multiplier: float = 1.3
    multiple_of: int = 1024
    norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    max_seq_len: int = 8192

    @property
    def ffn_hidden(self) -> int:
        hidden = int(2 * (4 * self.dim) / 3)
        hidden = int(self.ffn_dim_multiplier * hidden)
        return self.multiple_of * ((hidden + self.multiple_of - 1) // self.multiple_of)


LLAMA3_8B = LlamaConfig()  # FFN 14336
LLAMA3_70B = LlamaConfig(dim=8192, n_layers=80, n_heads=64, n_kv_heads=8, ffn_dim_multiplier=1.3,
                         multiple_of=4096)  # FFN 28672
# one block of the single-block configuration: dim 1024, 16 heads, FFN 4096
BLOCK_1K = LlamaConfig(dim=1024, n_layers=1, n_heads=16, n_kv_heads=16, vocab_size=32000, ffn_dim_multiplier=1.5,
                       multiple_of=256, max_seq_len=2048)


def rotary_table(head_dim: int, length: int, theta: float) -> torch.Tensor:
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2)[: head_dim // 2].float() / head_dim))
    angles = torch.outer(torch.arange(length, dtype=torch.float32), inv)
    return torch.polar(torch.ones_like(angles), angles)  # complex64 [length, head_dim / 2]


def rotate(x: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """x: [b, s, h, d] real; table: [s, d/2] complex."""
    xc = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2))
    t = table.view(1, xc.shape[1], 1, xc.shape[3])
    return torch.view_as_real(xc * t).flatten(3).type_as(x)


def causal_attention(q, k, v):
    """Causal scaled-dot-product attention on [b, h, s, d] operands.  On fake tensors the
    flash-attention operator is named directly so that the captured graph holds the same
    attention nodes (forward and backward) whatever device the trace runs on; real
    tensors go through the public functional."""
    from torch._subclasses.fake_tensor import is_fake

    if is_fake(q):
        return torch.ops.aten._scaled_dot_product_flash_attention(q, k, v, 0.0, True, False)[0]
    return F.scaled_dot_product_attention(q, k, v, is_causal=True)


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x):
        h = x.float()
        h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.eps)
        return h.type_as(x) * self.weight


class Attention(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.n_heads, self.n_kv = cfg.n_heads, cfg.n_kv_heads
        self.head_dim = cfg.dim // cfg.n_heads
        self.wq = nn.Linear(cfg.dim, cfg.n_heads * self.head_dim, bias=False)
        self.wk = nn.Linear(cfg.dim, cfg.n_kv_heads * self.head_dim, bias=False)
        self.wv = nn.Linear(cfg.dim, cfg.n_kv_heads * self.head_dim, bias=False)
        self.wo = nn.Linear(cfg.n_heads * self.head_dim, cfg.dim, bias=False)

    def forward(self, x, table):
        b, s, _ = x.shape
        q = self.wq(x).view(b, s, -1, self.head_dim)
        k = self.wk(x).view(b, s, -1, self.head_dim)
        v = self.wv(x).view(b, s, -1, self.head_dim)
        q, k = rotate(q, table), rotate(k, table)
        rep = self.n_heads // self.n_kv
        if rep > 1:  # grouped-query attention: repeat each kv head
            k = k[:, :, :, None, :].expand(b, s, self.n_kv, rep, self.head_dim).reshape(b, s, -1, self.head_dim)
            v = v[:, :, :, None, :].expand(b, s, self.n_kv, rep, self.head_dim).reshape(b, s, -1, self.head_dim)
        out = causal_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
        return self.wo(out.transpose(1, 2).contiguous().view(b, s, -1))


class FeedForward(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.w1 = nn.Linear(cfg.dim, cfg.ffn_hidden, bias=False)
        self.w2 = nn.Linear(cfg.ffn_hidden, cfg.dim, bias=False)
        self.w3 = nn.Linear(cfg.dim, cfg.ffn_hidden, bias=False)

    def forward(self, x):
        return self.w2(F.silu(self.w1(x)) * self.w3(x))


class Block(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.attention = Attention(cfg)
        self.feed_forward = FeedForward(cfg)
        self.attention_norm = RMSNorm(cfg.dim, cfg.norm_eps)
        self.ffn_norm = RMSNorm(cfg.dim, cfg.norm_eps)

    def forward(self, x, table):
        h = x + self.attention(self.attention_norm(x), table)
        return h + self.feed_forward(self.ffn_norm(h))


class Llama(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.cfg = cfg
        self.tok_embeddings = nn.Embedding(cfg.vocab_size, cfg.dim)
        self.layers = nn.ModuleList(Block(cfg) for _ in range(cfg.n_layers))
        self.norm = RMSNorm(cfg.dim, cfg.norm_eps)
        self.output = nn.Linear(cfg.dim, cfg.vocab_size, bias=False)
        self.register_buffer("rope", rotary_table(cfg.dim // cfg.n_heads, cfg.max_seq_len, cfg.rope_theta),
                             persistent=False)

    def forward(self, tokens):
        h = self.tok_embeddings(tokens)
        table = self.rope[: tokens.shape[1]]
        for layer in self.layers:
            h = layer(h, table)
        return self.output(self.norm(h))


class SingleBlock(nn.Module):
    """One decoder block on activations (the single-transformer-block configuration)."""

    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.cfg = cfg
        self.block = Block(cfg)
        self.register_buffer("rope", rotary_table(cfg.dim // cfg.n_heads, cfg.max_seq_len, cfg.rope_theta),
                             persistent=False)

    def forward(self, x):
        return self.block(x, self.rope[: x.shape[1]])
