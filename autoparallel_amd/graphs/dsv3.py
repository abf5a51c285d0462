"""A DeepSeek-V3 style mixture-of-experts decoder, used only to give the planner a benchmark
graph of that shape (traced on fake tensors; no weights are ever materialised).

Architecture (public DeepSeek-V3 model card): multi-head latent attention (low-rank query
and key/value projections with a decoupled rotary part), a dense SwiGLU feed-forward in the
first layers and, in the others, a mixture of experts: a sigmoid router picks ``top_k`` of
``n_routed_experts`` per token, a shared expert sees every token.

The routed experts run inside one ``local_map`` region per layer, as in the reference's
planning model (autoparallel/_testing/models/dsv3.py:878-985): the region's author fixes
the placements at its boundary (tokens sharded over every rank, experts sharded over the
expert-parallel mesh dim), and the planner treats the region as a single node with that
one strategy.  What happens inside (token dispatch to the ranks that own the experts,
grouped expert matmuls, combine) is invisible to planning; the body below is the local
computation on one rank's tokens and experts with evenly filled experts.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F
from torch import nn

from .llama3 import RMSNorm, rotary_table, rotate


@dataclass
class DeepSeekV3Config:
    dim: int = 7168
    n_layers: int = 16
    n_dense_layers: int = 1
    n_heads: int = 128
    q_lora_rank: int = 1536
    kv_lora_rank: int = 512
    qk_nope_head_dim: int = 128
    qk_rope_head_dim: int = 64
    v_head_dim: int = 128
    inter_dim: int = 18432       # dense feed-forward
    moe_inter_dim: int = 2048    # one expert
    n_routed_experts: int = 256
    n_shared_experts: int = 1
    top_k: int = 8
    token_shard_dim: int = 1     # dim of [batch, seq, dim] activations the expert regions shard tokens along
    route_scale: float = 2.5
    vocab_size: int = 129280
    norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    max_seq_len: int = 4096


DSV3_16L = DeepSeekV3Config()


def attention_unequal_heads(q, k, v, scale):
    """Causal attention whose value heads are narrower than its query/key heads, on
    [b, h, s, d] operands.  On fake tensors the memory-efficient attention operator (the one
    that accepts such shapes) is named directly, so the captured graph is the same on every
    device."""
    from torch._subclasses.fake_tensor import is_fake

    if torch.compiler.is_compiling() or is_fake(q):  # (Dynamo cannot trace is_fake: it is asked first)
        return torch.ops.aten._scaled_dot_product_efficient_attention(q, k, v, None, True, 0.0, True, scale=scale)[0]
    return F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=scale)


class LatentAttention(nn.Module):
    def __init__(self, cfg: DeepSeekV3Config):
        super().__init__()
        self.h = cfg.n_heads
        self.nope, self.rope, self.vd = cfg.qk_nope_head_dim, cfg.qk_rope_head_dim, cfg.v_head_dim
        self.kv_rank = cfg.kv_lora_rank
        self.wq_a = nn.Linear(cfg.dim, cfg.q_lora_rank, bias=False)
        self.q_norm = RMSNorm(cfg.q_lora_rank, cfg.norm_eps)
        self.wq_b = nn.Linear(cfg.q_lora_rank, cfg.n_heads * (self.nope + self.rope), bias=False)
        self.wkv_a = nn.Linear(cfg.dim, cfg.kv_lora_rank + self.rope, bias=False)
        self.kv_norm = RMSNorm(cfg.kv_lora_rank, cfg.norm_eps)
        self.wkv_b = nn.Linear(cfg.kv_lora_rank, cfg.n_heads * (self.nope + self.vd), bias=False)
        self.wo = nn.Linear(cfg.n_heads * self.vd, cfg.dim, bias=False)
        self.scale = (self.nope + self.rope) ** -0.5

    def forward(self, x, table):
        b, s, _ = x.shape
        q = self.wq_b(self.q_norm(self.wq_a(x))).view(b, s, self.h, self.nope + self.rope)
        q = torch.cat([q[..., : self.nope], rotate(q[..., self.nope:], table)], dim=-1)
        kv = self.wkv_a(x)
        k_pe = rotate(kv[..., self.kv_rank:].unsqueeze(2), table)  # one rotary key shared by all heads
        kv = self.wkv_b(self.kv_norm(kv[..., : self.kv_rank])).view(b, s, self.h, self.nope + self.vd)
        k = torch.cat([kv[..., : self.nope], k_pe.expand(b, s, self.h, self.rope)], dim=-1)
        v = kv[..., self.nope:]
        out = attention_unequal_heads(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), self.scale)
        return self.wo(out.transpose(1, 2).contiguous().view(b, s, self.h * self.vd))


class SwiGLU(nn.Module):
    def __init__(self, dim: int, hidden: int):
        super().__init__()
        self.w1 = nn.Linear(dim, hidden, bias=False)
        self.w2 = nn.Linear(hidden, dim, bias=False)
        self.w3 = nn.Linear(dim, hidden, bias=False)

    def forward(self, x):
        return self.w2(F.silu(self.w1(x)) * self.w3(x))


def routed_experts(x, indices, scores, w1, w3, w2, out, top_k: int):
    """One rank's share of the routed experts (the body of the ``local_map`` region).
    x, out: [b, s, dim]; indices / scores: [b, s, top_k]; w1, w3: [e, hidden, dim];
    w2: [e, dim, hidden].  Token copies are grouped by expert, every expert takes an equal
    share of them, and the weighted expert outputs are added onto ``out``.  (Arguments are
    declared in the order the body first uses them: Dynamo lifts a region's inputs in that
    order and insists that the declared placements follow it.)"""
    e, dim = w1.shape[0], x.shape[-1]
    tokens = x.reshape(-1, dim)
    order = torch.argsort(indices.reshape(-1), stable=True)
    token_of_copy = order // top_k
    weight = scores.reshape(-1)[order]
    routed = (tokens[token_of_copy].float() * weight[:, None]).to(x.dtype).view(e, -1, dim)
    hidden = F.silu(torch.bmm(routed, w1.transpose(1, 2))) * torch.bmm(routed, w3.transpose(1, 2))
    routed_out = torch.bmm(hidden, w2.transpose(1, 2)).view(-1, dim)
    out = out.reshape(-1, dim).index_add(0, token_of_copy, routed_out).view(x.shape)
    load = torch.histc(indices.reshape(-1).float(), bins=e, min=0, max=e)
    return out, load[None, :]


class MixtureOfExperts(nn.Module):
    def __init__(self, cfg: DeepSeekV3Config, mesh):
        super().__init__()
        self.cfg = cfg
        self.mesh = mesh
        e, d, h = cfg.n_routed_experts, cfg.dim, cfg.moe_inter_dim
        self.gate = nn.Linear(d, e, bias=False)
        self.w1 = nn.Parameter(torch.empty(e, h, d))
        self.w2 = nn.Parameter(torch.empty(e, d, h))
        self.w3 = nn.Parameter(torch.empty(e, h, d))
        self.shared = SwiGLU(d, h * cfg.n_shared_experts)

    def forward(self, x):
        from torch.distributed._tensor.experimental import local_map
        from torch.distributed.tensor.placement_types import Replicate, Shard

        affinity = torch.sigmoid(self.gate(x).float())
        scores, indices = torch.topk(affinity, self.cfg.top_k, dim=-1)
        scores = scores / scores.sum(dim=-1, keepdim=True) * self.cfg.route_scale
        shared = self.shared(x)
        nd = self.mesh.ndim
        # tokens over every rank, along the dim the configuration names (the sequence by default:
        # a batch smaller than the mesh cannot be split over it); experts over the expert-parallel
        # (first) mesh dim; the per-expert load is a small statistic and comes back replicated
        token_sharded = (Shard(self.cfg.token_shard_dim),) * nd
        expert_sharded = (Shard(0),) + (Replicate(),) * (nd - 1)
        replicated = (Replicate(),) * nd
        region = local_map(
            routed_experts,
            out_placements=(token_sharded, replicated),
            in_placements=(token_sharded, token_sharded, token_sharded, expert_sharded, expert_sharded,
                           expert_sharded, token_sharded, None),
            redistribute_inputs=True, in_grad_placements=None, device_mesh=self.mesh)
        out, _load = region(x, indices, scores, self.w1, self.w3, self.w2, shared, self.cfg.top_k)
        return out


class MoEBlock(nn.Module):
    def __init__(self, cfg: DeepSeekV3Config, mesh, dense: bool):
        super().__init__()
        self.attention = LatentAttention(cfg)
        self.feed_forward = SwiGLU(cfg.dim, cfg.inter_dim) if dense else MixtureOfExperts(cfg, mesh)
        self.attention_norm = RMSNorm(cfg.dim, cfg.norm_eps)
        self.ffn_norm = RMSNorm(cfg.dim, cfg.norm_eps)

    def forward(self, x, table):
        h = x + self.attention(self.attention_norm(x), table)
        return h + self.feed_forward(self.ffn_norm(h))


class DeepSeekV3(nn.Module):
    """``mesh`` is the logical device mesh the expert regions are declared on (the same one
    the planner plans for)."""

    def __init__(self, cfg: DeepSeekV3Config, mesh):
        super().__init__()
        self.cfg = cfg
        self.tok_embeddings = nn.Embedding(cfg.vocab_size, cfg.dim)
        self.layers = nn.ModuleList(MoEBlock(cfg, mesh, dense=i < cfg.n_dense_layers) for i in range(cfg.n_layers))
        self.norm = RMSNorm(cfg.dim, cfg.norm_eps)
        self.output = nn.Linear(cfg.dim, cfg.vocab_size, bias=False)
        self.register_buffer("rope", rotary_table(cfg.qk_rope_head_dim, cfg.max_seq_len, cfg.rope_theta),
                             persistent=False)

    def forward(self, tokens):
        h = self.tok_embeddings(tokens)
        table = self.rope[: tokens.shape[1]]
        for layer in self.layers:
            h = layer(h, table)
        return self.output(self.norm(h))
