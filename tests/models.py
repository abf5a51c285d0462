"""Small models used by the planner tests: the two architectures the reference's planner
tests plan (a two-layer FFN with pass-through inputs and a transformer block:
tests/test_optimize_placement.py:65-135), written for this repository."""

import torch
from torch import nn


def _attention(q, k, v):
    from torch._subclasses.fake_tensor import is_fake

    if is_fake(q):
        # name the memory-efficient attention operator so the traced graph is the same on
        # every device (it is what a CUDA / HIP device dispatches to for these shapes)
        return torch.ops.aten._scaled_dot_product_efficient_attention(q, k, v, None, True)[0]
    return nn.functional.scaled_dot_product_attention(q, k, v)


class TwoLayerFFN(nn.Module):
    def __init__(self, dim1, dim2):
        super().__init__()
        self.linear1 = nn.Linear(dim1, dim2, bias=False)
        self.linear2 = nn.Linear(dim2, dim1, bias=False)

    def forward(self, x, y):
        return y + 2, self.linear2(self.linear1(x)), y + 2


class AttentionMLPBlock(nn.Module):
    def __init__(self, nheads, dim1, dim2):
        super().__init__()
        self.nheads = nheads
        self.wq = nn.Linear(dim1, dim1, bias=False)
        self.wk = nn.Linear(dim1, dim1, bias=False)
        self.wv = nn.Linear(dim1, dim1, bias=False)
        self.wo = nn.Linear(dim1, dim1, bias=False)
        self.w1 = nn.Linear(dim1, dim2, bias=False)
        self.w2 = nn.Linear(dim2, dim1, bias=False)

    def forward(self, x):
        def heads(t):
            return t.unflatten(-1, (self.nheads, -1)).permute(0, 2, 1, 3)

        o = _attention(heads(self.wq(x)), heads(self.wk(x)), heads(self.wv(x)))
        o = self.wo(o.permute(0, 2, 1, 3).flatten(-2))
        h = o + x
        return h + self.w2(torch.relu(self.w1(h)))


class LocalMapAttentionBlock(nn.Module):
    """The transformer block with its attention inside a ``local_map`` region whose author
    fixes the placements on a 3-D (dp, tp, cp) mesh: context-parallel attention, query
    sharded over the sequence, key / value gathered
    (tests/test_optimize_placement.py:371-423)."""

    def __init__(self, nheads, dim1, dim2, mesh):
        super().__init__()
        self.nheads = nheads
        self.mesh = mesh
        self.wq = nn.Linear(dim1, dim1, bias=False)
        self.wk = nn.Linear(dim1, dim1, bias=False)
        self.wv = nn.Linear(dim1, dim1, bias=False)
        self.wo = nn.Linear(dim1, dim1, bias=False)
        self.w1 = nn.Linear(dim1, dim2, bias=False)
        self.w2 = nn.Linear(dim2, dim1, bias=False)

    def forward(self, x):
        from torch.distributed._tensor.experimental import local_map
        from torch.distributed.tensor.placement_types import Replicate, Shard

        @local_map(out_placements=((Shard(0), Shard(1), Shard(2)),),
                   in_placements=((Shard(0), Shard(1), Shard(2)), (Shard(0), Shard(1), Replicate()),
                                  (Shard(0), Shard(1), Replicate())),
                   redistribute_inputs=True, in_grad_placements=None, device_mesh=self.mesh)
        def context_parallel_attention(query, key, value):
            return (nn.functional.scaled_dot_product_attention(query=query, key=key, value=value, is_causal=False),)

        def heads(t):
            return t.unflatten(-1, (self.nheads, -1)).permute(0, 2, 1, 3)

        o = context_parallel_attention(heads(self.wq(x)), heads(self.wk(x)), heads(self.wv(x)))[0]
        o = self.wo(o.permute(0, 2, 1, 3).flatten(-2))
        h = o + x
        return h + self.w2(torch.relu(self.w1(h)))


class AddSmallParameter(nn.Module):
    """x + a parameter with fewer elements than the mesh has ranks
    (tests/test_optimize_placement.py:496-533)."""

    def __init__(self, dim):
        super().__init__()
        self.param = nn.Parameter(torch.rand(dim))

    def forward(self, x):
        return x + self.param


def make_model_and_inputs(mesh, kind):
    if kind == "ffn":
        bs, d1, d2 = 2048 * mesh.shape[0], 1024, 4096
        return (lambda: TwoLayerFFN(d1, d2)), (lambda: (torch.randn(bs, d1), torch.randn(bs, 1)))
    if kind == "block":
        bs, d1, nheads = 8 * mesh.shape[0], 6144, 48
        return (lambda: AttentionMLPBlock(nheads, d1, d1 * 4)), (lambda: torch.randn(bs, 256, d1, requires_grad=True))
    if kind == "local_map_block":
        bs, d1, nheads = 8 * mesh.shape[0], 6144, 48
        return (lambda: LocalMapAttentionBlock(nheads, d1, d1 * 4, mesh)), \
            (lambda: torch.randn(bs, 256, d1, requires_grad=True))
    if kind == "small_param":
        dim = mesh.shape[0] // 2
        return (lambda: AddSmallParameter(dim)), (lambda: (torch.rand(512, dim),))
    raise ValueError(kind)
