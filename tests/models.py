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


def make_model_and_inputs(mesh, kind):
    if kind == "ffn":
        bs, d1, d2 = 2048 * mesh.shape[0], 1024, 4096
        return (lambda: TwoLayerFFN(d1, d2)), (lambda: (torch.randn(bs, d1), torch.randn(bs, 1)))
    if kind == "block":
        bs, d1, nheads = 8 * mesh.shape[0], 6144, 48
        return (lambda: AttentionMLPBlock(nheads, d1, d1 * 4)), (lambda: torch.randn(bs, 256, d1, requires_grad=True))
    raise ValueError(kind)
