"""The traced benchmark workloads: model, synthetic input and logical mesh of every named
configuration (Llama-3 8B / 70B decoders, the single transformer block, the DeepSeek-V3
style mixture of experts)."""

from __future__ import annotations

import dataclasses
import warnings

import torch

from .dsv3 import DSV3_16L, DeepSeekV3
from .llama3 import BLOCK_1K, LLAMA3_8B, LLAMA3_70B, Llama, SingleBlock


def logical_mesh(mesh_sizes, names=None):
    """A DeviceMesh over a "fake" process group: ranks are modelled, nothing communicates
    (as the reference's planner tests and examples do, tests/test_optimize_placement.py:20-62)."""
    import math

    import torch.distributed as dist
    from torch.distributed.device_mesh import init_device_mesh
    from torch.testing._internal.distributed.fake_pg import FakeStore

    world = math.prod(mesh_sizes)
    if not dist.is_initialized():
        dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=max(world, 512))
    elif dist.get_world_size() < world:
        raise RuntimeError(f"process group has {dist.get_world_size()} ranks, the mesh needs {world}")
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        return init_device_mesh("cpu", tuple(mesh_sizes), mesh_dim_names=names)


WORKLOADS = {
    # name: (config, logical mesh, batch, sequence length)
    "llama3_8b": (LLAMA3_8B, (32, 8), 32, 8192),
    "llama3_70b": (LLAMA3_70B, (8, 8, 8), 64, 8192),
    "block_1k": (BLOCK_1K, (64,), 8, 2048),
    "dsv3_moe": (DSV3_16L, (64, 4), 16, 4096),
}


def build_model(name: str, mesh, n_layers=None, batch=None, seq=None, config=None):
    """-> (model on the meta device, input_fn, description, needs_dynamo) for a named
    workload planned on ``mesh``.  ``needs_dynamo``: the model has ``local_map`` regions, so
    its forward must be captured with Dynamo before the joint export."""
    cfg, _, batch_default, seq_default = WORKLOADS[name]
    cfg = config or cfg
    if n_layers is not None:
        cfg = dataclasses.replace(cfg, n_layers=n_layers)
    batch, seq = batch or batch_default, seq or seq_default
    with torch.device("meta"):
        if name == "block_1k":
            model = SingleBlock(cfg)
        elif name == "dsv3_moe":
            model = DeepSeekV3(cfg, mesh)
        else:
            model = Llama(cfg)
    if name == "block_1k":
        def input_fn():
            return torch.randn(batch, seq, cfg.dim, dtype=torch.bfloat16, requires_grad=True)
    else:
        def input_fn():
            return torch.randint(0, cfg.vocab_size, (batch, seq))
    desc = (f"{name} joint fwd+bwd graph ({cfg.n_layers} layers, dim {cfg.dim}, batch {batch}, seq {seq}, "
            f"bf16 params / fp32 reduce), logical mesh {tuple(mesh.shape)}")
    return model, input_fn, desc, name == "dsv3_moe"
