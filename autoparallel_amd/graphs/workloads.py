"""The benchmark workloads as encoded cost tables.

``llama3_tables`` traces a Llama-3 style decoder (joint forward+backward, bf16 parameter
casts, alias nodes), enumerates the placement strategies of every node on a logical mesh
and flattens them; the per-strategy flop / byte counts still have to be filled in from the
device's shard-shape table (see ``finish_strategy_inputs``).
"""

from __future__ import annotations

import dataclasses
import time
import warnings

import torch

from .capture import capture_joint_graph
from .cost_inputs import fill_flops_and_bytes
from .encode import encode_graph
from .llama3 import BLOCK_1K, LLAMA3_8B, LLAMA3_70B, Llama, SingleBlock
from .strategies import StrategyEnumerator


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
    # name: (config, mesh, batch, seq, param dtype, reduce dtype)
    "llama3_8b": (LLAMA3_8B, (32, 8), 32, 8192),
    "llama3_70b": (LLAMA3_70B, (8, 8, 8), 64, 8192),
    "block_1k": (BLOCK_1K, (64,), 8, 2048),
}


def traced_tables(name: str, n_layers=None, mesh_sizes=None):
    """Returns (encoded graph, strategies, context) for a named workload; ``context`` keeps
    the capture alive (fake tensors are needed until the flop / byte inference is done) and
    carries the host-side timings."""
    cfg, mesh_default, batch, seq = WORKLOADS[name]
    mesh_sizes = tuple(mesh_sizes or mesh_default)
    if n_layers is not None:
        cfg = dataclasses.replace(cfg, n_layers=n_layers)
    mesh = logical_mesh(mesh_sizes)
    timings = {}
    with torch.device("meta"):
        model = SingleBlock(cfg) if name == "block_1k" else Llama(cfg)
    if name == "block_1k":
        def input_fn():
            return torch.randn(batch, seq, cfg.dim, dtype=torch.bfloat16, requires_grad=True)
    else:
        def input_fn():
            return torch.randint(0, cfg.vocab_size, (batch, seq))
    t0 = time.perf_counter()
    ctx = capture_joint_graph(model, input_fn, param_dtype=torch.bfloat16)
    gm, joint = ctx.__enter__()
    timings["capture_s"] = time.perf_counter() - t0
    try:
        t0 = time.perf_counter()
        enumerator = StrategyEnumerator(mesh)
        strats = enumerator.enumerate(gm.graph)
        timings["enumerate_s"] = time.perf_counter() - t0
        from torch._functorch._aot_autograd.fx_utils import get_param_and_grad_nodes

        grads = set(g for _, g in get_param_and_grad_nodes(gm.graph).values() if g is not None)
        t0 = time.perf_counter()
        encoded = encode_graph(gm.graph, strats, mesh_sizes, grads)
        timings["encode_s"] = time.perf_counter() - t0
    except BaseException:
        ctx.__exit__(None, None, None)
        raise
    info = {"ctx": ctx, "gm": gm, "mesh": mesh, "timings": timings, "config": cfg, "batch": batch, "seq": seq,
            "mesh_sizes": mesh_sizes}
    return encoded, strats, info


def finish_strategy_inputs(encoded, strats, local_shape, local_stride, info):
    t0 = time.perf_counter()
    stats = {}
    fill_flops_and_bytes(encoded, strats, local_shape, local_stride, stats)
    info["timings"]["flops_bytes_s"] = time.perf_counter() - t0
    info["cost_input_stats"] = stats
