"""The benchmark tables at their full size, every entry against the C oracle: the 80-layer
Llama-3-70B graph on (8, 8, 8) and the 16-layer DeepSeek-V3 style mixture of experts at its
stated width on (64, 4) through the planner, and the 200 000-node synthetic DAG on (16, 8, 4).
(The Llama-3-8B graph at full depth: test_traced_graphs.py.)"""

import numpy as np
import pytest
import torch

from autoparallel_amd import CostModelParams
from autoparallel_amd.api import AutoParallelPlanner
from autoparallel_amd.device_tables import DeviceCostTables
from autoparallel_amd.graphs.cost_inputs import fill_flops_and_bytes
from autoparallel_amd.graphs.llama3 import LLAMA3_70B
from autoparallel_amd.synthetic import stress_dag
from oracle import c_oracle
from oracle import cost_oracle as po
from test_traced_graphs import _planner

pytestmark = pytest.mark.gpu


def _progress(what):
    print(f"[full size] {what}", flush=True)  # (a long test keeps telling where it is)


def test_full_depth_llama3_70b_on_mesh_8x8x8(gpu_device, fake_pg):
    """Configuration 3 at full size (examples/example_llama3.py:69-80): 80 layers, batch 64 x 8192
    tokens, mesh (8, 8, 8), linked layers, 73 M cost entries.  Flop / byte counts from the device
    against the host path under torch's flop counter; compute costs, every comm / transition /
    cost entry and the row minima against the C oracle; then the pruned solve: its plan is
    feasible and its objective is the sum of the oracle's costs of the chosen entries."""
    mesh = (8, 8, 8)
    with _planner(AutoParallelPlanner, LLAMA3_70B, mesh, 64, 8192, repeated_subgraphs=True) as autop:
        o = autop.sharding_optimizer
        enc, tb = o.encoded, o.encoded.tables
        _progress("planner built")
        assert tb.n_entries == 73_251_434 and o.cost_input_stats["strategy_inputs"] == "device"
        assert o.backend.launches == ("input_tables", "redistribute_tables")
        # flop / byte counts: what the device wrote against the reference's way, on the host
        device_counts = {k: getattr(tb, k).copy() for k in ("strat_flops", "strat_rw_bytes", "strat_dtype", "strat_zero_cost")}
        _, lshape, lstride, _, _ = c_oracle.spec_tables(tb.as_dict(), mesh)
        fill_flops_and_bytes(enc, o.strats, np.asarray(lshape), np.asarray(lstride))
        for k, v in device_counts.items():
            assert np.array_equal(getattr(tb, k), v), k
        _progress("flop / byte counts equal the host path's")
        params = po.make_params(mesh, rescale=2.2)
        want_compute, want_per_arg = c_oracle.compute_costs(tb.as_dict(), params)[:2]
        assert np.array_equal(o.compute_cost, want_compute) and np.array_equal(o.compute_cost_per_arg, want_per_arg)
        want = c_oracle.build_tables(tb.as_dict(), params, per_arg=want_per_arg)
        _progress("oracle tables built")
        for name in ("cost", "comm", "transition"):
            # (through the backend: the capture's fake-tensor mode is active inside this block)
            assert np.array_equal(o.backend.host_array(name), want[name]), name
            _progress(f"{name} equal")
        mins, args = o.row_minima()
        want_min, want_arg = c_oracle.segmented_min(want["cost"], tb.row_ptr())
        assert np.array_equal(mins, want_min) and np.array_equal(args, want_arg)
        _progress("row minima equal")
        from torch.distributed.tensor.placement_types import Replicate, Shard

        autop.add_parameter_memory_constraint(low=None, high=None)  # examples/example_llama3.py:205-218 on a 3-D mesh
        autop.add_input_constraints([(Shard(0), Replicate(), Replicate())])
        autop.add_output_constraints([(Shard(0), Replicate(), Replicate())])
        autop.optimize_placement()
        stats = o.solve_stats
        assert stats["incumbent"] is not None and stats["columns_after_pruning"] < 0.01 * stats["columns"], stats
        assert stats["lower_bound"] <= stats["incumbent"] * (1 + 1e-9)
        entries = np.asarray(o.res_entries, np.int64)
        assert o.objective_value() == float(want["cost"][entries].sum()) > 0
        assert np.isfinite(want["cost"][entries]).all()


def test_full_width_dsv3_moe_on_mesh_64x4(gpu_device, fake_pg):
    """Configuration 4 at its stated size (_testing/models/dsv3.py:1161-1227, 1523): 16 layers, dim
    7168, multi-head latent attention (q_lora 1536, kv_lora 512, 128 heads, rope dim 64), 256 routed
    experts of width 2048 with 8 active plus one shared expert, batch 16 x 4096 tokens, mesh (64, 4),
    the expert regions as ``local_map`` calls, captured through Dynamo.  (The seeded Zipf routing does
    not enter: planning sees static shapes.)  Flop / byte counts, compute costs, every comm /
    transition / cost entry and the row minima against the C oracle and the host path; then the
    pruned solve: its objective is the sum of the oracle's costs of the chosen entries."""
    from autoparallel_amd.graphs import workloads
    from autoparallel_amd.graphs.dsv3 import DSV3_16L

    cfg = DSV3_16L
    assert (cfg.n_layers, cfg.dim, cfg.n_routed_experts, cfg.top_k, cfg.n_shared_experts) == (16, 7168, 256, 8, 1)
    assert (cfg.q_lora_rank, cfg.kv_lora_rank, cfg.n_heads, cfg.qk_rope_head_dim, cfg.moe_inter_dim) == (1536, 512, 128, 64, 2048)
    mesh_sizes = (64, 4)
    mesh = workloads.logical_mesh(mesh_sizes)
    model, input_fn, _, needs_dynamo = workloads.build_model("dsv3_moe", mesh)
    assert needs_dynamo and tuple(input_fn().shape) == (16, 4096)
    with AutoParallelPlanner(model, input_fn, mesh, param_dtype=torch.bfloat16, reduce_dtype=torch.float32,
                             repeated_subgraphs=True, dynamo=True) as autop:
        o = autop.sharding_optimizer
        enc, tb = o.encoded, o.encoded.tables
        _progress(f"planner built: {len(o.nodes)} nodes, {tb.n_entries} entries, {o.clustering_used}")
        assert tb.n_entries == 1_073_460
        assert o.backend.launches == ("build_tables_packed",), "a table this small is one launch over packed tiles"
        assert sum("local_map_kwargs" in n.meta for n in o.graph.nodes) >= 2 * (cfg.n_layers - cfg.n_dense_layers)
        device_counts = {k: getattr(tb, k).copy() for k in ("strat_flops", "strat_rw_bytes", "strat_dtype", "strat_zero_cost")}
        if o.cost_input_stats["strategy_inputs"] == "device":
            _, lshape, lstride, _, _ = c_oracle.spec_tables(tb.as_dict(), mesh_sizes)
            fill_flops_and_bytes(enc, o.strats, np.asarray(lshape), np.asarray(lstride))
            for k, v in device_counts.items():
                assert np.array_equal(getattr(tb, k), v), k
            _progress("flop / byte counts equal the host path's")
        params = po.make_params(mesh_sizes, rescale=2.2)
        want_compute, want_per_arg = c_oracle.compute_costs(tb.as_dict(), params)[:2]
        assert np.array_equal(o.compute_cost, want_compute) and np.array_equal(o.compute_cost_per_arg, want_per_arg)
        want = c_oracle.build_tables(tb.as_dict(), params, per_arg=want_per_arg)
        for name in ("cost", "comm", "transition"):
            assert np.array_equal(o.backend.host_array(name), want[name]), name
            _progress(f"{name} equal")
        mins, args = o.row_minima()
        want_min, want_arg = c_oracle.segmented_min(want["cost"], tb.row_ptr())
        assert np.array_equal(mins, want_min) and np.array_equal(args, want_arg)
        _progress("row minima equal")
        from torch.distributed.tensor.placement_types import Replicate, Shard

        autop.add_parameter_memory_constraint(low=None, high=None)
        # the batch (16) does not divide the mesh's first dim: the sequence is pinned instead
        autop.add_input_constraints([(Shard(1), Replicate())])
        autop.add_output_constraints([(Shard(1), Replicate())])
        autop.optimize_placement()
        stats = o.solve_stats
        _progress(f"solved: {stats.get('solved_by')}, {stats.get('columns')} -> {stats.get('columns_after_pruning')} columns")
        assert stats["incumbent"] is not None and stats["lower_bound"] <= stats["incumbent"] * (1 + 1e-9)
        entries = np.asarray(o.res_entries, np.int64)
        assert np.isfinite(want["cost"][entries]).all()
        assert o.objective_value() == float(want["cost"][entries].sum()) > 0


def test_stress_table_at_full_size(gpu_device):
    """Configuration 5 at full size: 200 000 nodes, 426 918 edges, 464 M cost entries on mesh
    (16, 8, 4).  The planner's pass (cost alone) and the tables of its first launch against the
    C oracle, every entry."""
    mesh = (16, 8, 4)
    tb = stress_dag(seed=0, n_nodes=200_000, mesh_sizes=mesh)
    assert tb.n_entries == 464_235_576
    _progress("tables generated")
    dev = DeviceCostTables(tb, CostModelParams.from_mesh(mesh, rescale=2.2), device=gpu_device)
    step = dev.planner_pass()
    assert tuple(step) == ("input_tables", "redistribute_tables")
    for launch in step.values():
        launch()
    torch.cuda.synchronize()
    dev.check_error_flag()
    params = po.make_params(mesh, rescale=2.2)
    want_compute, want_per_arg = c_oracle.compute_costs(tb.as_dict(), params)[:2]
    assert np.array_equal(dev.compute_cost.cpu().numpy(), want_compute)
    wb, wc = c_oracle.tensor_tables(tb.as_dict())
    assert np.array_equal(dev.tensor_bytes.cpu().numpy(), wb) and np.array_equal(dev.tensor_contiguous.cpu().numpy(), wc)
    assert dev.comm is None and dev.transition is None
    # the oracle by ranges of edges (a tenth of the table at a time), the device array by the same ranges
    eb = tb.edge_entry_begin
    cost = dev.cost
    bounds = np.linspace(0, tb.n_edges, 11).astype(np.int64)
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        want = c_oracle.build_tables(tb.as_dict(), params, edge_range=(int(lo), int(hi)), per_arg=want_per_arg)["cost"]
        assert np.array_equal(cost[int(eb[lo]):int(eb[hi])].cpu().numpy(), want), (lo, hi)
        _progress(f"edges {lo} .. {hi} equal")
