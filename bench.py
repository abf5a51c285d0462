"""Benchmark of the sharding-cost table build on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama3_8b|llama3_70b|block_1k|stress]

A step is one complete device-side pass of the hot path over the workload's flattened
tables, already resident in HBM: tensor byte/contiguity table, local shard shapes,
per-strategy compute costs, the redistribution-cost matrices with assembled ILP costs, and
the row minima.  The default workload is the Llama-3-8B joint forward+backward graph
planned on a (32, 8) logical mesh; ``stress`` is the seeded 200k-node synthetic DAG on a
(16, 8, 4) mesh.

One JSON line is printed: whole-pass throughput in cost entries/s (``value``), the
redistribution-cost kernel against the HBM roofline (``roofline``), and the CPU oracle
timed on a bounded sample of the same tables (``cpu_baseline``).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E

# HBM bytes per launch of the kernel that writes the cost matrices, measured with rocprofv3 --pmc
# (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, KiB per dispatch; the factors come from the same
# counters read on a plain 1 GiB copy, --calibrate-copy).  A hardware counter cannot be read
# from inside this process, so the figure is the one of the profiled run of the same command
# and only reported for exactly that table: (entries, tiles, algorithmic bytes) must match.
MEASURED_TRAFFIC_BYTES = {
    (1_821_368, 1_616, 73_586_428): (3_184.3 * 2.000 + 68_345.1) * 1024,           # llama3_8b, mesh (32, 8), all tables and the row minima in one launch
    (1_821_368, 1_616, 71_794_420): (3_037.5 * 2.000 + 65_983.1) * 1024,           # the same, --row-min separate
    (1_821_368, 1_616, 32_348_914): (670.7 * 2.000 + 31_445.9) * 1024,             # the same, --table-launches 2
    (1_073_460, 1_387, 47_179_580): (2_310.1 * 2.000 + 43_498.1) * 1024,            # dsv3_moe, mesh (64, 4)
    (2_986, 129, 374_304): (249.0 * 2.000 + 317.4) * 1024,                          # block_1k, mesh (64,)
    (73_251_434, 40_727, 1_255_915_920): (12_322.6 * 2.000 + 1_221_016.0) * 1024,   # llama3_70b, mesh (8, 8, 8)
    (464_235_576, 426_918, 8_178_099_438): (165_040.2 * 2.000 + 7_953_223.0) * 1024,  # stress, mesh (16, 8, 4), row minima in the tiles
    (464_235_576, 426_918, 8_003_825_874): (159_776.0 * 2.000 + 7_760_473.5) * 1024,  # the same, --row-min separate
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="llama3_8b", choices=["llama3_8b", "llama3_70b", "dsv3_moe", "block_1k", "stress"])
    ap.add_argument("--layers", type=int, default=None, help="override the number of decoder layers")
    ap.add_argument("--stress-nodes", type=int, default=200_000)
    ap.add_argument("--tile-entries", type=int, default=None, help="entries per tile (default: chosen from the table)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target CPU-baseline sample duration")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-solve", action="store_true", help="skip the ILP leg of the plan wall-time")
    ap.add_argument("--no-clustering", action="store_true", help="one ILP variable per entry (no variable sharing)")
    ap.add_argument("--no-dedupe", action="store_true", help="tile every edge even if an identical one exists")
    ap.add_argument("--max-copies", type=int, default=8, help="identical edges served by one tiled edge")
    ap.add_argument("--table-launches", type=int, default=None, choices=[1, 2, 4],
                    help="launches that build the tables of a pass: 1 = everything in one (apc_build_tables), "
                         "2 = input tables, then cost matrices, 4 = tensor, spec and compute-cost tables on their own "
                         "(default: 1 for tables up to 128 MiB, else 2)")
    ap.add_argument("--row-min", choices=["auto", "tiles", "separate"], default="auto",
                    help="where the row minima of a pass are taken: by the launch that writes the cost matrices "
                         "(tiles), by a segmented_min launch that reads them back (separate); auto = tiles whenever "
                         "every matrix row lies inside one tile")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain 1 GiB device-to-device copy three times (reference reading for the "
                         "FETCH_SIZE / WRITE_SIZE counters) and exit")
    return ap.parse_args()


def build_workload(args):
    """-> (tables, params, description, device tables or None, planner or None, host timings)"""
    from autoparallel_amd import CostModelParams

    if args.workload == "stress":
        from autoparallel_amd.synthetic import stress_dag

        mesh = (16, 8, 4)
        t0 = time.perf_counter()
        tables = stress_dag(seed=0, n_nodes=args.stress_nodes, mesh_sizes=mesh)
        timings = {"generate_s": time.perf_counter() - t0}
        desc = {"workload": f"synthetic stress DAG, seed 0, {args.stress_nodes} nodes, mesh {mesh}",
                "mesh": list(mesh)}
        return tables, CostModelParams.from_mesh(mesh, rescale=2.2), desc, None, None, timings

    # traced workloads go through the product path: capture -> ShardingOptimizer (which
    # enumerates, clusters, encodes, builds the device tables and copies them back)
    import torch

    from autoparallel_amd.api import AutoParallelPlanner
    from autoparallel_amd.graphs import workloads
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    mesh_sizes = workloads.WORKLOADS[args.workload][1]
    mesh = workloads.logical_mesh(mesh_sizes)
    model, input_fn, workload_desc, needs_dynamo = workloads.build_model(args.workload, mesh, n_layers=args.layers)

    class Optimizer(ShardingOptimizer):
        tile_entries = args.tile_entries
        dedupe = not args.no_dedupe
        max_copies = args.max_copies

    class Planner(AutoParallelPlanner):
        optimizer_cls = Optimizer

    planner = Planner(model, input_fn, mesh, param_dtype=torch.bfloat16, reduce_dtype=torch.float32,
                      repeated_subgraphs=not args.no_clustering, dynamo=needs_dynamo)
    planner.__enter__()
    opt = planner.sharding_optimizer
    desc = {"workload": workload_desc, "mesh": list(mesh_sizes), "graph_nodes": len(opt.nodes), "ilp_variables": opt.n_variables,
            "clustered_nodes": len(opt.node_representative)}
    return opt.encoded.tables, opt.params, desc, opt.backend.dev, planner, dict(planner.timings)


def solve_plan(planner, args):
    """The ILP leg of the plan (input / output constraints of the reference's Llama example:
    examples/example_llama3.py:205-218)."""
    from torch.distributed.tensor.placement_types import Replicate, Shard

    t0 = time.perf_counter()
    planner.add_parameter_memory_constraint(low=None, high=None)
    nd = planner.mesh.ndim
    x_sharding = (Shard(0),) + (Replicate(),) * (nd - 1)
    out_sharding = (Shard(0), Shard(2)) if (nd == 2 and args.workload != "block_1k") else x_sharding
    if args.workload in ("block_1k", "dsv3_moe"):
        # the batch (8 / 16) does not divide the mesh's first dim, so no batch-sharded placement
        # exists (the default constraint would raise, as the reference's does): pin the sequence
        x_sharding = out_sharding = (Shard(1),) + (Replicate(),) * (nd - 1)
    planner.add_input_constraints([x_sharding])
    planner.add_output_constraints([out_sharding])
    constraints_s = time.perf_counter() - t0
    planner.optimize_placement()
    opt = planner.sharding_optimizer
    t0 = time.perf_counter()
    _, lower_bound = opt.greedy_strategies()  # row minima -> per-strategy bounds -> per-node minima, on the device
    bound_s = time.perf_counter() - t0
    return {"constraints_s": constraints_s, "solve_s": planner.timings["solve_s"],
            "objective": opt.objective_value(), "ilp_rows": getattr(opt.prob, "rows_after_dedupe", None),
            "ilp_variables": opt.n_variables, "lower_bound_from_row_minima": lower_bound, "lower_bound_s": bound_s}


def cpu_baseline(tables, params, target_seconds):
    """The scalar Python oracle (the reference executes this path as interpreted Python) on
    a prefix of the workload's edges sized for about ``target_seconds`` of CPU work."""
    import numpy as np

    from oracle import c_oracle
    from oracle import cost_oracle as po

    op = po.make_params(params.mesh_sizes, device_name=params.device_name, rescale=params.rescale)
    enc = tables.as_dict()
    eb = tables.edge_entry_begin
    # calibrate on ~20k entries
    cal_hi = int(np.searchsorted(eb, 20_000, side="left"))
    cal_hi = max(1, min(cal_hi, tables.n_edges))
    t0 = time.perf_counter()
    po.build_tables(enc, op, edge_range=(0, cal_hi))
    dt = time.perf_counter() - t0
    rate = max(int(eb[cal_hi]), 1) / max(dt, 1e-9)
    want = int(rate * target_seconds)
    hi = int(np.searchsorted(eb, want, side="left"))
    hi = max(1, min(hi, tables.n_edges))
    t0 = time.perf_counter()
    out = po.build_tables(enc, op, edge_range=(0, hi))
    dt = time.perf_counter() - t0
    n = len(out["comm"])
    # the plain-C restatement on the whole workload, for scale
    t0 = time.perf_counter()
    c_oracle.build_tables(enc, op)
    c_dt = time.perf_counter() - t0
    return {
        "value": n / dt, "unit": "entries/s", "cores": 1, "kind": "port",
        "sample": f"scalar Python oracle over the first {hi} of {tables.n_edges} edges ({n} entries, {dt:.1f} s), "
                  f"compute costs + redistribution costs + assembly",
        "c_port_entries_per_s": tables.n_entries / c_dt, "host_cpu_count": os.cpu_count(),
    }


def main():
    args = parse_args()
    # stage-by-stage progress of the (long, CPU-side) set-up goes to stderr
    import logging

    logging.basicConfig(stream=sys.stderr, level=logging.INFO, format="[bench %(relativeCreated)8.0f ms] %(message)s")
    log = logging.getLogger("bench")
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; cost tables shard by edge range without any exchange step, "
              "but no multi-GPU path is part of it. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a HIP device (there is no CPU path for the product)", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    if args.calibrate_copy:
        src = torch.ones(1 << 27, dtype=torch.float64, device="cuda:0")  # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes_read": src.numel() * 8, "calibrate_copy_bytes_written": src.numel() * 8,
                          "copies": 3}))
        return
    from autoparallel_amd.device_tables import DeviceCostTables

    t_setup = time.perf_counter()
    tables, params, desc, dev, planner, host_timings = build_workload(args)
    # a traced workload keeps its capture context (a fake-tensor mode) open until the plan is
    # solved; the measurements below work on real device buffers
    from autoparallel_amd.device_tables import _real_tensors

    guard = _real_tensors()
    guard.__enter__()
    t0 = time.perf_counter()
    if dev is None:
        if args.tile_entries:
            tables.build_tiles(args.tile_entries)
        dev = DeviceCostTables(tables, params, device="cuda:0")
    log.info("tables resident: %d entries, %d tiles", tables.n_entries, tables.n_tiles)
    step = dev.prepare_step(row_min=True, fused_inputs=args.table_launches != 4,
                            one_launch=None if args.table_launches is None else args.table_launches == 1,
                            row_min_in_tiles={"auto": None, "tiles": True, "separate": False}[args.row_min])
    row_min_in_tiles = "segmented_min" not in step
    args.table_launches = 1 if "build_tables" in step else 2 if "input_tables" in step else 4
    torch.cuda.synchronize()
    host_timings["upload_and_prepare_s"] = time.perf_counter() - t0
    host_timings["setup_total_s"] = time.perf_counter() - t_setup

    names = list(step)
    launchers = [step[k] for k in names]
    for _ in range(args.warmup):
        for launch in launchers:
            launch()
    torch.cuda.synchronize()

    # ---- timed region: exactly K steps -------------------------------------------------------
    K = args.steps
    ev = {k: [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(K)]
          for k in names}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(K):
        for k, launch in zip(names, launchers):
            a, b = ev[k][i]
            a.record()
            launch()
            b.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kernel_ms = {k: float(np.mean([a.elapsed_time(b) for a, b in ev[k]])) for k in names}
    kernel_ms_min = {k: float(np.min([a.elapsed_time(b) for a, b in ev[k]])) for k in names}

    # the same K steps without per-kernel events: the whole-pass rate.  One event pair brackets
    # the region on the launch stream: when a pass is a single kernel, region / K is that kernel's
    # average duration back to back, without the 1 - 2 us an event pair adds to every launch.
    region = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    region[0].record()
    for i in range(K):
        for launch in launchers:
            launch()
    region[1].record()
    torch.cuda.synchronize()
    wall_plain = time.perf_counter() - t0
    region_ms = region[0].elapsed_time(region[1])

    # copy-back of the results, for the PCIe-inclusive figure
    t0 = time.perf_counter()
    host_out = [x.cpu() for x in (dev.comm, dev.transition, dev.cost) if x is not None]
    copy_back_s = time.perf_counter() - t0
    del host_out

    log.info("timed region done: %.3f ms/step", wall_plain / K * 1e3)
    E = tables.n_entries
    # the launch that writes the cost matrices; in one-launch mode it also writes the input tables
    main = "build_tables" if args.table_launches == 1 else "redistribute_tables"
    alg_bytes = tables.algorithmic_bytes(comm=True, transition=True, cost=True)
    if args.table_launches == 1:
        alg_bytes += tables.algorithmic_bytes_input_tables()
    n_rows = int(tables.edge_n_tgt.astype(np.int64).sum())
    if row_min_in_tiles:
        alg_bytes += 12 * n_rows  # minimum f64 + argmin i32 per matrix row, written by the same launch
    t_kernel_pair = kernel_ms[main] * 1e-3  # an event pair around every launch
    single_kernel_pass = len(names) == 1
    t_kernel = region_ms * 1e-3 / K if single_kernel_pass else t_kernel_pair
    achieved = alg_bytes / t_kernel / 1e9
    ms_per_step = wall_plain / K * 1e3
    result = {
        "metric": "redistribution_cost_entries_per_s",
        "value": E * K / wall_plain,
        "unit": "entries/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": {**desc, "edges": tables.n_edges, "strategies": tables.n_strategies, "specs": tables.n_specs,
                   "entries": E, "tiles": tables.n_tiles, "tiling": tables.tiling,
                   "edges_deduplicated": int((tables.edge_canonical != np.arange(tables.n_edges)).sum()), "device_row": params.device_name,
                   "devices_per_host": 8,
                   "step": {1: "build_tables(tensor, spec and compute-cost tables + comm, transition, cost: one launch)",
                            2: "input_tables(tensor + spec + compute-cost tables, one launch) + "
                               "redistribute_tables(comm, transition, cost)",
                            4: "tensor_tables + spec_tables + compute_costs + redistribute_tables(comm, transition, cost)"
                            }[args.table_launches] +
                           (", row minima taken by that launch" if row_min_in_tiles else " + segmented_min(rows)"),
                   "matrix_rows": n_rows},
        "roofline": {"bound": "hbm", "kernel": "build_tables_kernel" if args.table_launches == 1 else
                     "redistribute_tiles_row_min_kernel" if row_min_in_tiles else "redistribute_tiles_kernel",
                     "achieved": achieved,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get((E, tables.n_tiles, alg_bytes)),
                     "algorithmic_bytes_input_tables": tables.algorithmic_bytes_input_tables() if args.table_launches == 1 else 0,
                     "algorithmic_bytes_per_launch": alg_bytes,
                     "bytes_written_per_entry": {"comm_f64": 8, "transition_u8": 1, "cost_f64": 8},
                     "bytes_written_per_matrix_row": 12 if row_min_in_tiles else 0,
                     "avg_launch_us": t_kernel * 1e6,
                     "avg_launch_us_event_pair_per_launch": t_kernel_pair * 1e6,
                     "frac_event_pair_per_launch": alg_bytes / t_kernel_pair / 1e9 / HBM_PEAK_GBPS,
                     "min_launch_us_event_pair_per_launch": kernel_ms_min[main] * 1e3,
                     "timing": ("one HIP event pair on the launch stream around the K back-to-back launches of the timed "
                                "region (the pass is this one kernel), / K" if single_kernel_pass else
                                "HIP events around every launch of the kernel inside the timed region")},
        "kernel_us": {k: v * 1e3 for k, v in kernel_ms.items()},
        "ms_per_step_with_events": wall / K * 1e3,
        "host_timings_s": {k: round(v, 4) for k, v in host_timings.items()},
        "copy_back_s": copy_back_s,
        "entries_per_s_including_copy_back": E / (ms_per_step * 1e-3 + copy_back_s),
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(tables, params, args.cpu_seconds)
    guard.__exit__(None, None, None)
    if planner is not None:
        plan = {"stages_s": {k: round(v, 4) for k, v in host_timings.items()}}
        if not args.no_solve:
            log.info("solving the ILP: %d variables", planner.sharding_optimizer.n_variables)
            plan.update(solve_plan(planner, args))
        table_stage = host_timings.get("optimizer_tables_s", 0.0)
        other = host_timings.get("capture_s", 0.0) + host_timings.get("optimizer_s", 0.0) - table_stage \
            + plan.get("constraints_s", 0.0) + plan.get("solve_s", 0.0)
        plan["total_with_gpu_tables_s"] = other + table_stage
        if "cpu_baseline" in result:
            # the same plan with the tables built by the CPU port: only the table stage differs
            cpu_tables = E / result["cpu_baseline"]["value"]
            plan["cpu_table_stage_s"] = cpu_tables
            plan["total_with_cpu_tables_s"] = other + cpu_tables
        result["plan_wall_time"] = plan
        planner.__exit__(None, None, None)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
