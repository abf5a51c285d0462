"""Benchmark of the sharding-cost table build on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama3_8b|llama3_70b|dsv3_moe|block_1k|stress]

A step is the device pass ``ShardingOptimizer.build_ds`` issues once the flop / byte counts
are in the strategy table (``DeviceCostTables.planner_pass``): the tensor byte / contiguity
table, the per-strategy compute costs and the assembled cost of every entry of every
redistribution-cost matrix, with the row minima where taking them there is cheaper than
reading the matrices back; tables already resident in HBM.  On the default workload, the
Llama-3-8B joint forward+backward graph planned on a (32, 8) logical mesh, that is ONE launch.
``stress`` is the seeded 200k-node synthetic DAG on a (16, 8, 4) mesh.

One JSON line is printed: whole-pass throughput in cost entries/s (``value``), the launch that
writes the cost matrices against the HBM roofline (``roofline``), the CPU oracle timed on a
bounded sample of the same tables (``cpu_baseline``), the plan wall-time by stage, and under
``extra`` the same roofline figures on the two tables large enough to be bandwidth-bound
(Llama-3-70B on (8, 8, 8) and the stress DAG).  Outside the timed region the pass's outputs are
compared with the launch-by-launch build of all arrays and with the C oracle; a mismatch fails
the run.
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
ORACLE_CHECK_MAX_ENTRIES = 60_000_000  # larger tables are checked against the C oracle on a prefix of their edges

WORKLOADS = ["llama3_8b", "llama3_70b", "dsv3_moe", "block_1k", "stress"]


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="llama3_8b", choices=WORKLOADS)
    ap.add_argument("--layers", type=int, default=None, help="override the number of decoder layers")
    ap.add_argument("--stress-nodes", type=int, default=200_000)
    ap.add_argument("--tile-entries", type=int, default=None, help="entries per tile (default: chosen from the table)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target CPU-baseline sample duration")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-solve", action="store_true", help="skip the ILP leg of the plan wall-time")
    ap.add_argument("--no-clustering", action="store_true", help="one ILP variable per entry (no variable sharing)")
    ap.add_argument("--no-dedupe", action="store_true", help="tile every edge even if an identical one exists")
    ap.add_argument("--max-copies", type=int, default=16, help="identical edges served by one tiled edge")
    ap.add_argument("--pass", dest="pass_kind", choices=["planner", "all"], default="planner",
                    help="planner: the pass build_ds issues (assembled cost, no spec table); all: every table and all "
                         "three per-entry arrays (the composite of the earlier benchmark, labelled as such)")
    ap.add_argument("--extra", default="llama3_70b,stress",
                    help="comma-separated workloads measured after the main one and reported under 'extra' "
                         "(fewer steps, no CPU baseline, no solve); '' for none")
    ap.add_argument("--no-verify", action="store_true", help="skip the comparison of the pass's outputs (timing runs)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain 1 GiB device-to-device copy three times (reference reading for the "
                         "FETCH_SIZE / WRITE_SIZE counters) and exit")
    ap.add_argument("--calibrate-launch", action="store_true",
                    help="only time an empty kernel launched back to back and plain fills of the bytes the three "
                         "workloads' launches move (what roofline.launch_floor_us / fill_us come from) and exit")
    ap.add_argument("--no-cpu-plan", action="store_true",
                    help="skip the measured plan with the tables built on the host (about 15 s on the default workload)")
    ap.add_argument("--no-traffic", action="store_true",
                    help="skip the HBM-traffic reading (four short child runs of this script under rocprofv3 --pmc)")
    ap.add_argument("--replay-tables", default=None,
                    help="(child of the traffic reading) load the encoded tables from this .npz, run the pass three "
                         "times and exit")
    return ap.parse_args()


# ---- HBM traffic of the dominant launch, read from the hardware counters --------------------------
# A counter cannot be read from inside the process, so the pass is replayed in child processes
# under ``rocprofv3 --pmc`` (one counter per run: FETCH_SIZE, then WRITE_SIZE, KiB per dispatch),
# each scaled by what the same counter reads for a plain 1 GiB device-to-device copy.  The
# children load the parent's encoded tables from a temporary file, so they take seconds.
TABLE_FIELDS_SKIP = ("mesh_sizes", "tiling")


def save_tables(tables, params, pass_kind, path):
    import numpy as np

    arrays = {k: v for k, v in tables.as_dict().items() if isinstance(v, np.ndarray)}
    np.savez(path, **arrays, _mesh=np.asarray(tables.mesh_sizes), _rescale=np.asarray([params.rescale]),
             _pass=np.asarray([pass_kind]))


def replay_tables(path):
    """Child process: the pass over tables loaded from ``path``, three times."""
    import numpy as np
    import torch

    from autoparallel_amd import CostModelParams
    from autoparallel_amd.device_tables import DeviceCostTables
    from autoparallel_amd.encoding import CostTables

    z = np.load(path)
    mesh = tuple(int(x) for x in z["_mesh"])
    fields = {k: z[k] for k in z.files if not k.startswith("_")}
    tables = CostTables(mesh_sizes=mesh, **fields)
    dev = DeviceCostTables(tables, CostModelParams.from_mesh(mesh, rescale=float(z["_rescale"][0])), device="cuda:0",
                           validate=False)
    step = prepare(dev, str(z["_pass"][0]))
    for _ in range(3):
        for launch in step.values():
            launch()
    torch.cuda.synchronize()
    print(json.dumps({"replayed": list(step), "entries": tables.n_entries}))


def read_counter(counter, child_args, kernel_substring, log, timeout_s=120):
    """Average ``counter`` per dispatch of the kernels whose name contains ``kernel_substring`` in a
    child run of this script under rocprofv3; None (and a log line) if anything goes wrong."""
    import csv
    import glob
    import shutil
    import signal
    import subprocess
    import tempfile

    rocprof = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not os.path.exists(rocprof):
        log.info("traffic: rocprofv3 not found")
        return None
    out_dir = tempfile.mkdtemp(prefix="apc_pmc_", dir="/tmp")
    cmd = [rocprof, "--pmc", counter, "-d", out_dir, "-o", "pmc", "--output-format", "csv", "--",
           sys.executable, os.path.abspath(__file__), *child_args]
    try:
        proc = subprocess.Popen(cmd, cwd="/tmp", env={**os.environ, "TMPDIR": "/tmp"}, stdout=subprocess.DEVNULL,
                                stderr=subprocess.DEVNULL, start_new_session=True)
        try:
            rc = proc.wait(timeout=timeout_s)
        except subprocess.TimeoutExpired:
            os.killpg(proc.pid, signal.SIGKILL)  # the child's own process group, nothing else
            proc.wait()
            log.info("traffic: %s run timed out", counter)
            return None
        if rc != 0:
            log.info("traffic: %s run exited with %d", counter, rc)
            return None
        files = glob.glob(os.path.join(out_dir, "**", "*counter_collection.csv"), recursive=True)
        values = []
        for f in files:
            with open(f) as fh:
                for row in csv.DictReader(fh):
                    if kernel_substring in row["Kernel_Name"] and row["Counter_Name"] == counter:
                        values.append(float(row["Counter_Value"]))
        return sum(values) / len(values) if values else None
    except OSError as e:
        log.info("traffic: %s", e)
        return None
    finally:
        shutil.rmtree(out_dir, ignore_errors=True)


def measure_traffic(tables, params, pass_kind, kernel, log, factor=None):
    """-> dict for ``roofline`` (traffic in bytes per launch and how it was read) or None.
    ``factor``: the copy-kernel scale factors of an earlier reading in this run (not read again)."""
    import tempfile

    gib_kib = float(1 << 20)  # a 1 GiB copy reads and writes 2^20 KiB
    path = os.path.join(tempfile.mkdtemp(prefix="apc_tables_", dir="/tmp"), "tables.npz")
    try:
        save_tables(tables, params, pass_kind, path)
        reading, factor = {}, dict(factor or {})
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            if counter not in factor:
                copy = read_counter(counter, ["--calibrate-copy"], "copyBuffer", log)
                if not copy:
                    return None
                factor[counter] = gib_kib / copy
            value = read_counter(counter, ["--replay-tables", path], kernel, log, timeout_s=240)
            if value is None:
                return None
            reading[counter] = value
        traffic = (reading["FETCH_SIZE"] * factor["FETCH_SIZE"] + reading["WRITE_SIZE"] * factor["WRITE_SIZE"]) * 1024.0
        return {"traffic": traffic,
                "traffic_reading": {"kib_per_dispatch": reading, "scale_from_1gib_copy": factor,
                                    "how": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (one run each) over a replay of this "
                                           "pass on the same tables in a child process; each scaled by the same "
                                           "counter's reading of a plain 1 GiB device-to-device copy"}}
    finally:
        import shutil

        shutil.rmtree(os.path.dirname(path), ignore_errors=True)


def build_workload(name, args):
    """-> (tables, params, description, device tables or None, planner or None, host timings)"""
    from autoparallel_amd import CostModelParams

    if name == "stress":
        from autoparallel_amd.synthetic import stress_dag

        mesh = (16, 8, 4)
        t0 = time.perf_counter()
        tables = stress_dag(seed=0, n_nodes=args.stress_nodes, mesh_sizes=mesh)
        timings = {"generate_s": time.perf_counter() - t0}
        desc = {"workload": f"synthetic stress DAG, seed 0, {args.stress_nodes} nodes, mesh {mesh}",
                "mesh": list(mesh)}
        return tables, CostModelParams.from_mesh(mesh, rescale=2.2), desc, None, None, timings

    # traced workloads go through the product path: capture -> ShardingOptimizer (which
    # enumerates, clusters, encodes, runs the table pass and takes the objective vector back)
    import torch

    from autoparallel_amd.api import AutoParallelPlanner
    from autoparallel_amd.graphs import workloads
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    mesh_sizes = workloads.WORKLOADS[name][1]
    mesh = workloads.logical_mesh(mesh_sizes)
    model, input_fn, workload_desc, needs_dynamo = workloads.build_model(name, mesh, n_layers=args.layers)

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
            "clustered_nodes": len(opt.node_representative), "planner_launches": list(opt.backend.launches)}
    return opt.encoded.tables, opt.params, desc, opt.backend.dev, planner, dict(planner.timings)


def solve_plan(planner, workload, compare_full=True):
    """The ILP leg of the plan (input / output constraints of the reference's Llama example:
    examples/example_llama3.py:205-218)."""
    from torch.distributed.tensor.placement_types import Replicate, Shard

    t0 = time.perf_counter()
    planner.add_parameter_memory_constraint(low=None, high=None)
    nd = planner.mesh.ndim
    x_sharding = (Shard(0),) + (Replicate(),) * (nd - 1)
    out_sharding = (Shard(0), Shard(2)) if (nd == 2 and workload != "block_1k") else x_sharding
    if workload in ("block_1k", "dsv3_moe"):
        # the batch (8 / 16) does not divide the mesh's first dim, so no batch-sharded placement
        # exists (the default constraint would raise, as the reference's does): pin the sequence
        x_sharding = out_sharding = (Shard(1),) + (Replicate(),) * (nd - 1)
    planner.add_input_constraints([x_sharding])
    planner.add_output_constraints([out_sharding])
    constraints_s = time.perf_counter() - t0
    opt = planner.sharding_optimizer
    upper = opt.prob.upper.copy()
    planner.optimize_placement()
    out = {"constraints_s": constraints_s, "solve_s": planner.timings["solve_s"],
           "objective": opt.objective_value(), "ilp_rows": getattr(opt.prob, "rows_after_dedupe", None),
           "ilp_variables": opt.n_variables}
    out.update({k: v for k, v in getattr(opt, "solve_stats", {}).items()})
    if compare_full and "columns_after_pruning" in out:
        # the same program without the pruning in front of the solver, for scale
        x = opt.prob.x.copy()
        opt.prob.upper = upper
        t0 = time.perf_counter()
        opt.prob.solve(time_limit=opt.solver_time_limit, mip_rel_gap=opt.solver_rel_gap)
        out["solve_s_without_pruning"] = time.perf_counter() - t0
        out["objective_without_pruning"] = float(opt.prob.objective @ opt.prob.x)
        out["objective_of_pruned_plan_in_full_program"] = float(opt.prob.objective @ x)
        opt.prob.x = x
    return out


def plan_with_cpu_tables(workload, args, log):
    """The same plan with the table stage on the host, measured: the planner of this package
    (capture, enumeration, clustering, encoding, constraints, solver unchanged) with the scalar
    Python oracle as its table source, the form in which the reference executes this path
    (examples/example_llama3.py:243-245 times the same stages around ``optimize_placement``).
    The pruning in front of the solver is off on this leg (its dual ascent runs on the device; the
    reference has none): the solver receives the full program, as it does in
    ``solve_s_without_pruning`` of the device leg.  -> stage times in seconds."""
    import numpy as np
    import torch

    tests_dir = os.path.join(ROOT, "tests")
    if tests_dir not in sys.path:
        sys.path.insert(0, tests_dir)
    from oracle_backend import OracleBackend  # the checker's table source behind the planner's backend interface

    from autoparallel_amd.api import AutoParallelPlanner
    from autoparallel_amd.graphs import workloads
    from autoparallel_amd.optimize_sharding import ShardingOptimizer
    from oracle import cost_oracle as po

    stage = {}

    class PythonTables(OracleBackend):
        def launch_tables(self):
            t0 = time.perf_counter()
            out = po.build_tables(self.tables.as_dict(), self.params)
            self.out = {k: np.asarray(v, np.uint8 if k == "transition" else np.float64) for k, v in out.items()}
            self.cost = self.out["cost"]
            self.launches = ("python oracle",)
            stage["cpu_tables_s"] = time.perf_counter() - t0

    class Optimizer(ShardingOptimizer):
        backend_cls = PythonTables
        prune_before_solve = False
        tile_entries = args.tile_entries
        dedupe = not args.no_dedupe
        max_copies = args.max_copies

    class Planner(AutoParallelPlanner):
        optimizer_cls = Optimizer

    mesh = workloads.logical_mesh(workloads.WORKLOADS[workload][1])
    model, input_fn, _, needs_dynamo = workloads.build_model(workload, mesh, n_layers=args.layers)
    t_all = time.perf_counter()
    with Planner(model, input_fn, mesh, param_dtype=torch.bfloat16, reduce_dtype=torch.float32,
                 repeated_subgraphs=not args.no_clustering, dynamo=needs_dynamo) as planner:
        stage.update({k: v for k, v in planner.timings.items() if k in ("capture_s", "optimizer_s")})
        plan = solve_plan(planner, workload, compare_full=False)
        stage["constraints_s"], stage["solve_s"], stage["objective"] = plan["constraints_s"], plan["solve_s"], plan["objective"]
    stage["total_s"] = time.perf_counter() - t_all
    log.info("plan with the tables built on the host: %.1f s (tables %.1f s)", stage["total_s"], stage["cpu_tables_s"])
    return stage


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
    # the plain-C restatement on the whole workload, for scale (second of two runs: the first
    # one pays for the page faults of its fresh output arrays)
    c_dt = float("inf")
    for _ in range(2):
        t0 = time.perf_counter()
        c_oracle.build_tables(enc, op)
        c_dt = min(c_dt, time.perf_counter() - t0)
    return {
        "value": n / dt, "unit": "entries/s", "cores": 1, "kind": "port",
        "sample": f"scalar Python oracle over the first {hi} of {tables.n_edges} edges ({n} entries, {dt:.1f} s), "
                  f"compute costs + redistribution costs + assembly",
        "c_port_entries_per_s": tables.n_entries / c_dt, "host_cpu_count": os.cpu_count(),
    }


def prepare(dev, pass_kind):
    if pass_kind == "planner":
        return dev.planner_pass()
    return dev.prepare_step(row_min=True, fused_inputs=True)


def time_pass(dev, step, steps, warmup):
    """Warm-up, then exactly ``steps`` passes twice: once with a HIP event pair around every
    launch (per-kernel durations), once plain with one event pair around the whole region (the
    pass rate; when a pass is one kernel, region / steps is that kernel's back-to-back duration
    without the 1 - 2 us an event pair adds to a launch)."""
    import numpy as np
    import torch

    names = list(step)
    launchers = [step[k] for k in names]
    for _ in range(warmup):
        for launch in launchers:
            launch()
    torch.cuda.synchronize()
    ev = {k: [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
          for k in names}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        for k, launch in zip(names, launchers):
            a, b = ev[k][i]
            a.record()
            launch()
            b.record()
    torch.cuda.synchronize()
    wall_events = time.perf_counter() - t0
    kernel_ms = {k: float(np.mean([a.elapsed_time(b) for a, b in ev[k]])) for k in names}
    kernel_ms_min = {k: float(np.min([a.elapsed_time(b) for a, b in ev[k]])) for k in names}
    region = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    region[0].record()
    for i in range(steps):
        for launch in launchers:
            launch()
    region[1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return {"names": names, "wall_s": wall, "wall_events_s": wall_events, "region_ms": region[0].elapsed_time(region[1]),
            "kernel_ms": kernel_ms, "kernel_ms_min": kernel_ms_min}


def verify_pass(dev, tables, params, log):
    """Outside the timed region: what the timed launches left in HBM against (1) the
    launch-by-launch build of every array on a second set of buffers and (2) the C oracle
    (whole table up to ORACLE_CHECK_MAX_ENTRIES, else a prefix of the edges)."""
    import numpy as np
    import torch

    from autoparallel_amd.device_tables import DeviceCostTables
    from oracle import c_oracle
    from oracle import cost_oracle as po

    torch.cuda.synchronize()
    dev.check_error_flag()
    ref = DeviceCostTables(tables, params, device=dev.device, validate=False)
    ref.build_all()
    torch.cuda.synchronize()
    checked = []

    def same(name, a, b):
        if a is None:
            return
        if not torch.equal(a, b):
            raise SystemExit(f"bench.py: PARITY FAILURE: {name} of the timed pass differs from the launch-by-launch build")
        checked.append(name)

    same("cost", dev.cost, ref.cost)
    same("comm", dev.comm, ref.comm)
    same("transition", dev.transition, ref.transition)
    same("compute_cost", dev.compute_cost, ref.compute_cost)
    same("compute_cost_per_arg", dev.compute_cost_per_arg, ref.compute_cost_per_arg)
    same("tensor_bytes", dev.tensor_bytes, ref.tensor_bytes)
    ref_min, ref_arg = ref.row_minima()
    if dev.row_min is not None:
        same("row_min", dev.row_min, ref_min)
        same("row_argmin", dev.row_argmin, ref_arg)
    # the C oracle
    op = po.make_params(params.mesh_sizes, device_name=params.device_name, rescale=params.rescale)
    enc = tables.as_dict()
    eb = tables.edge_entry_begin
    hi = tables.n_edges
    if tables.n_entries > ORACLE_CHECK_MAX_ENTRIES:
        hi = max(1, int(np.searchsorted(eb, ORACLE_CHECK_MAX_ENTRIES, side="right")) - 1)
    n = int(eb[hi])
    want_cc, want_pa = c_oracle.compute_costs(enc, op)
    want = c_oracle.build_tables(enc, op, edge_range=(0, hi), per_arg=want_pa)
    if not np.array_equal(dev.cost[:n].cpu().numpy(), want["cost"]):
        raise SystemExit("bench.py: PARITY FAILURE: cost of the timed pass differs from the C oracle")
    if not np.array_equal(dev.compute_cost.cpu().numpy(), want_cc):
        raise SystemExit("bench.py: PARITY FAILURE: compute costs of the timed pass differ from the C oracle")
    if not np.array_equal(ref.comm[:n].cpu().numpy(), want["comm"]) or \
            not np.array_equal(ref.transition[:n].cpu().numpy(), want["transition"]):
        raise SystemExit("bench.py: PARITY FAILURE: comm / transition differ from the C oracle")
    n_rows = int(tables.edge_n_tgt[:hi].astype(np.int64).sum())
    wm, wa = c_oracle.segmented_min(want["cost"], tables.row_ptr()[:n_rows + 1])
    if not (np.array_equal(ref_min[:n_rows].cpu().numpy(), wm) and np.array_equal(ref_arg[:n_rows].cpu().numpy(), wa)):
        raise SystemExit("bench.py: PARITY FAILURE: row minima differ from the C oracle")
    del ref
    torch.cuda.empty_cache()
    log.info("verified: %s equal to the launch-by-launch build; %d of %d entries equal to the C oracle",
             ", ".join(checked), n, tables.n_entries)
    return {"timed_pass_equals_launch_by_launch_build": checked, "entries_equal_to_c_oracle": n,
            "entries": tables.n_entries, "bit_exact": True}


def calibrate_launch(nbytes, grid, threads):
    """What a launch of this shape costs before it does any work, and what a kernel that only
    writes ``nbytes`` takes (the library's measurement kernels, back to back on the current stream,
    one HIP event pair around the run): -> (launch_floor_us, fill_us, the fill's doubles per workgroup,
    whether the fastest fill wrote through to memory)."""
    import ctypes

    import torch

    from autoparallel_amd import _native

    lib = _native.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def timed(fn, k):
        for _ in range(max(3, k // 10)):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(k):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / k

    k = 200 if nbytes < (256 << 20) else 20

    def empty():
        _native.check(lib.apc_calibrate_launch(ctypes.c_int64(grid), ctypes.c_int32(threads), stream), "apc_calibrate_launch")

    floor_us = timed(empty, 200)
    n = nbytes // 8
    buf = torch.empty(n + 2, dtype=torch.float64, device="cuda:0")
    best = None
    for through in (0, 1):
        for per in (512, 2048, 8192, 16384):
            def fill():
                _native.check(lib.apc_calibrate_fill(ctypes.c_void_p(buf.data_ptr()), ctypes.c_int64(n), ctypes.c_int64(per),
                                                     ctypes.c_double(1.0), ctypes.c_int32(through), stream), "apc_calibrate_fill")
            us = timed(fill, k)
            if best is None or us < best[0]:
                best = (us, per, through)
    del buf
    return floor_us, best[0], best[1], best[2]


def roofline_of(dev, tables, timing, steps, pass_kind):
    """The launch that writes the cost matrices against the HBM peak, two ways: over the bytes
    that launch must move (``frac``) and over fixed per-unit prices (``frac_survey_8d``: 8 B per
    entry for each fp64 array the launch writes and 1 B for the transition flag if it does, the
    spec lists and a 64-byte header per edge, 25 B per strategy when the launch also builds the
    compute costs, 12 B per row minimum it takes); and against two measured ceilings of this
    system: an empty launch of the same grid (``launch_floor_us``) and a kernel that only writes
    the same bytes (``fill_us``; ``frac_of_fill`` = fill_us / the launch's duration)."""
    import numpy as np

    names = timing["names"]
    packed = "build_tables_packed" in names
    one_launch = packed or "build_tables" in names
    main = "build_tables_packed" if packed else "build_tables" if one_launch else "redistribute_tables"
    in_tiles = dev.row_min is not None and "segmented_min" not in names
    outputs = tuple(k for k in ("comm", "transition", "cost") if getattr(dev, k) is not None)
    spec_table = pass_kind == "all"
    m = len(tables.mesh_sizes)
    per_edge = int(((tables.edge_n_src.astype(np.int64) + tables.edge_n_tgt.astype(np.int64)) * m + 64).sum())
    per_entry = 8 * ("comm" in outputs) + 1 * ("transition" in outputs) + 8 * ("cost" in outputs)
    launch_bytes = per_entry * tables.n_entries + per_edge + (12 * tables.n_rows if in_tiles else 0)
    priced = per_entry * tables.n_entries + per_edge + (12 * tables.n_rows if in_tiles else 0)
    if one_launch:
        launch_bytes += tables.algorithmic_bytes_input_tables(spec_table=spec_table)
        priced += 25 * tables.n_strategies
    t_pair = timing["kernel_ms"][main] * 1e-3
    single = len(names) == 1
    t_kernel = timing["region_ms"] * 1e-3 / steps if single else t_pair
    grid, threads = launch_shape(dev, tables, main)
    floor_us, fill_us, fill_per_wg, fill_through = calibrate_launch(priced, grid, threads)
    return {
        "bound": "hbm",
        "kernel": ("build_tables_packed_kernel" if packed else "build_tables_kernel" if one_launch else
                   "redistribute_tiles_row_min_kernel" if in_tiles else "redistribute_tiles_kernel"),
        "launch": main + (" (the one launch of the pass)" if single else ""),
        "arrays_written_per_entry": list(outputs),
        "row_minima_taken_by_this_launch": bool(in_tiles),
        # algorithmic bytes at fixed per-unit prices: 8 B per entry and fp64 array written (+ 1 B for the
        # transition flag), the two spec lists and a 64-byte header per edge, 25 B per strategy when the
        # launch builds the compute costs, 12 B per row minimum it takes
        "achieved": priced / t_kernel / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": priced / t_kernel / 1e9 / HBM_PEAK_GBPS,
        # every byte the launch reads or writes (the tensor and strategy table rows in full)
        "frac_bytes_moved": launch_bytes / t_kernel / 1e9 / HBM_PEAK_GBPS,
        "traffic": None,  # filled in by measure_traffic for the main workload
        "bytes_per_launch": priced, "bytes_moved_per_launch": launch_bytes,
        "avg_launch_us": t_kernel * 1e6,
        "launch_floor_us": floor_us, "fill_us": fill_us, "frac_of_fill": fill_us / (t_kernel * 1e6),
        "calibration": f"apc_calibrate_launch: an empty kernel of the launch's grid ({grid} workgroups of {threads} threads) "
                       f"back to back; apc_calibrate_fill: a kernel that only writes bytes_per_launch ({fill_per_wg} doubles "
                       f"per workgroup, stores {'written through to memory' if fill_through else 'left to the L2'}: the fastest "
                       "of four splits x two kinds of store), same timing",
        "avg_launch_us_event_pair_per_launch": t_pair * 1e6,
        "min_launch_us_event_pair_per_launch": timing["kernel_ms_min"][main] * 1e3,
        "timing": ("one HIP event pair on the launch stream around the K back-to-back launches of the timed "
                   "region (the pass is this one kernel), / K" if single else
                   "HIP events around every launch of the kernel inside the timed region"),
    }


def launch_shape(dev, tables, main):
    """(workgroups, threads) of the launch that writes the matrices, as the library sizes it."""
    n_tiles = tables.n_tiles
    tile_blocks = (n_tiles + 7) // 8 * 8
    if main == "build_tables_packed":
        return tile_blocks + (tables.n_tensors + 255) // 256 + (tables.n_strategies + 255) // 256, 256
    per_tile = tables.n_entries // max(n_tiles, 1)
    if main == "build_tables":
        threads = 256 if per_tile >= 1536 else 128 if per_tile >= 512 else 64
        return tile_blocks + (tables.n_tensors + threads - 1) // threads + (tables.n_strategies + threads - 1) // threads, threads
    threads = 256 if per_tile >= 4096 else 128 if per_tile >= 512 else 64
    return tile_blocks, threads


def measure(name, args, log, steps, warmup, main_run):
    """Builds one workload, times its pass, verifies it; -> (result dict, planner or None, ...)."""
    import numpy as np
    import torch

    from autoparallel_amd._device_thread import call as on_device_thread
    from autoparallel_amd.device_tables import DeviceCostTables

    t_setup = time.perf_counter()
    tables, params, desc, dev, planner, host_timings = build_workload(name, args)

    # a traced workload keeps its capture context (a fake-tensor mode) open in this thread until
    # the plan is solved; the measurements work on real device buffers, so they run where the
    # package's own device work runs
    def on_real_tensors(dev):
        t0 = time.perf_counter()
        if dev is None:
            if args.tile_entries:
                tables.build_tiles(args.tile_entries)
            dev = DeviceCostTables(tables, params, device="cuda:0")
        log.info("%s: tables resident: %d entries, %d tiles", name, tables.n_entries, tables.n_tiles)
        step = prepare(dev, args.pass_kind)
        torch.cuda.synchronize()
        host_timings["upload_and_prepare_s"] = time.perf_counter() - t0
        host_timings["setup_total_s"] = time.perf_counter() - t_setup
        timing = time_pass(dev, step, steps, warmup)
        ms_per_step = timing["wall_s"] / steps * 1e3
        log.info("%s: timed region done: %.4f ms/step", name, ms_per_step)
        parity = None if args.no_verify else verify_pass(dev, tables, params, log)
        roof = roofline_of(dev, tables, timing, steps, args.pass_kind)
        # the planner's follow-up launch: the ILP objective summed on the device from the cost
        # array (its own kernel, after the host has numbered the variables; not part of the table
        # pass); without a planner every entry is its own variable
        objective_us = None
        if dev.cost is not None:
            if planner is not None:
                groups = planner.sharding_optimizer.objective_groups
            else:
                eb = tables.edge_entry_begin.astype(np.int64)
                live = np.nonzero(np.diff(eb) > 0)[0]
                groups = (tables.n_entries, np.concatenate([eb[:-1][live], [tables.n_entries]]),
                          np.arange(len(live) + 1, dtype=np.int64), eb[:-1][live])
            pair = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            dev.cost_objective(*groups)
            torch.cuda.synchronize()
            pair[0].record()
            dev.cost_objective(*groups)
            pair[1].record()
            torch.cuda.synchronize()
            objective_us = pair[0].elapsed_time(pair[1]) * 1e3
            # the kernel alone: index arrays resident, launches back to back
            from autoparallel_amd import _native
            from autoparallel_amd.device_tables import _to_device

            gv, gm, me = (_to_device(np.ascontiguousarray(a, np.int64), dev.device) for a in groups[1:])
            reps = 20 if tables.n_entries < 10_000_000 else 5
            call = lambda: _native.torch_ops().cost_objective(int(groups[0]), gv, gm, me, dev.cost, 10000.0)  # noqa: E731
            call()
            torch.cuda.synchronize()
            pair[0].record()
            for _ in range(reps):
                call()
            pair[1].record()
            torch.cuda.synchronize()
            objective_kernel_us = pair[0].elapsed_time(pair[1]) * 1e3 / reps
            # the planner's device stage as one figure: the pass and the objective reduction that follows it,
            # alternating, back to back
            for launch in step.values():
                launch()
            call()
            torch.cuda.synchronize()
            pair[0].record()
            for _ in range(reps):
                for launch in step.values():
                    launch()
                call()
            pair[1].record()
            torch.cuda.synchronize()
            device_stage_us = pair[0].elapsed_time(pair[1]) * 1e3 / reps
            objective_bytes = 8 * sum(int(x) for x in np.diff(groups[1]) * np.diff(groups[2])) + 9 * int(groups[0])
        E = tables.n_entries
        out = {
            "value": E * steps / timing["wall_s"], "ms_per_step": ms_per_step,
            "config": {**desc, "edges": tables.n_edges, "strategies": tables.n_strategies, "specs": tables.n_specs,
                       "entries": E, "tiles": tables.n_tiles, "tiling": tables.tiling, "matrix_rows": tables.n_rows,
                       "edges_deduplicated": int((tables.edge_canonical != np.arange(tables.n_edges)).sum()),
                       "device_row": params.device_name, "devices_per_host": 8,
                       "step": " + ".join(timing["names"]) + (
                           ": DeviceCostTables.planner_pass, the launches ShardingOptimizer.build_ds issues "
                           "(tensor + compute-cost tables and the assembled cost of every entry"
                           + (", row minima taken by the same launch" if roof["row_minima_taken_by_this_launch"] else "")
                           + "; the spec table was built before, comm / transition are written only on request)"
                           if args.pass_kind == "planner" else
                           ": every table and all three per-entry arrays (composite pass, not what the planner issues)")},
            "roofline": roof,
            "kernel_us": {k: v * 1e3 for k, v in timing["kernel_ms"].items()},
            "objective_reduction_us_including_index_upload": objective_us,
            "objective_kernel": None if objective_us is None else {
                "avg_launch_us_back_to_back": objective_kernel_us, "variables": int(groups[0]), "groups": len(groups[1]) - 1,
                "bytes": objective_bytes, "frac_of_hbm_peak": objective_bytes / (objective_kernel_us * 1e-6) / 8e12,
                "pass_plus_objective_us": device_stage_us,
                "note": "bytes = 8 per entry read + 9 per variable written (objective f64, forced-to-zero u8); the "
                        "output arrays are allocated by the operator on every call; pass_plus_objective_us: the "
                        "planner's device stage, the launches of the pass and the reduction alternating back to back "
                        "(two host calls per iteration: on a small table the host's dispatch, about 10 us per call, "
                        "is part of the figure)"},
            "ms_per_step_with_events": timing["wall_events_s"] / steps * 1e3,
            "host_timings_s": {k: round(v, 6) for k, v in host_timings.items()},
            "parity": parity,
            "params": params,
        }
        if main_run and not args.no_cpu_baseline:
            out["cpu_baseline"] = cpu_baseline(tables, params, args.cpu_seconds)
        return out

    out = on_device_thread(on_real_tensors, dev)
    return out, planner, tables, host_timings


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
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a HIP device (there is no CPU path for the product)", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    if args.replay_tables:
        replay_tables(args.replay_tables)
        return
    if args.calibrate_launch:
        # the three workloads' launch shapes and bytes (bytes_per_launch of their roofline objects)
        for name, nbytes, grid, threads in (("llama3_8b", 20_766_135, 1352, 256), ("llama3_70b", 596_653_014, 11736, 256),
                                           ("stress", 3_825_705_690, 426920, 128)):
            floor_us, fill_us, per, through = calibrate_launch(nbytes, grid, threads)
            print(json.dumps({"workload": name, "bytes": nbytes, "grid": grid, "threads": threads, "launch_floor_us": floor_us,
                              "fill_us": fill_us, "fill_doubles_per_workgroup": per, "fill_written_through": bool(through),
                              "fill_TBps": nbytes / fill_us / 1e6}))
        return
    if args.calibrate_copy:
        src = torch.ones(1 << 27, dtype=torch.float64, device="cuda:0")  # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes_read": src.numel() * 8, "calibrate_copy_bytes_written": src.numel() * 8,
                          "copies": 3}))
        return

    K = args.steps
    copy_factor = None
    out, planner, tables, host_timings = measure(args.workload, args, log, K, args.warmup, main_run=True)
    result = {
        "metric": "redistribution_cost_entries_per_s",
        "value": out["value"],
        "unit": "entries/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": args.warmup,
        "ms_per_step": out["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": out["config"],
        "roofline": out["roofline"],
        "kernel_us": out["kernel_us"],
        "objective_reduction_us_including_index_upload": out["objective_reduction_us_including_index_upload"],
        "objective_kernel": out["objective_kernel"],
        "ms_per_step_with_events": out["ms_per_step_with_events"],
        "host_timings_s": out["host_timings_s"],
        "parity": out["parity"],
    }
    if "cpu_baseline" in out:
        result["cpu_baseline"] = out["cpu_baseline"]
    if not args.no_traffic:
        t0 = time.perf_counter()
        read = measure_traffic(tables, out["params"], args.pass_kind, out["roofline"]["kernel"], log)
        log.info("traffic reading: %.1f s", time.perf_counter() - t0)
        if read is not None:
            result["roofline"].update(read)
            result["roofline"]["traffic_over_bytes_moved"] = read["traffic"] / result["roofline"]["bytes_moved_per_launch"]
            copy_factor = read["traffic_reading"]["scale_from_1gib_copy"]
    if planner is not None:
        plan = {"stages_s": {k: round(v, 6) for k, v in host_timings.items()}}
        if not args.no_solve:
            log.info("solving the ILP: %d variables", planner.sharding_optimizer.n_variables)
            plan.update(solve_plan(planner, args.workload))
        table_stage = host_timings.get("optimizer_tables_s", 0.0)
        other = host_timings.get("capture_s", 0.0) + host_timings.get("optimizer_s", 0.0) - table_stage \
            + plan.get("constraints_s", 0.0) + plan.get("solve_s", 0.0)
        plan["total_with_gpu_tables_s"] = other + table_stage
        if "cpu_baseline" in result:
            # (derived, not a run: the device plan's other stages + the table size / the CPU port's rate)
            cpu_tables = tables.n_entries / result["cpu_baseline"]["value"]
            plan["derived_cpu_table_stage_s"] = cpu_tables
            plan["derived_total_with_cpu_tables_s"] = other + cpu_tables
        result["plan_wall_time"] = plan
        planner.__exit__(None, None, None)
        planner = None
        if not args.no_cpu_plan and not args.no_solve and not args.no_cpu_baseline:
            measured = plan_with_cpu_tables(args.workload, args, log)
            plan["measured_with_cpu_tables"] = {
                "what": "the same planner run once more with the scalar Python oracle as its table source (1 core), "
                        "pruning off: capture + optimizer construction (enumerate, cluster, encode, tables) + "
                        "constraints + solve of the full program",
                **{k: (round(v, 6) if k != "objective" else v) for k, v in measured.items()}}
            if "solve_s_without_pruning" in plan:
                plan["total_with_gpu_tables_without_pruning_s"] = \
                    plan["total_with_gpu_tables_s"] - plan.get("solve_s", 0.0) + plan["solve_s_without_pruning"]
            if abs(measured["objective"] - plan.get("objective", measured["objective"])) > 1e-6 * abs(measured["objective"]):
                raise SystemExit("bench.py: the plan from host-built tables has another objective than the device's")
    del planner, tables
    # ---- the bandwidth-bound tables, beside the headline ---------------------------------------
    extra = {}
    for name in [x for x in args.extra.split(",") if x and x != args.workload]:
        if name not in WORKLOADS:
            raise SystemExit(f"bench.py: unknown extra workload {name}")
        import gc

        gc.collect()
        torch.cuda.empty_cache()
        k = max(5, min(K, 20))
        o, pl, tb, _ = measure(name, args, log, k, min(args.warmup, 5), main_run=False)
        if pl is not None:
            pl.__exit__(None, None, None)
        if not args.no_traffic and copy_factor is not None:
            read = measure_traffic(tb, o["params"], args.pass_kind, o["roofline"]["kernel"], log, factor=copy_factor)
            if read is not None:
                o["roofline"].update(read)
                o["roofline"]["traffic_over_bytes_moved"] = read["traffic"] / o["roofline"]["bytes_moved_per_launch"]
        del tb
        extra[name] = {"workload": o["config"]["workload"], "entries": o["config"]["entries"], "steps": k,
                       "ms_per_step": o["ms_per_step"], "entries_per_s": o["value"], "step": o["config"]["step"],
                       "tiles": o["config"]["tiles"], "roofline": o["roofline"], "kernel_us": o["kernel_us"],
                       "objective_kernel": o["objective_kernel"], "parity": o["parity"], "host_timings_s": o["host_timings_s"]}
        del o, pl
    if extra:
        result["extra"] = extra
    print(json.dumps(result))


if __name__ == "__main__":
    main()
