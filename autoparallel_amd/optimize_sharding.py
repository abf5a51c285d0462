"""``ShardingOptimizer``: the planner class of the reference
(autoparallel/optimize_sharding.py:129-958) with its cost-table build replaced by one
batched pass over HIP kernels.

Same constructor, attributes and methods as the reference class, so its callers
(autoparallel/api.py:273-282, 398-445) can use it unchanged:

    opt = ShardingOptimizer(gm, mesh, rescale_grad_comm_cost_for_mp=1.0, repeated_subgraphs=False)
    opt.strats, opt.ds, opt.num_inp_out, opt.num_args, opt.prob, opt.res, opt.cluster_links
    opt.add_grad_param_constraints(), add_parameter_memory_constraint(), add_node_constraint(),
    add_sharded_input_constraint(), add_sharded_output_constraint(), get_solution(), get_log(),
    print_costs_for_node()

What differs underneath:
  * ``build_ds`` flattens ``strats`` once (graphs/encode.py), sends the tables to the GPU,
    runs the integer shard-shape kernel, the compute-cost kernel and the redistribution-cost
    kernel, and copies the three result arrays back.  ``ds`` is a read-only mapping view over
    those arrays: a record dict is materialised only when a key is looked up.
  * every ILP variable is an entry index of the flattened tables; constraints are emitted
    as sparse index arrays and solved by HiGHS through scipy (PuLP / CBC are not required).
  * the environment inputs the reference reads implicitly (devices per host, device row)
    are explicit: class attributes ``devices_per_host`` / ``device_name``, defaulting to the
    values the reference's own tests patch in (8, "H100").
There is no CPU path for the tables: without a HIP device construction raises.
"""

from __future__ import annotations

import logging
import math
import time
from collections.abc import Mapping
from typing import Optional

import numpy as np
import torch
from torch.distributed.tensor._dtensor_spec import DTensorSpec
from torch.distributed.tensor._op_schema import OpStrategy
from torch.distributed.tensor.placement_types import Placement, Replicate, Shard

from ._device_thread import on_device_thread
from .cost_model import CostModelParams
from .graphs.cost_inputs import fill_flops_and_bytes, strategy_recipes
from .graphs.encode import EncodedGraph, all_input_nodes, encode_graph
from .graphs.strategies import StrategyEnumerator
from .ilp import BinaryProgram, next_name

logger = logging.getLogger(__name__)


class DeviceBackend:
    """Runs the table kernels on the GPU (the only backend of the product).

    The table pass is enqueued and left running while the host numbers the ILP variables;
    what comes back afterwards is one objective coefficient and one forced-to-zero flag per
    variable plus the per-strategy compute costs.  The per-entry arrays stay in HBM and are
    copied (``comm`` and ``transition`` are even computed) only when a report asks for them.

    Methods that handle device tensors run on the package's device thread: the planner calls
    them under the fake-tensor mode of its graph capture, which that thread does not see."""

    def __init__(self, tables, params: CostModelParams, device="cuda:0"):
        from .device_tables import DeviceCostTables

        self.dev = DeviceCostTables(tables, params, device=device)
        self.timings = {}
        self.launches = ()

    @staticmethod
    def warm_up(device="cuda:0"):
        """Starts what the first use of the device costs a process (torch's first host-to-device
        copy, 0.15 s; loading the library's code object with its first launch, 15 ms) on the
        device thread and returns at once: a planner calls it before it captures the graph, so
        that the two overlap.  Failures are left to the real construction to report."""
        from . import _device_thread

        def first_use():
            try:
                if not torch.cuda.is_available():
                    return
                from . import _native

                ops = _native.torch_ops()
                one = torch.ones(1, dtype=torch.int32).to(device)
                row = torch.ones((1, _native.APC_MAX_RANK), dtype=torch.int64).to(device)
                ops.tensor_tables(one, one, row, row)
                torch.cuda.synchronize(device)
            except Exception as e:  # noqa: BLE001 (reported by the construction that follows)
                logger.debug("device warm-up: %s", e)

        return _device_thread.submit(first_use)

    @on_device_thread
    def local_shapes(self):
        out = self.dev.run_spec_tables()
        return out["local_shape"].cpu().numpy(), out["local_stride"].cpu().numpy()

    @on_device_thread
    def strategy_inputs(self, recipes):
        """Flop and byte counts of every strategy on the device (spec table, then
        ``apc_strategy_inputs`` over the per-node recipes); the host's strategy table receives
        copies (identical edges are found on the host, and flop / byte counts are part of an
        edge's identity)."""
        flops, rw_bytes, dtype, zero = self.dev.run_strategy_inputs(recipes)
        tb = self.dev.tables
        tb.strat_flops[:] = flops.cpu().numpy()
        tb.strat_rw_bytes[:] = rw_bytes.cpu().numpy()
        tb.strat_dtype[:] = dtype.cpu().numpy()
        tb.strat_zero_cost[:] = zero.cpu().numpy()
        self._strategy_inputs_on_device = True

    def upload_strategy_inputs(self, tables, tile_entries=None, dedupe=True, max_copies=16):
        """The strategy table is final: tile the edges (identical edges once) and send both."""
        tables.build_tiles(tile_entries, dedupe=dedupe, max_copies=max_copies)
        tables.validate(self.dev.params)
        names = ("tile_records", "dup_entry_begin", "dup_row_begin")
        if not getattr(self, "_strategy_inputs_on_device", False):
            names = ("strat_flops", "strat_rw_bytes", "strat_dtype", "strat_zero_cost") + names
        self.dev.refresh(*names)

    @on_device_thread
    def launch_tables(self):
        """Enqueues the planner's table pass (``DeviceCostTables.planner_pass``) and returns."""
        d = self.dev
        step = d.planner_pass()
        self.launches = tuple(step)
        self._events = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
        with torch.cuda.device(d.device):
            self._events[0].record()
            for launch in step.values():
                launch()
            self._events[1].record()

    @on_device_thread
    def finish(self, n_vars, group_var_begin, group_member_begin, member_entry_begin):
        """Sums the ILP objective on the device and copies back what the planner needs:
        -> {"objective", "forced_zero", "compute", "compute_per_arg"} (host arrays)."""
        d = self.dev
        with torch.cuda.device(d.device):
            obj, forced = d.cost_objective(n_vars, group_var_begin, group_member_begin, member_entry_begin)
            torch.cuda.synchronize(d.device)
        d.check_error_flag()
        self.timings["kernels_s"] = self._events[0].elapsed_time(self._events[1]) * 1e-3
        t0 = time.perf_counter()
        out = {
            "objective": obj.cpu().numpy(),
            "forced_zero": forced.cpu().numpy().astype(bool),
            "compute": d.compute_cost.cpu().numpy(),
            "compute_per_arg": d.compute_cost_per_arg.cpu().numpy(),
        }
        self.timings["copy_back_s"] = time.perf_counter() - t0
        for k in ("kernels_s", "copy_back_s"):
            logger.info("%s %.6f s", k, self.timings[k])
        return out

    @on_device_thread
    def host_array(self, name):
        """``comm`` / ``transition`` / ``cost`` of every entry, copied (computed first, if the
        table pass did not write it) now."""
        return self.dev.fetch(name).cpu().numpy()

    @on_device_thread
    def gather(self, name, entries):
        """The values of a few entries of ``comm`` / ``transition`` / ``cost``."""
        idx = torch.from_numpy(np.ascontiguousarray(entries, np.int64)).to(self.dev.device)
        return self.dev.fetch(name)[idx].cpu().numpy()

    def diffusion_sweeps(self, graph, theta, unary, n_sweeps):
        """Sweeps of the dual ascent that prunes the program (pruning.py), on the device."""
        return self.dev.diffusion_sweeps(graph, theta, unary, n_sweeps)

    @on_device_thread
    def row_min(self, row_ptr):
        if self._are_matrix_rows(row_ptr):  # taken by the table launch, or one read of every distinct row
            mins, args = self.dev.row_minima()
        else:
            mins, args = self.dev.segmented_min(self.dev.fetch("cost"), row_ptr)
        return mins.cpu().numpy(), args.cpu().numpy()

    def _are_matrix_rows(self, row_ptr) -> bool:
        tb = self.dev.tables
        return len(row_ptr) == tb.n_rows + 1 and np.array_equal(row_ptr, tb.row_ptr())

    @on_device_thread
    def greedy(self, row_ptr):
        """-> (bound per strategy, min per node, argmin per node) from the row minima of the cost table"""
        if self._are_matrix_rows(row_ptr):
            mins, _ = self.dev.row_minima()
        else:
            mins, _ = self.dev.segmented_min(self.dev.fetch("cost"), row_ptr)
        return tuple(x.cpu().numpy() for x in self.dev.greedy_strategies(mins))


class CostRecords(Mapping):
    """``ds``: (s_i, argi, ss, ii) -> record, backed by the flat result arrays."""

    def __init__(self, optimizer: "ShardingOptimizer"):
        self._o = optimizer

    def _index(self, key) -> int:
        s_i, argi, ss, ii = key
        enc = self._o.encoded
        e = enc.edge_of.get((s_i, argi))
        if e is None:
            raise KeyError(key)
        tb = enc.tables
        ns, nt = int(tb.edge_n_src[e]), int(tb.edge_n_tgt[e])
        if not (0 <= ss < nt and 0 <= ii < ns):
            raise KeyError(key)
        return int(tb.edge_entry_begin[e]) + ss * ns + ii

    def __getitem__(self, key):
        o = self._o
        idx = self._index(key)
        s_i, argi, ss, _ = key
        full = o.strats[o.nodes[s_i]].strategies[ss]
        return {
            "va": int(o.vars_of(idx)),
            "cost": float(o.cost[idx]),
            "compute_cost": float(o.compute_cost_per_arg[o.encoded.strat_begin[s_i] + ss]),
            "comm_cost": float(o.comm_cost[idx]),
            "sharding_transition_cost": int(o.transition_cost[idx]),
            "full_strat": full,
            "out_strat": full.output_specs,
            "inp_strat": full.input_specs[argi],
        }

    def __contains__(self, key):
        try:
            self._index(key)
            return True
        except (KeyError, TypeError, ValueError):
            return False

    def __len__(self):
        return self._o.encoded.tables.n_entries

    def __iter__(self):
        enc = self._o.encoded
        tb = enc.tables
        for e, (s_i, argi) in enumerate(enc.edge_keys):
            ns, nt = int(tb.edge_n_src[e]), int(tb.edge_n_tgt[e])
            for ss in range(nt):
                for ii in range(ns):
                    yield (s_i, argi, ss, ii)

    def key_of_entry(self, idx: int):
        return self.keys_of_entries(np.asarray([idx], np.int64))[0]

    def keys_of_entries(self, entries) -> list:
        tb = self._o.encoded.tables
        entries = np.asarray(entries, np.int64)
        # the last edge that starts at or before the entry and is not empty
        e = np.searchsorted(tb.edge_entry_begin, entries, side="right") - 1
        ns = tb.edge_n_src[e].astype(np.int64)
        local = entries - tb.edge_entry_begin[e]
        keys = self._o.encoded.edge_keys
        return [(*keys[ee], int(r), int(c)) for ee, r, c in zip(e.tolist(), (local // ns).tolist(), (local % ns).tolist())]


class ClusterLinks(Mapping):
    """``cluster_links``: key of a linked entry -> key of the entry whose ILP variable it
    shares (optimize_sharding.py:211-231), derived from the node representatives."""

    def __init__(self, optimizer: "ShardingOptimizer"):
        self._o = optimizer

    def _rep(self, key):
        s_i, argi, ss, ii = key
        o = self._o
        if key not in o.ds:
            raise KeyError(key)
        rep = o.node_representative.get(o.nodes[s_i])
        if rep is None:
            raise KeyError(key)
        return (o.node_map[rep], argi, ss, ii)

    def __getitem__(self, key):
        return self._rep(key)

    def __contains__(self, key):
        try:
            self._rep(key)
            return True
        except (KeyError, TypeError, ValueError):
            return False

    def __iter__(self):
        o = self._o
        for key in o.ds:
            if o.nodes[key[0]] in o.node_representative:
                yield key

    def __len__(self):
        return self._o.n_linked_entries


class ShardingOptimizer:
    # environment of the cost model, explicit (the reference reads torch.cuda.device_count()
    # and torch.cuda.get_device_name(); its tests patch them to 8 and "H100")
    devices_per_host = 8
    device_name = "H100"
    device = "cuda:0"
    backend_cls = DeviceBackend
    solver_time_limit: Optional[float] = None
    # relative gap at which the solver may stop: 0 = prove optimality (the reference's CBC default);
    # None = the solver's own default (1e-4)
    solver_rel_gap: Optional[float] = 0.0
    # tiling of the edge matrices: entries per tile (None: chosen from the table), whether
    # identical edges (repeated layers) are evaluated once, and how many copies one evaluated
    # edge may serve at most
    tile_entries = None
    dedupe = True
    max_copies = 16
    # ILP formulation: besides the reference's one binary per cost entry, one binary per (node,
    # strategy) tied to the entry variables of that strategy's row.  Only these need to be
    # declared integral: with a node's and its producers' choices fixed to unit vectors the
    # row / column sum constraints leave exactly one feasible (integral) value for every entry
    # variable.  Same feasible plans and optimum, far fewer branching variables for the solver.
    # How repeated subgraphs are found when the constructor is asked for them.
    #   "regions": the reference's region growing over torch's region tracker with the reference's
    #       links (graph_clustering.py:101-206, optimize_sharding.py:211-231); raises the reference's own
    #       "Duplicate node ... in region group" where the reference does (every Llama-shaped graph
    #       under torch 2.10);
    #   "neighbourhood": this package's refinement of node keys by their surroundings;
    #   "reference" (default): "regions", and "neighbourhood" only where "regions" ends in that
    #       error, so that a graph the reference can plan gets the reference's program.  torch's
    #       region tracker keeps the set of all ancestors of every node (quadratic: 0.9 s on 2 600
    #       nodes, 16.7 s on the 10 372 nodes of Llama-3-8B, where it then raises), so graphs of
    #       more than ``regions_max_nodes`` nodes go to "neighbourhood" directly.
    # ``clustering_used`` records which one produced the links, and why.
    clustering = "reference"
    regions_max_nodes = 3000
    # during enumeration torch's own redistribute_cost (whose values the table build replaces) is
    # stubbed by a constant; False leaves it alone (same tables, slower enumeration)
    cheap_enumeration_costs = True
    # flop / byte counts of the strategies from per-node recipes on the device (apc_strategy_inputs);
    # False: on the host, every distinct (operator, local shapes) on fake tensors under torch's
    # flop counter, as the reference does
    strategy_inputs_on_device = True
    node_choice_variables = True
    compact_constraints = True  # with choice variables: the structural constraints written through them
    # Before the solver runs: a dual ascent over the program's labelling form (row / column minima
    # of the reparametrised cost matrices, on the device), an incumbent rounded from it, and every
    # strategy and strategy pair whose bound exceeds the incumbent fixed to zero (pruning.py).
    # Sweeps are run in these chunks; after each the bound and the incumbent are re-evaluated and
    # the ascent stops once they agree to ``prune_gap``.
    prune_before_solve = True
    prune_sweep_chunks = (40, 40, 80, 80, 160)
    prune_gap = 2e-4
    # Where the rounding does not reach the bound (the relaxation has a gap, or the ascent is not
    # through: a mixture-of-experts graph has four times the classes of a Llama graph), the
    # ascent goes on in chunks twice the last one's size while a chunk still lifts the bound by more
    # than ``prune_gap / 4`` (relative), up to ``prune_max_sweeps`` in all; then the program is solved
    # restricted to the variables whose bound is within a slack of the lower bound, slack =
    # ``prune_slacks`` x |bound| in turn, capped by the incumbent's distance.  A restricted optimum
    # that is itself within the slack is the optimum: everything left out costs more.
    prune_max_sweeps = 3200
    prune_slacks = (1e-4, 1e-3, 1e-2)
    # copy ``comm`` back and write it into every OpSpec.redistribute_cost at construction
    # (optimize_sharding.py:361-363); off: ``materialize_redistribute_costs()`` does it on request
    write_back_redistribute_cost = False

    def __init__(self, gm, mesh, rescale_grad_comm_cost_for_mp=1.0, repeated_subgraphs=False):
        # Construction allocates millions of small long-lived objects (strategies, cost rows)
        # and no reference cycles worth collecting: the cyclic collector's full passes over
        # them were a fifth of the construction time on the 70B graph.
        import gc

        was_enabled = gc.isenabled()
        gc.disable()
        try:
            self._construct(gm, mesh, rescale_grad_comm_cost_for_mp, repeated_subgraphs)
        finally:
            if was_enabled:
                gc.enable()

    def _construct(self, gm, mesh, rescale_grad_comm_cost_for_mp, repeated_subgraphs):
        self.gm = gm
        self.graph = gm.graph
        self.nodes = list(self.graph.nodes)
        self.mesh = mesh
        self.rescale_grad_comm_cost_for_mp = rescale_grad_comm_cost_for_mp
        self.node_map = {node: i for i, node in enumerate(self.graph.nodes)}
        self.timings = {}
        t0 = time.perf_counter()
        self.strats = self.build_sharding_metadata()
        self.timings["enumerate_s"] = time.perf_counter() - t0
        logger.info("%s %.3f s", "enumerate_s", self.timings["enumerate_s"])

        self.node_representative = {}
        self.clustering_used = None
        if repeated_subgraphs:
            from .graphs import clustering

            t0 = time.perf_counter()
            self.node_representative, self.clustering_used = self._find_repeated_subgraphs(clustering)
            logger.info("repeated subgraphs: %s", self.clustering_used)
            self.timings["cluster_s"] = time.perf_counter() - t0
            logger.info("%s %.3f s", "cluster_s", self.timings["cluster_s"])
        self.ds, self.num_inp_out, self.num_args = self.build_ds()
        self.validate()
        self.cluster_links = ClusterLinks(self)
        self.create_cluster_links()
        self._finish_tables()
        self.prob = BinaryProgram(self.n_variables + self.n_choice_variables, "AutoParallel")
        self.res = None
        # what the user constraints mean on the labelling form (read by _label_graph)
        self._label_masks = {}  # s_i -> allowed strategies
        self._pair_ties = []  # (s_i, s_j, [(strategy of i, strategy of j) that go together])
        self._linear_rows = []  # ([(s_i, coefficient per strategy)], lower, upper)
        self.solve_stats = {}
        self.add_default_constraints()

    # ------------------------------------------------------------------------------------
    def _find_repeated_subgraphs(self, clustering):
        """-> (node -> representative, which algorithm produced it and why)."""
        if self.clustering == "neighbourhood":
            return clustering.cluster_nodes(self.graph, self.strats), "neighbourhood (asked for)"
        if self.clustering == "regions":
            return clustering.cluster_regions(self.graph, self.strats), "regions (asked for)"
        if self.clustering != "reference":
            raise ValueError(f"clustering must be 'reference', 'regions' or 'neighbourhood', not {self.clustering!r}")
        n_nodes = len(self.graph.nodes)
        if n_nodes > self.regions_max_nodes:
            return clustering.cluster_nodes(self.graph, self.strats), (
                f"neighbourhood ({n_nodes} nodes: torch's region tracker is quadratic, regions_max_nodes = "
                f"{self.regions_max_nodes})")
        try:
            return clustering.cluster_regions(self.graph, self.strats), "regions (the reference's links)"
        except RuntimeError as e:
            if "Duplicate node" not in str(e):
                raise
            return clustering.cluster_nodes(self.graph, self.strats), f"neighbourhood (the reference's algorithm raised: {e})"

    def build_sharding_metadata(self):
        self.enumerator = StrategyEnumerator(self.mesh, cheap_costs=self.cheap_enumeration_costs)
        return self.enumerator.enumerate(self.graph)

    def _grad_param_nodes(self):
        from torch._functorch._aot_autograd.fx_utils import get_param_and_grad_nodes

        try:
            return set(x[1] for x in get_param_and_grad_nodes(self.graph).values())
        except (KeyError, AttributeError):
            return set()  # a graph without AOT descriptors has no parameter gradients to rescale

    def cost_model_params(self) -> CostModelParams:
        return CostModelParams.from_mesh(tuple(self.mesh.shape), device_name=self.device_name,
                                         devices_per_host=self.devices_per_host,
                                         rescale=self.rescale_grad_comm_cost_for_mp)

    def build_ds(self):
        """Batched table build: encode -> shard-shape kernel -> flop / byte inference ->
        compute-cost kernel -> redistribution-cost kernel -> copy back."""
        t0 = time.perf_counter()
        self.encoded: EncodedGraph = encode_graph(self.graph, self.strats, tuple(self.mesh.shape),
                                                  self._grad_param_nodes())
        self.timings["encode_s"] = time.perf_counter() - t0
        logger.info("%s %.3f s", "encode_s", self.timings["encode_s"])
        self.params = self.cost_model_params()
        tb = self.encoded.tables
        t0 = time.perf_counter()
        self.backend = self.backend_cls(tb, self.params, self.device)
        self.cost_input_stats = {}
        # flop / byte counts of every strategy (compute_estimation.py:232-299, 334-349): on the
        # device from per-node recipes; on the host, operator by operator on fake tensors of the
        # local shapes, when the graph holds an operator no recipe covers (or the backend has
        # no device)
        recipes = strategy_recipes(self.encoded, self.strats, tuple(self.mesh.shape)) if self.strategy_inputs_on_device else None
        on_device = recipes is not None and not recipes.host_nodes and hasattr(self.backend, "strategy_inputs")
        self.cost_input_stats["strategy_inputs"] = "device" if on_device else "host"
        if on_device:
            self.backend.strategy_inputs(recipes)
        else:
            local_shape, local_stride = self.backend.local_shapes()
        self.timings["upload_and_shapes_s"] = time.perf_counter() - t0
        logger.info("%s %.3f s", "upload_and_shapes_s", self.timings["upload_and_shapes_s"])
        t0 = time.perf_counter()
        if not on_device:
            fill_flops_and_bytes(self.encoded, self.strats, local_shape, local_stride, self.cost_input_stats)
        self.backend.upload_strategy_inputs(tb, self.tile_entries, self.dedupe, self.max_copies)
        self.timings["flops_bytes_s"] = time.perf_counter() - t0
        logger.info("%s %.3f s", "flops_bytes_s", self.timings["flops_bytes_s"])
        # the table pass runs on the device while the host numbers the ILP variables;
        # _finish_tables() collects what the planner needs of it
        t0 = time.perf_counter()
        self.backend.launch_tables()
        self.timings["launch_tables_s"] = time.perf_counter() - t0
        self._host_arrays = {}
        self._inf_entries = None
        if self.write_back_redistribute_cost:
            self.materialize_redistribute_costs()
        return CostRecords(self), self.encoded.num_inp_out, self.encoded.num_args

    def _finish_tables(self):
        """Objective coefficients, forced-to-zero flags and compute costs from the backend: one
        number per ILP variable instead of three arrays per entry (optimize_sharding.py:522-536,
        650-655, evaluated where the costs are)."""
        t0 = time.perf_counter()
        tb = self.encoded.tables
        begin = tb.edge_entry_begin.astype(np.int64)
        sizes = begin[1:] - begin[:-1]
        live = sizes > 0
        roots = np.nonzero(self.edge_is_representative & live)[0]
        members = np.nonzero(live)[0]
        members = members[np.argsort(self.edge_rep[members], kind="stable")]  # grouped by root, ascending inside
        group_var_begin = np.concatenate([self.edge_var_base[roots], [self.n_variables]]).astype(np.int64)
        counts = np.bincount(np.searchsorted(roots, self.edge_rep[members]), minlength=len(roots))
        group_member_begin = np.zeros(len(roots) + 1, np.int64)
        np.cumsum(counts, out=group_member_begin[1:])
        self.objective_groups = (self.n_variables, group_var_begin, group_member_begin, begin[:-1][members])
        out = self.backend.finish(*self.objective_groups)
        self.objective_vector = out["objective"]
        self.forced_zero_vars = out["forced_zero"]
        self.compute_cost = out["compute"]  # per (node, strategy), before the division by num_args
        self.compute_cost_per_arg = out["compute_per_arg"]
        self.timings["tables_s"] = self.timings.pop("launch_tables_s") + time.perf_counter() - t0
        logger.info("%s %.3f s", "tables_s", self.timings["tables_s"])
        self.timings.update({f"backend_{k}": v for k, v in getattr(self.backend, "timings", {}).items()})

    # ---- per-entry arrays: they stay with the backend until somebody reads them --------------------
    def _host_array(self, name):
        a = self._host_arrays.get(name)
        if a is None:
            a = self.backend.host_array(name)
            if name == "cost":
                # optimize_sharding.py:531-533: a cost that is not finite reads 10000.0 afterwards
                bad = ~np.isfinite(a)
                self._inf_entries = np.nonzero(bad)[0]
                a = np.where(bad, self.params.inf_replacement_cost, a)
            self._host_arrays[name] = a
        return a

    @property
    def comm_cost(self):
        return self._host_array("comm")

    @property
    def transition_cost(self):
        return self._host_array("transition")

    @property
    def cost(self):
        return self._host_array("cost")

    @property
    def inf_entries(self):
        self._host_array("cost")
        return self._inf_entries

    def _values(self, name, entries):
        """A few entries of a per-entry array, without copying the whole array to the host."""
        entries = np.asarray(entries, np.int64)
        if name in self._host_arrays:
            return self._host_arrays[name][entries]
        v = self.backend.gather(name, entries)
        if name == "cost":
            v = np.where(np.isfinite(v), v, self.params.inf_replacement_cost)
        return v

    def create_cluster_links(self):
        """Entries of a linked node share the ILP variables of its representative's entries
        (same argument, same strategy pair).  Variables are numbered edge by edge over the
        edges that are their own representative; a linked edge takes its representative's
        block of numbers."""
        tb = self.encoded.tables
        n_edges = tb.n_edges
        begin = tb.edge_entry_begin.astype(np.int64)
        sizes = begin[1:] - begin[:-1]
        edge_rep = np.arange(n_edges, dtype=np.int64)
        edge_of = self.encoded.edge_of
        linked, roots = [], []
        for node, rep in self.node_representative.items():
            s1, s0 = self.node_map[node], self.node_map[rep]
            assert self.num_args[s1] == self.num_args[s0], f"clustering linked {node} and {rep} with different arity"
            for argi in range(self.num_args[s1]):
                linked.append(edge_of[(s1, argi)])
                roots.append(edge_of[(s0, argi)])
        linked, roots = np.asarray(linked, np.int64), np.asarray(roots, np.int64)
        differ = (tb.edge_n_tgt[linked] != tb.edge_n_tgt[roots]) | (tb.edge_n_src[linked] != tb.edge_n_src[roots])
        if differ.any():
            e1, e0 = int(linked[differ][0]), int(roots[differ][0])
            node, rep = (self.nodes[self.encoded.edge_keys[e][0]] for e in (e1, e0))
            raise AssertionError(f"Problem with graph clustering: {rep} and {node} don't have the same number of "
                                 "input/output placements. Please report a bug")
        edge_rep[linked] = roots
        while not np.array_equal(edge_rep[edge_rep], edge_rep):  # representatives are roots already; be safe
            edge_rep = edge_rep[edge_rep]
        is_root = edge_rep == np.arange(n_edges)
        base = np.zeros(n_edges, np.int64)
        base[is_root] = np.cumsum(sizes[is_root]) - sizes[is_root]
        self.edge_var_base = base[edge_rep]
        self.edge_rep = edge_rep
        self.edge_is_representative = is_root
        self._var_of_entry = None  # (one number per entry: made when somebody asks, see var_of_entry)
        self.n_variables = int(sizes[is_root].sum())
        self.n_linked_entries = int(sizes[~is_root].sum())
        # choice variables: one per (node, strategy), shared with the node's representative
        self.n_choice_variables = 0
        self.choice_var_of_strategy = None
        self.node_choice_base = {}
        if self.node_choice_variables:
            # the strategies of every node that represents itself, numbered in node order; a linked
            # node's strategies take its representative's numbers
            nsb = np.asarray(tb.node_strat_begin, np.int64)
            n_strat = nsb[1:] - nsb[:-1]
            own = np.array([node.op != "output" and node not in self.node_representative for node in self.nodes], bool)
            node_base = np.full(len(self.nodes), -1, np.int64)
            node_base[own] = self.n_variables + np.cumsum(n_strat[own]) - n_strat[own]
            next_free = self.n_variables + int(n_strat[own].sum())
            for node, rep in self.node_representative.items():
                s1, s0 = self.node_map[node], self.node_map[rep]
                assert n_strat[s1] == n_strat[s0]
                node_base[s1] = node_base[s0]
            has = node_base >= 0
            self.node_choice_base = {int(s_i): int(node_base[s_i]) for s_i in np.nonzero(has)[0]}
            strat_node = np.repeat(np.arange(len(self.nodes)), n_strat)
            choice = node_base[strat_node] + (np.arange(tb.n_strategies, dtype=np.int64) - nsb[:-1][strat_node])
            choice[~has[strat_node]] = 0
            self.choice_var_of_strategy = choice
            self.n_choice_variables = next_free - self.n_variables

    # ---- entries <-> ILP variables -------------------------------------------------------------
    def vars_of(self, entries):
        """ILP variables of the given entries (an entry of a linked edge has its representative's)."""
        begin = self.encoded.tables.edge_entry_begin
        entries = np.asarray(entries, np.int64)
        e = np.searchsorted(begin, entries, side="right") - 1  # (an empty edge shares its begin with the next one)
        return self.edge_var_base[e] + (entries - begin[e])

    @property
    def var_of_entry(self):
        """The variable of every entry, as one array (n_entries numbers: planning itself asks
        ``vars_of`` about the few entries it needs)."""
        if getattr(self, "_var_of_entry", None) is None:
            self._var_of_entry = self.vars_of(np.arange(self.encoded.tables.n_entries, dtype=np.int64))
        return self._var_of_entry

    def _chosen_entries(self):
        """Entries whose variable is 1 in the solution, ascending.  Every edge's block of
        variables holds exactly one (its unique-decision row), so each edge, linked ones included,
        contributes the entry at that offset; anything else falls back to a pass over all entries."""
        tb = self.encoded.tables
        begin = tb.edge_entry_begin.astype(np.int64)
        sizes = begin[1:] - begin[:-1]
        ones = np.nonzero(self.prob.x[:self.n_variables] == 1)[0]
        roots = np.nonzero(self.edge_is_representative & (sizes > 0))[0]
        root_base = self.edge_var_base[roots]  # ascending: blocks are numbered in edge order
        block = np.searchsorted(root_base, ones, side="right") - 1
        if len(ones) != len(roots) or not np.array_equal(block, np.arange(len(roots))):
            return np.nonzero(self.prob.x[self.var_of_entry] == 1)[0]
        offset_of_root = np.zeros(tb.n_edges, np.int64)
        offset_of_root[roots] = ones - root_base
        live = np.nonzero(sizes > 0)[0]
        return begin[:-1][live] + offset_of_root[self.edge_rep[live]]

    def materialize_redistribute_costs(self):
        """Writes the recomputed communication costs into ``OpSpec.redistribute_cost`` of every
        strategy (optimize_sharding.py:361-363).  Nothing in the planner reads them there
        (``print_costs_for_node`` takes the flat array), so this copy of the whole ``comm`` array
        is made only on request, or at construction with ``write_back_redistribute_cost = True``."""
        tb = self.encoded.tables
        comm = self.comm_cost
        for strategy in self.strats.values():  # nodes of one memo entry share their OpSpec objects until now
            if isinstance(strategy, OpStrategy):
                StrategyEnumerator.own_specs(strategy)
        for e, (s_i, argi) in enumerate(self.encoded.edge_keys):
            ns, nt = int(tb.edge_n_src[e]), int(tb.edge_n_tgt[e])
            b = int(tb.edge_entry_begin[e])
            rows = comm[b:b + ns * nt].reshape(nt, ns).tolist()
            for s, row in zip(self.strats[self.nodes[s_i]].strategies, rows):
                s.redistribute_cost[argi] = row

    # ------------------------------------------------------------------------------------
    def _all_input_nodes(self, node):
        return all_input_nodes(node)

    def walk_over_options(self, node, constrain_arg=None):
        tgt = self.strats[node]
        for argi in range(len(tgt.strategies[0].input_specs)):
            if constrain_arg is not None and argi != constrain_arg:
                continue
            for oi, s in enumerate(tgt.strategies):
                for ii in range(len(s.redistribute_cost[argi])):
                    yield argi, oi, ii

    def _edge(self, s_i, argi):
        e = self.encoded.edge_of[(s_i, argi)]
        tb = self.encoded.tables
        return int(tb.edge_entry_begin[e]), int(tb.edge_n_tgt[e]), int(tb.edge_n_src[e])

    # ---- default constraints (optimize_sharding.py:402-542) --------------------------------
    # Linked nodes share variable blocks, so most constraints of a repeated layer are literally
    # the rows of its representative layer.  A row is determined by the variable blocks (and
    # shapes) it is built from; every emitter below skips a combination it has already emitted
    # instead of materialising the row and leaving it to the solver front-end to drop.
    def add_unique_decision_constraint(self):
        """For every (node, argument): exactly one (output, input) strategy pair."""
        tb = self.encoded.tables
        sizes = (tb.edge_entry_begin[1:] - tb.edge_entry_begin[:-1])[self.edge_is_representative]
        self.prob.add_rows(np.arange(self.n_variables, dtype=np.int64), 1.0, sizes, 1.0, 1.0, "unique_decision")

    def _edge_vars(self, s_i, argi):
        """(variable block start, consumer strategies, producer strategies) of one edge."""
        e = self.encoded.edge_of[(s_i, argi)]
        tb = self.encoded.tables
        return int(self.edge_var_base[e]), int(tb.edge_n_tgt[e]), int(tb.edge_n_src[e])

    def add_same_output_across_args_constraint(self):
        """All arguments of a node agree on the node's output strategy."""
        cols, vals, lens, seen = [], [], [], set()
        for s_i, node in enumerate(self.nodes):
            if node.op != "call_function" or len(self._all_input_nodes(node)) <= 1:
                continue
            b0, nt, ns0 = self._edge_vars(s_i, 0)
            for argi in range(1, len(self._all_input_nodes(node))):
                ba, nta, nsa = self._edge_vars(s_i, argi)
                assert nta == nt
                key = (b0, ba, nt, ns0, nsa)
                if key in seen:
                    continue
                seen.add(key)
                first = b0 + np.arange(nt)[:, None] * ns0 + np.arange(ns0)[None, :]
                other = ba + np.arange(nt)[:, None] * nsa + np.arange(nsa)[None, :]
                cols.append(np.concatenate([first, other], axis=1).ravel())
                vals.append(np.tile(np.concatenate([np.ones(ns0), -np.ones(nsa)]), nt))
                lens.append(np.full(nt, ns0 + nsa))
        if cols:
            self.prob.add_rows(np.concatenate(cols), np.concatenate(vals), np.concatenate(lens), 0.0, 0.0,
                               "same_across_args")

    def add_output_input_consistent_constraint(self):
        """The producer's chosen output strategy is the column its consumers read."""
        cols, vals, lens, seen = [], [], [], set()
        for s_i, node in enumerate(self.nodes):
            if node.op == "output":
                continue
            bp, ntp, nsp = self._edge_vars(s_i, 0)
            for user in node.users:
                if user.op == "output":
                    continue
                s_j = self.node_map[user]
                argj = [i for i, n in enumerate(user.all_input_nodes) if n == node]
                assert len(argj) == 1
                bc, ntc, nsc = self._edge_vars(s_j, argj[0])
                assert nsc == ntp, f"{node} has {ntp} strategies, {user} arg {argj[0]} reads {nsc}"
                key = (bp, bc, ntp, nsp, ntc)
                if key in seen:
                    continue
                seen.add(key)
                prod = bp + np.arange(ntp)[:, None] * nsp + np.arange(nsp)[None, :]  # row o of producer
                cons = bc + np.arange(ntc)[None, :] * nsc + np.arange(nsc)[:, None]  # column o of consumer
                cols.append(np.concatenate([prod, cons], axis=1).ravel())
                vals.append(np.tile(np.concatenate([np.ones(nsp), -np.ones(ntc)]), ntp))
                lens.append(np.full(ntp, nsp + ntc))
        if cols:
            self.prob.add_rows(np.concatenate(cols), np.concatenate(vals), np.concatenate(lens), 0.0, 0.0,
                               "output_input_consistent")

    def add_inf_cost_constraint(self):
        """Non-finite costs become 10000 and their variable is forced to 0 (the flags come with
        the objective vector: one per variable, set where any entry of the variable is not finite)."""
        self.prob.force_zero(np.nonzero(self.forced_zero_vars)[0])

    def add_choice_link_constraint(self):
        """choice[node, strategy] = sum of the entry variables of that strategy's row of the
        node's first argument; entry variables become continuous."""
        cols, vals, lens, seen = [], [], [], set()
        for s_i, node in enumerate(self.nodes):
            if node.op == "output":
                continue
            b, nt, ns = self._edge_vars(s_i, 0)
            cb = self.node_choice_base[s_i]
            if (b, cb) in seen:
                continue
            seen.add((b, cb))
            entries = b + np.arange(nt)[:, None] * ns + np.arange(ns)[None, :]
            choice = (cb + np.arange(nt))[:, None]
            cols.append(np.concatenate([entries, choice], axis=1).ravel())
            vals.append(np.tile(np.concatenate([np.ones(ns), [-1.0]]), nt))
            lens.append(np.full(nt, ns + 1))
        if cols:
            self.prob.add_rows(np.concatenate(cols), np.concatenate(vals), np.concatenate(lens), 0.0, 0.0,
                               "choice_link")
        self.prob.integrality[:self.n_variables] = 0.0

    def add_compact_constraints(self):
        """The feasible plans of the reference's three structural constraints, written through
        the per-(node, strategy) choice variables y instead of entry variables against entry
        variables:
          * every node takes one strategy: sum_s y[n, s] = 1;
          * every edge's matrix row sums are its consumer's choice:
            sum_ii x[e, ss, ii] = y[consumer, ss]  (unique decision per edge, agreement of a
            node's arguments and the choice link, optimize_sharding.py:402-455, in one family);
          * the columns a consumer reads are its producer's choice:
            sum_ss x[e, ss, o] = y[producer, o]  for exactly the (producer, user, argument
            index) triples the reference couples (optimize_sharding.py:457-520, including its
            use of the user's de-duplicated input list as the argument index).
        Row sums equal to y make the reference's producer-row = consumer-column equation the
        third family, so the feasible set is the same; the rows are shorter (a consistency
        row no longer carries the producer's whole first matrix), about half as many nonzeros,
        and nothing is left for the solver's presolve to discover as redundant."""
        seen = set()
        one_cols, one_lens = [], []
        cols, vals, lens = [], [], []
        # which class of nodes labels the rows / the columns of which block of entry variables
        # (read again by the pruning in front of the solver)
        self._block_sides = sides = {}
        for s_i, node in enumerate(self.nodes):
            if node.op == "output":
                continue
            cb = self.node_choice_base[s_i]
            n = len(self.strats[node].strategies)
            if ("one", cb) not in seen:
                seen.add(("one", cb))
                one_cols.append(cb + np.arange(n))
                one_lens.append(n)
            for argi in range(self.num_args[s_i]):
                b, nt, ns = self._edge_vars(s_i, argi)
                assert nt == n
                if ("row", b, cb) in seen:
                    continue
                seen.add(("row", b, cb))
                sides.setdefault(b, [nt, ns, [], []])[2].append(cb)
                entries = b + np.arange(nt)[:, None] * ns + np.arange(ns)[None, :]
                cols.append(np.concatenate([entries, (cb + np.arange(nt))[:, None]], axis=1).ravel())
                vals.append(np.tile(np.concatenate([np.ones(ns), [-1.0]]), nt))
                lens.append(np.full(nt, ns + 1))
            for user in node.users:
                if user.op == "output":
                    continue
                s_j = self.node_map[user]
                argj = [i for i, x in enumerate(user.all_input_nodes) if x == node]
                assert len(argj) == 1
                bc, ntc, nsc = self._edge_vars(s_j, argj[0])
                assert nsc == n, f"{node} has {n} strategies, {user} arg {argj[0]} reads {nsc}"
                if ("col", bc, cb) in seen:
                    continue
                seen.add(("col", bc, cb))
                sides.setdefault(bc, [ntc, nsc, [], []])[3].append(cb)
                entries = bc + np.arange(ntc)[None, :] * nsc + np.arange(nsc)[:, None]  # column o of the consumer
                cols.append(np.concatenate([entries, (cb + np.arange(nsc))[:, None]], axis=1).ravel())
                vals.append(np.tile(np.concatenate([np.ones(ntc), [-1.0]]), nsc))
                lens.append(np.full(nsc, ntc + 1))
        if one_cols:
            self.prob.add_rows(np.concatenate(one_cols), 1.0, np.asarray(one_lens), 1.0, 1.0, "one_strategy")
        if cols:
            self.prob.add_rows(np.concatenate(cols), np.concatenate(vals), np.concatenate(lens), 0.0, 0.0, "choice_link")
        self.prob.integrality[:self.n_variables] = 0.0

    def add_default_constraints(self):
        if self.node_choice_variables and self.compact_constraints:
            self.add_compact_constraints()
            self.add_inf_cost_constraint()
            return
        if self.node_choice_variables:
            self.add_choice_link_constraint()
        self.add_unique_decision_constraint()
        self.add_same_output_across_args_constraint()
        self.add_output_input_consistent_constraint()
        self.add_inf_cost_constraint()

    # ---- solve (optimize_sharding.py:648-701) ------------------------------------------------
    def get_solution(self, verbose=False):
        # linked entries share a variable: their costs add up (summed where the costs are)
        obj = np.zeros(self.prob.n_vars, np.float64)
        obj[:self.n_variables] = self.objective_vector
        self.prob.objective = obj
        if getattr(self, "_upper_unpruned", None) is not None:  # (a second solve, maybe under more constraints)
            self.prob.upper = self._upper_unpruned.copy()
        self.solve_stats = {"columns": int((self.prob.upper > 0).sum())}
        self._solved_while_pruning = False
        if self.prune_before_solve and self.node_choice_variables:
            self.prune()
        t0 = time.perf_counter()
        if self._solved_while_pruning:  # (the restricted program's optimum, proven to be the program's)
            status = self.prob.status
            solver_s = self.solve_stats["near_bound_solver_s"]
        else:
            status = self.prob.solve(verbose=verbose, time_limit=self.solver_time_limit, mip_rel_gap=self.solver_rel_gap)
            solver_s = time.perf_counter() - t0 + self.solve_stats.get("near_bound_solver_s", 0.0)
        self.solve_stats.update(solver_s=solver_s, solved_by=self.prob.solved_by,
                                columns_solved=getattr(self.prob, "cols_after_fixing", None))
        if status == -1:
            print(self.get_violated_constraints_log())
            raise RuntimeError("Unsolvable problem")
        chosen = self._chosen_entries()
        self.res = self.ds.keys_of_entries(chosen)
        self.res_entries = chosen

        # one strategy pair per (node, argument), one strategy per node (optimize_sharding.py:676-696)
        nodes = self.nodes
        seen = set()
        chosen_strategy = {}
        for s_i, argi, ss, _ in self.res:
            node = nodes[s_i]
            if (s_i, argi) in seen:
                raise RuntimeError(f"Multiple solutions for {node}, key={(s_i, argi)}, solutions: "
                                   f"{[str(self.strats[node].strategies[k[2]]) for k in self.res if k[0] == s_i]}")
            seen.add((s_i, argi))
            first = chosen_strategy.setdefault(node, ss)
            assert first == ss or self.strats[node].strategies[first] == self.strats[node].strategies[ss], \
                f"{node}: arguments chose different strategies {first} and {ss}"
        return {node: self.strats[node].strategies[ss] for node, ss in chosen_strategy.items()}

    # ---- pruning before the solve (no counterpart in the reference, see pruning.py) ----------------
    def _label_graph(self):
        """The program as a pairwise labelling problem over classes of nodes that must take the
        same strategy (linked nodes, and nodes tied through a shared variable block)."""
        from . import pruning

        parent = {}

        def find(x):
            parent.setdefault(x, x)
            while parent[x] != x:
                parent[x] = parent[parent[x]]
                x = parent[x]
            return x

        raw = getattr(self, "_block_sides", None)  # var base -> [nt, ns, row choice bases, column choice bases]
        if raw is None:
            raw = {}
            for s_i, node in enumerate(self.nodes):
                if node.op == "output":
                    continue
                cb = self.node_choice_base[s_i]
                for argi in range(self.num_args[s_i]):
                    b, nt, ns = self._edge_vars(s_i, argi)
                    raw.setdefault(b, [nt, ns, [], []])[2].append(cb)
                for user in node.users:
                    if user.op == "output":
                        continue
                    s_j = self.node_map[user]
                    argj = [i for i, x in enumerate(user.all_input_nodes) if x == node]
                    bc, ntc, nsc = self._edge_vars(s_j, argj[0])
                    raw.setdefault(bc, [ntc, nsc, [], []])[3].append(cb)
        for nt, ns, rows, cols in raw.values():
            for side in (rows, cols):
                for cb in side[1:]:
                    parent[find(cb)] = find(side[0])
        class_id, class_sizes, members = {}, [], []
        size_of = {}  # choice base -> number of strategies
        for nt, ns, rows, cols in raw.values():
            for cb in rows:
                size_of[cb] = nt
            for cb in cols:
                size_of[cb] = ns
        for cb in sorted(size_of):
            root = find(cb)
            if root not in class_id:
                class_id[root] = len(class_sizes)
                class_sizes.append(size_of[cb])
                members.append(set())
            members[class_id[root]].add(cb)
            assert class_sizes[class_id[root]] == size_of[cb], "nodes tied through a block have the same strategies"
        cls = lambda cb: class_id[find(cb)]  # noqa: E731
        blocks = [pruning.Block(b, nt, ns, cls(rows[0]), cls(cols[0]) if cols else -1)
                  for b, (nt, ns, rows, cols) in raw.items()]
        forbidden = self.forced_zero_vars | (self.prob.upper[:self.n_variables] == 0)

        def block_costs(b):
            sl = slice(b.var_begin, b.var_begin + b.nt * b.ns)
            return np.where(forbidden[sl], np.inf, self.objective_vector[sl]).reshape(b.nt, b.ns)

        masks = {}
        for s_i, allowed in self._label_masks.items():
            c = cls(self.node_choice_base[s_i])
            masks[c] = masks.get(c, True) & allowed
        # a linear row over the strategies of several nodes: a strategy whose coefficient cannot be
        # made up for by the best choices of all other nodes is infeasible
        for per_node, lo, hi in self._linear_rows:
            least = math.fsum(min(r) for _, r in per_node)
            most = math.fsum(max(r) for _, r in per_node)
            for s_i, ratios in per_node:
                r = np.asarray(ratios)
                ok = (r - r.min() <= (hi - least) + 1e-9) & (r.max() - r <= (most - lo) + 1e-9)
                c = cls(self.node_choice_base[s_i])
                masks[c] = masks.get(c, True) & ok
        ties = []
        for s_i, s_j, pairs in self._pair_ties:
            ci, cj = cls(self.node_choice_base[s_i]), cls(self.node_choice_base[s_j])
            m = np.zeros((class_sizes[ci], class_sizes[cj]))
            for a, b in pairs:  # strategy a of the parameter goes with strategy b of its gradient, and only with it
                m[a, :] = np.inf
            for a, b in pairs:
                col = np.full(class_sizes[ci], np.inf)
                col[[x for x, y in pairs if y == b]] = 0.0
                m[:, b] = col
            ties.append((ci, cj, m))
        graph = pruning.build_label_graph(blocks, class_sizes, block_costs, masks, ties)
        graph.members = members
        return graph

    def _plan_vector(self, graph, labels):
        """The 0/1 vector of the program for a labelling of the classes."""
        x = np.zeros(self.prob.n_vars, np.float64)
        for c, bases in enumerate(graph.members):
            for cb in bases:
                x[cb + labels[c]] = 1.0
        forbidden = self.forced_zero_vars | (self.prob.upper[:self.n_variables] == 0)
        for b in graph.blocks:
            r = int(labels[b.row_class])
            if b.col_class >= 0:
                col = int(labels[b.col_class])
            else:
                row = slice(b.var_begin + r * b.ns, b.var_begin + (r + 1) * b.ns)
                col = int(np.argmin(np.where(forbidden[row], np.inf, self.objective_vector[row])))
            x[b.var_begin + r * b.ns + col] = 1.0
        return x

    def prune(self):
        """Fixes to zero the variables that the bound proves to be in no optimal plan; where the
        incumbent stays above the bound, solves the program restricted to the variables near the
        bound (``prune_slacks``) and keeps the solution once it is proven optimal."""
        from . import pruning

        t0 = time.perf_counter()
        stats = self.solve_stats
        self._solved_while_pruning = False
        # what an earlier call fixed was decided under the constraints of that call: start again
        # from the bounds of the unpruned program (nothing but pruning changes them after construction)
        if getattr(self, "_upper_unpruned", None) is not None:
            self.prob.upper = self._upper_unpruned.copy()
        self._upper_unpruned = self.prob.upper.copy()
        graph = self._label_graph()
        stats["prune_graph_s"] = time.perf_counter() - t0
        t_sweeps = t_round = 0.0
        if graph.n_classes == 0 or int(np.diff(graph.label_begin).max()) > pruning.MAX_LABELS:
            stats["pruning"] = "skipped"
            return
        theta, unary = graph.theta.copy(), graph.unary.copy()
        best_ub, best_x, sweeps, bound = math.inf, None, 0, -math.inf
        chunks = list(self.prune_sweep_chunks)
        k = 0
        while k < len(chunks):
            chunk = chunks[k]
            k += 1
            t1 = time.perf_counter()
            theta, unary = self.backend.diffusion_sweeps(graph, theta, unary, chunk)
            t_sweeps += time.perf_counter() - t1
            t1 = time.perf_counter()
            sweeps += chunk
            before = bound
            bound = pruning.lower_bound(graph, theta, unary)[0]
            labels = pruning.refine(graph, theta, unary, pruning.decode(graph, theta, unary))
            x = self._plan_vector(graph, labels)
            if (x <= self.prob.upper).all() and not self.prob.violated_constraints(x):
                ub = float(self.prob.objective @ x)
                if ub < best_ub:
                    best_ub, best_x = ub, x
            t_round += time.perf_counter() - t1
            if best_ub - bound <= self.prune_gap * abs(best_ub):
                break
            if k == len(chunks) and bound - before > 0.25 * self.prune_gap * abs(bound):  # the ascent is not through
                more = 2 * chunk if k == len(self.prune_sweep_chunks) else chunk  # (twice the last planned chunk, repeated)
                if sweeps + more <= self.prune_max_sweeps:
                    chunks.append(more)
        stats.update(prune_sweeps_s=t_sweeps, prune_rounding_s=t_round)
        stats.update(prune_sweeps=sweeps, lower_bound=bound, incumbent=best_ub if best_x is not None else None,
                     label_classes=graph.n_classes, label_edges=graph.n_edges)
        if best_x is not None:
            self.incumbent = best_x
            state = (graph, theta, unary)
            if best_ub - bound <= self.prune_gap * abs(best_ub) or not self.prune_slacks:
                self._fix_above(state, best_ub, best_x)
            else:
                self._solve_near_the_bound(state, bound, best_ub, best_x)
        stats["columns_after_pruning"] = int((self.prob.upper > 0).sum())
        stats["prune_s"] = time.perf_counter() - t0

    def _fix_above(self, state, limit, feasible_x=None):
        """Upper bound 0 for every variable whose bound (min-marginal of its strategy / strategy
        pair under the reparametrised costs) exceeds ``limit``."""
        from . import pruning

        graph, theta, unary = state
        dead_label, dead_pair = pruning.prune_masks(graph, theta, unary, limit)
        lb = graph.label_begin
        off = []
        for c, bases in enumerate(graph.members):
            d = np.nonzero(dead_label[lb[c]:lb[c + 1]])[0]
            off.extend(cb + d for cb in bases)
        for b in graph.blocks:
            dead = dead_label[lb[b.row_class]:lb[b.row_class + 1]][:, None] & np.ones((1, b.ns), bool)
            if b.col_class >= 0:
                pair = graph.matrix(dead_pair, b.edge)
                dead = dead | (pair.T if b.transposed else pair)
            off.append(b.var_begin + np.nonzero(dead.ravel())[0])
        off = np.concatenate(off) if off else np.zeros(0, np.int64)
        if feasible_x is not None:
            assert not feasible_x[off].any(), "the incumbent uses a variable the bound rules out"
        self.prob.force_zero(off)

    def _solve_near_the_bound(self, state, bound, best_ub, best_x):
        """Solves the program restricted to the variables whose bound is at most ``bound +
        slack`` for growing slacks.  A plan that uses a variable left out costs more than ``bound
        + slack``, so a restricted optimum of at most that value is an optimum of the full
        program (and no optimal plan was left out).  The last slack is the incumbent's distance,
        where that always holds: the incumbent itself lies inside."""
        stats = self.solve_stats
        upper0 = self.prob.upper.copy()
        tries = []
        t_solver = 0.0
        for rel in tuple(self.prune_slacks) + (math.inf,):
            slack = min(rel * abs(bound), best_ub - bound)
            last = slack >= best_ub - bound
            self.prob.upper = upper0.copy()
            self._fix_above(state, bound + slack, best_x if last else None)
            t1 = time.perf_counter()
            status = self.prob.solve(time_limit=self.solver_time_limit, mip_rel_gap=self.solver_rel_gap)
            dt = time.perf_counter() - t1
            t_solver += dt
            value = self.prob.objective_value if status == 1 else None
            tries.append({"slack": slack, "columns": int(self.prob.cols_after_fixing), "seconds": dt, "value": value,
                          "solved_by": self.prob.solved_by})
            if value is not None and value <= bound + slack:
                self._solved_while_pruning = True
                break
            if value is not None and value < best_ub:  # a better incumbent: the cap of the next slack
                best_ub, best_x = value, self.prob.x.astype(np.float64)
                self.incumbent = best_x
            if last:
                break
        stats["near_bound_solves"] = tries
        stats["near_bound_solver_s"] = t_solver
        if not self._solved_while_pruning:  # (a solver time limit: leave the decision to the full solve)
            self.prob.upper = upper0.copy()
            self._fix_above(state, best_ub, best_x)

    def objective_value(self) -> float:
        return float(self._values("cost", self.res_entries).sum())

    def get_violated_constraints_log(self):
        names = self.prob.violated_constraints()
        return f"Violated constraints: {names}"

    # ---- user constraints (optimize_sharding.py:703-906) ---------------------------------------
    def _add_node_constraint(self, node, output_constraint_indices, constraint_name=None):
        if constraint_name is None:
            constraint_name = "user_constraint"
        s_i = self.node_map[node]
        rows = np.asarray(sorted(output_constraint_indices), np.int64)
        allowed = np.zeros(len(self.strats[node].strategies), bool)
        allowed[rows] = True
        self._label_masks[s_i] = self._label_masks.get(s_i, True) & allowed
        for argi in range(self.num_args[s_i]):
            b, nt, ns = self._edge(s_i, argi)
            idx = (b + rows[:, None] * ns + np.arange(ns)[None, :]).ravel()
            self.prob.add_row(self.vars_of(idx), 1.0, 1.0, 1.0, next_name(constraint_name))

    def add_grad_param_constraints(self):
        """A parameter and its gradient choose the same placement."""
        from torch._functorch._aot_autograd.fx_utils import get_param_and_grad_nodes

        for param, grad in get_param_and_grad_nodes(self.graph).values():
            if grad is None:
                continue
            s_i, s_j = self.node_map[param], self.node_map[grad]
            num_out = self.num_inp_out[(s_i, 0)]["num_output_strat"]
            num_inp_g = self.num_inp_out[(s_j, 0)]["num_input_strat"]
            strat_p = [str(s.output_specs) for s in self.strats[param].strategies]
            assert num_out == len(strat_p)
            strat_gp = [str(s.output_specs) for s in self.strats[grad].strategies]
            bp, _, nsp = self._edge(s_i, 0)
            bg, _, nsg = self._edge(s_j, 0)
            self._pair_ties.append((s_i, s_j, [(oi, strat_gp.index(sp)) for oi, sp in enumerate(strat_p) if sp in strat_gp]))
            for oi in range(num_out):
                sp = strat_p[oi]
                if sp not in strat_gp:
                    continue
                ooi = strat_gp.index(sp)
                g = bg + ooi * nsg + np.arange(num_inp_g)
                cols = np.concatenate([g, [bp + oi * nsp]])
                vals = np.concatenate([np.ones(num_inp_g), [-1.0]])
                self.prob.add_row(self.vars_of(cols), vals, 0.0, 0.0, next_name("grad_param_constraint"))

    def add_parameter_memory_constraint(self, memory_factor_low: float, memory_factor_high: float):
        """Sum over parameters of (local size / global size) stays within [low, high] x #params."""
        from torch._functorch._aot_autograd.fx_utils import get_param_nodes

        world_size = math.prod(self.mesh.shape)
        cols, vals = [], []
        considered = 0
        per_node = []
        for node in get_param_nodes(self.graph):
            s_i = self.node_map[node]
            if node.meta["val"].numel() < world_size:
                continue
            considered += 1
            b, nt, ns = self._edge(s_i, 0)
            ratios = []
            for oi in range(self.num_inp_out[(s_i, 0)]["num_output_strat"]):
                spec: DTensorSpec = self.strats[node].strategies[oi].input_specs[0]
                shape = list(spec.tensor_meta.shape)
                old = math.prod(shape)
                for n, p in zip(self.mesh.shape, spec.placements):
                    if p.is_shard():
                        shape[p.dim] = (shape[p.dim] + n - 1) // n
                cols.append(b + oi * ns)
                ratios.append(math.prod(shape) / old)
            vals.extend(ratios)
            per_node.append((s_i, ratios) if ns == 1 else None)
        cols = self.vars_of(np.asarray(cols, np.int64))
        self.prob.add_row(cols, vals, -np.inf, memory_factor_high * considered, "memory_constraint_high")
        self.prob.add_row(cols, vals, memory_factor_low * considered, np.inf, "memory_constraint_low")
        if all(x is not None for x in per_node):  # (a parameter's only column is its own strategy)
            self._linear_rows.append((per_node, memory_factor_low * considered, memory_factor_high * considered))

    def add_node_constraint(self, node, placement=None, constraint_name=None):
        assert node in self.strats, (node, self.strats.keys())
        if placement is None:
            placement = (Shard(0),) + (Replicate(),) * (self.mesh.ndim - 1)
        wanted = [i for i, s in enumerate(self.strats[node].strategies) if s.output_specs.placements == placement]
        if not wanted:
            raise RuntimeError(f"Couldn't find appropriate constraint {node} {constraint_name} {placement}")
        self._add_node_constraint(node, output_constraint_indices=wanted, constraint_name=constraint_name)

    def add_sharded_input_constraint(self, input_placements: Optional[list[Optional[tuple[Placement, ...]]]] = None):
        from torch._functorch._aot_autograd.descriptors import PlainAOTInput
        from torch._functorch._aot_autograd.fx_utils import get_plain_input_and_grad_nodes

        pending = None if input_placements is None else dict(enumerate(input_placements))
        for desc, (node, grad_node) in get_plain_input_and_grad_nodes(self.graph).items():
            if pending is None:
                placement = None
            else:
                assert isinstance(desc, PlainAOTInput)
                placement = pending.pop(desc.idx)
            self.add_node_constraint(node, placement, constraint_name="input_constraint")
            if grad_node is not None:
                self.add_node_constraint(grad_node, placement, constraint_name="grad_input_constraint")
        ignored = [i for i, p in (pending or {}).items() if p is not None]
        if ignored:
            raise RuntimeError(
                f"We were unable to respect placements for inputs at indices {ignored}.  The traced joint graph has "
                "no dedicated placeholder node for these inputs (typically because inputs alias each other); "
                "remove the explicit placement (use None) or clone the inputs before tracing.")

    def add_sharded_output_constraint(self, output_placements=None):
        from torch._functorch._aot_autograd.descriptors import PlainAOTOutput
        from torch._functorch._aot_autograd.fx_utils import get_plain_output_and_tangent_nodes

        pending = None if output_placements is None else dict(enumerate(output_placements))
        for desc, (node, tangent_node) in get_plain_output_and_tangent_nodes(self.graph).items():
            if pending is None:
                placement = None
            else:
                assert isinstance(desc, PlainAOTOutput)
                placement = pending.pop(desc.idx)
            self.add_node_constraint(node, placement, constraint_name="output_constraint")
            if tangent_node is not None:
                self.add_node_constraint(tangent_node, placement, constraint_name="grad_output_constraint")
        ignored = [i for i, p in (pending or {}).items() if p is not None]
        if ignored:
            raise RuntimeError(
                f"We were unable to respect placements for outputs at indices {ignored}.  The traced joint graph has "
                "no dedicated output node for these outputs (typically because outputs alias each other); "
                "remove the explicit placement (use None) or clone the outputs before returning them.")

    # ---- reporting (optimize_sharding.py:569-646) ------------------------------------------------
    def get_log(self, colored=False):
        from torch.fx.graph import _color_fns, _identity

        opt = {}
        nodes = self.nodes
        for key in self.res:
            opt.setdefault(nodes[key[0]], []).append(self.ds[key])
        code = self.graph.python_code("self", colored=colored).src.strip().split("\n")
        txt_color = _color_fns["blue"] if colored else _identity
        attr_color = _color_fns["red"] if colored else _identity
        l_id = 1
        plc_txt, cost_txt = txt_color("# placement="), txt_color(", cost=")
        for node in nodes:
            if node.op == "output":
                continue
            d = opt[node]
            strat = str(d[0]["full_strat"])
            costs = [(x["comm_cost"], x["compute_cost"], x["sharding_transition_cost"]) for x in d]
            line = f"  {plc_txt}{attr_color(strat)} {cost_txt}{attr_color(str(costs))}"
            if node.op == "placeholder":
                code.insert(l_id, f"    # {node.name}: {line}")
                l_id += 1
                continue
            while not code[l_id].lstrip().startswith(repr(node)):
                l_id += 1
            code[l_id] += line
            l_id += 1
        code = "\n".join(code)
        idx = self.res_entries
        strat_rows = np.asarray([self.encoded.strat_begin[k[0]] + k[2] for k in self.res], np.int64)
        code += f"\ntotal_cost: {self._values('cost', idx).sum():.2f}"
        code += f"\n  comm_cost: {self._values('comm', idx).sum():.2f}"
        code += f"\n  compute_cost: {self.compute_cost_per_arg[strat_rows].sum():.2f}"
        code += f"\n  transition_cost: {self._values('transition', idx).astype(np.float64).sum():.2f}"
        code += "\n" + self.get_violated_constraints_log()
        return code

    def print_costs_for_node(self, node, arg=0, **kwargs):
        """Prints the redistribution-cost matrix of ``node``'s ``arg``-th input edge: a row per
        strategy of ``node``, a column per strategy of the input (optimize_sharding.py:633-646),
        taken from the flat array the kernels filled."""
        from tabulate import tabulate
        from torch.distributed.tensor._op_schema import _pretty_print_spec

        begin, n_rows, n_cols = self._edge(self.node_map[node], arg)
        matrix = self.comm_cost[begin:begin + n_rows * n_cols].reshape(n_rows, n_cols)
        producer = self._all_input_nodes(node)[arg]
        header = [""] + [_pretty_print_spec(s.output_specs) for s in self.strats[producer].strategies]
        body = [[str(s), *matrix[i].tolist()] for i, s in enumerate(self.strats[node].strategies)]
        print(tabulate(body, headers=header, **kwargs))

    # ---- warm-start helpers built on the segmented min kernel -------------------------------------
    def row_minima(self):
        """min / first-argmin over producer strategies for every (edge, consumer strategy)."""
        return self.backend.row_min(self.encoded.tables.row_ptr())

    def edge_minima(self):
        """min / first-argmin (flattened consumer-strategy-major index) of every edge's whole matrix."""
        return self.backend.row_min(self.encoded.tables.edge_entry_begin)

    def greedy_strategies(self):
        """-> ({node: strategy index}, lower bound).  Every node takes the strategy that is
        cheapest when each of its input edges is charged the row minimum of that strategy.
        The choices of neighbouring nodes need not agree, so this is a starting point, not a
        plan; the sum of the per-node minima is a lower bound of every plan's objective (user
        constraints only remove plans).  No counterpart in the reference, which hands the
        table to the solver directly (optimize_sharding.py:648-659)."""
        _, node_min, node_arg = self.backend.greedy(self.encoded.tables.row_ptr())
        # (a node without strategies, the graph's output node, has argmin -1 and adds nothing)
        choice = {node: int(node_arg[i]) for i, node in enumerate(self.encoded.nodes) if node_arg[i] >= 0}
        return choice, math.fsum(m for m, a in zip(node_min.tolist(), node_arg.tolist()) if a >= 0)

    def lower_bound(self) -> float:
        return self.greedy_strategies()[1]

    # ---- structural checks (optimize_sharding.py:908-958) -------------------------------------------
    def validate(self):
        for node in self.graph.nodes:
            if node.op != "call_function":
                continue
            strat0 = self.strats[node].strategies[0]
            inputs = self._all_input_nodes(node)
            n_in = len(inputs)
            assert (len(strat0.redistribute_cost) == n_in) or (n_in == 0 and len(strat0.redistribute_cost) == 1), \
                f"{node}, {len(strat0.redistribute_cost)}, {n_in}"
            ospec = strat0.output_specs
            if isinstance(ospec, (list, tuple)):
                for spec in ospec:
                    if spec:
                        assert spec.tensor_meta is not None, f"{node} doesn't have a tensor_meta"
            elif ospec is not None:
                assert ospec.tensor_meta is not None, f"{node} doesn't have a tensor_meta"
            for ispec in strat0.input_specs:
                if isinstance(ispec, (list, tuple)):
                    for spec in ispec:
                        assert spec.tensor_meta is not None, f"{node} input_spec doesn't have a tensor_meta"
                elif ispec is not None:
                    assert ispec.tensor_meta is not None, f"{node} input_spec doesn't have a tensor_meta"
            for i, arg in enumerate(inputs):
                n_arg = len(self.strats[arg].strategies)
                assert len(strat0.redistribute_cost[i]) == n_arg, f"{node}, {len(strat0.redistribute_cost[i])}, {n_arg}"
