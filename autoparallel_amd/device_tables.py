"""Device-resident cost tables: uploads a ``CostTables`` encoding to HBM once and
runs the HIP kernels of libapcost.so over it through the operators of the torch layer
(``torch.ops.apcost``, csrc/apcost_torch.cpp: tensors in, tensors out, argument checks,
current stream and device guard on the C++ side).

torch is used for device memory and streams only; every computation is a kernel of the
library.  Without a HIP device (or without the built libraries) construction raises: there
is no CPU path.

Every method that allocates, launches or copies runs on the package's device thread
(``_device_thread``), where no dispatch mode of the caller (a graph capture's fake-tensor
mode) is active; the launchers of ``prepare_step`` enqueue from whichever thread calls them.
"""

from __future__ import annotations

import numpy as np
import torch

from . import _native
from ._device_thread import on_device_thread as _guarded
from .cost_model import CostModelParams
from .encoding import CostTables

_UPLOAD = (
    "tensor_rank", "tensor_itemsize", "tensor_shape", "tensor_stride", "spec_codes", "spec_tensor",
    "strat_flops", "strat_rw_bytes", "strat_dtype", "strat_zero_cost", "strat_num_args",
    "edge_src_begin", "edge_n_src", "edge_tgt_begin", "edge_n_tgt", "edge_flags", "edge_pt_begin",
    "edge_entry_begin", "edge_strat_begin", "pt_values", "tile_records", "dup_entry_begin",
    "dup_row_begin",
)


def _to_device(a: np.ndarray, device) -> torch.Tensor:
    if a.dtype == np.uint32:  # same bits; torch's uint32 support is partial
        a = a.view(np.int32)
    if a.dtype.names is not None:  # packed records travel as raw int32 words
        a = np.ascontiguousarray(a).view(np.int32).reshape(len(a), a.dtype.itemsize // 4)
    if a.size == 0:
        return torch.empty(a.shape, dtype=torch.from_numpy(np.zeros(1, a.dtype)).dtype, device=device)
    return torch.from_numpy(a).to(device, non_blocking=False)


_TORCH_DTYPE = {np.int32: torch.int32, np.int64: torch.int64, np.uint8: torch.uint8, np.float64: torch.float64,
                np.int8: torch.int8, np.uint32: torch.int32}


class DeviceCostTables:
    @_guarded
    def __init__(self, tables: CostTables, params: CostModelParams, device="cuda:0", validate=True):
        if not torch.cuda.is_available():
            raise RuntimeError("DeviceCostTables needs a HIP device; there is no CPU path")
        self.ops = _native.torch_ops()
        self.tables = tables
        self.params = params
        self.device = torch.device(device)
        if validate:
            tables.validate(params)
        self.c_params = params.to_c()
        self.p = _native.params_tensor(self.c_params)  # struct apc_params as the operators take it
        with torch.cuda.device(self.device):
            self.d = {k: _to_device(getattr(tables, k), self.device) for k in _UPLOAD}
        self.tensor_bytes = None
        self.tensor_contiguous = None
        self.compute_cost = None
        self.compute_cost_per_arg = None
        self.comm = None
        self.transition = None
        self.cost = None
        self.row_min = None  # minima / first argmins of the rows of ``cost``, when a table launch took them
        self.row_argmin = None

    @_guarded
    def refresh(self, *names):
        """Re-uploads host tables that changed after construction (strategy inputs filled in
        from the shard-shape table, tiles rebuilt with de-duplication)."""
        with torch.cuda.device(self.device):
            for k in names:
                self.d[k] = _to_device(getattr(self.tables, k), self.device)

    # ---- helpers -------------------------------------------------------------------------
    def _empty(self, shape, dtype):
        return torch.empty(shape, dtype=dtype, device=self.device)

    # (for the entry points of the C ABI that have no operator: raw pointers and the stream handle)
    @property
    def lib(self):
        return _native.lib()

    def _stream(self):
        return _native.vp(torch.cuda.current_stream(self.device).cuda_stream)

    def _p(self, key):
        t = self.d[key] if isinstance(key, str) else key
        return _native.vp(t.data_ptr() if t is not None and t.numel() else 0)

    def _tensor_table(self):
        d = self.d
        return d["tensor_rank"], d["tensor_itemsize"], d["tensor_shape"], d["tensor_stride"]

    def _strategy_table(self):
        d = self.d
        return d["strat_flops"], d["strat_rw_bytes"], d["strat_dtype"], d["strat_zero_cost"], d["strat_num_args"]

    # ---- integer tables ------------------------------------------------------------------
    @_guarded
    def run_tensor_tables(self):
        self.tensor_bytes, self.tensor_contiguous = self.ops.tensor_tables(*self._tensor_table())
        return self.tensor_bytes, self.tensor_contiguous

    @_guarded
    def run_spec_tables(self):
        width = self.tables.shape_width()  # rows as wide as the largest rank needs, not APC_MAX_RANK
        names = ("num_shards", "local_shape", "local_stride", "local_numel", "local_bytes")
        out = dict(zip(names, self.ops.shard_shapes_bytes(self.p, self.d["spec_codes"], self.d["spec_tensor"],
                                                          *self._tensor_table(), width)))
        self.spec_out = out
        return out

    # ---- per-strategy flop / byte counts -----------------------------------------------------
    @_guarded
    def run_strategy_inputs(self, recipes):
        """Flop and byte counts of every (node, strategy) from the spec table and the per-node
        ``recipes`` (``graphs.cost_inputs.StrategyRecipes``), on the device; the strategy table
        of later launches reads the results where they are.  -> (flops, rw_bytes, dtype_code,
        zero_cost) device tensors."""
        tb = self.tables
        spec = getattr(self, "spec_out", None) or self.run_spec_tables()
        n_nodes = tb.n_nodes
        for name in ("node_kind", "node_dtype", "node_const_bytes"):
            if len(getattr(recipes, name)) != n_nodes:
                raise ValueError(f"recipes.{name} must have one row per node")
        # every row a recipe names, plus the node's strategies, lies inside the spec table; the
        # tensors of a flop formula have the rank it reads
        n_strat = np.diff(tb.node_strat_begin).astype(np.int64)
        per_node = np.repeat(n_strat, np.diff(recipes.node_row_begin))
        if len(recipes.byte_rows) and int((recipes.byte_rows.astype(np.int64) + per_node).max()) > tb.n_specs:
            raise ValueError("a recipe's spec rows run past the spec table")
        with_formula = recipes.node_kind >= 2
        if with_formula.any():
            if int((recipes.node_flop_rows[with_formula].astype(np.int64).max(axis=1) + n_strat[with_formula]).max()) > tb.n_specs:
                raise ValueError("a flop formula's spec rows run past the spec table")
            need = 4 if (recipes.node_kind >= 4).any() else 3 if (recipes.node_kind == 3).any() else 2
            if spec["local_shape"].shape[1] < need:
                raise ValueError("the spec table's shape rows are narrower than a flop formula's tensors")
        strat_node = _to_device(np.repeat(np.arange(n_nodes, dtype=np.int32), n_strat), self.device)
        up = {k: _to_device(np.ascontiguousarray(getattr(recipes, k)), self.device) for k in (
            "node_kind", "node_dtype", "node_const_bytes", "node_row_begin", "byte_rows", "node_flop_rows")}
        node_strat_begin = _to_device(np.ascontiguousarray(tb.node_strat_begin, np.int64), self.device)
        out = self.ops.strategy_inputs(strat_node, node_strat_begin, up["node_kind"], up["node_dtype"], up["node_const_bytes"],
                                       up["node_row_begin"], up["byte_rows"], up["node_flop_rows"].reshape(-1),
                                       spec["local_shape"], spec["local_bytes"])
        for key, t in zip(("strat_flops", "strat_rw_bytes", "strat_dtype", "strat_zero_cost"), out):
            self.d[key] = t
        return out

    # ---- per-strategy compute cost ---------------------------------------------------------
    @_guarded
    def run_compute_costs(self):
        self.compute_cost, self.compute_cost_per_arg, err = self.ops.compute_cost(self.p, *self._strategy_table())
        if int(err.item()) != 0:
            # compute_estimation.py:198-201
            raise ValueError(f"a strategy with non-zero flops uses a dtype not supported on {self.params.device_name}")
        return self.compute_cost, self.compute_cost_per_arg

    # ---- redistribution-cost matrices ------------------------------------------------------
    @_guarded
    def alloc_outputs(self, comm=True, transition=True, cost=True):
        n = self.tables.n_entries
        self.comm = self._empty((n,), torch.float64) if comm else None
        self.transition = self._empty((n,), torch.uint8) if transition else None
        self.cost = self._empty((n,), torch.float64) if cost else None

    def _bind_redistribute_tables(self, comm, transition, cost, rows=None):
        """A bound launch of the table kernel over the tables already built, writing the given
        per-entry arrays (None: not written) and, with ``rows = (edge_row_begin, row_min,
        row_argmin)``, the row minima."""
        d = self.d
        erb, rmin, rarg = rows if rows is not None else (None, None, None)
        return self.ops.bind_redistribute_tables(
            self.p, self.tensor_bytes, self.tensor_contiguous, d["spec_codes"], d["spec_tensor"], d["pt_values"],
            self.compute_cost_per_arg, d["tile_records"], d["dup_entry_begin"], self.tables.n_entries, comm, transition, cost,
            erb, d["dup_row_begin"] if rows is not None else None, rmin, rarg)

    @_guarded
    def launch_redistribute_tables(self, row_min=False):
        """One enqueue of the table kernel over pre-allocated outputs.  ``row_min``: the launch
        also writes ``row_min`` / ``row_argmin`` (allocated by ``run_redistribute_tables``)."""
        rows = None
        if row_min:
            rows = (_to_device(self.tables.edge_row_begin(), self.device), self.row_min, self.row_argmin)
        self._bind_redistribute_tables(self.comm, self.transition, self.cost, rows).run()

    @_guarded
    def run_redistribute_tables(self, comm=True, transition=True, cost=True, row_min=None):
        """``row_min``: also take the row minima of ``cost`` in the same launch (``None``: when all
        three outputs are wanted and ``row_min_in_tiles_pays``)."""
        if self.tensor_bytes is None:
            self.run_tensor_tables()
        if cost and self.compute_cost_per_arg is None:
            self.run_compute_costs()
        self.alloc_outputs(comm, transition, cost)
        if row_min is None:
            row_min = self.row_min_in_tiles_pays()
        if row_min:
            self.tables.validate_row_minima()  # raises when some matrix row is spread over tiles
        self.row_min = self.row_argmin = None
        if row_min:
            n_rows = self.tables.n_rows
            self.row_min = self._empty((n_rows,), torch.float64)
            self.row_argmin = self._empty((n_rows,), torch.int32)
        self.launch_redistribute_tables(row_min=bool(row_min))
        return self.comm, self.transition, self.cost

    @_guarded
    def build_all(self):
        """tensor tables -> compute costs -> cost matrices, all on the current stream."""
        self.run_tensor_tables()
        self.run_compute_costs()
        return self.run_redistribute_tables()

    # ---- one full device-side pass with pre-bound arguments -------------------------------------
    # A pass over a table this small is bound by the ramp-up and drain of every launch, and
    # one launch for all tables wins (Llama-3-8B on a (32, 8) mesh, 78 MB: 25 us against 30 us
    # per pass); above it the tiles' own derivation of what they would otherwise read costs
    # more than a launch (measured crossover between 90 MB and 170 MB of tables).
    ONE_LAUNCH_MAX_BYTES = 128 << 20

    def row_min_in_tiles_pays(self) -> bool:
        """Whether the launch that writes the cost matrices should take the row minima itself.
        Inside the tiles the minima cost about 0.5 ns per tile (a barrier and the stores of the
        row results) plus 1.6 ps per entry a tile computes (identical edges are computed, and
        reduced, once for all their copies); a ``segmented_min`` launch costs about 4 us plus
        reading every stored entry back at about 4.5 TB/s.  Measured, in tiles / separate:
        Llama-3-8B on (32, 8), whose tiles compute an eighth of the entries they store, 18.8 /
        23.9 us per pass with all three arrays written; the 464 M-entry stress table, where every
        entry is computed, 2.42 ms for the launch that writes the cost alone with the minima
        against 1.45 ms without them plus 0.87 ms for the separate launch."""
        tb = self.tables
        if tb.n_tiles == 0 or not tb.rows_fit_tiles():
            return False
        computed = int((tb.tile_row_count.astype(np.int64) * tb.tile_col_count.astype(np.int64)).sum())
        return 0.5e-3 * tb.n_tiles + 1.6e-6 * computed < 4.0 + 8.0 * tb.n_entries / 4.5e6

    def _alloc_input_tables(self, spec_table: bool):
        """Allocates (does not fill) the outputs of the tensor, compute-cost and, when wanted,
        spec tables."""
        tb = self.tables
        self.tensor_bytes = self._empty((tb.n_tensors,), torch.int64)
        self.tensor_contiguous = self._empty((tb.n_tensors,), torch.uint8)
        self.compute_cost = self._empty((tb.n_strategies,), torch.float64)
        self.compute_cost_per_arg = self._empty((tb.n_strategies,), torch.float64)
        if not spec_table:
            return None
        n, width = tb.n_specs, tb.shape_width()
        self.spec_out = {
            "num_shards": self._empty((n,), torch.int64),
            "local_shape": self._empty((n, width), torch.int64),
            "local_stride": self._empty((n, width), torch.int64),
            "local_numel": self._empty((n,), torch.int64),
            "local_bytes": self._empty((n,), torch.int64),
        }
        return self.spec_out

    def pass_bytes(self, outputs=("comm", "transition", "cost"), spec_table=True, row_min_in_tiles=False) -> int:
        """Bytes a pass with these outputs must move at minimum (what its launches write, plus
        the spec lists and edge headers the tiles read)."""
        tb = self.tables
        total = tb.algorithmic_bytes(comm="comm" in outputs, transition="transition" in outputs, cost="cost" in outputs)
        total += tb.algorithmic_bytes_input_tables(spec_table=spec_table)
        if row_min_in_tiles:
            total += 12 * tb.n_rows
        return total

    # A table up to this many entries is bound by the latency of one workgroup: its planner pass
    # runs over packed tiles (every wavefront on its own, one round of loads, no LDS staging).
    # Above, the per-entry arithmetic of that kernel (direct evaluation) costs more than the
    # staging it saves.
    PACKED_MAX_ENTRIES = 4_000_000

    def packed_pass_pays(self) -> bool:
        tb = self.tables
        return tb.n_entries <= self.PACKED_MAX_ENTRIES and tb.packable()

    def _packed_tiles(self):
        """The device copy of ``CostTables.pack_tiles()`` (checked against the tables by the
        library's host-side validator), made once per tiling."""
        cached = getattr(self, "_packed_cache", None)
        if cached is not None and cached[0] is self.tables.tile_records:
            return cached[1]
        packed = self.tables.pack_tiles()
        self.tables.validate_packed(packed)
        with torch.cuda.device(self.device):
            dev = _to_device(packed, self.device)
        self._packed_cache = (self.tables.tile_records, dev)
        return dev

    @_guarded
    def prepare_step(self, row_min=True, fused_inputs=False, one_launch=None, row_min_in_tiles=None,
                     outputs=("comm", "transition", "cost"), spec_table=True, packed=None):
        """Allocates every output once and returns ``{kernel name: zero-argument launcher}``
        in launch order.  A launcher only enqueues (no allocation, no synchronisation), so a
        timed loop measures the kernels and not Python argument marshalling.  With
        ``fused_inputs`` the tensor, spec and compute-cost tables are one launch
        (``input_tables``) instead of three; with ``one_launch`` they and the cost matrices
        are one (``build_tables``); ``one_launch=None`` takes one launch for tables up to
        ``ONE_LAUNCH_MAX_BYTES`` when ``fused_inputs`` is set.  ``row_min_in_tiles``: the launch
        that writes the cost matrices takes the row minima too (no ``segmented_min`` launch, no
        second read of the matrices); it needs every row inside one tile
        (``CostTables.rows_fit_tiles``), and ``None`` takes it when ``row_min_in_tiles_pays``.
        ``outputs``: which of the per-entry arrays the pass writes; ``spec_table=False`` leaves
        the local shard shapes out (a planner has computed them before it could fill in the
        flop / byte counts this pass reads).  ``packed``: the one launch runs over packed tiles
        (``apc_build_tables_packed``: the assembled cost and the row minima, no spec table);
        ``None`` takes them when the pass is of that kind and ``packed_pass_pays``."""
        outputs = tuple(outputs)
        if not outputs or any(o not in ("comm", "transition", "cost") for o in outputs):
            raise ValueError(f"outputs must name some of comm, transition, cost: {outputs}")
        if not spec_table and not fused_inputs:
            raise ValueError("a pass without the spec table is built with fused_inputs")
        fits = self.tables.rows_fit_tiles()
        if row_min_in_tiles is None:
            row_min_in_tiles = self.row_min_in_tiles_pays()
        row_min_in_tiles = bool(row_min_in_tiles) and bool(row_min)
        if row_min_in_tiles and not fits:
            raise ValueError("row minima inside the table launch need every matrix row inside one tile")
        if row_min and not row_min_in_tiles and "cost" not in outputs:
            raise ValueError("a segmented_min launch over the rows reads the cost array: ask for it")
        total = self.pass_bytes(outputs, spec_table, row_min_in_tiles)
        if one_launch is None:
            one_launch = bool(fused_inputs) and total <= self.ONE_LAUNCH_MAX_BYTES
        packed_kind = bool(one_launch) and row_min_in_tiles and outputs == ("cost",) and not spec_table
        if packed is None:
            packed = packed_kind and self.packed_pass_pays()
        elif packed and not (packed_kind and self.tables.packable()):
            raise ValueError("a pass over packed tiles is one launch that writes the assembled cost and the row minima, "
                             "without the spec table, over tiles of whole rows")
        spec = self._alloc_input_tables(spec_table)
        self.alloc_outputs("comm" in outputs, "transition" in outputs, "cost" in outputs)
        self.row_min = self.row_argmin = None
        ops, d, tb = self.ops, self.d, self.tables
        err = torch.zeros((1,), dtype=torch.int32, device=self.device)
        self._step_keepalive = [err, spec]
        spec_outputs = [spec[k] for k in ("num_shards", "local_shape", "local_stride", "local_numel", "local_bytes")] \
            if spec_table else []
        width = spec["local_shape"].shape[1] if spec_table else tb.shape_width()
        input_tables = (self.p, *self._tensor_table(), self.tensor_bytes, self.tensor_contiguous, d["spec_codes"],
                        d["spec_tensor"], spec_outputs, width, *self._strategy_table(), self.compute_cost,
                        self.compute_cost_per_arg, err)

        def bind(bound):
            # a launcher only looks up the current stream (or takes the given one) and enqueues
            run, run_on = bound.run, bound.run_on

            def launch(on_stream=None):
                if on_stream is None:
                    run()
                else:
                    run_on(int(on_stream.cuda_stream))
            launch.bound = bound
            return launch

        rows = None
        if row_min:
            self.row_min = self._empty((tb.n_rows,), torch.float64)
            self.row_argmin = self._empty((tb.n_rows,), torch.int32)
        if row_min_in_tiles:
            rows = (_to_device(tb.edge_row_begin(), self.device), self.row_min, self.row_argmin)
        erb, rmin, rarg = rows if rows is not None else (None, None, None)
        dup_rows = d["dup_row_begin"] if rows is not None else None
        if packed:
            step = {"build_tables_packed": bind(ops.bind_cost_tables_packed(
                self.p, *self._tensor_table(), self.tensor_bytes, self.tensor_contiguous, *self._strategy_table(),
                self.compute_cost, self.compute_cost_per_arg, err, d["pt_values"], self._packed_tiles(), tb.n_entries, tb.n_rows,
                self.cost, self.row_min, self.row_argmin))}
        elif one_launch:
            step = {"build_tables": bind(ops.bind_cost_tables(
                *input_tables, d["pt_values"], d["tile_records"], d["dup_entry_begin"], tb.n_entries, self.comm,
                self.transition, self.cost, erb, dup_rows, rmin, rarg))}
        elif fused_inputs:
            step = {"input_tables": bind(ops.bind_input_tables(*input_tables))}
        else:
            step = {
                "tensor_tables": bind(ops.bind_tensor_tables(*self._tensor_table(), self.tensor_bytes,
                                                             self.tensor_contiguous)),
                "spec_tables": bind(ops.bind_spec_tables(self.p, d["spec_codes"], d["spec_tensor"],
                                                         *self._tensor_table(), spec_outputs, width)),
                "compute_costs": bind(ops.bind_compute_costs(self.p, *self._strategy_table(), self.compute_cost,
                                                             self.compute_cost_per_arg, err)),
            }
        if not one_launch and not packed:
            step["redistribute_tables"] = bind(self._bind_redistribute_tables(self.comm, self.transition, self.cost, rows))
        if row_min and not row_min_in_tiles:
            row_ptr = torch.from_numpy(tb.row_ptr()).to(self.device)
            assert row_ptr.numel() - 1 == self.row_min.numel()
            copies = self._row_copies()
            if copies is not None:  # identical edges: every distinct row is read once, its minimum stored to all
                selected, copy_ptr, copy_rows, n_read = copies
                step["segmented_min"] = bind(ops.bind_segmented_min(self.cost, row_ptr, selected, copy_ptr, copy_rows,
                                                                    n_read, self.row_min, self.row_argmin))
            else:
                step["segmented_min"] = bind(ops.bind_segmented_min(self.cost, row_ptr, None, None, None, 0,
                                                                    self.row_min, self.row_argmin))
        self._step_error_flag = err
        return step

    # ---- the planner's table build -------------------------------------------------------------
    PLANNER_OUTPUTS = ("cost",)

    def planner_pass(self, packed=None):
        """The launches ``ShardingOptimizer.build_ds`` issues once the flop / byte counts are in
        the strategy table (optimize_sharding.py:270-380 in one pass): the tensor and
        compute-cost tables and the assembled cost of every entry, the array the ILP objective
        is summed from, in one launch for tables up to ``ONE_LAUNCH_MAX_BYTES`` (else the input
        tables, then the matrices); the launch also takes the row minima when that is cheaper
        than reading the matrices back (``row_min_in_tiles_pays``), otherwise they are taken
        when asked for.  The spec table is not part of it (the planner needed the local shard
        shapes before it could count flops); ``comm`` and ``transition`` are written only when a
        report asks (``fetch``)."""
        return self.prepare_step(row_min=self.row_min_in_tiles_pays(), fused_inputs=True,
                                 outputs=self.PLANNER_OUTPUTS, spec_table=False, packed=packed)

    @_guarded
    def check_error_flag(self):
        """After a synchronisation: raises if a strategy with flops had an unsupported dtype."""
        err = getattr(self, "_step_error_flag", None)
        if err is not None and int(err.item()) != 0:
            # compute_estimation.py:198-201
            raise ValueError(f"a strategy with non-zero flops uses a dtype not supported on {self.params.device_name}")

    @_guarded
    def fetch(self, name: str) -> torch.Tensor:
        """The device array ``comm`` / ``transition`` / ``cost``; one that the pass did not write
        is computed now by a launch of the table kernel with that output alone (same values:
        the kernel evaluates an entry the same way whichever arrays it stores)."""
        have = {"comm": self.comm, "transition": self.transition, "cost": self.cost}
        if name not in have:
            raise KeyError(name)
        if have[name] is not None:
            return have[name]
        if self.tensor_bytes is None or self.compute_cost_per_arg is None:
            raise RuntimeError("no table pass has run yet")
        n = self.tables.n_entries
        out = self._empty((n,), torch.uint8 if name == "transition" else torch.float64)
        self._bind_redistribute_tables(*(out if k == name else None for k in have)).run()
        setattr(self, name, out)
        return out

    @_guarded
    def cost_objective(self, n_vars: int, group_var_begin, group_member_begin, member_entry_begin):
        """-> (objective f64[n_vars], forced_zero u8[n_vars]) on the device: the ILP objective
        summed from ``cost`` (``apc_cost_objective``).  The index arrays are host arrays."""
        gv = _to_device(np.ascontiguousarray(group_var_begin, np.int64), self.device)
        gm = _to_device(np.ascontiguousarray(group_member_begin, np.int64), self.device)
        me = _to_device(np.ascontiguousarray(member_entry_begin, np.int64), self.device)
        n_groups = len(group_var_begin) - 1
        if n_groups < 0 or len(group_member_begin) != n_groups + 1:
            raise ValueError("group_var_begin and group_member_begin must have n_groups + 1 rows")
        if n_groups and (int(group_var_begin[0]) != 0 or int(group_var_begin[-1]) != n_vars
                         or int(group_member_begin[-1]) != len(member_entry_begin)):
            raise ValueError("group pointers do not span the variables / members")
        if n_groups and not bool((np.diff(np.asarray(group_var_begin, np.int64)) > 0).all()):
            raise ValueError("every variable group needs at least one variable (the kernel takes one workgroup per group)")
        return self.ops.cost_objective(int(n_vars), gv, gm, me, self.fetch("cost"), float(self.params.inf_replacement_cost))

    @_guarded
    def capture_step_graph(self, step):
        """Records one pass (the launchers of ``prepare_step``) into a HIP graph: one launch per
        pass, and the three kernels that only read the uploaded tables (tensor, spec and
        compute-cost tables) sit on parallel branches, so they overlap on the device instead
        of queueing behind each other.  Returns the ``torch.cuda.CUDAGraph``; ``replay()``
        enqueues the pass on the current stream.  For callers that want a single launch per
        pass; it is not the fast way to loop over passes: on the Llama-3-8B table a replay was
        measured at 61 us against 39 us for the five plain launches in stream order (the
        runtime's per-node replay cost exceeds what the overlap saves), and equal on tables
        large enough to be bandwidth-bound."""
        graph = torch.cuda.CUDAGraph()
        branches = [torch.cuda.Stream(device=self.device) for _ in range(2)]  # default priority
        with torch.cuda.graph(graph):
            main = torch.cuda.current_stream()
            for b in branches:
                b.wait_stream(main)
            if "build_tables" in step:
                step["build_tables"](main)
            elif "input_tables" in step:
                step["input_tables"](main)
            else:
                step["spec_tables"](main)
                step["tensor_tables"](branches[0])
                step["compute_costs"](branches[1])
            for b in branches:
                main.wait_stream(b)
            if "redistribute_tables" in step:
                step["redistribute_tables"](main)
            if "segmented_min" in step:
                step["segmented_min"](main)
        self._step_keepalive.append(branches)
        return graph

    # ---- segmented min ---------------------------------------------------------------------
    def _row_copies(self):
        """Device arrays of ``CostTables.row_copies()`` when reading only the distinct rows saves
        at least a quarter of the matrix bytes, else None."""
        tb = self.tables
        if tb.dup_entry_begin is None or len(tb.dup_entry_begin) == 0:
            return None
        cached = getattr(self, "_row_copies_cache", None)
        if cached is not None and cached[0] is tb.tile_records:  # (a new tiling packs new records)
            return cached[1]
        selected, copy_ptr, copy_rows, n_read = tb.row_copies()
        out = None
        if n_read <= 0.75 * tb.n_entries:
            out = (_to_device(selected, self.device), _to_device(copy_ptr, self.device),
                   _to_device(copy_rows, self.device), n_read)
        self._row_copies_cache = (tb.tile_records, out)
        return out

    @_guarded
    def row_minima(self):
        """(min, first argmin) of every matrix row of ``cost``: what the table launch already took,
        else a segmented minimum that reads every distinct row once."""
        if self.row_min is not None:
            return self.row_min, self.row_argmin
        tb = self.tables
        copies = self._row_copies()
        row_ptr = _to_device(tb.row_ptr(), self.device)
        if copies is None:
            return self.segmented_min(self.fetch("cost"), row_ptr, check=False)
        selected, copy_ptr, copy_rows, n_read = copies
        n_rows = row_ptr.numel() - 1
        mins = self._empty((n_rows,), torch.float64)
        args = self._empty((n_rows,), torch.int32)
        self.ops.bind_segmented_min(self.fetch("cost"), row_ptr, selected, copy_ptr, copy_rows, n_read, mins, args).run()
        return mins, args  # (the index arrays stay cached with the tables)

    @_guarded
    def segmented_min(self, values: torch.Tensor, seg_ptr, check: bool = True):
        if not isinstance(seg_ptr, torch.Tensor):
            seg_ptr = torch.from_numpy(np.ascontiguousarray(seg_ptr, dtype=np.int64)).to(self.device)
        if values.dtype != torch.float64 or seg_ptr.dtype != torch.int64:
            raise TypeError("segmented_min takes float64 values and an int64 segment pointer")
        if not (values.is_contiguous() and seg_ptr.is_contiguous()):
            raise ValueError("segmented_min takes contiguous arrays")
        n_seg = seg_ptr.numel() - 1
        if n_seg < 0:
            raise ValueError("seg_ptr must have at least one element")
        if check and n_seg > 0:
            # the kernel trusts the pointer array: keep it inside the value array
            ok = bool((seg_ptr[1:] >= seg_ptr[:-1]).all()) and int(seg_ptr[0]) >= 0 and int(seg_ptr[-1]) <= values.numel()
            if not ok:
                raise ValueError("seg_ptr must be non-decreasing and end within the value array")
        return self.ops.segmented_min(values, seg_ptr)

    # ---- dual ascent over the planning program's labelling form ---------------------------------
    @_guarded
    def diffusion_sweeps(self, graph, theta: np.ndarray, unary: np.ndarray, n_sweeps: int):
        """``n_sweeps`` sweeps of min-sum diffusion (``apc_diffusion_sweeps``) over ``graph``
        (``pruning.LabelGraph``) starting from the host arrays ``theta`` / ``unary``; returns the
        updated pair as new host arrays (read-only: handed back to the next call unchanged, they
        are not uploaded again).  The graph's index arrays are uploaded once, as one buffer."""
        cached = getattr(self, "_diffusion_graph", None)
        if cached is None or cached[0] is not graph:
            names = ("color_nodes", "label_begin", "inc_begin", "inc_edge", "inc_side", "edge_begin", "edge_i", "edge_j")
            # one host buffer, one copy: every array at a 16-byte boundary, viewed with its own dtype on the device
            arrays = {k: np.ascontiguousarray(getattr(graph, k)) for k in names}
            offsets, size = {}, 0
            for k, a in arrays.items():
                offsets[k] = size
                size += -(-a.nbytes // 16) * 16
            packed = np.zeros(max(size, 16), np.uint8)
            for k, a in arrays.items():
                packed[offsets[k]:offsets[k] + a.nbytes] = a.view(np.uint8).reshape(-1)
            on_device = torch.from_numpy(packed).to(self.device)
            views = {k: on_device[offsets[k]:offsets[k] + a.nbytes].view(_TORCH_DTYPE[a.dtype.type]) for k, a in arrays.items()}
            cached = (graph, views, on_device)
            self._diffusion_graph = cached
            self._diffusion_state = None
        d = cached[1]
        state = getattr(self, "_diffusion_state", None)
        if state is not None and state[0] is theta and state[1] is unary:
            th, un = state[2], state[3]  # what the last call left on the device, returned as these very arrays
        else:
            th = torch.from_numpy(np.ascontiguousarray(theta, np.float64)).to(self.device)
            un = torch.from_numpy(np.ascontiguousarray(unary, np.float64)).to(self.device)
        color_begin = torch.from_numpy(np.ascontiguousarray(graph.color_begin, np.int64))
        max_labels = int(np.diff(graph.label_begin).max()) if graph.n_classes else 0
        self.ops.diffusion_sweeps_(int(n_sweeps), color_begin, d["color_nodes"], d["label_begin"], d["inc_begin"],
                                   d["inc_edge"], d["inc_side"], d["edge_begin"], d["edge_i"], d["edge_j"], max_labels,
                                   int(graph.label_begin[-1]), int(graph.edge_begin[-1]), th, un)
        theta_out, unary_out = th.cpu().numpy(), un.cpu().numpy()
        theta_out.setflags(write=False)
        unary_out.setflags(write=False)
        self._diffusion_state = (theta_out, unary_out, th, un)
        return theta_out, unary_out

    @_guarded
    def strategy_bounds(self, row_min: torch.Tensor) -> torch.Tensor:
        """Per-(node, strategy) sum of the row minima of the node's edges (``row_min`` in the
        order of ``CostTables.row_ptr()``)."""
        t = self.tables
        if row_min.dtype != torch.float64 or not row_min.is_contiguous():
            raise TypeError("strategy_bounds takes a contiguous float64 array of row minima")
        if row_min.numel() != t.n_rows:
            raise ValueError("row_min must hold one value per matrix row")
        if getattr(self, "_bound_index", None) is None:
            self._bound_index = {k: _to_device(v, self.device) for k, v in t.strategy_bound_index().items()}
            self._bound_index["node_strat_begin"] = _to_device(np.ascontiguousarray(t.node_strat_begin, np.int64), self.device)
        ix = self._bound_index
        return self.ops.strategy_bounds(ix["strat_node"], ix["node_strat_begin"], ix["node_edge_begin"], ix["edges_by_node"],
                                        ix["edge_row_begin"], row_min)

    @_guarded
    def greedy_strategies(self, row_min: torch.Tensor):
        """-> (bound per strategy, min per node, argmin per node): the cheapest strategy of every
        node when each of its edges is charged its row minimum."""
        bound = self.strategy_bounds(row_min)
        node_min, node_arg = self.segmented_min(bound, self._bound_index["node_strat_begin"], check=False)
        return bound, node_min, node_arg
