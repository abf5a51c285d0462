"""``dict[Node, OpStrategy]`` -> flattened ``CostTables``.

Walks the strategies in the order ``ShardingOptimizer.build_ds`` does
(autoparallel/optimize_sharding.py:299-379): nodes in graph order (the ``output`` node
skipped), for each node its arguments, for each argument the consumer strategies as matrix
rows and the producer's strategies as columns.  The producer of argument ``argi`` is the
``argi``-th ``fx.Node`` among the flattened ``node.args`` (duplicates kept, kwargs ignored:
:382-387); ``operator.getitem`` consumers read slot ``node.args[1]`` of the producer's
tuple of output specs (:333-334).  Where a producer or consumer spec is not a
``DTensorSpec`` the rule-provided ``redistribute_cost`` value is kept (pass-through).
"""

from __future__ import annotations

import operator
from dataclasses import dataclass, field

import numpy as np
import torch
from torch.distributed.tensor._dtensor_spec import DTensorSpec

from .._native import APC_MAX_RANK
from ..encoding import (EDGE_GRAD_RESCALE, EDGE_NO_PRODUCER, PARTIAL_OPS, CostTables, pack_codes, partial_code,
                        shard_code)


class PlacementCoder:
    """Placement -> one-byte code.  Plain Replicate / Partial(op) / Shard(d) have fixed
    codes; any other Partial or Shard flavour (masked partials, strided shards) is interned
    as a variant so that it compares equal only to itself, as ``Placement.__eq__`` would."""

    def __init__(self):
        self._partial_variants: dict = {}
        self._shard_variants: dict = {}

    def code(self, p) -> int:
        if p.is_replicate():
            return 0
        if p.is_partial():
            op = getattr(p, "reduce_op", "sum")
            if type(p).__name__ == "Partial" and op in PARTIAL_OPS:
                return partial_code(op)
            vid = self._partial_variants.setdefault(repr(p), len(PARTIAL_OPS) + len(self._partial_variants))
            return partial_code(vid)
        if p.is_shard():
            if type(p).__name__ == "Shard":
                return shard_code(p.dim)
            vid = self._shard_variants.setdefault(repr(p), 1 + len(self._shard_variants))
            if vid > 3:
                raise NotImplementedError("more than three distinct non-plain Shard placements in one graph")
            return shard_code(p.dim, vid)
        raise NotImplementedError(f"placement {p!r}")


def all_input_nodes(node) -> list:
    """node.all_input_nodes with duplicates kept, args only (optimize_sharding.py:382-387):
    the Nodes among the leaves of ``tree_flatten(node.args)``, in that order.  (Walked by hand:
    the planner asks this several times per node, and a pytree flatten is ten times the work.)"""
    out: list = []

    def walk(x):
        if isinstance(x, torch.fx.Node):
            out.append(x)
        elif isinstance(x, (tuple, list)):
            for y in x:
                walk(y)
        elif isinstance(x, dict):
            for y in x.values():
                walk(y)

    walk(node.args)
    return out


@dataclass
class EncodedGraph:
    tables: CostTables
    nodes: list  # graph nodes in order (including the output node: s_i indexes this list)
    strat_begin: dict  # s_i -> first row of the strategy table
    edge_of: dict  # (s_i, argi) -> edge row
    edge_keys: list  # edge row -> (s_i, argi)
    num_args: dict  # s_i -> number of arguments
    num_inp_out: dict  # (s_i, argi) -> {"num_input_strat", "num_output_strat"}
    input_spec_row: dict  # (s_i, argi) -> first spec row of that argument's consumer specs
    output_spec_row: dict  # (s_i, slot) -> first spec row of that output slot
    coder: PlacementCoder = field(default_factory=PlacementCoder)


def encode_graph(graph: torch.fx.Graph, strats: dict, mesh_sizes, grad_param_nodes=()) -> EncodedGraph:
    mesh_sizes = tuple(int(x) for x in mesh_sizes)
    M = len(mesh_sizes)
    coder = PlacementCoder()
    nodes = list(graph.nodes)
    grad_param_nodes = set(grad_param_nodes)

    tensor_ids: dict = {}
    t_rank, t_item, t_shape, t_stride = [], [], [], []

    def tensor_row(tm) -> int:
        key = (tuple(tm.shape), tuple(tm.stride), tm.dtype)
        row = tensor_ids.get(key)
        if row is None:
            row = len(t_rank)
            tensor_ids[key] = row
            r = len(tm.shape)
            if r > APC_MAX_RANK:
                raise NotImplementedError(f"tensor rank {r} above {APC_MAX_RANK}")
            t_rank.append(r)
            t_item.append(tm.dtype.itemsize)
            t_shape.append([int(x) for x in tm.shape] + [0] * (APC_MAX_RANK - r))
            t_stride.append([int(x) for x in tm.stride] + [0] * (APC_MAX_RANK - r))
        return row

    spec_codes: list = []
    spec_tensor: list = []
    spec_cache: dict = {}

    def row_of(spec) -> tuple:
        """(placement codes, tensor row) of a spec; (0, -1) for what is not a DTensorSpec"""
        if not isinstance(spec, DTensorSpec):
            return 0, -1
        hit = spec_cache.get(id(spec))
        if hit is None:
            codes = pack_codes([coder.code(p) for p in spec.placements])
            hit = (codes, tensor_row(spec.tensor_meta))
            spec_cache[id(spec)] = hit
        return hit

    def block_of(specs) -> tuple:
        rows = [row_of(spec) for spec in specs]
        return [r[0] for r in rows], [r[1] for r in rows]

    def add_block(block) -> None:
        spec_codes.extend(block[0])
        spec_tensor.extend(block[1])

    # Nodes enumerated from one memo entry (``_apc_origin``) share their OpSpec objects: their
    # spec rows are worked out once and appended per node.
    blocks_of_origin: dict = {}

    def spec_blocks(strategy) -> tuple:
        """-> (one block per output slot, one block per argument) of a node's strategies"""
        origin = getattr(strategy, "_apc_origin", None)
        if origin is not None:
            hit = blocks_of_origin.get(id(origin))
            if hit is not None:
                return hit
        strategies = strategy.strategies
        outs0 = strategies[0].output_specs
        if isinstance(outs0, (list, tuple)):
            outs = [block_of([s.output_specs[slot] for s in strategies]) for slot in range(len(outs0))]
        else:
            outs = [block_of([s.output_specs for s in strategies])]
        ins = [block_of([s.input_specs[argi] for s in strategies]) for argi in range(len(strategies[0].redistribute_cost))]
        if origin is not None:
            blocks_of_origin[id(origin)] = (outs, ins)
        return outs, ins

    strat_begin: dict = {}
    output_spec_row: dict = {}
    input_spec_row: dict = {}
    num_args: dict = {}
    num_inp_out: dict = {}
    n_strat_total = 0
    node_strat_begin = [0]
    strat_num_args: list = []

    # ---- pass 1: strategy rows, output spec rows, consumer input spec rows ------------------
    for s_i, node in enumerate(nodes):
        if node.op == "output":
            node_strat_begin.append(n_strat_total)
            continue
        strategies = strats[node].strategies
        if not strategies:
            raise RuntimeError(f"{node}: no strategy survives the divisibility filter")
        strat_begin[s_i] = n_strat_total
        n_strat_total += len(strategies)
        node_strat_begin.append(n_strat_total)
        na = len(strategies[0].input_specs)
        num_args[s_i] = na
        strat_num_args.extend([na] * len(strategies))
        outs, ins = spec_blocks(strats[node])
        for slot, block in enumerate(outs):
            output_spec_row[(s_i, slot)] = len(spec_codes)
            add_block(block)
        for argi, row in enumerate(strategies[0].redistribute_cost):
            num_inp_out[(s_i, argi)] = {"num_input_strat": len(row), "num_output_strat": len(strategies)}
            input_spec_row[(s_i, argi)] = len(spec_codes)
            add_block(ins[argi])

    node_index = {n: i for i, n in enumerate(nodes)}
    # producer-less pseudo arguments read a block of always-invalid spec rows appended below
    DUMMY = -1
    dummy_rows_needed = 1

    # ---- pass 2: edges -----------------------------------------------------------------------
    e_node, e_arg, e_src_begin, e_n_src, e_tgt_begin, e_n_tgt = [], [], [], [], [], []
    e_flags, e_pt_begin, e_strat_begin = [], [], []
    pt_values: list = []
    edge_of: dict = {}
    edge_keys: list = []
    for s_i, node in enumerate(nodes):
        if node.op == "output":
            continue
        strategies = strats[node].strategies
        inputs = all_input_nodes(node)
        for argi, row0 in enumerate(strategies[0].redistribute_cost):
            n_src, n_tgt = len(row0), len(strategies)
            flags = EDGE_GRAD_RESCALE if node in grad_param_nodes else 0
            needs_pt = False
            if inputs:
                producer = inputs[argi]
                p_i = node_index[producer]
                p_strats = strats[producer].strategies
                if len(p_strats) != n_src:
                    raise RuntimeError(f"{node} arg {argi}: cost row has {n_src} columns, producer {producer} has "
                                       f"{len(p_strats)} strategies")
                p_out0 = p_strats[0].output_specs
                if node.target == operator.getitem:
                    slot = node.args[1]
                    src_begin = output_spec_row[(p_i, slot)]
                elif isinstance(p_out0, (list, tuple)):
                    # a tuple of specs is not a DTensorSpec: every entry keeps the rule's value
                    src_begin, flags, needs_pt = DUMMY, flags | EDGE_NO_PRODUCER, True
                else:
                    src_begin = output_spec_row[(p_i, 0)]
            else:
                src_begin, flags, needs_pt = DUMMY, flags | EDGE_NO_PRODUCER, True
            if src_begin == DUMMY:
                dummy_rows_needed = max(dummy_rows_needed, n_src)
            tgt_begin = input_spec_row[(s_i, argi)]
            if not needs_pt:
                if any(t < 0 for t in spec_tensor[tgt_begin:tgt_begin + n_tgt]) or any(
                        t < 0 for t in spec_tensor[src_begin:src_begin + n_src]):
                    needs_pt = True
            if needs_pt:
                e_pt_begin.append(len(pt_values))
                for s in strategies:
                    r = s.redistribute_cost[argi]
                    if len(r) != n_src:
                        raise RuntimeError(f"{node} arg {argi}: ragged redistribute_cost rows")
                    pt_values.extend(float(v) for v in r)
            else:
                e_pt_begin.append(-1)
            edge_of[(s_i, argi)] = len(e_node)
            edge_keys.append((s_i, argi))
            e_node.append(s_i)
            e_arg.append(argi)
            e_src_begin.append(src_begin)
            e_n_src.append(n_src)
            e_tgt_begin.append(tgt_begin)
            e_n_tgt.append(n_tgt)
            e_flags.append(flags)
            e_strat_begin.append(strat_begin[s_i])
    dummy_begin = len(spec_codes)
    spec_codes.extend([0] * dummy_rows_needed)
    spec_tensor.extend([-1] * dummy_rows_needed)
    e_src_begin = [dummy_begin if b == DUMMY else b for b in e_src_begin]
    per_edge = np.asarray(e_n_src, np.int64) * np.asarray(e_n_tgt, np.int64)
    entry_begin = np.zeros(len(e_node) + 1, np.int64)
    np.cumsum(per_edge, out=entry_begin[1:])

    S = n_strat_total
    tables = CostTables(
        mesh_sizes=mesh_sizes,
        tensor_rank=t_rank, tensor_itemsize=t_item,
        tensor_shape=np.asarray(t_shape, np.int64).reshape(-1, APC_MAX_RANK),
        tensor_stride=np.asarray(t_stride, np.int64).reshape(-1, APC_MAX_RANK),
        spec_codes=np.asarray(spec_codes, np.uint32), spec_tensor=spec_tensor,
        strat_flops=np.zeros(S, np.int64), strat_rw_bytes=np.zeros(S, np.int64), strat_dtype=np.ones(S, np.int8),
        strat_zero_cost=np.ones(S, np.uint8), strat_num_args=strat_num_args,
        node_strat_begin=node_strat_begin,
        edge_node=e_node, edge_arg=e_arg, edge_src_begin=e_src_begin, edge_n_src=e_n_src,
        edge_tgt_begin=e_tgt_begin, edge_n_tgt=e_n_tgt, edge_flags=e_flags, edge_pt_begin=e_pt_begin,
        edge_entry_begin=entry_begin, edge_strat_begin=e_strat_begin, pt_values=pt_values,
    )
    return EncodedGraph(tables=tables, nodes=nodes, strat_begin=strat_begin, edge_of=edge_of, edge_keys=edge_keys,
                        num_args=num_args, num_inp_out=num_inp_out, input_spec_row=input_spec_row,
                        output_spec_row=output_spec_row, coder=coder)
