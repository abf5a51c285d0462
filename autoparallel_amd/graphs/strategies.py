"""Strategy enumeration: for every node of a joint FX graph, the list of DTensor
placement strategies (``OpStrategy``) the planner may choose from on a logical mesh.

This is the step that feeds the cost tables.  It reproduces the behaviour of the
reference's enumeration (autoparallel/optimize_sharding.py:156-209,
autoparallel/utils.py:36-192, autoparallel/propagation_rules.py) on top of torch's
DTensor strategy registry, which is where most per-op strategy functions live:

  placeholder            every {Replicate, Shard(d)}^mesh_ndim placement that divides evenly
  getitem / view / alias / unbind / split_with_sizes
                         whole-rule overrides working on the producer's strategy list
  factories, scalar_tensor, layer_norm fwd/bwd, convert_element_type, sdpa variants,
  reshape, expand, einsum, scatter.src
                         overrides working on an ``OpSchema``
  everything else        the strategy function torch registers for the op; ops without
                         one fall back to an all-Replicate strategy
then, for every call_function: output/input tensor metadata is filled in by running the op
once on the node's fake arguments, strategies that shard a dim unevenly are dropped and
duplicates (same input and output specs) are removed, first occurrence kept.

Transformer layers repeat: results are memoised on (op, the input strategies' output
specs, the non-tensor arguments), and every node with the same key gets its own
``OpStrategy`` around the memo entry's ``OpSpec`` objects (shared read-only;
``StrategyEnumerator.own_specs`` un-shares a node's before anything is written into them).
"""

from __future__ import annotations

import contextlib
import itertools
import logging
import math
import operator
import threading

import torch
from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
from torch.distributed.tensor._op_schema import OpSchema, OpSpec, OpStrategy, RuntimeSchemaInfo, TupleStrategy
from torch.distributed.tensor.placement_types import Placement, Replicate, Shard
from torch.utils._pytree import tree_flatten, tree_map_only

logger = logging.getLogger(__name__)
aten = torch.ops.aten

SHAPE_FACTORY_OPS = (aten.zeros.default, aten.ones.default, aten.full.default, aten.empty.memory_format,
                     aten.rand.default, aten.randn.default)
TENSOR_FACTORY_OPS = SHAPE_FACTORY_OPS + (aten.scalar_tensor.default,)

SDPA_OPS = (aten._scaled_dot_product_efficient_attention.default, aten._scaled_dot_product_flash_attention.default,
            aten._scaled_dot_product_flash_attention_backward.default,
            aten._scaled_dot_product_efficient_attention_backward.default)


def _registry():
    from torch.distributed.tensor import DTensor

    return DTensor._op_dispatcher.sharding_propagator


_COST_STUB_LOCK = threading.RLock()


@contextlib.contextmanager
def _cheap_placeholder_costs(enabled: bool):
    """torch's strategy functions fill ``redistribute_cost`` rows by calling its own
    redistribute_cost for every (producer strategy, input spec) pair.  The planner
    recomputes every such entry with its own model (and keeps a rule-provided value only where
    a side is not a DTensorSpec, which torch's function never sees), so during enumeration the
    call can be a constant.  The name is a module attribute of torch, so the stub is process-wide
    while it is in: one enumeration at a time holds it (a lock), and it is taken out again on
    any exit.  ``StrategyEnumerator(cheap_costs=False)`` leaves torch's function alone; the
    tables are the same either way (tests/test_traced_graphs.py)."""
    if not enabled:
        yield
        return
    import torch.distributed.tensor._ops.utils as ops_utils

    with _COST_STUB_LOCK:
        saved = ops_utils.redistribute_cost
        ops_utils.redistribute_cost = lambda current_spec, target_spec: 0.0
        try:
            yield
        finally:
            ops_utils.redistribute_cost = saved


def _tensor_meta(t) -> TensorMeta:
    return TensorMeta(t.shape, t.stride(), t.dtype)


def _meta_tensor(tm: TensorMeta):
    return torch.empty_strided(tm.shape, tm.stride, dtype=tm.dtype, device="meta")


def _zero_row(strategy: OpStrategy) -> list:
    return [0.0] * len(strategy.strategies)


def drop_uneven_shardings(strategy: OpStrategy, mesh) -> OpStrategy:
    """Keeps a strategy only if every Shard of every input and output spec divides its
    tensor dim evenly, mesh dim after mesh dim (propagation_rules.py:104-135)."""
    kept = []
    for s in strategy.strategies:
        out = s.output_specs
        if isinstance(out, DTensorSpec):
            out = [out]
        if s.input_specs is not None:
            specs = list(s.input_specs) + (list(out) if out is not None else [])
        else:
            specs = list(out)
        ok = True
        for spec in specs:
            if spec is None:
                continue
            shape = list(spec.tensor_meta.shape)
            for n, p in zip(mesh.shape, spec.placements):
                if p.is_shard():
                    if shape[p.dim] % n == 0:
                        shape[p.dim] //= n
                    else:
                        ok = False
                        break
        if ok:
            kept.append(s)
    return OpStrategy(kept)


def drop_duplicate_strategies(strategy: OpStrategy) -> OpStrategy:
    """First occurrence of each (input specs, output specs) pair (utils.py:132-151)."""
    seen = set()
    kept = []
    for s in strategy.strategies:
        ins, outs = s.input_specs, s.output_specs
        ins = tuple(ins) if isinstance(ins, list) else ins
        outs = tuple(outs) if isinstance(outs, list) else outs
        try:
            key = (ins, outs)
            if key in seen:
                continue
            seen.add(key)
        except TypeError:
            pass
        kept.append(s)
    return OpStrategy(kept)


def all_placements(mesh, tensor_meta: TensorMeta) -> OpStrategy:
    """{Replicate, Shard(0..rank-1)} per mesh dim in itertools.product order, uneven ones
    dropped; each strategy has itself as its single input spec and a [[0.0]] cost row
    (propagation_rules.py:161-178)."""
    options = [Replicate()] + [Shard(d) for d in range(len(tensor_meta.shape))]
    out = []
    for placements in itertools.product(options, repeat=mesh.ndim):
        spec = DTensorSpec(mesh, placements, tensor_meta=tensor_meta)
        out.append(OpSpec(spec, input_specs=[spec], redistribute_cost=[[0.0]]))
    return drop_uneven_shardings(OpStrategy(out), mesh)


class StrategyEnumerator:
    def __init__(self, mesh, memoize: bool = True, cheap_costs: bool = True):
        self.mesh = mesh
        self.memoize = memoize
        self.cheap_costs = cheap_costs
        self.registry = _registry()
        self._sig_ids: dict = {}
        self._memo: dict = {}
        self.stats = {"nodes": 0, "memo_hits": 0, "implicit_replicate": set()}
        self._whole_rules = {
            operator.getitem: self._getitem,
            aten.view.default: self._view,
            aten.alias.default: self._alias,
            aten.unbind.int: self._unbind,
            aten.split_with_sizes.default: self._split_with_sizes,
            torch.ops.prims.iota.default: self._needs_hardening,
            aten.randperm.default: self._needs_hardening,
        }
        self._schema_rules = {
            aten.scalar_tensor.default: self._scalar_tensor,
            aten.native_layer_norm.default: self._layer_norm,
            aten.native_layer_norm_backward.default: self._layer_norm_backward,
            torch.ops.prims.convert_element_type.default: self._single_input,
            aten.split.Tensor: self._split_tensor,
            aten._unsafe_index.Tensor: self._needs_hardening,
            aten.index.Tensor: self._needs_hardening,
            aten.reshape.default: self._reshape,
            aten.expand.default: self._expand,
            aten.einsum.default: self._einsum,
            aten.scatter.src: self._scatter_src,
        }
        for op in SHAPE_FACTORY_OPS:
            self._schema_rules[op] = self._factory
        for op in SDPA_OPS:
            self._schema_rules[op] = self._sdpa

    # ------------------------------------------------------------------------------------
    # whole-graph walk (optimize_sharding.py:156-209)
    # ------------------------------------------------------------------------------------
    def enumerate(self, graph: torch.fx.Graph) -> dict:
        strats: dict = {}
        with _cheap_placeholder_costs(self.cheap_costs):
            for node in graph.nodes:
                self.stats["nodes"] += 1
                if node.op == "placeholder":
                    val = node.meta["val"]
                    strats[node] = self._placeholder(val)
                elif node.op == "call_function":
                    if node.meta.get("local_map_kwargs"):
                        strats[node] = self._local_map(node, strats)
                    else:
                        strats[node] = self._call_function(node, strats)
                elif node.op == "output":
                    strats[node] = tree_map_only(torch.fx.Node, lambda x: strats[x], node.args)
                else:
                    raise ValueError(f"unsupported node kind {node.op}")
        return strats

    # ------------------------------------------------------------------------------------
    def _local_map(self, node, strats) -> OpStrategy:
        """A ``local_map`` region (forward or backward call of the higher-order op) has exactly
        one strategy: the placements its author declared (optimize_sharding.py:174-196,
        utils.py:195-313).  Leading arguments beyond the declared ones are activations saved
        by the forward call and are replicated, as are outputs beyond the declared ones;
        ``None`` / SymInt slots carry no spec.  The cost rows are placeholders: the cost
        kernels recompute every entry from the specs."""
        kw = node.meta["local_map_kwargs"]
        if kw.get("in_placements") is None or kw.get("out_placements") is None:
            raise NotImplementedError(f"{node}: local_map regions need in_placements and out_placements")
        if kw.get("in_grad_placements") is not None:
            raise NotImplementedError(f"{node}: local_map in_grad_placements are not supported")
        if kw.get("device_mesh") not in (self.mesh, None):
            raise NotImplementedError(f"{node}: local_map region declared on another device mesh")
        if node.kwargs:
            raise NotImplementedError(f"{node}: keyword arguments of a local_map call")
        mesh = self.mesh
        replicated = tuple(Replicate() for _ in range(mesh.ndim))

        def spec_of(example, placements):
            if example is None or placements is None or not isinstance(example, torch.Tensor):
                return None
            if isinstance(placements, Placement):
                placements = (placements,)
            return DTensorSpec(mesh=mesh, placements=tuple(placements), tensor_meta=_tensor_meta(example))

        args = [a.meta["val"] if isinstance(a, torch.fx.Node) else a for a in node.args]
        in_placements = list(kw["in_placements"])
        n_saved = len(args) - len(in_placements)
        if n_saved < 0:
            raise RuntimeError(f"{node}: {len(in_placements)} input placements for {len(args)} arguments")
        in_specs = [spec_of(a, replicated) for a in args[:n_saved]]
        in_specs += [spec_of(a, p) for a, p in zip(args[n_saved:], in_placements)]
        val = node.meta["val"]
        outs = list(val) if isinstance(val, (list, tuple)) else [val]
        out_placements = list(kw["out_placements"])
        out_specs = [spec_of(o, p) for o, p in zip(outs, out_placements)]
        out_specs += [spec_of(o, replicated) for o in outs[len(out_placements):]]
        rows = []
        for a in node.args:
            producer = strats[a] if isinstance(a, torch.fx.Node) else None
            rows.append(_zero_row(producer) if isinstance(producer, OpStrategy) else [0.0])
        return OpStrategy([OpSpec(tuple(out_specs), input_specs=tuple(in_specs), redistribute_cost=rows)])

    def _signature(self, strategy) -> int:
        """A small integer naming the list of output specs of an OpStrategy."""
        if isinstance(strategy, OpStrategy):
            key = tuple(tuple(s.output_specs) if isinstance(s.output_specs, (list, tuple)) else s.output_specs
                        for s in strategy.strategies)
        else:
            key = ("const", repr(strategy))
        return self._sig_ids.setdefault(key, len(self._sig_ids))

    def _arg_key(self, x, strats):
        if isinstance(x, torch.fx.Node):
            val = x.meta.get("val")
            meta = (tuple(val.shape), tuple(val.stride()), val.dtype) if isinstance(val, torch.Tensor) else repr(val)
            s = strats[x]
            sig = getattr(s, "_apc_sig", None)
            if sig is None:
                origin = getattr(s, "_apc_origin", None)  # (the same list for every node of the memo entry)
                sig = getattr(origin, "_apc_sig", None) if origin is not None else None
                if sig is None:
                    sig = self._signature(s)
                    if origin is not None:
                        origin._apc_sig = sig
                s._apc_sig = sig
            return ("node", sig, meta)
        if isinstance(x, (list, tuple)):
            return (type(x).__name__,) + tuple(self._arg_key(y, strats) for y in x)
        if isinstance(x, dict):
            return ("dict",) + tuple((k, self._arg_key(v, strats)) for k, v in x.items())
        return ("const", repr(x))

    @staticmethod
    def _fresh_copy(strategy: OpStrategy) -> OpStrategy:
        """The node's own OpStrategy around the memo's OpSpec objects, which every node with
        the same key shares read-only (a planner that writes costs into
        ``OpSpec.redistribute_cost`` un-shares them first: ``own_specs``).  ``_apc_origin``
        names the memo entry, so that later passes (output signature, clustering key, spec
        encoding) do per distinct strategy list what they would otherwise do per node."""
        out = OpStrategy(list(strategy.strategies))
        out._apc_origin = strategy
        return out

    @staticmethod
    def own_specs(strategy: OpStrategy) -> None:
        """Replaces the shared OpSpec objects of a node's OpStrategy by copies of its own (with
        their own ``redistribute_cost`` lists)."""
        if getattr(strategy, "_apc_origin", None) is None:
            return
        strategy.strategies = [
            OpSpec(s.output_specs, input_specs=s.input_specs,
                   redistribute_cost=None if s.redistribute_cost is None else list(s.redistribute_cost))
            for s in strategy.strategies]
        strategy._apc_origin = None

    def _placeholder(self, val) -> OpStrategy:
        key = ("placeholder", tuple(val.shape), tuple(val.stride()), val.dtype)
        if self.memoize and key in self._memo:
            self.stats["memo_hits"] += 1
            return self._fresh_copy(self._memo[key])
        out = all_placements(self.mesh, _tensor_meta(val))
        if self.memoize:
            self._memo[key] = out
            return self._fresh_copy(out)
        return out

    def _call_function(self, node, strats) -> OpStrategy:
        key = None
        if self.memoize:
            key = (node.target, self._arg_key(node.args, strats), self._arg_key(node.kwargs, strats))
            hit = self._memo.get(key)
            if hit is not None:
                self.stats["memo_hits"] += 1
                return self._fresh_copy(hit)
        user_strats = tree_map_only(torch.fx.Node, lambda x: strats[x], node.args)
        user_args = tree_map_only(torch.fx.Node, lambda x: x.meta["val"], node.args)
        user_kwargs = tree_map_only(torch.fx.Node, lambda x: x.meta["val"], node.kwargs)
        out = self.placement_options(node.target, user_strats, user_args, user_kwargs)
        if self.memoize:
            self._memo[key] = out
            return self._fresh_copy(out)
        return out

    # ------------------------------------------------------------------------------------
    # one op (utils.py:154-192)
    # ------------------------------------------------------------------------------------
    def placement_options(self, op, specs, user_args, user_kwargs) -> OpStrategy:
        assert len(specs) == len(user_args)
        mesh = self.mesh
        if op in self._whole_rules:
            out = self._whole_rules[op](specs)
            return drop_duplicate_strategies(drop_uneven_shardings(out, mesh))

        schema_args = []
        needs_pytree = False
        for spec in specs:
            if isinstance(spec, list) and len(spec) > 0 and any(isinstance(x, OpStrategy) for x in spec):
                schema_args.append(TupleStrategy(spec))
                needs_pytree = True
            else:
                schema_args.append(spec)
        schema = OpSchema(op, tuple(schema_args), {}, RuntimeSchemaInfo(needs_pytree=needs_pytree))
        if op in self._schema_rules:
            out = self._schema_rules[op](schema)
        else:
            out = self._registered(op, schema)
        self._fill_tensor_meta(op, user_args, user_kwargs, out)
        self._fill_missing_costs(op, specs, out)
        return drop_duplicate_strategies(drop_uneven_shardings(out, mesh))

    def _registered(self, op, schema) -> OpStrategy:
        """torch's own strategy function; ops without one are planned all-Replicate
        (dtensor_util/utils.py:208-229)."""
        funcs = self.registry.op_strategy_funcs
        if op in funcs:
            return funcs[op](schema)
        from torch.distributed.tensor._ops.utils import replicate_op_strategy

        if op not in self.stats["implicit_replicate"]:
            self.stats["implicit_replicate"].add(op)
            logger.warning("no sharding strategy registered for %s: planning it replicated", op)
        return replicate_op_strategy(schema)

    def _fill_tensor_meta(self, op, user_args, user_kwargs, out: OpStrategy) -> None:
        """utils.py:36-109: run the op once on the fake arguments and attach the resulting
        metadata to the output specs (None outputs that are tensors become Replicate) and
        the arguments' metadata to input specs that lack it."""
        result = op(*user_args, **user_kwargs)
        if isinstance(result, torch.Tensor):
            out_meta = _tensor_meta(result)
        else:
            out_meta = tree_map_only(torch.Tensor, _tensor_meta, result)
        arg_metas = tuple(_tensor_meta(x) for x in tree_flatten(user_args)[0] if isinstance(x, torch.Tensor))
        for s in out.strategies:
            if isinstance(out_meta, TensorMeta):
                s.output_spec.tensor_meta = out_meta
            else:
                mesh = s.mesh
                filled = []
                for spec, tm in zip(s.output_specs, out_meta):
                    if spec is None and isinstance(tm, TensorMeta):
                        spec = DTensorSpec(mesh=mesh, placements=(Replicate(),) * mesh.ndim)
                    filled.append(spec)
                s.output_specs = tuple(filled)
                for spec, tm in zip(s.output_specs, out_meta):
                    if spec is not None and spec.tensor_meta != tm:
                        if spec.tensor_meta is None:
                            spec.tensor_meta = tm
                        else:
                            assert tm is None
            if s.input_specs is None:
                allowed = {torch.ops.prims.convert_element_type.default, aten.clone.default, aten.slice.Tensor}
                assert op in allowed, f"{op}: strategy without input_specs"
                s.input_specs = (s.output_specs,)
                assert s.redistribute_cost is None
            if op in TENSOR_FACTORY_OPS:
                assert len(arg_metas) == 0 and len(s.input_specs) == 1, op
            else:
                assert len(arg_metas) == len(s.input_specs), f"{op}: {len(arg_metas)} tensors, {len(s.input_specs)} specs"
            for tm, spec in zip(arg_metas, s.input_specs):
                if spec.tensor_meta is None:
                    spec.tensor_meta = tm

    def _fill_missing_costs(self, op, specs, out: OpStrategy) -> None:
        """utils.py:112-129."""
        for s in out.strategies:
            if s.redistribute_cost is None:
                allowed = {aten.ones_like.default, aten.full_like.default, aten.empty_like.default,
                           torch.ops.prims.convert_element_type.default, aten.slice.Tensor}
                assert op in allowed, f"{op}: strategy without redistribute_cost"
                s.redistribute_cost = [_zero_row(specs[0])]

    # ------------------------------------------------------------------------------------
    # whole rules (propagation_rules.py:186-343)
    # ------------------------------------------------------------------------------------
    def _getitem(self, specs) -> OpStrategy:
        producer, index = specs[0], specs[1]
        out = []
        for s in producer.strategies:
            picked = s.output_specs[index]
            spec = OpSpec(picked, input_specs=(picked,))
            spec.redistribute_cost = [_zero_row(producer)]
            out.append(spec)
        return OpStrategy(out)

    def _view(self, specs) -> OpStrategy:
        from torch.distributed.tensor._ops._view_ops import dim_maps, propagate_shape_and_sharding

        producer, shape = specs[0], specs[1]
        rules = dim_maps[torch.Tensor.view](producer, shape)
        global_shape = producer.shape
        in_meta = producer.strategies[0].output_specs.tensor_meta
        out_meta = _tensor_meta(aten.view.default(_meta_tensor(in_meta), shape))
        out = []
        for s in producer.strategies:
            src = s.output_specs
            in_placements, out_placements = propagate_shape_and_sharding(
                src.placements, global_shape, rules, self.mesh.shape, strict_view=False)
            in_spec = DTensorSpec(mesh=self.mesh, placements=tuple(in_placements), tensor_meta=src.tensor_meta)
            out_spec = DTensorSpec(mesh=self.mesh, placements=tuple(out_placements), tensor_meta=out_meta)
            out.append(OpSpec(out_spec, input_specs=(in_spec,), redistribute_cost=[_zero_row(producer)]))
        return OpStrategy(out)

    def _alias(self, specs) -> OpStrategy:
        producer = specs[0]
        tm = producer.strategies[0].output_specs.tensor_meta
        out = []
        for s in all_placements(self.mesh, tm).strategies:
            spec = OpSpec(s.output_specs, input_specs=(s.output_specs,))
            spec.redistribute_cost = [_zero_row(producer)]
            out.append(spec)
        return OpStrategy(out)

    def _split_like(self, producer, dim, split):
        banned = {i for i, s in enumerate(producer.strategies)
                  if any(p.is_shard(dim) or p.is_partial() for p in s.output_spec.placements)}
        out = []
        for s in producer.strategies:
            src = s.output_spec
            if any(p.is_shard(dim) or p.is_partial() for p in src.placements):
                continue
            pieces = split(_meta_tensor(src.tensor_meta))
            outs = tuple(DTensorSpec(self.mesh, src.placements, tensor_meta=_tensor_meta(t)) for t in pieces)
            row = _zero_row(producer)
            for b in banned:
                row[b] = math.inf
            spec = OpSpec(outs, input_specs=(src,))
            spec.redistribute_cost = [row]
            out.append(spec)
        return OpStrategy(out)

    def _unbind(self, specs) -> OpStrategy:
        dim = specs[1]
        return self._split_like(specs[0], dim, lambda t: t.unbind(dim))

    def _split_with_sizes(self, specs) -> OpStrategy:
        sizes = specs[1]
        dim = specs[2] if len(specs) > 2 else 0
        return self._split_like(specs[0], dim, lambda t: t.split(sizes, dim))

    def _needs_hardening(self, *_):
        raise NotImplementedError("Needs hardening, only tested on a few cases")

    # ------------------------------------------------------------------------------------
    # schema rules (propagation_rules.py:385-874)
    # ------------------------------------------------------------------------------------
    def _scalar_tensor(self, schema) -> OpStrategy:
        dtype = torch.get_default_dtype()
        if len(schema.args_schema) >= 2 and schema.args_schema[1] is not None:
            dtype = schema.args_schema[1]
        spec = DTensorSpec(self.mesh, (Replicate(),) * self.mesh.ndim, tensor_meta=TensorMeta((), (), dtype))
        return OpStrategy([OpSpec(output_specs=spec, input_specs=[spec], redistribute_cost=[[0.0]])])

    def _factory(self, schema) -> OpStrategy:
        from torch.distributed.tensor._ops.utils import is_tensor_shardable

        shape = schema.args_schema[0]
        assert isinstance(shape, (torch.Size, list))
        stride = torch.empty(shape, device="meta").stride()
        dtype = torch.get_default_dtype()
        if len(schema.args_schema) >= 3:
            dtype = schema.args_schema[2]
            assert isinstance(dtype, torch.dtype), dtype
        # Replicate last: listing the sharded options first nudges the solver towards them
        per_dim = [Shard(i) for i in range(len(shape))] + [Replicate()]
        combos = list(itertools.product(per_dim, repeat=self.mesh.ndim))
        out = []
        for placements in combos:
            spec = DTensorSpec(self.mesh, tuple(placements))
            spec.tensor_meta = TensorMeta(shape, stride, dtype)
            if not is_tensor_shardable(shape, spec):
                continue
            out.append(OpSpec(output_specs=spec, input_specs=[spec], redistribute_cost=[[0.0] * len(combos)]))
        return OpStrategy(out)

    def _norm_axis(self, input_strategy, normalized_shape):
        from torch.distributed.tensor._ops._math_ops import normalize_to_torch_size

        return input_strategy.ndim - len(normalize_to_torch_size(normalized_shape))

    def _layer_norm(self, schema) -> OpStrategy:
        from torch.distributed.tensor._ops._math_ops import normalize_to_torch_size
        from torch.distributed.tensor._ops._pointwise_ops import pointwise_strategy

        assert len(schema.args_schema) == 5
        input_strategy, normalized_shape = schema.args_schema[0], schema.args_schema[1]
        n_norm = len(normalize_to_torch_size(normalized_shape))
        axis = input_strategy.ndim - n_norm
        kept = []
        for s in pointwise_strategy(schema, linearity=False).strategies:
            if any(p.is_shard() and p.dim >= axis for p in s.input_specs[0].placements):
                continue  # would need a reduction over a sharded dim
            out_spec, in_spec = s.output_specs, s.input_specs[0]
            out_spec.tensor_meta = in_spec.tensor_meta
            stat_shape = in_spec.tensor_meta.shape[:axis] + (1,) * n_norm
            stat_meta = _tensor_meta(torch.empty(stat_shape, dtype=torch.float32, device="meta"))
            stat = DTensorSpec(mesh=s.mesh, placements=out_spec.placements, tensor_meta=stat_meta)
            s.output_specs = (out_spec, stat, stat)
            kept.append(s)
        return OpStrategy(kept)

    def _layer_norm_backward(self, schema) -> OpStrategy:
        from torch.distributed.tensor._ops._pointwise_ops import pointwise_strategy

        assert len(schema.args_schema) == 8
        input_strategy, normalized_shape = schema.args_schema[1], schema.args_schema[2]
        axis = self._norm_axis(input_strategy, normalized_shape)
        kept = []
        for s in pointwise_strategy(schema, linearity=False).strategies:
            in_spec = s.input_specs[1]
            if any(p.is_shard() and p.dim >= axis for p in in_spec.placements):
                continue
            grad_in = DTensorSpec(mesh=s.mesh, placements=s.output_specs.placements, tensor_meta=in_spec.tensor_meta)
            w, b = s.input_specs[4], s.input_specs[5]
            s.output_specs = (grad_in,
                              DTensorSpec(mesh=s.mesh, placements=w.placements, tensor_meta=w.tensor_meta),
                              DTensorSpec(mesh=s.mesh, placements=b.placements, tensor_meta=b.tensor_meta))
            kept.append(s)
        return OpStrategy(kept)

    def _single_input(self, schema) -> OpStrategy:
        from torch.distributed.tensor._ops._tensor_ops import propagate_single_input_strategy

        return propagate_single_input_strategy(schema)

    def _split_tensor(self, schema) -> OpStrategy:
        """propagation_rules.py:649-671.  The reference applies torch's per-spec split rule (in
        the torch it pins; the function is gone from current torch, so what it did is restated
        here) to every strategy of the producer: a producer with a Partial placement is not
        supported, one sharded on the split dim yields no strategy (the old rule asked for a
        redistribution instead), any other keeps its placements on every piece.  A kept
        strategy accepts only the producer strategy it came from (cost 0, all others inf)."""
        args = schema.args_schema
        producer, size = args[0], args[1]
        dim = args[2] if len(args) > 2 else 0
        out = []
        for i, s in enumerate(producer.strategies):
            src = s.output_spec
            if any(p.is_partial() for p in src.placements):
                raise NotImplementedError(f"splitting distributed tensor with Partial placement is not implemented: {src}")
            d = dim + src.ndim if dim < 0 else dim
            if any(p.is_shard(d) for p in src.placements):
                continue
            n = src.tensor_meta.shape[d]
            pieces = len(size) if isinstance(size, (list, tuple)) else max(-(-n // size), 1)
            outs = tuple(DTensorSpec(self.mesh, src.placements) for _ in range(pieces))
            spec = OpSpec(outs, input_specs=(src,))
            row = [math.inf] * len(producer.strategies)
            row[i] = 0.0
            spec.redistribute_cost = [row]
            out.append(spec)
        return OpStrategy(out)

    def _sdpa(self, schema) -> OpStrategy:
        out = self._registered(schema.op, schema)
        # drop context-parallel strategies (sequence dim of the first operand sharded)
        out.strategies = [s for s in out.strategies if Shard(2) not in s.input_specs[0].placements]
        return out

    def _reshape(self, schema) -> OpStrategy:
        out = self._registered(aten.reshape.default, schema)
        if self.mesh.ndim == 1 and len(out.strategies) > 2 and str(out.strategies[2]) == str(out.strategies[0]):
            out.strategies.pop(2)
        return out

    def _expand(self, schema_) -> OpStrategy:
        import copy

        from torch._subclasses.fake_tensor import unset_fake_temporarily

        op = aten.expand.default
        with unset_fake_temporarily():
            schema = copy.deepcopy(schema_)
        input_strategy = schema.args_schema[0]
        src_shape = input_strategy.strategies[0].output_specs.tensor_meta.shape
        dst_shape = schema.args_schema[1]
        expanded = [i for i, (a, b) in enumerate(zip(src_shape, dst_shape)) if a == 1 and b != a]
        if len(expanded) != 1:
            assert len(expanded) == 0
            return self._registered(op, schema)
        dim = expanded[0]
        hidden = [i for i, s in enumerate(input_strategy.strategies)
                  if any(p.is_shard(dim) for p in s.output_spec.placements)]
        for i in reversed(hidden):
            input_strategy.strategies.pop(i)
        out = self._registered(op, schema)
        for s in out.strategies:
            for i in hidden:
                s.redistribute_cost[0].insert(i, math.inf)
        return out

    def _einsum(self, schema) -> OpStrategy:
        from torch.distributed.tensor._ops._matrix_ops import _mm_like_strategy

        equation, operands = schema.args_schema
        assert isinstance(equation, str) and isinstance(operands, TupleStrategy)
        assert len(operands.children) == 2, "only two-operand einsum is supported"
        a, b = operands.children
        return _mm_like_strategy(equation, self.mesh, OpSchema(aten.einsum.default, (a, b), {}))

    def _scatter_src(self, schema) -> OpStrategy:
        from torch.distributed.tensor._ops._tensor_ops import expand_to_full_mesh_op_strategy, normalize_dim

        input_strategy, dim, index_strategy = schema.args_schema[0], schema.args_schema[1], schema.args_schema[2]
        assert isinstance(input_strategy, OpStrategy) and isinstance(index_strategy, OpStrategy)
        dim = normalize_dim(dim, input_strategy.ndim)
        in_shape, idx_shape = input_strategy.shape, index_strategy.shape
        # placements of [output, input, index, src]
        options = [[Replicate()] * 4]
        if len(in_shape) == len(idx_shape):
            for d in range(len(in_shape)):
                if d != dim and in_shape[d] == idx_shape[d]:
                    options.append([Shard(d)] * 4)
        return expand_to_full_mesh_op_strategy(input_strategy.mesh, schema, options, input_index=1)


def enumerate_strategies(gm: torch.fx.GraphModule, mesh, memoize: bool = True, cheap_costs: bool = True):
    en = StrategyEnumerator(mesh, memoize=memoize, cheap_costs=cheap_costs)
    return en.enumerate(gm.graph), en
