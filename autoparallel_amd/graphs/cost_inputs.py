"""Per-(node, strategy) flop and byte counts: the integer inputs of the compute-cost
kernel.

The reference obtains them by running each op on fake tensors of the *local shard* shape
under ``FlopCounterMode`` and summing the element bytes of all tensor arguments and
outputs (autoparallel/compute_estimation.py:232-299, 334-349).  Output sizes are therefore
whatever the op's own shape function yields, which has no closed form across ops.  Here
the local shard shapes and strides come from the device's integer kernel (one row per
spec); this module only runs the op's shape function once per *distinct* (op, local
shapes, strides, dtypes, other arguments) combination and fills the flattened strategy
table.  Nodes the reference costs at zero (non call_function, non-OpOverload targets such
as getitem, views: compute_estimation.py:279-291) never reach the shape function.
"""

from __future__ import annotations

import math

import numpy as np
import torch
from torch.utils._pytree import tree_flatten
from torch.utils.flop_counter import FlopCounterMode

from ..cost_model import DTYPE_CODES

UNSUPPORTED_DTYPE_CODE = 7


def einsum_flop(equation, tensors, out=None, **kwargs) -> int:
    """The flop count the reference registers for ``aten.einsum`` (compute_estimation.py:16-40): two
    operands; [b, m, k] x [k, n] counts b m n k 2, two rank-3 operands [b, m, k] x [b, m, k2] (the
    weight-gradient form) count (b m) k k2 2; any other pair of ranks is an error.  The equation
    string itself is not read."""
    assert len(tensors) == 2
    a_shape, b_shape = [x.shape for x in tensors]
    if len(a_shape) == 3 and len(b_shape) == 3:
        b, m, k = a_shape
        b1, n, k2 = b_shape
        assert b == b1
        assert m == n
        return (b * m) * k * k2 * 2
    if len(a_shape) == 3 and len(b_shape) == 2:
        b, m, k = a_shape
        k2, n = b_shape
        assert k == k2
        return b * m * n * k * 2
    raise NotImplementedError(f"Unsupported einsum shapes: {a_shape} {b_shape}")


def register_einsum_flop_formula() -> bool:
    """Registers ``einsum_flop`` in torch's flop registry the way the reference does when it is
    imported (``register_flop_formula(torch.ops.aten.einsum, get_raw=True)``,
    compute_estimation.py:16), unless a formula for the operator is already there (the reference
    itself, in the same process).  Whether ``FlopCounterMode`` consults it is torch's business and
    the same for both: the installed torch (2.10) looks an operator's overload up before it
    decomposes it, finds no entry under ``aten.einsum.default`` and counts the matrix products
    of the decomposition, which for the shapes above are the same numbers."""
    from torch.utils.flop_counter import flop_registry, register_flop_formula

    if torch.ops.aten.einsum in flop_registry:
        return False
    register_flop_formula(torch.ops.aten.einsum, get_raw=True)(einsum_flop)
    return True


register_einsum_flop_formula()

_DTYPE_TO_CODE = {getattr(torch, name): code for name, code in DTYPE_CODES.items()}


def has_zero_cost(node) -> bool:
    if node.op != "call_function":
        return True
    if not isinstance(node.target, torch._ops.OpOverload):
        return True
    return bool(node.target.is_view)


def _const_key(x):
    if isinstance(x, (torch.dtype, torch.device, torch.layout, torch.memory_format, int, float, bool, str,
                      type(None))):
        return x
    if isinstance(x, torch.Tensor):  # a non-Node tensor constant in args: shape only
        return ("tensor", tuple(x.shape), x.dtype)
    return repr(x)


# what a node's flop count is to the device kernel (APC_NODE_* of include/apcost.h)
NODE_ZERO_COST, NODE_BYTES_ONLY, NODE_MM, NODE_BMM, NODE_SDPA, NODE_SDPA_BACKWARD = range(6)

# operator packet -> (kind, positions among the node's tensor arguments of the tensors the
# formula reads, the rank it expects of them): torch/utils/flop_counter.py mm_flop, addmm_flop,
# bmm_flop, baddbmm_flop, sdpa_flop, sdpa_backward_flop
_aten = torch.ops.aten
_CLOSED_FORMS = {
    _aten.mm: (NODE_MM, (0, 1), 2),
    _aten.addmm: (NODE_MM, (1, 2), 2),
    _aten.bmm: (NODE_BMM, (0, 1), 3),
    _aten.baddbmm: (NODE_BMM, (1, 2), 3),
    _aten._scaled_dot_product_flash_attention: (NODE_SDPA, (0, 1, 2), 4),
    _aten._scaled_dot_product_efficient_attention: (NODE_SDPA, (0, 1, 2), 4),
    _aten._scaled_dot_product_cudnn_attention: (NODE_SDPA, (0, 1, 2), 4),
    _aten._scaled_dot_product_flash_attention_backward: (NODE_SDPA_BACKWARD, (1, 2, 3), 4),
    _aten._scaled_dot_product_efficient_attention_backward: (NODE_SDPA_BACKWARD, (1, 2, 3), 4),
    _aten._scaled_dot_product_cudnn_attention_backward: (NODE_SDPA_BACKWARD, (1, 2, 3), 4),
}


class StrategyRecipes:
    """Per-node recipes from which the device computes the flop and byte count of every
    (node, strategy) out of the spec table (``apc_strategy_inputs``): ``node_kind``,
    ``node_dtype``, ``node_const_bytes``, ``node_row_begin`` / ``byte_rows`` (CSR of first spec
    rows whose local bytes add up) and ``node_flop_rows`` [n_nodes, 4].  ``host_nodes`` lists
    the nodes no recipe covers (an operator torch's flop counter knows but the kernel has no
    formula for, or one that decomposes under the counter): with any of them the planner takes
    the host path (``fill_flops_and_bytes``) for the whole graph."""

    def __init__(self, n_nodes: int):
        self.node_kind = np.zeros(n_nodes, np.int32)
        self.node_dtype = np.ones(n_nodes, np.int8)  # the strategy table's initial dtype code
        self.node_const_bytes = np.zeros(n_nodes, np.int64)
        self.node_row_begin = np.zeros(n_nodes + 1, np.int64)
        self.byte_rows = np.zeros(0, np.int32)
        self.node_flop_rows = np.zeros((n_nodes, 4), np.int32)
        self.host_nodes: list = []


def _local_shape_stride(tables, row: int, mesh_sizes):
    """Local shape and stride of spec row ``row`` on the host (compute_estimation.py:211-229:
    the sharded dim ceil-divided by the mesh dim's size, the stride of the dim before it as
    well when that dim is not the first) -- the rule the spec-table kernel applies to every
    row; here for the one row per operator that the recipe check below evaluates."""
    from ..encoding import KIND_SHARD, code_dim, code_kind, unpack_codes

    t = int(tables.spec_tensor[row])
    r = int(tables.tensor_rank[t])
    shape = [int(x) for x in tables.tensor_shape[t][:r]]
    stride = [int(x) for x in tables.tensor_stride[t][:r]]
    for n, c in zip(mesh_sizes, unpack_codes(int(tables.spec_codes[row]), len(mesh_sizes))):
        if code_kind(c) == KIND_SHARD:
            d = code_dim(c)
            shape[d] = (shape[d] + n - 1) // n
            if d - 1 > 0:
                stride[d - 1] = (stride[d - 1] + n - 1) // n
    return tuple(shape), tuple(stride)


def _recipe_holds(encoded, s_i, node, vals, tensor_pos, node_args, flat_args, treespec, kw_vals, kw_spec, out_rows,
                  const_bytes, mesh_sizes, n_strategies) -> bool:
    """Whether a bytes-only recipe gives what the reference's evaluation gives for ``node``
    (compute_estimation.py:232-243, 334-349 adds the bytes of what the operator RETURNS on the
    local-shaped arguments; the recipe adds the local bytes of the output specs: equal only
    while the operator's output shape follows its sharded inputs).  One strategy is evaluated
    on the host: the first one that shards an argument or an output (a fully replicated
    strategy cannot tell the two apart), and its flops must be zero."""
    from ..encoding import KIND_SHARD, code_kind, unpack_codes

    tb = encoded.tables
    arg_rows = [encoded.input_spec_row[(s_i, k)] for k in range(len(node_args))]
    M = len(mesh_sizes)

    def sharded(row):
        return int(tb.spec_tensor[row]) >= 0 and any(code_kind(c) == KIND_SHARD for c in unpack_codes(int(tb.spec_codes[row]), M))

    pick = 0
    for ss in range(n_strategies):
        if any(sharded(r + ss) for r in arg_rows + out_rows):
            pick = ss
            break
    if any(int(tb.spec_tensor[r + pick]) < 0 for r in arg_rows):
        return False  # an argument without a spec: nothing to take a local shape from
    local = {i: _local_shape_stride(tb, arg_rows[k] + pick, mesh_sizes) for k, i in enumerate(node_args)}
    shapes = [local.get(i, (tuple(vals[i].shape), tuple(vals[i].stride()))) for i in tensor_pos]
    mode = getattr(vals[tensor_pos[0]], "fake_mode", None)
    try:
        flops, rw_bytes, _ = _evaluate(node.target, vals, tensor_pos, shapes, treespec, kw_vals, kw_spec, mode)
    except Exception:
        return False  # the host path reports what the operator cannot run on
    want = const_bytes
    for r in arg_rows + out_rows:
        row = r + pick
        t = int(tb.spec_tensor[row])
        if t >= 0:
            want += math.prod(_local_shape_stride(tb, row, mesh_sizes)[0]) * int(tb.tensor_itemsize[t])
    return flops == 0 and rw_bytes == want


def tb_codes(encoded, rows, n_strategies):
    """The placement codes of the spec rows of a node (its strategies one after the other per
    argument / output slot), as bytes: two nodes with the same operator, shapes and codes have
    the same recipe check."""
    tb = encoded.tables
    return [np.ascontiguousarray(tb.spec_codes[r:r + n_strategies]).tobytes() for r in rows]


def strategy_recipes(encoded, strats, mesh_sizes=None) -> StrategyRecipes:
    """One recipe per graph node (no per-strategy work on the host).  What the reference does
    per strategy (compute_estimation.py:232-299, 334-349): run the operator on fake tensors of
    the local shard shapes under ``FlopCounterMode`` and add the bytes of every tensor among
    the arguments and the outputs.  Per node that is: the local bytes of the strategy's input
    specs and output specs (rows of the spec table) plus the bytes of tensor constants; for an
    operator without tensor arguments (a factory) the operator runs on its own arguments, so
    its output is the global tensor whatever the strategy: a constant; flops as the closed
    form of the operator's entry in torch's flop registry, zero outside the registry.

    A bytes-only recipe (an operator outside the flop registry) rests on the operator's output
    having the local shape of its output spec.  With ``mesh_sizes`` given, that is checked once
    per distinct (operator, constants, argument shapes and dtypes) by evaluating one sharded
    strategy on the host the reference's way; a node whose recipe does not hold is listed in
    ``host_nodes``."""
    from torch.utils.flop_counter import flop_registry

    n_nodes = len(encoded.nodes)
    rc = StrategyRecipes(n_nodes)
    rows: list = []
    checked: dict = {}  # (operator, constants, argument shapes / strides / dtypes) -> the recipe holds
    slots_of: dict = {}
    for (s_i, slot), row in encoded.output_spec_row.items():
        slots_of.setdefault(s_i, []).append(row)
    for s_i, node in enumerate(encoded.nodes):
        rc.node_row_begin[s_i] = len(rows)
        if node.op == "output" or has_zero_cost(node):
            continue  # NODE_ZERO_COST, dtype code 1
        flat_args, treespec = tree_flatten(node.args)
        vals = [a.meta["val"] if isinstance(a, torch.fx.Node) else a for a in flat_args]
        tensor_pos = [i for i, v in enumerate(vals) if isinstance(v, torch.Tensor)]
        kw_flat, kw_spec = tree_flatten(node.kwargs)
        kw_vals = [a.meta["val"] if isinstance(a, torch.fx.Node) else a for a in kw_flat]
        for v in kw_vals:
            # compute_estimation.py:254-256: tensors are expected in args only
            assert not isinstance(v, torch.Tensor), f"{node}: tensor keyword arguments are not supported"
        rc.node_kind[s_i] = NODE_BYTES_ONLY
        dtype = vals[tensor_pos[0]].dtype if tensor_pos else torch.float32
        rc.node_dtype[s_i] = _DTYPE_TO_CODE.get(dtype, UNSUPPORTED_DTYPE_CODE)
        packet = node.target.overloadpacket
        if not tensor_pos:
            # a factory: the reference runs it on its own (global) arguments for every strategy
            mode = getattr(node.meta.get("val"), "fake_mode", None)
            flops, rw_bytes, code = _evaluate(node.target, vals, [], [], treespec, kw_vals, kw_spec, mode)
            if flops != 0:
                rc.host_nodes.append(node)
            rc.node_const_bytes[s_i] = rw_bytes
            rc.node_dtype[s_i] = code
            continue
        node_args = [i for i in tensor_pos if isinstance(flat_args[i], torch.fx.Node)]
        if len(node_args) != encoded.num_args[s_i]:
            rc.host_nodes.append(node)  # input specs do not line up with the tensor arguments
            continue
        for i in tensor_pos:
            if not isinstance(flat_args[i], torch.fx.Node):  # a tensor constant keeps its size
                rc.node_const_bytes[s_i] += vals[i].numel() * vals[i].element_size()
        arg_rows = [encoded.input_spec_row[(s_i, k)] for k in range(len(node_args))]
        rows.extend(arg_rows)
        rows.extend(slots_of.get(s_i, []))
        form = _CLOSED_FORMS.get(packet)
        if form is not None:
            kind, positions, rank = form
            reads = [tensor_pos[p] for p in positions] if max(positions) < len(tensor_pos) else None
            if reads is None or any(not isinstance(flat_args[i], torch.fx.Node) or vals[i].dim() != rank for i in reads):
                rc.host_nodes.append(node)
                continue
            rc.node_kind[s_i] = kind
            for t, i in enumerate(reads):
                rc.node_flop_rows[s_i, t] = arg_rows[node_args.index(i)]
        elif packet in flop_registry or torch._C._dispatch_has_kernel_for_dispatch_key(
                node.target.name(), "CompositeImplicitAutograd"):
            rc.host_nodes.append(node)  # counted by torch, no formula here (or decomposes under the counter)
        elif mesh_sizes is not None:
            key = (node.target, tuple(_const_key(v) for i, v in enumerate(vals) if i not in tensor_pos), str(treespec),
                   tuple(_const_key(v) for v in kw_vals), str(kw_spec),
                   tuple((tuple(vals[i].shape), tuple(vals[i].stride()), vals[i].dtype, isinstance(flat_args[i], torch.fx.Node))
                         for i in tensor_pos),
                   tuple(tb_codes(encoded, arg_rows + slots_of.get(s_i, []), len(strats[node].strategies))))
            ok = checked.get(key)
            if ok is None:
                ok = checked[key] = _recipe_holds(encoded, s_i, node, vals, tensor_pos, node_args, flat_args, treespec, kw_vals,
                                                  kw_spec, slots_of.get(s_i, []), int(rc.node_const_bytes[s_i]), mesh_sizes,
                                                  len(strats[node].strategies))
            if not ok:
                rc.host_nodes.append(node)
    rc.node_row_begin[n_nodes] = len(rows)
    rc.byte_rows = np.asarray(rows, np.int32)
    return rc


def fill_flops_and_bytes(encoded, strats, local_shape: np.ndarray, local_stride: np.ndarray, stats=None) -> None:
    """Writes strat_flops / strat_rw_bytes / strat_dtype / strat_zero_cost of
    ``encoded.tables`` in place.  ``local_shape`` / ``local_stride`` are the [n_specs, width]
    outputs of the spec-table kernel."""
    tb = encoded.tables
    memo: dict = {}
    node_memo: dict = {}  # node key -> first strategy row of the node that was evaluated
    n_eval = 0
    for s_i, node in enumerate(encoded.nodes):
        if node.op == "output":
            continue
        base = encoded.strat_begin[s_i]
        strategies = strats[node].strategies
        n = len(strategies)
        if has_zero_cost(node):
            tb.strat_zero_cost[base:base + n] = 1
            continue
        tb.strat_zero_cost[base:base + n] = 0
        flat_args, treespec = tree_flatten(node.args)
        vals = [a.meta["val"] if isinstance(a, torch.fx.Node) else a for a in flat_args]
        tensor_pos = [i for i, v in enumerate(vals) if isinstance(v, torch.Tensor)]
        kw_flat, kw_spec = tree_flatten(node.kwargs)
        kw_vals = [a.meta["val"] if isinstance(a, torch.fx.Node) else a for a in kw_flat]
        for v in kw_vals:
            # compute_estimation.py:254-256: tensors are expected in args only
            assert not isinstance(v, torch.Tensor), f"{node}: tensor keyword arguments are not supported"
        const_key = (tuple(_const_key(v) for i, v in enumerate(vals) if i not in tensor_pos), str(treespec),
                     tuple(_const_key(v) for v in kw_vals), str(kw_spec))
        ranks = [vals[i].dim() for i in tensor_pos]
        dtypes = tuple(vals[i].dtype for i in tensor_pos)
        n_specs = encoded.num_args[s_i]
        spec_rows = [encoded.input_spec_row[(s_i, a)] for a in range(n_specs)]
        mode = None
        for v in vals:
            if isinstance(v, torch.Tensor):
                mode = getattr(v, "fake_mode", None)
                break
        if mode is None:
            out_val = node.meta.get("val")
            mode = getattr(out_val, "fake_mode", None) if isinstance(out_val, torch.Tensor) else None
        # a node of a repeated layer has the rows of its first occurrence: same op, constants,
        # dtypes and local shapes / strides of every strategy
        node_key = (node.target, const_key, dtypes, tuple(ranks), n,
                    tuple(local_shape[spec_rows[k]:spec_rows[k] + n, :r].tobytes() +
                          local_stride[spec_rows[k]:spec_rows[k] + n, :r].tobytes() for k, r in enumerate(ranks)))
        seen = node_memo.get(node_key)
        if seen is not None:
            tb.strat_flops[base:base + n] = tb.strat_flops[seen:seen + n]
            tb.strat_rw_bytes[base:base + n] = tb.strat_rw_bytes[seen:seen + n]
            tb.strat_dtype[base:base + n] = tb.strat_dtype[seen:seen + n]
            continue
        node_memo[node_key] = base
        for ss in range(n):
            shapes = []
            for k, r in enumerate(ranks):
                row = spec_rows[k] + ss
                shapes.append((tuple(int(x) for x in local_shape[row, :r]), tuple(int(x) for x in local_stride[row, :r])))
            key = (node.target, tuple(shapes), dtypes, const_key)
            hit = memo.get(key)
            if hit is None:
                hit = _evaluate(node.target, vals, tensor_pos, shapes, treespec, kw_vals, kw_spec, mode)
                memo[key] = hit
                n_eval += 1
            flops, rw_bytes, dtype_code = hit
            tb.strat_flops[base + ss] = flops
            tb.strat_rw_bytes[base + ss] = rw_bytes
            tb.strat_dtype[base + ss] = dtype_code
    if stats is not None:
        stats["shape_function_calls"] = n_eval
        stats["distinct_keys"] = len(memo)


def _evaluate(op, vals, tensor_pos, shapes, treespec, kw_vals, kw_spec, mode):
    import contextlib

    ctx = mode if mode is not None else contextlib.nullcontext()
    with ctx:
        new_vals = list(vals)
        for (shape, stride), i in zip(shapes, tensor_pos):
            x = vals[i]
            new_vals[i] = torch.empty_strided(shape, stride, device=x.device, dtype=x.dtype)
        args = treespec.unflatten(new_vals)
        kwargs = kw_spec.unflatten(kw_vals)
        with FlopCounterMode(display=False) as counter:
            out = op(*args, **kwargs)
        flops = counter.get_total_flops()
        rw_bytes = 0
        for x in tree_flatten(args)[0]:
            if isinstance(x, torch.Tensor):
                rw_bytes += x.numel() * x.element_size()
        for x in tree_flatten(out)[0]:
            if isinstance(x, torch.Tensor):
                rw_bytes += x.numel() * x.element_size()
    dtype = torch.float32
    for x in tree_flatten(args)[0]:
        if isinstance(x, torch.Tensor):
            dtype = x.dtype
            break
    return int(flops), int(rw_bytes), _DTYPE_TO_CODE.get(dtype, UNSUPPORTED_DTYPE_CODE)
