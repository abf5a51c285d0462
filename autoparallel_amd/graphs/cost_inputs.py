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

import numpy as np
import torch
from torch.utils._pytree import tree_flatten
from torch.utils.flop_counter import FlopCounterMode

from ..cost_model import DTYPE_CODES

UNSUPPORTED_DTYPE_CODE = 7

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
