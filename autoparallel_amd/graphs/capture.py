"""Joint forward+backward graph capture on fake tensors, and the graph preparation
that decides which nodes and edges the cost tables see.

What the reference does at this step (autoparallel/api.py:50-107, 310-384 and
autoparallel/graph_utils.py:17-39, 76-150), restated with torch's public AOT export:
  * the model's parameters and buffers become FakeTensors (no storage is allocated);
  * ``aot_export_joint_with_descriptors`` traces forward and backward into one FX graph
    whose placeholders / outputs carry descriptors (parameter, plain input, tangent, grad);
  * the inductor decomposition table is used minus a few ops that must stay whole, and
    ``addmm`` is decomposed to ``self + mat1 @ mat2`` so the planner sees a bare ``mm``;
  * dead code, no-op and assert nodes are removed;
  * an ``aten.alias`` node is inserted after every tensor node with two or more users and
    in front of every graph output, which gives the planner a redistribution point there.
Low-precision parameters are modelled by a cast parametrization on every parameter, so a
``convert_element_type`` node follows each parameter placeholder.
"""

from __future__ import annotations

import contextlib
import copy

import torch
from torch import nn
from torch._subclasses import FakeTensorMode


def decomposition_table():
    from torch._inductor.decomposition import select_decomp_table

    table = copy.copy(select_decomp_table())
    aten = torch.ops.aten
    for op in (aten.full_like.default, aten.empty_like.default, aten.threshold_backward.default,
               aten.native_layer_norm.default, aten.embedding_dense_backward.default,
               aten.native_layer_norm_backward.default, aten._softmax_backward_data.default,
               aten._softmax.default, aten.addmm.default):
        table.pop(op, None)

    def addmm_as_add_mm(self, mat1, mat2, beta=1, alpha=1):
        return self + mat1 @ mat2

    table[aten.addmm.default] = addmm_as_add_mm
    return table


def fakeify_(model: nn.Module, fake_mode: FakeTensorMode, device="cpu") -> nn.Module:
    """Replaces every parameter / buffer (typically created on the meta device) by a
    FakeTensor of the same shape, stride and dtype on ``device``."""
    with fake_mode:
        for mod in model.modules():
            for name, p in list(mod._parameters.items()):
                if p is not None:
                    fake = torch.empty_strided(p.shape, p.stride(), dtype=p.dtype, device=device)
                    mod._parameters[name] = nn.Parameter(fake, requires_grad=p.requires_grad)
            for name, b in list(mod._buffers.items()):
                if b is not None:
                    mod._buffers[name] = torch.empty_strided(b.shape, b.stride(), dtype=b.dtype, device=device)
    return model


class _CastTo(nn.Module):
    def __init__(self, dtype):
        super().__init__()
        self.dtype = dtype

    def forward(self, x):
        return x.to(self.dtype)


def cast_parameters_(model: nn.Module, dtype: torch.dtype) -> nn.Module:
    """Every floating-point parameter is read through a cast to ``dtype`` (parameters stay
    in their storage dtype; gradients flow back through the cast)."""
    from torch.nn.utils import parametrize

    for mod in list(model.modules()):
        if parametrize.is_parametrized(mod):
            continue
        for name, p in list(mod._parameters.items()):
            if p is not None and p.is_floating_point() and p.dtype != dtype:
                parametrize.register_parametrization(mod, name, _CastTo(dtype), unsafe=True)
    return model


def cleanup_graph(gm: torch.fx.GraphModule) -> None:
    """Dead code, no-op and assert removal on ``gm.graph``.  The module's Python code is not
    regenerated here (a quarter of a second per pass on a 10 000-node graph, and planning only
    reads the graph): the caller recompiles once when the graph is final."""
    from torch._inductor.fx_passes.post_grad import remove_assert_ops, remove_noop_ops

    gm.graph.eliminate_dead_code()
    remove_noop_ops(gm.graph)
    remove_assert_ops(gm.graph)
    gm.graph.eliminate_dead_code()
    gm.graph.lint()


def add_alias_nodes(gm: torch.fx.GraphModule) -> torch.fx.GraphModule:
    """``aten.alias`` after every tensor-valued node with >= 2 users (placed before its
    first user) and before every graph output."""
    graph = gm.graph
    nodes = list(graph.nodes)
    position = {n: i for i, n in enumerate(nodes)}
    alias = torch.ops.aten.alias.default

    def reroute(node, anchor, before):
        ctx = graph.inserting_before(anchor) if before else graph.inserting_after(anchor)
        with ctx:
            new = graph.call_function(alias, args=(node,))
        new.meta.update(node.meta)
        node.replace_all_uses_with(new, delete_user_cb=lambda user: user is not new)

    for node in nodes:
        if len(node.users) >= 2 and isinstance(node.meta.get("val"), torch.Tensor):
            first_user = nodes[min(position[u] for u in node.users)]
            reroute(node, first_user, before=True)
    (output,) = graph.find_nodes(op="output")
    for node in output.all_input_nodes:
        reroute(node, node, before=False)
    gm.recompile()
    return gm


def dynamo_capture(model: nn.Module, inputs: tuple) -> torch.fx.GraphModule:
    """The model's forward as a Dynamo-captured graph module whose parameters keep their
    fully qualified names, with every ``local_map``-decorated function kept as one
    higher-order-op call instead of being traced through (api.py:152-192).  The joint
    export of that module then carries a forward and a backward ``call_local_map`` node per
    region, tagged with the region's declared placements (``meta["local_map_kwargs"]``)."""
    from torch._dynamo.functional_export import _dynamo_graph_capture_for_export
    from torch._dynamo.variables.higher_order_ops import LocalMapWrappedHigherOrderVariable
    from torch._higher_order_ops import local_map as local_map_module
    from torch.export._trace import _restore_state_dict

    def forward(*args):
        return model(*args)

    with LocalMapWrappedHigherOrderVariable.enable(), local_map_module.defer_inlining(), \
            torch._dynamo.utils._disable_saved_tensors_hooks_during_tracing(), \
            torch._dynamo.config.patch(install_free_tensors=True):
        gm = _dynamo_graph_capture_for_export(forward)(*inputs)
        _restore_state_dict(model, gm)
    return gm


@contextlib.contextmanager
def capture_joint_graph(model: nn.Module, input_fn, param_dtype: torch.dtype | None = None, device="cpu",
                        add_aliases: bool = True, dynamo: bool = False, prepare: bool = True):
    """Context manager yielding ``(gm, joint_with_descriptors)`` for ``model`` (built on
    the meta device) and ``input_fn`` (called under the fake mode; returns a tensor or a
    tuple of tensors).  The fake mode stays usable inside the ``with`` block.  ``dynamo``
    captures the forward with Dynamo first (needed for models with ``local_map`` regions,
    which plain AOT tracing would inline).  ``prepare=False`` yields the exported graph as it
    is, before dead-code / no-op removal and alias insertion."""
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors

    fake_mode = FakeTensorMode()
    model = fakeify_(copy.deepcopy(model), fake_mode, device)
    if param_dtype is not None:
        cast_parameters_(model, param_dtype)
    with fake_mode:
        inputs = input_fn()
    if not isinstance(inputs, tuple):
        inputs = (inputs,)
    with contextlib.ExitStack() as stack:
        if dynamo:
            from torch._higher_order_ops import local_map as local_map_module

            # the joint export must not inline the regions either
            stack.enter_context(local_map_module.defer_inlining())
            model = dynamo_capture(model, inputs)
        joint = aot_export_joint_with_descriptors(stack, model, inputs, decompositions=decomposition_table())
        gm = joint.graph_module
        for node in gm.graph.nodes:
            if node.op == "call_function" and getattr(node.target, "namespace", "") == "_c10d_functional":
                raise RuntimeError(f"the model already contains a collective ({node.target}); "
                                   "planning needs a single-device graph")
        if prepare:
            cleanup_graph(gm)
            if add_aliases:
                add_alias_nodes(gm)
            else:
                gm.recompile()
        yield gm, joint
