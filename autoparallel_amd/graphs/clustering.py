"""Repeated-subgraph detection for ILP variable sharing.

Transformer layers repeat, and the planner may decide once for all of them.  The
reference finds identical *regions* with dynamo's region tracker seeded by a per-node
hash of (source line, argument metadata, the node's strategies, its producers' output
placements) and links the ILP variables of corresponding nodes
(autoparallel/graph_clustering.py:88-206, autoparallel/optimize_sharding.py:211-231).

Here the same per-node key is refined a fixed number of rounds with the keys of the
node's producers (by argument position) and consumers (as a multiset), Weisfeiler-Lehman
style: two nodes end up with the same key exactly when their neighbourhoods of that radius
look the same, which is what "the same position in another layer" means, while nodes that
merely share an op and shapes inside one layer (the two up-projections of a SwiGLU block)
are told apart by what consumes them.  Nodes with equal final keys form a cluster; the
first one in graph order represents it.
"""

from __future__ import annotations

import hashlib

import torch
from torch.utils._pytree import tree_flatten

from .encode import all_input_nodes


def _const_repr(x):
    if isinstance(x, torch.fx.Node):
        val = x.meta.get("val")
        if isinstance(val, torch.Tensor):
            return ("node", tuple(val.shape), tuple(val.stride()), str(val.dtype))
        return ("node", repr(val))
    return repr(x)


def _digest(obj) -> bytes:
    return hashlib.blake2b(repr(obj).encode(), digest_size=16).digest()


def cluster_nodes(graph: torch.fx.Graph, strats: dict, rounds: int = 2) -> dict:
    """node -> representative node, for every call_function node that shares its final key
    with an earlier node (placeholders and the output node are never linked)."""
    interned: dict = {}

    def strategy_id(node, output_only: bool) -> int:
        s = strats[node]
        if not hasattr(s, "strategies"):
            return -1
        rows = []
        for st in s.strategies:
            outs = st.output_specs
            outs = tuple(outs) if isinstance(outs, (list, tuple)) else outs
            if output_only:
                rows.append(outs)
            else:
                ins = tuple(st.input_specs) if st.input_specs is not None else None
                rows.append((ins, outs))
        key = (output_only, tuple(rows))
        return interned.setdefault(key, len(interned))

    nodes = [n for n in graph.nodes if n.op == "call_function"]
    key = {}
    for n in graph.nodes:
        if n.op == "call_function":
            flat, spec = tree_flatten((n.args, dict(sorted(n.kwargs.items()))))
            key[n] = _digest((str(n.target), n.meta.get("stack_trace"), tuple(_const_repr(a) for a in flat), str(spec),
                              strategy_id(n, False), tuple(strategy_id(a, True) for a in all_input_nodes(n))))
        elif n.op == "placeholder":
            val = n.meta.get("val")
            meta = (tuple(val.shape), tuple(val.stride()), str(val.dtype)) if isinstance(val, torch.Tensor) else repr(val)
            key[n] = _digest(("placeholder", meta))
        else:
            key[n] = _digest((n.op,))
    for _ in range(rounds):
        new = {}
        for n in graph.nodes:
            ins = tuple(key[a] for a in all_input_nodes(n)) if n.op != "output" else ()
            outs = tuple(sorted(key[u] for u in n.users))
            new[n] = _digest((key[n], ins, outs))
        key = new
    first: dict = {}
    rep: dict = {}
    for n in nodes:
        r = first.setdefault(key[n], n)
        if r is not n:
            rep[n] = r
    return rep
