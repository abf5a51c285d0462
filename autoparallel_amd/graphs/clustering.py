"""Repeated-subgraph detection for ILP variable sharing.

Transformer layers repeat, and the planner may decide once for all of them.  The
reference finds identical *regions* with dynamo's region tracker seeded by a per-node
hash of (source line, argument metadata, the node's strategies, its producers' output
placements) and links the ILP variables of corresponding nodes
(autoparallel/graph_clustering.py:88-206, autoparallel/optimize_sharding.py:211-231).

Two algorithms live here.  ``cluster_regions`` restates the reference's: the same per-node key,
identical regions grown with torch's own region tracker, regions of a group paired node by
node; on the graphs where the reference's function returns, its links are reproduced exactly
(the test fixtures hold the reference's own output).  Under torch 2.10 the reference's function
ends in its own sanity check ("Duplicate node ... in region group") on every Llama-shaped graph
tried, and ``cluster_regions`` raises the same way, so the planner's default is the second one,
``cluster_nodes``:

the same per-node key is refined a fixed number of rounds with the keys of the
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
    known: dict = {}  # (node, output_only) -> id: a producer is asked about once per consumer

    def strategy_id(node, output_only: bool) -> int:
        found = known.get((node, output_only))
        if found is None:
            found = known[(node, output_only)] = intern_strategies(node, output_only)
        return found

    by_origin: dict = {}  # nodes enumerated from one memo entry hold the same strategy list

    def intern_strategies(node, output_only: bool) -> int:
        s = strats[node]
        if not hasattr(s, "strategies"):
            return -1
        origin = getattr(s, "_apc_origin", None)
        if origin is None:
            return intern_list(s, output_only)
        found = by_origin.get((id(origin), output_only))
        if found is None:
            found = by_origin[(id(origin), output_only)] = intern_list(s, output_only)
        return found

    def intern_list(s, output_only: bool) -> int:
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


def _output_placements(strategy) -> str:
    """The output placements of every strategy of a node, as text (graph_clustering.py:58-74)."""
    from torch.distributed.tensor._dtensor_spec import DTensorSpec

    parts = []
    for s in strategy.strategies:
        specs = s.output_specs
        if isinstance(specs, DTensorSpec):
            specs = [specs]
        inner = ["(None)" if spec is None else "(" + ",".join(str(p) for p in spec.placements) + ")" for spec in specs]
        parts.append("(" + ",".join(inner) + ")")
    return ", ".join(parts)


def cluster_regions(graph: torch.fx.Graph, strats: dict) -> dict:
    """node -> representative node, with the reference's semantics
    (autoparallel/graph_clustering.py:88-206 and the pairing of optimize_sharding.py:211-231):

      * every node but the placeholders is keyed by (source line, argument metadata, its
        strategies as text, the output placements of its producers) (:88-98);
      * nodes with equal keys seed groups of one-node regions; groups are visited from the latest
        in the graph to the earliest and each is grown backwards through the arguments, one node
        at a time and only while the candidate nodes of all regions are again identical, unseen
        and acyclic: torch's ``fully_expand_region_group`` (the library routine the reference calls);
      * groups whose regions stayed single nodes are dropped; every region of a group is paired
        node by node, in graph order, with the group's first region.
    Raises ``RuntimeError`` when a node ends up in two groups, as the reference's own check does."""
    import math
    from collections import defaultdict

    from torch._dynamo.graph_region_tracker import (InputPickler, _populate_recursive_ancestor_map,
                                                    fully_expand_region_group)
    from torch._inductor.codecache import sha256_hash

    rank = {node: i for i, node in enumerate(graph.nodes)}
    ancestors = _populate_recursive_ancestor_map(graph)
    pickler = InputPickler()

    def arg_value(a):
        if isinstance(a, torch.fx.Node):
            return a.meta.get("val")
        return a if isinstance(a, (torch.Tensor, int)) else None

    def strategy_text(node):
        s = strats.get(node)
        if s is None and node.op == "output":  # (the reference keys the output node by its producers' strategies)
            s = [strats[x] for x in node.all_input_nodes]
        return str(s)

    same_key = defaultdict(list)
    group_of = {}
    for node in graph.nodes:
        if node.op == "placeholder":
            continue
        flat_args, _ = tree_flatten(node.args)
        flat_kwargs, _ = tree_flatten(sorted(node.kwargs.items(), key=lambda kv: kv[0]))
        key = (node.meta.get("stack_trace"),
               (tuple(sorted(node.kwargs)), tuple(arg_value(a) for a in flat_args + flat_kwargs)),
               strategy_text(node),
               tuple(_output_placements(strats[p]) for p in node.all_input_nodes))
        bucket = same_key[sha256_hash(pickler.dumps(key))]
        bucket.append(node)
        group_of[node] = bucket

    def identical(a, b):
        return a is not b and a in group_of and b in group_of and group_of[a] is group_of[b]

    groups = [([[n] for n in bucket], min(rank[n] for n in bucket)) for bucket in same_key.values() if len(bucket) > 1]
    groups.sort(key=lambda g: -g[1])
    seen: set = set()
    grown = []
    for regions, _ in groups:
        if regions[0][0] in seen:
            continue
        fully_expand_region_group(regions, seen, ancestors, identical)
        for region in regions:
            region.sort(key=rank.__getitem__)
        grown.append(regions)
    grown = [regions for regions in grown if len(regions[0]) > 1]
    for regions in grown:
        regions.sort(key=lambda region: rank[region[0]])
    grown.sort(key=lambda regions: rank[regions[0][0]])
    claimed: set = set()
    rep: dict = {}
    for regions in grown:
        for region in regions:
            for node in region:
                if node in claimed:
                    raise RuntimeError(f"Duplicate node {node} in region group")
                claimed.add(node)
        first = regions[0]
        for region in regions[1:]:
            assert len(region) == len(first)
            for n0, ni in zip(first, region):
                rep[ni] = n0
    return rep
