"""Seeded synthetic strategy graphs in flattened form.

``stress_dag`` draws the raw-throughput workload: an FX-like DAG with a
matmul / elementwise / reduction / view op mix, tensors of rank 2-4 with
power-of-two dims, bf16 / fp32, a uniform number of strategies per node and
Poisson fan-out, on an arbitrary logical mesh.  Every placement drawn is valid
in the sense of the reference's divisibility filter
(autoparallel/propagation_rules.py:104-135): a sharded tensor dim is divisible by
the product of the mesh dims that shard it.

The per-strategy flop and byte counts follow closed forms on the local shard
shapes (the definition of this workload; on traced graphs they come from the
op's own shape function):
    view         zero cost
    elementwise  flops 0, bytes = sum(local input bytes) + local output bytes
    reduction    flops 0, bytes as above
    matmul       flops = 2 * local_numel(out) * K / prod(mesh dims where the output
                 is Partial), bytes as above
"""

from __future__ import annotations

import numpy as np

from ._native import APC_MAX_RANK
from .encoding import EDGE_GRAD_RESCALE, EDGE_NO_PRODUCER, CostTables

OP_MATMUL, OP_ELEMENTWISE, OP_REDUCTION, OP_VIEW = 0, 1, 2, 3


def _random_codes(rng, n, rank, mesh_sizes, shape, p_replicate, p_partial, allow_partial):
    """n packed placement tuples for tensors of the given per-row rank / shape.
    Shards that would split a dim unevenly (sequential divisibility over mesh dims)
    are turned into Replicate."""
    M = len(mesh_sizes)
    u = rng.random((n, M))
    dims = (rng.random((n, M)) * rank[:, None]).astype(np.int64)
    codes = np.where(u < p_replicate, 0, 0x80 | dims)
    part = (u >= p_replicate) & (u < p_replicate + p_partial) & allow_partial[:, None]
    codes = np.where(part, 0x40, codes)
    remaining = shape.copy()
    for i in range(M):
        is_shard = (codes[:, i] >> 6) == 2
        d = codes[:, i] & 0x0F
        cur = remaining[np.arange(n), d]
        ok = is_shard & (cur % mesh_sizes[i] == 0) & (cur >= mesh_sizes[i])
        codes[:, i] = np.where(is_shard & ~ok, 0, codes[:, i])
        remaining[np.arange(n)[ok], d[ok]] = cur[ok] // mesh_sizes[i]
    packed = np.zeros(n, np.uint32)
    for i in range(M):
        packed |= (codes[:, i].astype(np.uint32) & 0xFF) << np.uint32(8 * i)
    return packed, remaining


def _local_bytes(packed, tensor_idx, t_shape, t_rank, t_item, mesh_sizes):
    n = len(packed)
    shape = t_shape[tensor_idx].copy()
    for i, m in enumerate(mesh_sizes):
        c = (packed >> np.uint32(8 * i)) & np.uint32(0xFF)
        is_shard = (c >> 6) == 2
        d = (c & 0x0F).astype(np.int64)
        rows = np.arange(n)[is_shard]
        shape[rows, d[is_shard]] = -(-shape[rows, d[is_shard]] // m)
    mask = np.arange(APC_MAX_RANK)[None, :] < t_rank[tensor_idx][:, None]
    numel = np.where(mask, shape, 1).prod(axis=1)
    return numel, numel * t_item[tensor_idx]


def stress_dag(seed: int = 0, n_nodes: int = 200_000, mesh_sizes=(16, 8, 4), min_strategies: int = 4,
               max_strategies: int = 64, fanout_lambda: float = 2.0, window: int = 256,
               op_mix=(0.4, 0.3, 0.2, 0.1), min_log2_dim: int = 6, max_log2_dim: int = 14,
               max_log2_numel: int = 36, frac_noncontiguous: float = 0.1, frac_grad_nodes: float = 0.05,
               frac_nonspec_nodes: float = 0.005, p_match_producer: float = 0.5,
               tile_entries=None) -> CostTables:
    rng = np.random.Generator(np.random.PCG64(seed))
    mesh_sizes = tuple(int(m) for m in mesh_sizes)
    M = len(mesh_sizes)
    N = int(n_nodes)

    # ---- nodes: op class, output tensor, strategy counts ------------------------------------
    op = rng.choice(4, size=N, p=np.asarray(op_mix, dtype=np.float64))
    rank = rng.integers(2, 5, size=N)
    log2 = rng.integers(min_log2_dim, max_log2_dim + 1, size=(N, APC_MAX_RANK))
    col = np.arange(APC_MAX_RANK)[None, :]
    log2 = np.where(col < rank[:, None], log2, 0)
    # keep numel <= 2**max_log2_numel by shaving the largest dim (never below the minimum)
    for _ in range(64):
        over = log2.sum(axis=1) - max_log2_numel
        rows = np.nonzero(over > 0)[0]
        if rows.size == 0:
            break
        big = log2[rows].argmax(axis=1)
        cut = np.minimum(over[rows], log2[rows, big] - min_log2_dim)
        cut = np.maximum(cut, 0)
        log2[rows, big] -= cut
        if (cut == 0).all():
            break
    shape = np.where(col < rank[:, None], np.int64(1) << log2, 0).astype(np.int64)
    itemsize = np.where(rng.random(N) < 0.5, 2, 4).astype(np.int32)
    dtype_code = np.where(itemsize == 2, 3, 1).astype(np.int8)  # bfloat16 / float32
    # contiguous strides; a fraction has its last two dims swapped in memory
    stride = np.zeros_like(shape)
    run = np.ones(N, np.int64)
    for d in range(APC_MAX_RANK - 1, -1, -1):
        live = d < rank
        stride[:, d] = np.where(live, run, 0)
        run = np.where(live, run * shape[:, d], run)
    swap = rng.random(N) < frac_noncontiguous
    rows = np.nonzero(swap)[0]
    last = rank[rows] - 1
    inner = stride[rows, last].copy()
    stride[rows, last] = inner * shape[rows, last - 1]  # a transposed view of the last two dims
    stride[rows, last - 1] = inner
    nonspec = rng.random(N) < frac_nonspec_nodes
    n_strat = rng.integers(min_strategies, max_strategies + 1, size=N).astype(np.int64)
    node_strat_begin = np.zeros(N + 1, np.int64)
    np.cumsum(n_strat, out=node_strat_begin[1:])
    S = int(node_strat_begin[-1])
    strat_node = np.repeat(np.arange(N), n_strat)

    # ---- edges: Poisson fan-out to later nodes ----------------------------------------------
    fan = rng.poisson(fanout_lambda, size=N)
    room = np.minimum(window, N - 1 - np.arange(N))
    fan = np.where(room > 0, fan, 0)
    prod = np.repeat(np.arange(N), fan)
    cons = prod + 1 + (rng.random(prod.size) * room[prod]).astype(np.int64)
    order = np.lexsort((prod, cons))
    prod, cons = prod[order], cons[order]
    n_in = np.bincount(cons, minlength=N)
    # nodes without inputs get one producer-less pseudo argument (placeholders / factories)
    src_less = np.nonzero(n_in == 0)[0]
    e_node = np.concatenate([cons, src_less])
    e_prod = np.concatenate([prod, np.full(src_less.size, -1, np.int64)])
    order = np.lexsort((np.arange(e_node.size), e_node))
    e_node, e_prod = e_node[order], e_prod[order]
    E = e_node.size
    first_of_node = np.searchsorted(e_node, np.arange(N))
    e_arg = np.arange(E) - first_of_node[e_node]
    num_args = np.maximum(n_in, 1)
    has_prod = e_prod >= 0
    e_src_node = np.where(has_prod, e_prod, e_node)

    # ---- spec table: [output specs of every strategy] ++ [input specs per edge row] ---------
    out_tensor = np.where(nonspec, -1, np.arange(N))[strat_node]
    allow_partial = (op[strat_node] == OP_MATMUL) | (op[strat_node] == OP_REDUCTION)
    out_codes, _ = _random_codes(rng, S, rank[strat_node], mesh_sizes, shape[strat_node], 0.4, 0.15, allow_partial)
    out_codes = np.where(out_tensor < 0, np.uint32(0), out_codes)

    e_n_src = np.where(has_prod, n_strat[e_src_node], 1)
    e_n_tgt = n_strat[e_node]
    e_src_begin = np.where(has_prod, node_strat_begin[e_src_node], 0)
    e_tgt_begin = S + (np.cumsum(e_n_tgt) - e_n_tgt)
    T_in = int(e_n_tgt.sum())
    in_edge = np.repeat(np.arange(E), e_n_tgt)
    in_row = np.arange(T_in) - np.repeat(np.cumsum(e_n_tgt) - e_n_tgt, e_n_tgt)
    in_src_node = e_src_node[in_edge]
    in_tensor = np.where(nonspec[in_src_node], -1, in_src_node)
    rnd_codes, _ = _random_codes(rng, T_in, rank[in_src_node], mesh_sizes, shape[in_src_node], 0.4, 0.05,
                                 np.ones(T_in, bool))
    pick = node_strat_begin[in_src_node] + (rng.random(T_in) * n_strat[in_src_node]).astype(np.int64)
    match = rng.random(T_in) < p_match_producer
    in_codes = np.where(match, out_codes[pick], rnd_codes)
    # a producer-less argument's input spec is the strategy's own output spec
    own = node_strat_begin[e_node[in_edge]] + in_row
    in_codes = np.where(has_prod[in_edge], in_codes, out_codes[own])
    in_tensor = np.where(has_prod[in_edge], in_tensor, out_tensor[own])
    in_codes = np.where(in_tensor < 0, np.uint32(0), in_codes)
    # producer-less edges read one (unused) producer spec row: point it at the node's first strategy
    e_src_begin = np.where(has_prod, e_src_begin, node_strat_begin[e_node])

    spec_codes = np.concatenate([out_codes, in_codes]).astype(np.uint32)
    spec_tensor = np.concatenate([out_tensor, in_tensor]).astype(np.int32)

    # ---- entries, pass-through values, flags -------------------------------------------------
    per_edge = e_n_src.astype(np.int64) * e_n_tgt.astype(np.int64)
    entry_begin = np.zeros(E + 1, np.int64)
    np.cumsum(per_edge, out=entry_begin[1:])
    needs_pt = ~has_prod | nonspec[e_src_node]
    pt_len = np.where(needs_pt, per_edge, 0)
    pt_begin = np.where(needs_pt, np.cumsum(pt_len) - pt_len, -1)
    pt_values = np.where(rng.random(int(pt_len.sum())) < 0.1, np.inf, 0.0)
    # producer-less pseudo arguments carry the rule's [[0.0]] row
    is_srcless_pt = np.repeat(~has_prod, pt_len)
    pt_values = np.where(is_srcless_pt, 0.0, pt_values)
    grad_node = rng.random(N) < frac_grad_nodes
    flags = np.where(grad_node[e_node], EDGE_GRAD_RESCALE, 0) | np.where(has_prod, 0, EDGE_NO_PRODUCER)

    # ---- per-strategy flops / bytes -----------------------------------------------------------
    t_rank = rank.astype(np.int32)
    safe_out = np.maximum(out_tensor, 0)
    out_numel, out_bytes = _local_bytes(out_codes, safe_out, shape, t_rank, itemsize, mesh_sizes)
    out_bytes = np.where(out_tensor < 0, 0, out_bytes)
    safe_in = np.maximum(in_tensor, 0)
    _, in_bytes = _local_bytes(in_codes, safe_in, shape, t_rank, itemsize, mesh_sizes)
    in_bytes = np.where(in_tensor < 0, 0, in_bytes)
    in_strat = node_strat_begin[e_node[in_edge]] + in_row
    rw_bytes = out_bytes.astype(np.int64)
    np.add.at(rw_bytes, in_strat, in_bytes.astype(np.int64))
    k_log2 = rng.integers(min_log2_dim, max_log2_dim + 1, size=N)
    partial_div = np.ones(S, np.int64)
    for i, m in enumerate(mesh_sizes):
        c = (out_codes >> np.uint32(8 * i)) & np.uint32(0xFF)
        partial_div *= np.where((c >> 6) == 1, m, 1)
    k_local = np.maximum((np.int64(1) << k_log2[strat_node]) // partial_div, 1)
    flops = np.where(op[strat_node] == OP_MATMUL, 2 * out_numel * k_local, 0)
    flops = np.where(out_tensor < 0, 0, flops)
    zero_cost = ((op[strat_node] == OP_VIEW) | (out_tensor < 0)).astype(np.uint8)

    tables = CostTables(
        mesh_sizes=mesh_sizes,
        tensor_rank=t_rank, tensor_itemsize=itemsize, tensor_shape=shape, tensor_stride=stride,
        spec_codes=spec_codes, spec_tensor=spec_tensor,
        strat_flops=flops, strat_rw_bytes=rw_bytes, strat_dtype=dtype_code[strat_node],
        strat_zero_cost=zero_cost, strat_num_args=num_args[strat_node],
        node_strat_begin=node_strat_begin,
        edge_node=e_node, edge_arg=e_arg, edge_src_begin=e_src_begin, edge_n_src=e_n_src,
        edge_tgt_begin=e_tgt_begin, edge_n_tgt=e_n_tgt, edge_flags=flags, edge_pt_begin=pt_begin,
        edge_entry_begin=entry_begin, edge_strat_begin=node_strat_begin[e_node],
        pt_values=pt_values,
    )
    if tile_entries is not None:
        tables.build_tiles(tile_entries)
    tables.node_op = op
    return tables
