"""Flattened strategy / placement encoding: the object graph
``dict[Node, OpStrategy] -> OpSpec -> DTensorSpec`` that the reference walks in
``ShardingOptimizer.build_ds`` (autoparallel/optimize_sharding.py:270-380; types at
torch/distributed/tensor/_op_schema.py:94-141) laid out as CSR arrays over tensors,
specs, strategies, edges and entries, ready to sit in HBM.

Layout
------
tensor table   one row per distinct (shape, stride, dtype): ``tensor_rank``,
               ``tensor_itemsize``, ``tensor_shape[T, 8]``, ``tensor_stride[T, 8]``.
spec table     one row per DTensorSpec occurrence: ``spec_codes`` (uint32, byte i =
               placement code of mesh dim i) and ``spec_tensor`` (row of the tensor
               table, -1 for "not a DTensorSpec": ``None`` outputs, scalars).
strategy table one row per (node, strategy): ``strat_flops``, ``strat_rw_bytes``,
               ``strat_dtype``, ``strat_zero_cost``, ``strat_num_args``;
               ``node_strat_begin[N + 1]`` is its CSR pointer.
edge table     one row per (consumer node, argument): producer output specs are spec
               rows ``[edge_src_begin, +edge_n_src)``, consumer input specs are
               ``[edge_tgt_begin, +edge_n_tgt)``; the edge's cost matrix occupies
               entries ``[edge_entry_begin[e], edge_entry_begin[e + 1])``, row-major by
               consumer strategy (= ``redistribute_cost[argi][ii]`` of strategy ``ss``).
pt_values      rule-provided costs that survive where either side is not a
               DTensorSpec (optimize_sharding.py:336-355).
tiles          rectangles of edge matrices, one per workgroup.

Placement codes: 0x00 Replicate; 0x40|op Partial(op) (op 0 = sum); 0x80|v<<4|d Shard(d)
with v a variant id (0 = plain ``Shard``).
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass, fields
from typing import Optional

import numpy as np

from . import _native
from ._native import APC_MAX_RANK, APC_PACKED_MAX_DUPS, APC_TILE_MAX_COLS, APC_TILE_MAX_DUPS, APC_TILE_MAX_ROWS

REPLICATE = 0x00
PARTIAL_SUM = 0x40
KIND_REPLICATE, KIND_PARTIAL, KIND_SHARD = 0, 1, 2

# reduce ops of Partial; index = code payload
PARTIAL_OPS = ("sum", "avg", "min", "max", "product", "band", "bor", "bxor")

EDGE_GRAD_RESCALE = _native.EDGE_GRAD_RESCALE
EDGE_NO_PRODUCER = _native.EDGE_NO_PRODUCER

# Tiling chosen when the caller names no tile size (measured on one MI355X): an edge matrix of
# up to 64 x 64 entries is best served by one tile (its producer specs and cost terms are
# staged once); a table that would then have too few tiles to fill the chip several times
# over is cut finer (fewer copies per tiled edge first, then smaller tiles), as long as a
# tile still stores a few thousand entries.  (Llama-3-70B on (8, 8, 8), 73 M entries: 126 us with
# 11 732 tiles of 2048 entries and 4 copies; 134 us with 8 130 of 4096 / 4, 130 us with 16 192 of
# 4096 / 2, 140 us with 23 376 of 2048 / 2, 155 us with 40 727 of 1024 / 2, 164 us with 2 085 of
# 4096 / 16.)
AUTO_MIN_TILES = 10000
AUTO_MIN_STORED_PER_TILE = 2048
AUTO_MIN_TILE_ENTRIES = 512
# A table this small is bound by the latency of one workgroup, not by work: it keeps the largest
# tiles and up to 16 copies per tiled edge (Llama-3-8B on (32, 8), 1.8 M entries: 13.3 us with
# 840 tiles of 16 copies against 14.6 us with 1 616 tiles of 8 and 17.7 us with 3 168 of 4).
AUTO_SMALL_TABLE_ENTRIES = 4_000_000

# numpy mirror of the C struct apc_tile (64 bytes)
TILE_DTYPE = np.dtype([
    ("edge", "<i4"), ("row_begin", "<i4"), ("col_begin", "<i4"), ("counts", "<i4"),
    ("src_begin", "<i4"), ("n_src", "<i4"), ("tgt_begin", "<i4"), ("flags", "<i4"), ("strat_begin", "<i4"),
    ("tensor", "<i4"), ("entry_begin", "<i8"), ("pt_begin", "<i8"), ("dup_begin", "<i4"), ("dup_count", "<i4"),
])
assert TILE_DTYPE.itemsize == 64


# numpy mirror of the C struct apc_packed_tile: everything one tile reads, in one record
PACKED_MIXED = 0x100
PACKED_TILE_DTYPE = np.dtype([
    ("rows", "<i4"), ("cols", "<i4"), ("flags", "<i4"), ("dup_count", "<i4"), ("tensor", "<i4"), ("tensor_rank", "<i4"),
    ("tensor_itemsize", "<i4"), ("edge", "<i4"), ("entry_begin", "<i8"), ("row_begin", "<i8"), ("pt_begin", "<i8"),
    ("reserved", "<i8"), ("tensor_shape", "<i8", (APC_MAX_RANK,)), ("tensor_stride", "<i8", (APC_MAX_RANK,)),
    ("dup_entry_begin", "<i8", (APC_PACKED_MAX_DUPS,)), ("dup_row_begin", "<i8", (APC_PACKED_MAX_DUPS,)),
    ("col_codes", "<u4", (APC_TILE_MAX_COLS,)), ("col_tensor", "<i4", (APC_TILE_MAX_COLS,)),
    ("row_codes", "<u4", (APC_TILE_MAX_ROWS,)), ("row_tensor", "<i4", (APC_TILE_MAX_ROWS,)),
    ("row_flops", "<i8", (APC_TILE_MAX_ROWS,)), ("row_rw_bytes", "<i8", (APC_TILE_MAX_ROWS,)),
    ("row_meta", "<i4", (APC_TILE_MAX_ROWS,)),
])
assert PACKED_TILE_DTYPE.itemsize == 2752


def shard_code(dim: int, variant: int = 0) -> int:
    if not 0 <= dim < 16:
        raise ValueError(f"Shard dim {dim} outside [0, 16)")
    if not 0 <= variant < 4:
        raise ValueError(f"Shard variant {variant} outside [0, 4)")
    return 0x80 | (variant << 4) | dim


def partial_code(op: int | str = 0) -> int:
    if isinstance(op, str):
        op = PARTIAL_OPS.index(op)
    if not 0 <= op < 64:
        raise ValueError(f"Partial op id {op} outside [0, 64)")
    return 0x40 | op


def code_kind(code: int) -> int:
    return code >> 6


def code_dim(code: int) -> int:
    return code & 0x0F


def pack_codes(codes) -> int:
    out = 0
    for i, c in enumerate(codes):
        out |= (int(c) & 0xFF) << (8 * i)
    return out


def unpack_codes(packed: int, ndim: int) -> tuple:
    return tuple((int(packed) >> (8 * i)) & 0xFF for i in range(ndim))


def _i32(x):
    return np.ascontiguousarray(x, dtype=np.int32)


def _i64(x):
    return np.ascontiguousarray(x, dtype=np.int64)


@dataclass
class CostTables:
    mesh_sizes: tuple
    tensor_rank: np.ndarray
    tensor_itemsize: np.ndarray
    tensor_shape: np.ndarray
    tensor_stride: np.ndarray
    spec_codes: np.ndarray
    spec_tensor: np.ndarray
    strat_flops: np.ndarray
    strat_rw_bytes: np.ndarray
    strat_dtype: np.ndarray
    strat_zero_cost: np.ndarray
    strat_num_args: np.ndarray
    node_strat_begin: np.ndarray
    edge_node: np.ndarray
    edge_arg: np.ndarray
    edge_src_begin: np.ndarray
    edge_n_src: np.ndarray
    edge_tgt_begin: np.ndarray
    edge_n_tgt: np.ndarray
    edge_flags: np.ndarray
    edge_pt_begin: np.ndarray
    edge_entry_begin: np.ndarray
    edge_strat_begin: np.ndarray
    pt_values: np.ndarray
    tile_edge: np.ndarray = None
    tile_row_begin: np.ndarray = None
    tile_row_count: np.ndarray = None
    tile_col_begin: np.ndarray = None
    tile_col_count: np.ndarray = None
    tile_records: np.ndarray = None
    edge_canonical: np.ndarray = None  # edge -> the identical edge that is tiled (itself unless de-duplicated)
    dup_entry_begin: np.ndarray = None  # entry offsets of the duplicates, grouped by canonical edge
    dup_row_begin: np.ndarray = None  # their first matrix rows (rows numbered as in ``row_ptr()``)
    edge_dup_begin: np.ndarray = None
    edge_dup_count: np.ndarray = None
    tiling: dict = None  # tile size and copies per tiled edge of the current tiling

    _DTYPES = {
        "tensor_rank": np.int32, "tensor_itemsize": np.int32, "tensor_shape": np.int64,
        "tensor_stride": np.int64, "spec_codes": np.uint32, "spec_tensor": np.int32,
        "strat_flops": np.int64, "strat_rw_bytes": np.int64, "strat_dtype": np.int8,
        "strat_zero_cost": np.uint8, "strat_num_args": np.int32, "node_strat_begin": np.int64,
        "edge_node": np.int32, "edge_arg": np.int32, "edge_src_begin": np.int32,
        "edge_n_src": np.int32, "edge_tgt_begin": np.int32, "edge_n_tgt": np.int32,
        "edge_flags": np.int32, "edge_pt_begin": np.int64, "edge_entry_begin": np.int64,
        "edge_strat_begin": np.int32, "pt_values": np.float64, "tile_edge": np.int32,
        "tile_row_begin": np.int32, "tile_row_count": np.int32, "tile_col_begin": np.int32,
        "tile_col_count": np.int32,
    }

    def __post_init__(self):
        self.mesh_sizes = tuple(int(x) for x in self.mesh_sizes)
        for name, dt in self._DTYPES.items():
            v = getattr(self, name)
            if v is not None:
                setattr(self, name, np.ascontiguousarray(v, dtype=dt))
        if self.tensor_shape.ndim != 2 or self.tensor_shape.shape[1] != APC_MAX_RANK:
            raise ValueError(f"tensor_shape must be [T, {APC_MAX_RANK}]")
        if self.tensor_stride.shape != self.tensor_shape.shape:
            raise ValueError("tensor_stride must have the shape of tensor_shape")
        if self.tile_edge is None:
            self.build_tiles()
        elif self.tile_records is None:
            self.pack_tile_records()

    # ---- sizes -------------------------------------------------------------------------
    @property
    def n_tensors(self) -> int:
        return len(self.tensor_rank)

    @property
    def n_specs(self) -> int:
        return len(self.spec_codes)

    @property
    def n_strategies(self) -> int:
        return len(self.strat_flops)

    @property
    def n_nodes(self) -> int:
        return len(self.node_strat_begin) - 1

    @property
    def n_edges(self) -> int:
        return len(self.edge_n_src)

    @property
    def n_entries(self) -> int:
        return int(self.edge_entry_begin[-1])

    @property
    def n_tiles(self) -> int:
        return len(self.tile_edge)

    def algorithmic_bytes(self, comm=True, transition=True, cost=True) -> int:
        """Bytes one table build must move at minimum: the outputs written per entry,
        the placement codes of both spec lists of every edge and a 64-byte edge header."""
        per_entry = 8 * int(comm) + 1 * int(transition) + 8 * int(cost)
        m = len(self.mesh_sizes)
        per_edge = (self.edge_n_src.astype(np.int64) + self.edge_n_tgt.astype(np.int64)) * m + 64
        return per_entry * self.n_entries + int(per_edge.sum())

    def shape_width(self) -> int:
        """Values per row of the local shape / stride tables: the largest tensor rank, rounded up
        to even (rows leave the kernel as 16-byte pairs), at least 2."""
        top = int(self.tensor_rank.max()) if self.n_tensors else 0
        return max(2, top + (top & 1))

    def algorithmic_bytes_input_tables(self, spec_table: bool = True) -> int:
        """Bytes the tensor, spec and compute-cost tables must move at minimum: per tensor 136 B
        read (rank, itemsize, shape, stride) and 9 B written; per spec 8 B read and 24 B + two
        rows of ``shape_width()`` values written (shard count, local element and byte counts,
        local shape and stride); per strategy 22 B read and 16 B written."""
        spec = (32 + 16 * self.shape_width()) * self.n_specs if spec_table else 0
        return 145 * self.n_tensors + spec + 38 * self.n_strategies

    def algorithmic_bytes_priced_per_unit(self, row_minima: bool = True) -> int:
        """The same pass priced by fixed per-unit figures, whatever arrays a launch happens to
        write: 8 B (one fp64 cost) + 1 B (transition flag) per entry; per edge its two spec lists
        (one byte per mesh dim and spec) and a 64-byte header; 8 B written + 17 B read per
        (node, strategy) compute cost; 12 B written per row minimum."""
        m = len(self.mesh_sizes)
        per_edge = (self.edge_n_src.astype(np.int64) + self.edge_n_tgt.astype(np.int64)) * m + 64
        return 9 * self.n_entries + int(per_edge.sum()) + 25 * self.n_strategies + (12 * self.n_rows if row_minima else 0)

    @property
    def n_rows(self) -> int:
        """Matrix rows over all edges: one per (edge, consumer strategy)."""
        return int(self.edge_n_tgt.astype(np.int64).sum())

    def validate_row_minima(self) -> None:
        """Raises unless every matrix row lies inside one tile (the precondition of the
        ``apc_*_row_min`` entry points), through the library's host-side check."""
        def p(a):
            return a.ctypes.data_as(ctypes.c_void_p)

        rc = _native.lib().apc_validate_row_minima_host(ctypes.c_int64(self.n_edges), p(self.edge_n_src), p(self.edge_n_tgt),
                                                        ctypes.c_int64(self.n_tiles), p(self.tile_records))
        _native.check(rc, "apc_validate_row_minima_host")

    # ---- tiles -------------------------------------------------------------------------
    def edge_signatures(self) -> list:
        """One digest per edge over everything its matrix depends on: both spec lists
        (codes and tensor rows), flags, the consumer strategies' compute-cost inputs and
        the pass-through values.  Equal digests = bit-identical comm / transition / cost."""
        import hashlib

        sb, ns = self.edge_src_begin.astype(np.int64), self.edge_n_src.astype(np.int64)
        tb, nt = self.edge_tgt_begin.astype(np.int64), self.edge_n_tgt.astype(np.int64)
        st = self.edge_strat_begin.astype(np.int64)
        codes, tensor = self.spec_codes, self.spec_tensor
        strat = np.rec.fromarrays([self.strat_flops, self.strat_rw_bytes, self.strat_dtype, self.strat_zero_cost,
                                   self.strat_num_args])
        out = []
        for e in range(self.n_edges):
            h = hashlib.blake2b(digest_size=16)
            h.update(np.array([ns[e], nt[e], self.edge_flags[e]], np.int64).tobytes())
            h.update(codes[sb[e]:sb[e] + ns[e]].tobytes())
            h.update(tensor[sb[e]:sb[e] + ns[e]].tobytes())
            h.update(codes[tb[e]:tb[e] + nt[e]].tobytes())
            h.update(tensor[tb[e]:tb[e] + nt[e]].tobytes())
            h.update(strat[st[e]:st[e] + nt[e]].tobytes())
            if self.edge_pt_begin[e] >= 0:
                b = int(self.edge_pt_begin[e])
                h.update(self.pt_values[b:b + int(ns[e] * nt[e])].tobytes())
            out.append(h.digest())
        return out

    def build_tiles(self, tile_entries: Optional[int] = None, dedupe: bool = False, max_copies: int = 16,
                    signatures=None, rows_per_wavefront_pass: Optional[int] = None) -> None:
        """Cuts every edge matrix into rectangles of about ``tile_entries`` entries:
        whole rows when a row fits the LDS column budget, column chunks otherwise.  With
        ``dedupe`` only the first of every group of identical edges is tiled; its tiles
        store their values to all copies.  (Call it after the strategy table is final:
        the compute-cost inputs are part of an edge's identity.)  One tiled edge serves at
        most ``max_copies - 1`` duplicates, so a long run of identical edges still spreads
        over many workgroups.  ``tile_entries=None`` chooses tile size and copies per tiled
        edge from the table (``tiling`` records the choice).  ``rows_per_wavefront_pass = w``: a
        tile of whole rows holds at most ``w * (64 // columns)`` of them, what ``w`` wavefronts that
        each walk ``64 // columns`` whole rows at a time cover in one pass (the packed-tile launch
        of a small table, whose slowest workgroup decides the launch; the automatic choice sets it
        to 4 for such a table)."""
        if tile_entries is None:
            sigs = self.edge_signatures() if dedupe and self.n_edges else None
            te, mc = APC_TILE_MAX_ROWS * APC_TILE_MAX_COLS, int(max_copies)
            small = self.n_entries <= AUTO_SMALL_TABLE_ENTRIES
            while True:
                self.build_tiles(te, dedupe, mc, signatures=sigs, rows_per_wavefront_pass=4 if small else None)
                n = self.n_tiles
                if n == 0 or n >= AUTO_MIN_TILES or self.n_entries / n <= AUTO_MIN_STORED_PER_TILE \
                        or self.n_entries <= AUTO_SMALL_TABLE_ENTRIES:
                    break
                if dedupe and mc > 4:
                    mc //= 2
                elif te > 2048:
                    te //= 2
                elif dedupe and mc > 2:
                    mc //= 2
                elif te > AUTO_MIN_TILE_ENTRIES:
                    te //= 2
                else:
                    break
            return
        self.tiling = {"tile_entries": int(tile_entries), "max_copies": int(max_copies) if dedupe else 1}
        if rows_per_wavefront_pass:
            self.tiling["rows_per_wavefront_pass"] = int(rows_per_wavefront_pass)
        ns = self.edge_n_src.astype(np.int64)
        nt = self.edge_n_tgt.astype(np.int64)
        canonical = np.arange(self.n_edges, dtype=np.int64)
        if dedupe and self.n_edges:
            first: dict = {}  # signature -> [canonical edge, copies it already serves]
            for e, sig in enumerate(signatures if signatures is not None else self.edge_signatures()):
                slot = first.get(sig)
                if slot is None or slot[1] >= min(APC_TILE_MAX_DUPS, max(int(max_copies) - 1, 0)):
                    first[sig] = [e, 0]  # a new canonical edge (also when the previous one is full)
                else:
                    canonical[e] = slot[0]
                    slot[1] += 1
        self.edge_canonical = canonical
        is_dup = canonical != np.arange(self.n_edges)
        # duplicates grouped by canonical edge (stable: in edge order)
        dup_edges = np.nonzero(is_dup)[0]
        order = np.argsort(canonical[dup_edges], kind="stable")
        dup_edges = dup_edges[order]
        self.dup_entry_begin = _i64(self.edge_entry_begin[:-1][dup_edges]) if self.n_edges else _i64([])
        self.dup_row_begin = _i64(self.edge_row_begin()[dup_edges]) if self.n_edges else _i64([])
        self.edge_dup_count = np.bincount(canonical[dup_edges], minlength=self.n_edges).astype(np.int64)
        self.edge_dup_begin = np.cumsum(self.edge_dup_count) - self.edge_dup_count
        live = (ns > 0) & (nt > 0) & ~is_dup
        ns1 = np.maximum(ns, 1)
        nt1 = np.maximum(nt, 1)
        ncc = -(-ns1 // APC_TILE_MAX_COLS)  # column chunks per edge
        cw = -(-ns1 // ncc)  # chunk width
        rpt = np.clip(tile_entries // cw, 1, APC_TILE_MAX_ROWS)
        if rows_per_wavefront_pass:
            rpt = np.where(ncc == 1, np.minimum(rpt, int(rows_per_wavefront_pass) * np.maximum(64 // cw, 1)), rpt)
        nrt = -(-nt1 // rpt)  # row tiles per edge
        rpt = -(-nt1 // nrt)  # balanced rows per tile
        per_edge = np.where(live, ncc * nrt, 0)
        total = int(per_edge.sum())
        te = np.repeat(np.arange(self.n_edges, dtype=np.int64), per_edge)
        first_tile = np.cumsum(per_edge) - per_edge
        k = np.arange(total, dtype=np.int64) - np.repeat(first_tile, per_edge)
        ci = k % ncc[te]
        ri = k // ncc[te]
        col_begin = ci * cw[te]
        row_begin = ri * rpt[te]
        self.tile_edge = _i32(te)
        self.tile_col_begin = _i32(col_begin)
        self.tile_col_count = _i32(np.minimum(cw[te], ns[te] - col_begin))
        self.tile_row_begin = _i32(row_begin)
        self.tile_row_count = _i32(np.minimum(rpt[te], nt[te] - row_begin))
        self.pack_tile_records()

    def pack_tile_records(self) -> None:
        """The tile rectangles plus the fields of their edge, as the packed records the
        table kernel reads (C struct ``apc_tile``)."""
        te = self.tile_edge.astype(np.int64)
        if self.edge_canonical is None or len(self.edge_canonical) != self.n_edges:
            self.edge_canonical = np.arange(self.n_edges, dtype=np.int64)
            self.dup_entry_begin = _i64([])
            self.dup_row_begin = _i64([])
            self.edge_dup_count = np.zeros(self.n_edges, np.int64)
            self.edge_dup_begin = np.zeros(self.n_edges, np.int64)
        rec = np.zeros(len(te), TILE_DTYPE)
        inside = (te >= 0) & (te < self.n_edges)
        tc = np.where(inside, te, 0)  # (out-of-range tiles are reported by validate())
        rec["edge"] = self.tile_edge
        rec["row_begin"], rec["col_begin"] = self.tile_row_begin, self.tile_col_begin
        rec["counts"] = (self.tile_row_count.astype(np.int64) & 0xFFFF) | ((self.tile_col_count.astype(np.int64) & 0x7FFF) << 16)
        if len(te) and self.n_edges:
            rec["src_begin"] = self.edge_src_begin[tc]
            rec["n_src"] = self.edge_n_src[tc]
            rec["tgt_begin"] = self.edge_tgt_begin[tc]
            rec["flags"] = self.edge_flags[tc]
            rec["strat_begin"] = self.edge_strat_begin[tc]
            rec["entry_begin"] = self.edge_entry_begin[:-1][tc]
            rec["pt_begin"] = self.edge_pt_begin[tc]
            rec["dup_begin"] = self.edge_dup_begin[tc]
            rec["dup_count"] = self.edge_dup_count[tc]
        if len(te) and self.n_specs and self.n_edges:
            # (indices are clipped here; validate() reports ranges that fall outside the table)
            first = np.clip(self.edge_src_begin[tc].astype(np.int64) + self.tile_col_begin, 0, self.n_specs - 1)
            rec["tensor"] = self.spec_tensor[first]
        self.tile_records = rec

    # ---- packed tiles ------------------------------------------------------------------
    def packable(self) -> bool:
        """Every tile holds whole rows of at most APC_TILE_MAX_COLS columns and serves at most
        APC_PACKED_MAX_DUPS identical edges: the table can be built from packed tiles."""
        if self.n_tiles == 0 or not self.rows_fit_tiles():
            return False
        if int(self.tile_records["dup_count"].max()) > APC_PACKED_MAX_DUPS:
            return False
        return bool(self.n_strategies == 0 or int(self.strat_num_args.max()) <= 0x7FFF)

    def pack_tiles(self) -> np.ndarray:
        """One ``apc_packed_tile`` record per tile: the tile's header, its tensor's row, the
        first entries / rows of its identical edges, its producer and consumer specs and its
        consumer strategies' rows of the strategy table, copied out of the tables (after the
        strategy table is final).  A workgroup then loads nothing whose address depends on
        another load."""
        if not self.packable():
            raise RuntimeError("packed tiles need whole rows in every tile and at most "
                               f"{APC_PACKED_MAX_DUPS} identical edges per tile")
        rec = self.tile_records
        n = len(rec)
        pk = np.zeros(n, PACKED_TILE_DTYPE)
        rows = (rec["counts"] & 0xFFFF).astype(np.int64)
        cols = (rec["counts"] >> 16).astype(np.int64)
        rb = rec["row_begin"].astype(np.int64)
        edge = rec["edge"].astype(np.int64)
        first = rb * cols
        pk["rows"], pk["cols"], pk["dup_count"], pk["tensor"], pk["edge"] = rows, cols, rec["dup_count"], rec["tensor"], rec["edge"]
        pk["entry_begin"] = rec["entry_begin"] + first
        pk["row_begin"] = self.edge_row_begin()[edge] + rb
        pk["pt_begin"] = np.where(rec["pt_begin"] < 0, -1, rec["pt_begin"] + first)
        t = rec["tensor"].astype(np.int64)
        has = t >= 0
        tc = np.where(has, t, 0)
        if self.n_tensors:
            pk["tensor_rank"] = np.where(has, self.tensor_rank[tc], 0)
            pk["tensor_itemsize"] = np.where(has, self.tensor_itemsize[tc], 0)
            pk["tensor_shape"] = np.where(has[:, None], self.tensor_shape[tc], 0)
            pk["tensor_stride"] = np.where(has[:, None], self.tensor_stride[tc], 0)
        j = np.arange(APC_TILE_MAX_COLS, dtype=np.int64)[None, :]
        # producer specs
        live = j < cols[:, None]
        sp = np.where(live, rec["src_begin"].astype(np.int64)[:, None] + j, 0)
        pk["col_codes"] = np.where(live, self.spec_codes[sp], 0)
        col_tensor = np.where(live, self.spec_tensor[sp], 0)
        pk["col_tensor"] = col_tensor
        mixed = (live & ((col_tensor < 0) | (col_tensor != rec["tensor"][:, None]))).any(axis=1)
        # consumer specs and their strategies
        live = j < rows[:, None]
        ts = np.where(live, (rec["tgt_begin"].astype(np.int64) + rb)[:, None] + j, 0)
        pk["row_codes"] = np.where(live, self.spec_codes[ts], 0)
        row_tensor = np.where(live, self.spec_tensor[ts], 0)
        pk["row_tensor"] = row_tensor
        mixed |= (live & (row_tensor < 0)).any(axis=1)
        sr = np.where(live, (rec["strat_begin"].astype(np.int64) + rb)[:, None] + j, 0)
        pk["row_flops"] = np.where(live, self.strat_flops[sr], 0)
        pk["row_rw_bytes"] = np.where(live, self.strat_rw_bytes[sr], 0)
        meta = (self.strat_dtype[sr].astype(np.int64) & 0xFF) | ((self.strat_zero_cost[sr] != 0).astype(np.int64) << 8) \
            | (self.strat_num_args[sr].astype(np.int64) << 16)
        pk["row_meta"] = np.where(live, meta, 0).astype(np.int32)
        pk["flags"] = rec["flags"] | np.where(mixed, PACKED_MIXED, 0)
        # identical edges
        d = np.arange(APC_PACKED_MAX_DUPS, dtype=np.int64)[None, :]
        live = d < rec["dup_count"].astype(np.int64)[:, None]
        if len(self.dup_entry_begin):
            at = np.where(live, rec["dup_begin"].astype(np.int64)[:, None] + d, 0)
            pk["dup_entry_begin"] = np.where(live, self.dup_entry_begin[at] + first[:, None], 0)
            pk["dup_row_begin"] = np.where(live, self.dup_row_begin[at] + rb[:, None], 0)
        return pk

    def validate_packed(self, packed: np.ndarray) -> None:
        """The packed records against the tables, through the library's host-side check."""
        def p(a):
            return np.ascontiguousarray(a).ctypes.data_as(ctypes.c_void_p)

        keep = [np.ascontiguousarray(a) for a in (
            self.tensor_rank, self.tensor_itemsize, self.tensor_shape, self.tensor_stride, self.spec_codes, self.spec_tensor,
            self.strat_flops, self.strat_rw_bytes, self.strat_dtype, self.strat_zero_cost, self.strat_num_args,
            self.edge_row_begin(), self.tile_records, self.dup_entry_begin, self.dup_row_begin, packed)]
        (rank, item, shape, stride, codes, owner, flops, rw, dt, zero, nargs, erb, tiles, dups, dup_rows, pk) = keep
        rc = _native.lib().apc_validate_packed_tiles_host(
            ctypes.c_int64(self.n_tensors), p(rank), p(item), p(shape), p(stride), ctypes.c_int64(self.n_specs), p(codes), p(owner),
            ctypes.c_int64(self.n_strategies), p(flops), p(rw), p(dt), p(zero), p(nargs), ctypes.c_int64(self.n_edges), p(erb),
            ctypes.c_int64(self.n_tiles), p(tiles), ctypes.c_int64(len(dups)), p(dups), p(dup_rows), p(pk))
        _native.check(rc, "apc_validate_packed_tiles_host")

    # ---- checks ------------------------------------------------------------------------
    def validate(self, params) -> None:
        """Structural check through the library's host-side validator; raises
        RuntimeError naming the first malformed row."""
        if tuple(params.mesh_sizes) != self.mesh_sizes:
            raise RuntimeError(f"tables were encoded for mesh {self.mesh_sizes}, params describe {params.mesh_sizes}")
        if len(self.edge_entry_begin) != self.n_edges + 1:
            raise RuntimeError("edge_entry_begin must have n_edges + 1 rows")
        for name in ("edge_src_begin", "edge_tgt_begin", "edge_flags", "edge_pt_begin", "edge_strat_begin",
                     "edge_n_tgt"):
            if len(getattr(self, name)) != self.n_edges:
                raise RuntimeError(f"{name} must have n_edges rows")
        if len(self.spec_tensor) != self.n_specs:
            raise RuntimeError("spec_tensor must have n_specs rows")
        for name in ("strat_rw_bytes", "strat_dtype", "strat_zero_cost", "strat_num_args"):
            if len(getattr(self, name)) != self.n_strategies:
                raise RuntimeError(f"{name} must have n_strategies rows")
        if self.n_strategies and int(self.strat_num_args.min()) < 1:
            raise RuntimeError("strat_num_args must be >= 1")
        if (self.strat_flops >= 2**53).any() or (self.strat_rw_bytes >= 2**53).any():
            raise RuntimeError("flop / byte counts must stay below 2**53 to convert to fp64 exactly")
        cp = params.to_c()
        if self.tile_records is None or len(self.tile_records) != self.n_tiles:
            raise RuntimeError("tile_records must have one record per tile (call pack_tile_records())")

        def p(a):
            return a.ctypes.data_as(ctypes.c_void_p)

        rc = _native.lib().apc_validate_tables_host(
            ctypes.byref(cp), ctypes.c_int64(self.n_tensors), p(self.tensor_rank),
            ctypes.c_int64(self.n_specs), p(self.spec_codes), p(self.spec_tensor),
            ctypes.c_int64(self.n_edges), p(self.edge_src_begin), p(self.edge_n_src), p(self.edge_tgt_begin),
            p(self.edge_n_tgt), p(self.edge_flags), p(self.edge_pt_begin), p(self.edge_entry_begin),
            p(self.edge_strat_begin), ctypes.c_int64(len(self.pt_values)), ctypes.c_int64(self.n_strategies),
            ctypes.c_int64(self.n_tiles), p(self.tile_records), ctypes.c_int64(len(self.dup_entry_begin)),
            p(self.dup_entry_begin))
        _native.check(rc, "apc_validate_tables_host")
        # every edge is either tiled completely or a duplicate of an edge that is
        area = np.zeros(self.n_edges, np.int64)
        np.add.at(area, self.tile_edge.astype(np.int64),
                  self.tile_row_count.astype(np.int64) * self.tile_col_count.astype(np.int64))
        want = self.edge_n_src.astype(np.int64) * self.edge_n_tgt.astype(np.int64)
        tiled = self.edge_canonical == np.arange(self.n_edges)
        if not np.array_equal(area[tiled], want[tiled]) or area[~tiled].any():
            raise RuntimeError("tiles do not cover every (non-duplicate) edge matrix exactly once")
        if int(self.edge_dup_count.sum()) != int((~tiled).sum()) or len(self.dup_entry_begin) != int((~tiled).sum()):
            raise RuntimeError("duplicate-edge lists do not account for every de-duplicated edge")
        # byte counts must convert to fp64 exactly (the kernels divide them as doubles)
        if self.n_tensors:
            r = np.arange(APC_MAX_RANK)[None, :] < self.tensor_rank[:, None]
            if (np.where(r, self.tensor_shape, 0) < 0).any():
                raise RuntimeError("tensor sizes must not be negative")
            numel = np.where(r, self.tensor_shape, 1).astype(object).prod(axis=1)
            if (numel * self.tensor_itemsize.astype(object) >= 2**53).any():
                raise RuntimeError("tensor byte counts must stay below 2**53")

    def as_dict(self) -> dict:
        """Plain-data view (numpy arrays) of every table."""
        out = {"mesh_sizes": self.mesh_sizes}
        for f in fields(self):
            if f.name != "mesh_sizes":
                out[f.name] = getattr(self, f.name)
        return out

    # ---- derived index arrays ------------------------------------------------------------
    def strategy_bound_index(self) -> dict:
        """Index arrays of the per-strategy lower bounds (C entry ``apc_strategy_bounds``):
        the node of every strategy, every node's edges (as consumer) in edge order, and the
        first matrix row of every edge in the order of ``row_ptr()``."""
        n_nodes = self.n_nodes
        n_strat = np.diff(self.node_strat_begin).astype(np.int64)
        node = self.edge_node.astype(np.int64)
        if self.n_edges and (node.min() < 0 or node.max() >= n_nodes):
            raise RuntimeError("edge_node outside the node table")
        if not np.array_equal(self.edge_n_tgt.astype(np.int64), n_strat[node]):
            raise RuntimeError("an edge's row count differs from its consumer node's strategy count")
        order = np.argsort(node, kind="stable")
        node_edge_begin = np.zeros(n_nodes + 1, np.int64)
        np.cumsum(np.bincount(node, minlength=n_nodes), out=node_edge_begin[1:])
        edge_row_begin = np.cumsum(self.edge_n_tgt.astype(np.int64)) - self.edge_n_tgt
        return {
            "strat_node": _i32(np.repeat(np.arange(n_nodes, dtype=np.int64), n_strat)),
            "node_edge_begin": node_edge_begin,
            "edges_by_node": _i32(order),
            "edge_row_begin": _i64(edge_row_begin),
        }

    def edge_row_begin(self) -> np.ndarray:
        """First matrix row of every edge: rows are numbered edge by edge, one per consumer
        strategy (the order of ``row_ptr()``)."""
        nt = self.edge_n_tgt.astype(np.int64)
        return _i64(np.cumsum(nt) - nt)

    def rows_fit_tiles(self) -> bool:
        """Every matrix row lies inside one tile (and none is empty), so the launch that writes
        the cost matrices can take the row minima itself."""
        ns = self.edge_n_src.astype(np.int64)
        nt = self.edge_n_tgt.astype(np.int64)
        with_rows = nt > 0
        if not bool(((ns[with_rows] >= 1) & (ns[with_rows] <= APC_TILE_MAX_COLS)).all()):
            return False
        te = self.tile_edge.astype(np.int64)
        return bool((self.tile_col_begin == 0).all() and (self.tile_col_count == ns[te]).all())

    def row_copies(self):
        """-> (selected, copy_ptr, copy_rows, n_values_selected): the matrix rows of the edges that
        are tiled, and for each of them the rows of the identical edges that receive the same
        values (rows numbered as in ``row_ptr()``).  A minimum taken over ``selected`` and
        stored to the copies covers every row while reading each distinct row once."""
        nt = self.edge_n_tgt.astype(np.int64)
        ns = self.edge_n_src.astype(np.int64)
        rb = self.edge_row_begin()
        canon = np.nonzero(self.edge_canonical == np.arange(self.n_edges))[0]
        ntc = nt[canon]
        n_sel = int(ntc.sum())
        first = np.cumsum(ntc) - ntc
        r = np.arange(n_sel, dtype=np.int64) - np.repeat(first, ntc)  # consumer strategy of every selected row
        selected = np.repeat(rb[canon], ntc) + r
        per_row = np.repeat(self.edge_dup_count[canon].astype(np.int64), ntc)
        copy_ptr = np.zeros(n_sel + 1, np.int64)
        np.cumsum(per_row, out=copy_ptr[1:])
        which = np.repeat(np.arange(n_sel, dtype=np.int64), per_row)
        k = np.arange(int(copy_ptr[-1]), dtype=np.int64) - copy_ptr[which]
        dup_first = np.repeat(self.edge_dup_begin[canon].astype(np.int64), ntc)
        copy_rows = self.dup_row_begin[dup_first[which] + k] + r[which] if len(which) else _i64([])
        return _i64(selected), _i64(copy_ptr), _i64(copy_rows), int((ns[canon] * ntc).sum())

    def row_ptr(self) -> np.ndarray:
        """CSR pointer of matrix rows over the entry array: one segment per
        (edge, consumer strategy), length = that edge's producer count."""
        ns = self.edge_n_src.astype(np.int64)
        nt = self.edge_n_tgt.astype(np.int64)
        lens = np.repeat(ns, nt)
        out = np.zeros(len(lens) + 1, np.int64)
        np.cumsum(lens, out=out[1:])
        return out
