"""Host-side checks that need no GPU: the C-ABI library loads and exports every
symbol the public header declares; the flattened encoding's tiles cover every
entry exactly once; the host validator rejects malformed tables; the cost-model
parameters reproduce the reference's environment lookups."""

import ctypes
import os
import re

import numpy as np
import pytest

from autoparallel_amd import CostModelParams, _native, get_device_limit, mesh_topology
from autoparallel_amd.encoding import (EDGE_NO_PRODUCER, CostTables, code_dim, code_kind, pack_codes, partial_code,
                                       shard_code, unpack_codes)
from autoparallel_amd.synthetic import stress_dag

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "apcost.h")).read()
    declared = set(re.findall(r"\b(apc_[a-z_0-9]+)\s*\(", header))
    assert declared, "no declarations found in include/apcost.h"
    lib = _native.lib()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in apcost.h but not exported"
    assert declared == set(_native.EXPORTS)
    # the header's constant, the library's answer and the binding's mirror agree
    version = int(re.search(r"#define APC_ABI_VERSION (\d+)", header).group(1))
    assert lib.apc_version() == version == _native.APC_ABI_VERSION


def test_params_struct_layout_matches_header(tmp_path):
    """The ctypes mirrors against the C compiler's own layout of include/apcost.h."""
    import subprocess

    fields_p = [name for name, _ in _native.ApcParams._fields_]
    fields_t = [name for name, _ in _native.ApcTile._fields_]
    src = tmp_path / "layout.c"
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "apcost.h"', 'int main(void) {',
             '  printf("%zu %zu\\n", sizeof(apc_params), sizeof(apc_tile));']
    lines += [f'  printf("%zu\\n", offsetof(apc_params, {f}));' for f in fields_p]
    lines += [f'  printf("%zu\\n", offsetof(apc_tile, {f}));' for f in fields_t]
    lines += ['  return 0;', '}']
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include"),
                    "-o", str(exe), str(src)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert [int(out[0]), int(out[1])] == [ctypes.sizeof(_native.ApcParams), ctypes.sizeof(_native.ApcTile)]
    want = [getattr(_native.ApcParams, f).offset for f in fields_p] + [getattr(_native.ApcTile, f).offset for f in fields_t]
    assert [int(x) for x in out[2:]] == want
    assert ctypes.sizeof(_native.ApcTile) == 64  # one record per scalar 64-byte load


def test_placement_codes_round_trip():
    codes = (0, partial_code("sum"), partial_code("max"), shard_code(3))
    assert unpack_codes(pack_codes(codes), 4) == codes
    assert [code_kind(c) for c in codes] == [0, 1, 1, 2]
    assert code_dim(shard_code(3)) == 3 and shard_code(2, variant=1) != shard_code(2)
    with pytest.raises(ValueError):
        shard_code(16)


def test_launch_entry_points_fail_loudly_without_a_device():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a HIP device is present")
    from autoparallel_amd.device_tables import DeviceCostTables

    tb = stress_dag(seed=0, n_nodes=10, mesh_sizes=(4, 2))
    with pytest.raises(RuntimeError, match="no CPU path"):
        DeviceCostTables(tb, CostModelParams.from_mesh((4, 2)))


@pytest.mark.parametrize("tile_entries", [64, 1000, 4096])
def test_tiles_cover_every_entry_exactly_once(tile_entries):
    tb = stress_dag(seed=3, n_nodes=300, mesh_sizes=(4, 4, 2), max_strategies=80, tile_entries=tile_entries)
    seen = np.zeros(tb.n_entries, np.int32)
    for t in range(tb.n_tiles):
        e = tb.tile_edge[t]
        ns = int(tb.edge_n_src[e])
        r0, rc, c0, cc = (int(x[t]) for x in (tb.tile_row_begin, tb.tile_row_count, tb.tile_col_begin, tb.tile_col_count))
        assert 1 <= rc <= _native.APC_TILE_MAX_ROWS and 1 <= cc <= _native.APC_TILE_MAX_COLS
        rows = np.arange(r0, r0 + rc)[:, None] * ns + np.arange(c0, c0 + cc)[None, :]
        seen[int(tb.edge_entry_begin[e]) + rows.ravel()] += 1
    assert (seen == 1).all()


def twin_graph(tb: CostTables) -> CostTables:
    """A copy of every node, spec and edge appended to the tables (tensors shared): every
    edge then has an identical twin, like the layers of a transformer."""
    S, NS, NP = tb.n_strategies, tb.n_specs, len(tb.pt_values)
    cat = np.concatenate
    eb = tb.edge_entry_begin
    return CostTables(
        mesh_sizes=tb.mesh_sizes, tensor_rank=tb.tensor_rank, tensor_itemsize=tb.tensor_itemsize,
        tensor_shape=tb.tensor_shape, tensor_stride=tb.tensor_stride,
        spec_codes=cat([tb.spec_codes, tb.spec_codes]), spec_tensor=cat([tb.spec_tensor, tb.spec_tensor]),
        strat_flops=cat([tb.strat_flops] * 2), strat_rw_bytes=cat([tb.strat_rw_bytes] * 2),
        strat_dtype=cat([tb.strat_dtype] * 2), strat_zero_cost=cat([tb.strat_zero_cost] * 2),
        strat_num_args=cat([tb.strat_num_args] * 2),
        node_strat_begin=cat([tb.node_strat_begin, tb.node_strat_begin[1:] + S]),
        edge_node=cat([tb.edge_node, tb.edge_node + tb.n_nodes]), edge_arg=cat([tb.edge_arg] * 2),
        edge_src_begin=cat([tb.edge_src_begin, tb.edge_src_begin + NS]), edge_n_src=cat([tb.edge_n_src] * 2),
        edge_tgt_begin=cat([tb.edge_tgt_begin, tb.edge_tgt_begin + NS]), edge_n_tgt=cat([tb.edge_n_tgt] * 2),
        edge_flags=cat([tb.edge_flags] * 2),
        edge_pt_begin=cat([tb.edge_pt_begin, np.where(tb.edge_pt_begin >= 0, tb.edge_pt_begin + NP, -1)]),
        edge_entry_begin=cat([eb, eb[1:] + eb[-1]]), edge_strat_begin=cat([tb.edge_strat_begin, tb.edge_strat_begin + S]),
        pt_values=cat([tb.pt_values] * 2))


def test_deduplicated_tiles_write_every_entry_exactly_once():
    base = stress_dag(seed=8, n_nodes=120, mesh_sizes=(4, 2), max_strategies=20)
    tb = twin_graph(base)
    tb.build_tiles(256, dedupe=True)
    tb.validate(CostModelParams.from_mesh((4, 2)))
    n_dup = int((tb.edge_canonical != np.arange(tb.n_edges)).sum())
    assert n_dup >= base.n_edges  # every appended edge has its original as twin
    seen = np.zeros(tb.n_entries, np.int32)
    rec = tb.tile_records
    for t in range(tb.n_tiles):
        e = int(rec["edge"][t])
        ns = int(tb.edge_n_src[e])
        rc, cc = int(rec["counts"][t]) & 0xFFFF, int(rec["counts"][t]) >> 16
        local = (np.arange(rec["row_begin"][t], rec["row_begin"][t] + rc)[:, None] * ns
                 + np.arange(rec["col_begin"][t], rec["col_begin"][t] + cc)[None, :]).ravel()
        seen[int(tb.edge_entry_begin[e]) + local] += 1
        for d in range(int(rec["dup_count"][t])):
            seen[int(tb.dup_entry_begin[int(rec["dup_begin"][t]) + d]) + local] += 1
    assert (seen == 1).all()
    # edges that differ in anything their matrix depends on are not merged
    other = twin_graph(base)
    other.strat_flops[other.n_strategies // 2:] += 1
    other.build_tiles(256, dedupe=True)
    assert int((other.edge_canonical != np.arange(other.n_edges)).sum()) < n_dup


def test_row_minimum_entry_points_reject_incomplete_arguments():
    """Argument checks of apc_*_row_min run on the host before anything is launched: a NULL
    descriptor, a descriptor without its arrays, identical edges without their rows; the host
    check of the whole-row precondition; the objective's argument checks."""
    import ctypes

    lib = _native.lib()
    p = CostModelParams.from_mesh((4, 2)).to_c()
    one = ctypes.c_void_p(8)  # a non-NULL placeholder: every call below fails before it is read
    tables = (ctypes.byref(p), one, one, one, one, None, one, ctypes.c_int64(1), one, None, ctypes.c_int64(1))

    def error_of(rc):
        assert rc != 0
        return lib.apc_last_error().decode()

    assert "NULL rows" in error_of(lib.apc_redistribute_tables_row_min(*tables, one, one, one, None, None))
    empty = _native.ApcRowMinima(None, None, None, None)
    assert "NULL row-minimum array" in error_of(
        lib.apc_redistribute_tables_row_min(*tables, one, one, one, ctypes.byref(empty), None))
    rows = _native.ApcRowMinima(one, None, one, one)
    with_dups = tables[:9] + (one,) + tables[10:]
    assert "dup_row_begin" in error_of(
        lib.apc_redistribute_tables_row_min(*with_dups, one, one, one, ctypes.byref(rows), None))
    assert "NULL selection" in error_of(lib.apc_segmented_min_copies(
        one, one, ctypes.c_int64(3), None, None, None, ctypes.c_int64(9), one, one, None))
    assert "no group" in error_of(lib.apc_cost_objective(
        ctypes.c_int64(4), ctypes.c_int64(0), one, one, one, one, ctypes.c_double(10000.0), one, one, None))
    assert "NULL array" in error_of(lib.apc_cost_objective(
        ctypes.c_int64(4), ctypes.c_int64(1), one, one, one, None, ctypes.c_double(10000.0), one, one, None))


def test_row_minimum_precondition_is_checked_on_the_host():
    """apc_validate_row_minima_host: tiles of whole rows pass; an edge with more producer
    strategies than a tile holds, or a tile cut by columns, is named."""
    tb = stress_dag(seed=5, n_nodes=60, mesh_sizes=(4, 2))
    tb.build_tiles(4096)
    assert tb.rows_fit_tiles()
    tb.validate_row_minima()
    wide = stress_dag(seed=5, n_nodes=60, mesh_sizes=(4, 2), max_strategies=100)
    wide.build_tiles(4096)
    assert not wide.rows_fit_tiles()
    with pytest.raises(RuntimeError, match="producer strategies"):
        wide.validate_row_minima()
    # cut one tile by columns: same edge, half the columns
    rec = tb.tile_records.copy()
    t = int(np.argmax((rec["counts"] >> 16) >= 2))
    rc, cc = int(rec["counts"][t]) & 0xFFFF, int(rec["counts"][t]) >> 16
    assert cc >= 2
    rec["counts"][t] = rc | ((cc // 2) << 16)
    tb.tile_records = rec
    with pytest.raises(RuntimeError, match="not the whole rows"):
        tb.validate_row_minima()


def test_row_copies_cover_every_row_once_and_pair_identical_rows():
    """``row_copies``: the rows of the tiled edges plus their copies are every matrix row exactly
    once; a copy is the same consumer strategy of an identical edge; rows are numbered as in
    ``row_ptr`` / ``edge_row_begin`` (what the row-minimum launches write to)."""
    tb = twin_graph(stress_dag(seed=3, n_nodes=150, mesh_sizes=(4, 2), frac_nonspec_nodes=0.03))
    tb.build_tiles(1024, dedupe=True, max_copies=8)
    selected, copy_ptr, copy_rows, n_read = tb.row_copies()
    n_rows = int(tb.edge_n_tgt.sum())
    seen = np.zeros(n_rows, np.int64)
    np.add.at(seen, selected, 1)
    np.add.at(seen, copy_rows, 1)
    assert (seen == 1).all() and len(copy_rows) > 0
    row_edge = np.repeat(np.arange(tb.n_edges), tb.edge_n_tgt)
    rb = tb.edge_row_begin()
    assert np.array_equal(rb, np.cumsum(tb.edge_n_tgt.astype(np.int64)) - tb.edge_n_tgt)
    which = np.repeat(np.arange(len(selected)), np.diff(copy_ptr))
    assert np.array_equal(tb.edge_canonical[row_edge[copy_rows]], row_edge[selected[which]])
    assert np.array_equal(copy_rows - rb[row_edge[copy_rows]], selected[which] - rb[row_edge[selected[which]]])
    lens = np.diff(tb.row_ptr())
    assert n_read == int(lens[selected].sum()) < tb.n_entries
    # the rows the tiles' duplicate lists name are the same ones
    for e in np.nonzero(tb.edge_dup_count)[0][:20]:
        dups = tb.dup_row_begin[tb.edge_dup_begin[e]:tb.edge_dup_begin[e] + tb.edge_dup_count[e]]
        assert np.array_equal(tb.edge_canonical[row_edge[dups]], np.full(len(dups), e))
    # without identical edges: every row selected, no copies
    plain = stress_dag(seed=3, n_nodes=50, mesh_sizes=(4, 2))
    selected, copy_ptr, copy_rows, n_read = plain.row_copies()
    assert np.array_equal(selected, np.arange(int(plain.edge_n_tgt.sum()))) and len(copy_rows) == 0
    assert n_read == plain.n_entries and plain.rows_fit_tiles()


def test_validator_rejects_bad_duplicate_offsets():
    tb = twin_graph(stress_dag(seed=8, n_nodes=60, mesh_sizes=(4, 2), max_strategies=10))
    tb.build_tiles(256, dedupe=True)
    tb.dup_entry_begin[0] += 1
    with pytest.raises(RuntimeError, match="duplicate offset"):
        tb.validate(CostModelParams.from_mesh((4, 2)))


def test_wide_edges_are_cut_into_column_chunks():
    # one consumer with 3 strategies reading a producer with 2500 strategies
    n_src, n_tgt = 2500, 3
    tb = CostTables(
        mesh_sizes=(4,), tensor_rank=[1], tensor_itemsize=[4], tensor_shape=[[64] + [0] * 7],
        tensor_stride=[[1] + [0] * 7], spec_codes=np.zeros(n_src + n_tgt, np.uint32),
        spec_tensor=np.zeros(n_src + n_tgt, np.int32), strat_flops=np.zeros(n_tgt), strat_rw_bytes=np.zeros(n_tgt),
        strat_dtype=np.ones(n_tgt), strat_zero_cost=np.zeros(n_tgt), strat_num_args=np.ones(n_tgt),
        node_strat_begin=[0, n_tgt], edge_node=[0], edge_arg=[0], edge_src_begin=[0], edge_n_src=[n_src],
        edge_tgt_begin=[n_src], edge_n_tgt=[n_tgt], edge_flags=[0], edge_pt_begin=[-1],
        edge_entry_begin=[0, n_src * n_tgt], edge_strat_begin=[0], pt_values=[])
    assert tb.n_tiles >= 3 and int(tb.tile_col_count.max()) <= _native.APC_TILE_MAX_COLS
    assert int(tb.tile_col_count.astype(np.int64).dot(tb.tile_row_count)) == n_src * n_tgt
    tb.validate(CostModelParams.from_mesh((4,)))


def _small():
    return stress_dag(seed=5, n_nodes=40, mesh_sizes=(4, 2), max_strategies=8)


def test_validator_accepts_generated_tables():
    _small().validate(CostModelParams.from_mesh((4, 2)))


@pytest.mark.parametrize("mutate, message", [
    (lambda t: t.tensor_rank.__setitem__(0, 9), "rank"),
    (lambda t: t.spec_tensor.__setitem__(3, 10**6), "tensor row"),
    (lambda t: t.spec_codes.__setitem__(0, 0xC0), "no meaning"),
    (lambda t: t.spec_codes.__setitem__(0, 0x01), "no meaning"),
    (lambda t: t.spec_codes.__setitem__(0, 0x8F), "Shard"),
    (lambda t: t.spec_codes.__setitem__(0, 0x800000), "beyond mesh ndim"),
    (lambda t: t.edge_entry_begin.__setitem__(2, int(t.edge_entry_begin[2]) + 1), "entry_begin"),
    (lambda t: t.edge_src_begin.__setitem__(1, t.n_specs), "producer spec range"),
    (lambda t: t.edge_strat_begin.__setitem__(1, t.n_strategies), "strategy rows"),
    (lambda t: t.edge_n_src.__setitem__(1, (1 << 22) + 1), "strategies"),
    (lambda t: t.tile_row_count.__setitem__(0, 10**4), "rows"),
    (lambda t: t.tile_col_begin.__setitem__(0, -1), "cols"),
])
def test_validator_rejects_malformed_tables(mutate, message):
    tb = _small()
    mutate(tb)
    tb.pack_tile_records()
    with pytest.raises(RuntimeError, match=message):
        tb.validate(CostModelParams.from_mesh((4, 2)))


def test_validator_rejects_tile_record_that_disagrees_with_its_edge():
    tb = _small()
    tb.tile_records["src_begin"][0] += 1
    with pytest.raises(RuntimeError, match="does not repeat"):
        tb.validate(CostModelParams.from_mesh((4, 2)))
    tb = _small()
    tb.tile_records["edge"][0] = tb.n_edges
    with pytest.raises(RuntimeError, match="out of range"):
        tb.validate(CostModelParams.from_mesh((4, 2)))


def test_validator_rejects_a_tile_with_more_identical_edges_than_the_kernels_stage():
    """The tile kernels stage APC_TILE_MAX_DUPS offsets of identical edges in LDS; a record with
    more (a tile array built against an older header, which allowed 127) is refused on the host."""
    tb = twin_graph(stress_dag(seed=8, n_nodes=60, mesh_sizes=(4, 2), max_strategies=10))
    tb.build_tiles(256, dedupe=True)
    params = CostModelParams.from_mesh((4, 2))
    tb.validate(params)
    t = int(np.nonzero(tb.tile_records["dup_count"] > 0)[0][0])
    assert int(re.search(r"#define APC_TILE_MAX_DUPS (\d+)", open(os.path.join(ROOT, "include", "apcost.h")).read()).group(1)) \
        == _native.APC_TILE_MAX_DUPS == 32
    for bad in (_native.APC_TILE_MAX_DUPS + 1, 127, -1):
        tb.tile_records["dup_count"][t] = bad
        with pytest.raises(RuntimeError, match="duplicate list"):
            tb.validate(params)


def test_validator_rejects_a_negative_tensor_size():
    tb = _small()
    tb.tensor_shape[0, 0] = -4
    with pytest.raises(RuntimeError, match="must not be negative"):
        tb.validate(CostModelParams.from_mesh((4, 2)))


def test_validator_needs_pass_through_values_for_producerless_edges():
    tb = _small()
    e = int(np.nonzero(tb.edge_flags & EDGE_NO_PRODUCER)[0][0])
    tb.edge_pt_begin[e] = -1
    tb.pack_tile_records()
    with pytest.raises(RuntimeError, match="pass-through"):
        tb.validate(CostModelParams.from_mesh((4, 2)))


def test_validator_rejects_mesh_mismatch():
    with pytest.raises(RuntimeError, match="mesh"):
        _small().validate(CostModelParams.from_mesh((2, 4)))


def test_cost_model_params_follow_reference_environment():
    assert mesh_topology((32, 8)) == ((87.7 * 0.22, 87.7), (2.7, 0.6))
    assert mesh_topology((8, 8, 8)) == ((87.7 * 0.22, 87.7 * 0.22, 87.7), (2.7, 2.7, 0.6))
    assert mesh_topology((64,))[0] == (87.7 * 0.22,)
    assert mesh_topology((8,))[0] == (87.7,)  # strict '>' on the device product
    p = CostModelParams.from_mesh((32, 8), rescale=2.2)
    assert p.hbm_bw == 3.35 * 1024**4 and p.gpu_flops[3] == 989e12 and p.gpu_flops[1] == 494e12
    assert p.gpu_flops[5] == 0.0
    assert get_device_limit("NVIDIA H100 80GB HBM3").name == "H100"
    with pytest.raises(ValueError, match="Unsupported device"):
        CostModelParams.from_mesh((8,), device_name="AMD Instinct MI355X")
    with pytest.raises(ValueError):
        CostModelParams.from_mesh((2, 2, 2, 2, 2))
    c = p.to_c()
    assert c.mesh_ndim == 2 and list(c.mesh_size)[:2] == [32, 8] and c.rescale == 2.2


def test_oracle_and_product_agree_on_constants():
    # the oracle restates the device table and codes independently; both must say the same
    from oracle import cost_oracle as po

    for mesh in [(64,), (32, 8), (16, 8, 4)]:
        a, b = po.make_params(mesh), CostModelParams.from_mesh(mesh)
        assert a.bw == b.bw and a.lat == b.lat and a.hbm_bw == b.hbm_bw and tuple(a.gpu_flops) == tuple(b.gpu_flops)
    assert po.shard(3) == shard_code(3) and po.partial(2) == partial_code(2)
    assert po.DTYPE_CODES == __import__("autoparallel_amd.cost_model", fromlist=["x"]).DTYPE_CODES


def test_missing_library_fails_loudly(tmp_path):
    """No library, no product: loading raises (there is no CPU path to fall back to), and so
    does everything built on it."""
    import subprocess
    import sys

    code = (
        "import sys\n"
        "from autoparallel_amd import _native\n"
        "try:\n"
        "    _native.lib()\n"
        "except RuntimeError as e:\n"
        "    assert 'missing' in str(e), e\n"
        "    sys.exit(42)\n"
        "sys.exit(0)\n"
    )
    env = dict(os.environ, APCOST_LIBRARY=str(tmp_path / "no_such_libapcost.so"))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, capture_output=True, text=True)
    assert proc.returncode == 42, proc.stderr[-2000:]
