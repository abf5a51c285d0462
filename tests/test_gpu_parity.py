"""GPU parity: every kernel, called through the C ABI, against the CPU oracle on the
same seeded tables.  Bar: bit-exact for integer / byte / index outputs AND for the fp64
costs (the kernels are built with FMA contraction off and evaluate in the reference's
operation order); the stated tolerance of the path is 1e-9 relative, asserted as well
so that a future relaxation of bit-exactness cannot silently exceed it."""

import math

import numpy as np
import pytest
import torch

from autoparallel_amd import CostModelParams
from autoparallel_amd.device_tables import DeviceCostTables
from autoparallel_amd.encoding import CostTables, pack_codes, partial_code, shard_code
from autoparallel_amd.synthetic import stress_dag
from oracle import c_oracle
from oracle import cost_oracle as po

pytestmark = pytest.mark.gpu

REL_TOL = 1e-9


def _assert_costs(got: np.ndarray, want: np.ndarray, what: str):
    assert got.shape == want.shape, what
    assert np.array_equal(np.isinf(got), np.isinf(want)), f"{what}: inf pattern differs"
    fin = np.isfinite(want)
    denom = np.maximum(np.abs(want[fin]), 1e-300)
    rel = np.abs(got[fin] - want[fin]) / denom
    assert rel.size == 0 or rel.max() <= REL_TOL, f"{what}: max rel err {rel.max()}"
    assert np.array_equal(got, want), f"{what}: not bit-identical ({int((got != want).sum())} entries differ)"


def _same_rows(got: np.ndarray, want) -> bool:
    """Device rows are ``shape_width()`` wide, the oracle's 8: equal where both exist, zero beyond."""
    want = np.asarray(want, dtype=np.int64)
    if got.ndim == 1:
        return np.array_equal(got, want)
    w = got.shape[1]
    return np.array_equal(got, want[:, :w]) and not want[:, w:].any()


def _run_and_compare(tb: CostTables, mesh, rescale, device):
    p = CostModelParams.from_mesh(mesh, rescale=rescale)
    op = po.make_params(mesh, rescale=rescale)
    d = DeviceCostTables(tb, p, device=device)
    comm, trans, cost = d.build_all()
    torch.cuda.synchronize()
    enc = tb.as_dict()
    want_cc, want_pa = c_oracle.compute_costs(enc, op)
    want = c_oracle.build_tables(enc, op, per_arg=want_pa)
    _assert_costs(d.compute_cost.cpu().numpy(), want_cc, "compute_cost")
    _assert_costs(d.compute_cost_per_arg.cpu().numpy(), want_pa, "compute_cost_per_arg")
    _assert_costs(comm.cpu().numpy(), want["comm"], "comm")
    _assert_costs(cost.cpu().numpy(), want["cost"], "cost")
    assert np.array_equal(trans.cpu().numpy(), want["transition"])
    # the planner's forms of the same tables (the assembled cost alone, with the row minima in
    # the tiles where every row lies in one tile): all tables in one launch, and two launches
    fits = tb.rows_fit_tiles()
    want_rows = c_oracle.segmented_min(want["cost"], tb.row_ptr()) if fits and tb.n_entries else None
    # ... and, where every tile holds whole rows, the launch over packed tiles (every wavefront on
    # its own, entries evaluated directly in registers)
    forms = [(True, False), (False, False)] + ([(True, True)] if tb.packable() else [])
    for one_launch, packed in forms:
        dp = DeviceCostTables(tb, p, device=device, validate=False)
        step = dp.prepare_step(row_min=fits, fused_inputs=True, one_launch=one_launch, row_min_in_tiles=fits,
                               outputs=("cost",), spec_table=False, packed=packed)
        assert tuple(step) == (("build_tables_packed",) if packed else ("build_tables",) if one_launch else
                               ("input_tables", "redistribute_tables"))
        for launch in step.values():
            launch()
        torch.cuda.synchronize()
        assert dp.comm is None and dp.transition is None
        assert np.array_equal(dp.cost.cpu().numpy(), want["cost"]), f"cost alone, one_launch={one_launch}, packed={packed}"
        assert np.array_equal(dp.compute_cost_per_arg.cpu().numpy(), want_pa)
        if want_rows is not None:
            assert np.array_equal(dp.row_min.cpu().numpy(), want_rows[0]) and np.array_equal(dp.row_argmin.cpu().numpy(), want_rows[1])
    return d, want


@pytest.mark.parametrize("mesh", [(64,), (32, 8), (8, 8, 8), (64, 4), (16, 8, 4), (6, 3), (5, 3, 2), (2, 3, 2, 2),
                                  (2, 4, 2, 2), (4, 1, 2), (1,), (2048, 1024, 1024), (65536, 65536)])
def test_tables_match_oracle_on_seeded_dags(gpu_device, mesh):
    # (power-of-two meshes take the kernels' per-exponent term arrays: up to 32 exponents, which
    # the mesh of 2^31 devices needs; the others, and the last one with 33, the per-state arrays)
    tb = stress_dag(seed=11, n_nodes=1500, mesh_sizes=mesh, frac_nonspec_nodes=0.02, frac_noncontiguous=0.2)
    d, want = _run_and_compare(tb, mesh, 2.2, gpu_device)
    # integer tables: bit-exact
    enc = tb.as_dict()
    wb, wc = c_oracle.tensor_tables(enc)
    assert np.array_equal(d.tensor_bytes.cpu().numpy(), wb)
    assert np.array_equal(d.tensor_contiguous.cpu().numpy(), wc)
    got = d.run_spec_tables()
    for key, w in zip(("num_shards", "local_shape", "local_stride", "local_numel", "local_bytes"),
                      c_oracle.spec_tables(enc, mesh)):
        assert _same_rows(got[key].cpu().numpy(), w), key
    assert got["local_shape"].shape[1] == tb.shape_width() <= 8


@pytest.mark.parametrize("mesh,threads", [((4, 2), None), ((8, 4, 2), "64"), ((8, 4, 2), "256"), ((3, 2), "128")])
def test_tiles_with_the_maximum_number_of_identical_edges(gpu_device, mesh, threads, monkeypatch):
    """A tile lists at most APC_TILE_MAX_DUPS identical edges (their first entries, and first
    matrix rows for the minima, are staged in LDS): 64 copies of a graph are served by two tiled
    edges per group, whatever ``max_copies`` asks for."""
    from autoparallel_amd._native import APC_TILE_MAX_DUPS
    from test_abi_and_encoding import twin_graph

    if threads:
        monkeypatch.setenv("APC_TILE_THREADS", threads)
    tb = stress_dag(seed=31, n_nodes=40, mesh_sizes=mesh, max_strategies=12, frac_nonspec_nodes=0.05,
                    frac_noncontiguous=0.2)
    for _ in range(6):  # 64 copies of every edge
        tb = twin_graph(tb)
    tb.build_tiles(None, dedupe=True, max_copies=100)
    assert int(tb.tile_records["dup_count"].max()) == APC_TILE_MAX_DUPS == 32 and tb.rows_fit_tiles()
    _run_and_compare(tb, mesh, 2.2, gpu_device)


@pytest.mark.parametrize("mesh", [(32, 8), (16, 8, 4), (2, 4, 2, 2)])
def test_per_state_term_arrays_on_power_of_two_meshes(gpu_device, mesh, monkeypatch):
    """The term arrays every mesh can use give the same bits on the meshes that normally take
    the per-exponent arrays (the library reads APC_GENERAL_TERMS at every launch)."""
    monkeypatch.setenv("APC_GENERAL_TERMS", "1")
    tb = stress_dag(seed=12, n_nodes=800, mesh_sizes=mesh, frac_nonspec_nodes=0.02, frac_noncontiguous=0.2)
    _run_and_compare(tb, mesh, 2.2, gpu_device)


def test_python_oracle_agrees_on_a_small_case(gpu_device):
    # the scalar Python restatement (not only its C twin) against the kernels
    mesh = (32, 8)
    tb = stress_dag(seed=2, n_nodes=40, mesh_sizes=mesh, max_strategies=10, frac_nonspec_nodes=0.1)
    p = CostModelParams.from_mesh(mesh, rescale=2.2)
    d = DeviceCostTables(tb, p, device=gpu_device)
    comm, trans, cost = d.build_all()
    want = po.build_tables(tb.as_dict(), po.make_params(mesh, rescale=2.2))
    assert np.array_equal(comm.cpu().numpy(), np.asarray(want["comm"]))
    assert np.array_equal(cost.cpu().numpy(), np.asarray(want["cost"]))
    assert np.array_equal(trans.cpu().numpy(), np.asarray(want["transition"], dtype=np.uint8))


def _two_node_tables(mesh, shape, stride, itemsize, src_codes, tgt_codes, flags=0, num_args=1, flops=0, rw=0):
    """producer node (strategies = src_codes) -> consumer node (input specs = tgt_codes)."""
    ns, nt = len(src_codes), len(tgt_codes)
    rank = len(shape)
    pad = [0] * (8 - rank)
    specs = [pack_codes(c) for c in src_codes] + [pack_codes(c) for c in tgt_codes]
    return CostTables(
        mesh_sizes=mesh, tensor_rank=[rank], tensor_itemsize=[itemsize], tensor_shape=[list(shape) + pad],
        tensor_stride=[list(stride) + pad], spec_codes=specs, spec_tensor=[0] * (ns + nt),
        strat_flops=[0] * ns + [flops] * nt, strat_rw_bytes=[0] * ns + [rw] * nt, strat_dtype=[3] * (ns + nt),
        strat_zero_cost=[1] * ns + [0 if (flops or rw) else 1] * nt, strat_num_args=[1] * ns + [num_args] * nt,
        node_strat_begin=[0, ns, ns + nt], edge_node=[1], edge_arg=[0], edge_src_begin=[0], edge_n_src=[ns],
        edge_tgt_begin=[ns], edge_n_tgt=[nt], edge_flags=[flags], edge_pt_begin=[-1],
        edge_entry_begin=[0, ns * nt], edge_strat_begin=[ns], pt_values=[])


@pytest.mark.parametrize("mesh", [(3, 5, 7), (64, 2), (6, 1, 1000003)])
def test_local_shapes_of_very_large_dims(gpu_device, mesh):
    """The shard-shape kernel divides through the mesh size's reciprocal with an integer
    correction below 2^52 and with the integer division above: dims and strides chosen at
    multiples of the mesh sizes +-1, near 2^52 and far above it, against Python integers."""
    M = len(mesh)
    rng = np.random.default_rng(5)
    dims = []
    for m in mesh:
        for k in (1, 2, 3, 1000, 2**20 + 1, 2**40 // m, 2**51 // m):
            dims += [k * m - 1, k * m, k * m + 1]
    dims += [2**52 - 1, 2**52, 2**52 + 1, 2**52 - 64, 1, 2, 0]
    shapes, strides = [], []
    for i, d in enumerate(dims):
        # rank 3, the large value as shape[1] (bytes stay below 2^53: the other dims are 1) and,
        # independently, stride[1] (the one Shard(2) divides) up to 2^62 (strides are not bounded by the bytes)
        big = int(rng.integers(2**52, 2**62)) if i % 3 == 0 else d
        shapes.append([1, d, 1] + [0] * 5)
        strides.append([dims[(i * 5 + 1) % len(dims)], big if i % 3 == 0 else dims[(i * 7 + 3) % len(dims)], 1] + [0] * 5)
    T = len(shapes)
    codes, tensor = [], []
    shard_sets = [[shard_code(1)] * M, [shard_code(2)] * M, [shard_code(1), 0, shard_code(2)][:M] + [0] * max(0, M - 3),
                  [shard_code(0)] * M]
    for t in range(T):
        for c in shard_sets:
            codes.append(pack_codes(c[:M]))
            tensor.append(t)
    n = len(codes)
    tb = CostTables(
        mesh_sizes=mesh, tensor_rank=[3] * T, tensor_itemsize=[1] * T, tensor_shape=shapes, tensor_stride=strides,
        spec_codes=codes, spec_tensor=tensor, strat_flops=[0] * n, strat_rw_bytes=[0] * n, strat_dtype=[3] * n,
        strat_zero_cost=[1] * n, strat_num_args=[1] * n, node_strat_begin=[0, n], edge_node=[], edge_arg=[],
        edge_src_begin=[], edge_n_src=[], edge_tgt_begin=[], edge_n_tgt=[], edge_flags=[], edge_pt_begin=[],
        edge_entry_begin=[0], edge_strat_begin=[], pt_values=[])
    d = DeviceCostTables(tb, CostModelParams.from_mesh(mesh), device=gpu_device, validate=False)
    got = d.run_spec_tables()
    torch.cuda.synchronize()
    want = po.spec_tables(tb.as_dict(), mesh)
    for key, w in zip(("num_shards", "local_shape", "local_stride", "local_numel", "local_bytes"), want):
        # (local numel / bytes of the 2^52-sized dims exceed nothing: the other dims are 1)
        assert _same_rows(got[key].cpu().numpy(), w), key
    assert got["local_shape"].shape[1] == 4  # rank 3, rounded up to even


def _golden():
    import json
    import os

    with open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")) as f:
        return json.load(f)


def test_known_answer_values_on_device(gpu_device):
    """The hand-derived values (tests/golden/known_answers.json) straight from the kernel."""
    R, P, S0, S1 = 0, partial_code(), shard_code(0), shard_code(1)
    named = {"R": R, "P": P, "S0": S0, "S1": S1, "S2": shard_code(2)}
    g = _golden()
    mesh = tuple(g["environment"]["mesh"])
    for cases, case_mesh in ((g["redistribute_cost_us"], mesh),
                             (g["mesh_8x8x8"]["redistribute_cost_us"], tuple(g["mesh_8x8x8"]["environment"]["mesh"]))):
        for case in cases:
            src, tgt = tuple(named[x] for x in case["src"]), tuple(named[x] for x in case["tgt"])
            tb = _two_node_tables(case_mesh, case["shape"], case["stride"], case["itemsize"], [src], [tgt])
            d = DeviceCostTables(tb, CostModelParams.from_mesh(case_mesh), device=gpu_device)
            comm, trans, _ = d.build_all()
            assert comm.cpu().numpy()[0] == case["value"], case["note"]
            assert trans.cpu().numpy()[0] == 1
            # the launch over packed tiles (direct evaluation in registers) gives the same value
            dp = DeviceCostTables(tb, CostModelParams.from_mesh(case_mesh), device=gpu_device)
            for launch in dp.planner_pass(packed=True).values():
                launch()
            assert dp.cost.cpu().numpy()[0] == case["value"] + 1, case["note"]  # + the transition cost; compute cost 0
    # one matrix with the special cases around them
    src = [(S0, S0), (P, P), (S0, S1), (R, R), (S0, R)]
    tgt = [(R, S0), (R, R), (S0, S0), (S0, R), (S0, S1), (P, R)]
    tb = _two_node_tables(mesh, [4096, 4096], [4096, 1], 2, src, tgt)
    d = DeviceCostTables(tb, CostModelParams.from_mesh(mesh), device=gpu_device)
    comm, trans, _ = d.build_all()
    m = comm.cpu().numpy().reshape(len(tgt), len(src))
    assert m[0, 0] == 286.43246022079404 and m[2, 1] == 609.0198034363015 and m[3, 2] == 27.543354475484605
    assert m[2, 0] == 0.0 and m[0, 3] == 0.0  # identity, replicated source
    assert math.isinf(m[5, 3]) and math.isinf(m[5, 0])  # -> Partial banned
    t = trans.cpu().numpy().reshape(len(tgt), len(src))
    assert t[2, 0] == 0 and t[0, 0] == 1 and t[3, 4] == 0


def test_compute_cost_known_answer_and_assembly(gpu_device):
    S0 = shard_code(0)
    kat = _golden()["compute_cost"]
    flops, rw = kat["flops"], kat["read_write_bytes"]
    assert kat["cost_us"] == 99.26256931388127
    tb = _two_node_tables((32, 8), [4096, 4096], [4096, 1], 2, [(S0, S0)], [(0, S0)], flags=1, num_args=2,
                          flops=flops, rw=rw)
    d = DeviceCostTables(tb, CostModelParams.from_mesh((32, 8), rescale=2.2), device=gpu_device)
    comm, trans, cost = d.build_all()
    cc = d.compute_cost.cpu().numpy()
    assert cc[1] == 99.26256931388127 and cc[0] == 0.0
    assert comm.cpu().numpy()[0] == 286.43246022079404 / 2.2  # grad rescale is a division
    assert cost.cpu().numpy()[0] == 286.43246022079404 / 2.2 + 99.26256931388127 / 2 + 1


def test_unsupported_dtype_raises(gpu_device):
    tb = _two_node_tables((4,), [64, 64], [64, 1], 2, [(0,)], [(0,)], flops=10, rw=10)
    tb.strat_dtype[:] = 6
    d = DeviceCostTables(tb, CostModelParams.from_mesh((4,)), device=gpu_device)
    d.run_tensor_tables()
    with pytest.raises(ValueError, match="dtype"):
        d.run_compute_costs()


def test_wide_and_degenerate_edges(gpu_device):
    """Column-chunked tiles (producer with > 1024 strategies), single-entry edges and a
    graph with zero edges."""
    rng = np.random.default_rng(0)
    n_src, n_tgt = 2600, 7
    opts = [0, partial_code(), shard_code(0), shard_code(1), shard_code(2)]
    src = [tuple(rng.choice(opts, 3)) for _ in range(n_src)]
    tgt = [tuple(rng.choice(opts, 3)) for _ in range(n_tgt)]
    tb = _two_node_tables((4, 2, 2), [64, 32, 16], [512, 16, 1], 4, src, tgt)
    assert int(tb.tile_col_count.max()) <= 1024 and tb.n_tiles > 1
    _run_and_compare(tb, (4, 2, 2), 1.0, gpu_device)
    tb = _two_node_tables((4,), [64], [1], 4, [(shard_code(0),)], [(0,)])
    _run_and_compare(tb, (4,), 1.0, gpu_device)
    empty = CostTables(
        mesh_sizes=(4,), tensor_rank=[], tensor_itemsize=[], tensor_shape=np.zeros((0, 8)),
        tensor_stride=np.zeros((0, 8)), spec_codes=[], spec_tensor=[], strat_flops=[], strat_rw_bytes=[],
        strat_dtype=[], strat_zero_cost=[], strat_num_args=[], node_strat_begin=[0], edge_node=[], edge_arg=[],
        edge_src_begin=[], edge_n_src=[], edge_tgt_begin=[], edge_n_tgt=[], edge_flags=[], edge_pt_begin=[],
        edge_entry_begin=[0], edge_strat_begin=[], pt_values=[])
    d = DeviceCostTables(empty, CostModelParams.from_mesh((4,)), device=gpu_device)
    comm, trans, cost = d.build_all()
    assert comm.numel() == 0 and trans.numel() == 0 and cost.numel() == 0


def test_deduplicated_edges_receive_identical_values(gpu_device):
    """Identical edges tiled once and stored to every copy: still bit-identical to the oracle,
    which evaluates every edge on its own."""
    from test_abi_and_encoding import twin_graph

    for mesh in [(32, 8), (4, 4, 2)]:
        tb = twin_graph(stress_dag(seed=21, n_nodes=600, mesh_sizes=mesh, frac_nonspec_nodes=0.02))
        tb.build_tiles(512, dedupe=True)
        assert int((tb.edge_canonical != np.arange(tb.n_edges)).sum()) >= tb.n_edges // 2
        _run_and_compare(tb, mesh, 2.2, gpu_device)


@pytest.mark.parametrize("threads", [64, 128, 256])
def test_wavefronts_per_tile_do_not_change_results(gpu_device, threads, monkeypatch):
    """The launcher picks one, two or four wavefronts per tile from the table's mean tile
    size; each choice (forced here through the tuning override, read at every launch) must
    give the oracle's bits, with and without identical edges stored to several copies."""
    from test_abi_and_encoding import twin_graph

    monkeypatch.setenv("APC_TILE_THREADS", str(threads))
    for mesh in [(32, 8), (16, 8, 4)]:
        tb = stress_dag(seed=9, n_nodes=500, mesh_sizes=mesh, frac_nonspec_nodes=0.02, frac_noncontiguous=0.2)
        _run_and_compare(tb, mesh, 2.2, gpu_device)
        tw = twin_graph(stress_dag(seed=10, n_nodes=300, mesh_sizes=mesh, frac_nonspec_nodes=0.02))
        tw.build_tiles(2048, dedupe=True)
        _run_and_compare(tw, mesh, 2.2, gpu_device)


def test_tile_size_does_not_change_results(gpu_device):
    mesh = (16, 8, 4)
    base = None
    for te in (64, 777, 4096, 16384):
        tb = stress_dag(seed=4, n_nodes=400, mesh_sizes=mesh, tile_entries=te)
        d = DeviceCostTables(tb, CostModelParams.from_mesh(mesh), device=gpu_device)
        out = [x.cpu().numpy() for x in d.build_all()]
        if base is None:
            base = out
        else:
            for a, b in zip(base, out):
                assert np.array_equal(a, b)


@pytest.mark.parametrize("max_len", [3, 40, 700])
def test_segmented_min_matches_oracle(gpu_device, max_len):
    rng = np.random.default_rng(max_len)
    lens = rng.integers(0, max_len + 1, size=5000)
    ptr = np.zeros(len(lens) + 1, np.int64)
    np.cumsum(lens, out=ptr[1:])
    vals = rng.choice([0.0, 1.0, 2.5, 7.0, 1e4, np.inf], size=int(ptr[-1]))
    tb = stress_dag(seed=0, n_nodes=5, mesh_sizes=(2,))
    d = DeviceCostTables(tb, CostModelParams.from_mesh((2,)), device=gpu_device)
    mins, args = d.segmented_min(torch.from_numpy(vals).to(gpu_device), ptr)
    wm, wa = c_oracle.segmented_min(vals, ptr)
    assert np.array_equal(mins.cpu().numpy(), wm)
    assert np.array_equal(args.cpu().numpy(), wa)
    nz = lens > 0
    assert np.array_equal(wm[nz], np.minimum.reduceat(vals, ptr[:-1][nz]))


def test_row_min_of_cost_tables(gpu_device):
    mesh = (32, 8)
    tb = stress_dag(seed=9, n_nodes=300, mesh_sizes=mesh)
    d, want = _run_and_compare(tb, mesh, 2.2, gpu_device)
    rp = tb.row_ptr()
    mins, args = d.segmented_min(d.cost, rp)
    wm, wa = c_oracle.segmented_min(want["cost"], rp)
    assert np.array_equal(mins.cpu().numpy(), wm) and np.array_equal(args.cpu().numpy(), wa)
    # a table this small has its row minima taken by the launch that wrote the matrices
    assert d.row_min_in_tiles_pays() and d.row_min is not None
    assert np.array_equal(d.row_min.cpu().numpy(), wm) and np.array_equal(d.row_argmin.cpu().numpy(), wa)
    d.run_redistribute_tables(row_min=False)
    assert d.row_min is None


@pytest.mark.parametrize("copies", [2, 8])
def test_row_minima_read_every_distinct_row_once(gpu_device, copies):
    """apc_segmented_min_copies on a table with identical edges (and some empty rows): the same
    minima and argmins as apc_segmented_min over every row and as the oracle, with a third of the
    rows written through the copy lists."""
    from test_abi_and_encoding import twin_graph

    mesh = (8, 8, 8)
    tb = twin_graph(stress_dag(seed=21, n_nodes=400, mesh_sizes=mesh, max_strategies=90, frac_nonspec_nodes=0.02))
    tb.build_tiles(1024, dedupe=True, max_copies=copies)
    assert not tb.rows_fit_tiles()  # producers with more than 64 strategies: the tiles cannot take the minima
    d, want = _run_and_compare(tb, mesh, 2.2, gpu_device)
    assert d.row_min is None and d._row_copies() is not None
    mins, args = d.row_minima()
    plain_min, plain_arg = d.segmented_min(d.cost, tb.row_ptr())
    wm, wa = c_oracle.segmented_min(want["cost"], tb.row_ptr())
    assert np.array_equal(mins.cpu().numpy(), wm) and np.array_equal(args.cpu().numpy(), wa)
    assert torch.equal(mins, plain_min) and torch.equal(args, plain_arg)


@pytest.mark.parametrize("mesh", [(32, 8), (16, 8, 4)])
def test_strategy_bounds_and_greedy_strategies_match_oracle(gpu_device, mesh):
    """Per-strategy sums of row minima and the per-node (min, argmin): same bits as the oracle
    (a node's edges are added in edge order on both sides)."""
    tb = stress_dag(seed=13, n_nodes=800, mesh_sizes=mesh, frac_nonspec_nodes=0.02)
    d, want = _run_and_compare(tb, mesh, 2.2, gpu_device)
    row_min, _ = d.segmented_min(d.cost, tb.row_ptr())
    bound, node_min, node_arg = d.greedy_strategies(row_min)
    torch.cuda.synchronize()
    enc = tb.as_dict()
    want_rows, _ = c_oracle.segmented_min(want["cost"], tb.row_ptr())
    wb, wm, wa, _ = po.greedy_strategies(enc, want_rows)
    assert np.array_equal(bound.cpu().numpy(), np.asarray(wb))
    assert np.array_equal(node_min.cpu().numpy(), np.asarray(wm))
    assert np.array_equal(node_arg.cpu().numpy(), np.asarray(wa))
    # wrong sizes are refused before any launch
    with pytest.raises(ValueError):
        d.strategy_bounds(row_min[:-1].contiguous())


def test_full_size_stress_properties(gpu_device):
    """The raw-throughput workload at a size the CPU cannot check entry by entry in test
    time: size-independent properties instead.  (a) the diagonal property: wherever the
    producer and consumer placements are identical the comm cost is exactly 0 and the
    transition flag 0; (b) a sampled 2000-edge slice is bit-identical to the oracle;
    (c) row minima are <= every sampled entry of their row."""
    mesh = (16, 8, 4)
    tb = stress_dag(seed=0, n_nodes=40_000, mesh_sizes=mesh)
    p = CostModelParams.from_mesh(mesh, rescale=2.2)
    d = DeviceCostTables(tb, p, device=gpu_device)
    comm, trans, cost = d.build_all()
    torch.cuda.synchronize()
    assert comm.numel() == tb.n_entries > 50_000_000
    # (b)
    lo, hi = 17_000, 19_000
    want = c_oracle.build_tables(tb.as_dict(), po.make_params(mesh, rescale=2.2), edge_range=(lo, hi))
    a, b = int(tb.edge_entry_begin[lo]), int(tb.edge_entry_begin[hi])
    assert np.array_equal(comm[a:b].cpu().numpy(), want["comm"])
    assert np.array_equal(cost[a:b].cpu().numpy(), want["cost"])
    assert np.array_equal(trans[a:b].cpu().numpy(), want["transition"])
    # (a) on the same slice, from the tables
    got_c, got_t = comm[a:b].cpu().numpy(), trans[a:b].cpu().numpy()
    off = 0
    for e in range(lo, hi):
        ns, nt = int(tb.edge_n_src[e]), int(tb.edge_n_tgt[e])
        if not (tb.edge_flags[e] & 2):
            s = tb.spec_codes[tb.edge_src_begin[e]:tb.edge_src_begin[e] + ns]
            t = tb.spec_codes[tb.edge_tgt_begin[e]:tb.edge_tgt_begin[e] + nt]
            valid = (tb.spec_tensor[tb.edge_src_begin[e]] >= 0)
            if valid:
                same = (t[:, None] == s[None, :]).ravel()
                assert (got_c[off:off + ns * nt][same] == 0.0).all()
                assert (got_t[off:off + ns * nt] == (~same).astype(np.uint8)).all()
        off += ns * nt
    # (c)
    mins, _ = d.segmented_min(cost, tb.row_ptr())
    rp = torch.from_numpy(tb.row_ptr()).to(gpu_device)
    seg_of_entry = torch.repeat_interleave(torch.arange(rp.numel() - 1, device=gpu_device)[:200_000],
                                           (rp[1:] - rp[:-1])[:200_000])
    assert bool((cost[: seg_of_entry.numel()] >= mins[seg_of_entry]).all())


@pytest.mark.parametrize("launches", [5, 2, 1])
def test_graph_replay_of_one_pass_matches_eager(gpu_device, launches):
    """One pass recorded as a HIP graph (five launches with the independent kernels on parallel
    branches, the one-launch build + row minima, or the one launch that takes the row minima
    too) gives the eager results on every replay, with eager work and synchronisations between
    replays."""
    mesh = (8, 4, 2)
    tb = stress_dag(seed=5, n_nodes=3000, mesh_sizes=mesh, frac_nonspec_nodes=0.02, frac_noncontiguous=0.2)
    d = DeviceCostTables(tb, CostModelParams.from_mesh(mesh, rescale=2.2), device=gpu_device)
    step = d.prepare_step(row_min=True, fused_inputs=launches <= 2, one_launch=launches <= 2,
                          row_min_in_tiles=launches == 1)
    assert len(step) == launches
    for launch in step.values():
        launch()
    torch.cuda.synchronize()
    outputs = {"comm": d.comm, "transition": d.transition, "cost": d.cost, "row_min": d.row_min,
               "row_argmin": d.row_argmin, "compute": d.compute_cost, "per_arg": d.compute_cost_per_arg,
               "bytes": d.tensor_bytes}
    want = {k: v.clone() for k, v in outputs.items()}
    enc = tb.as_dict()
    op = po.make_params(mesh, rescale=2.2)
    oracle = c_oracle.build_tables(enc, op, per_arg=c_oracle.compute_costs(enc, op)[1])
    assert np.array_equal(want["cost"].cpu().numpy(), oracle["cost"])
    graph = d.capture_step_graph(step)
    for replay in range(4):
        for v in outputs.values():
            v.zero_()  # eager work between replays; also proves the replay rewrites everything
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for k, v in outputs.items():
            assert torch.equal(v, want[k]), (replay, k)


@pytest.mark.parametrize("mesh", [(6,), (4, 8), (16, 2, 4), (2, 2, 2, 2), (5, 2, 3, 2)])
@pytest.mark.parametrize("contiguous", [True, False])
@pytest.mark.parametrize("threads", [None, 64, 128, 256])
def test_every_placement_pair(gpu_device, mesh, contiguous, threads, monkeypatch):
    """Brute force over the placement algebra: every producer placement against every consumer
    placement (Replicate, Partial(sum), Partial(avg), Shard of each tensor dim, on every mesh
    dim; a sample of 300 x 300 on the 4-D meshes), for a contiguous and a transposed tensor, with
    and without the gradient rescale, with the wavefronts per tile the library picks and with
    each of its three instantiations forced.  Kernel == C oracle bit for bit on all of them, ==
    the scalar Python oracle on the 1-D and 2-D meshes."""
    import itertools

    if threads is not None:
        monkeypatch.setenv("APC_TILE_THREADS", str(threads))

    M = len(mesh)
    options = [0, partial_code(0), partial_code(1), shard_code(0), shard_code(1), shard_code(2)]
    combos = list(itertools.product(options, repeat=M))
    if len(combos) > 300:
        rng = np.random.default_rng(7)
        keep = rng.choice(len(combos), 300, replace=False)
        combos = [combos[i] for i in sorted(keep)]
    shape = [96, 64, 32]
    stride = [2048, 32, 1] if contiguous else [1, 96, 6144]
    for flags, rescale in ((0, 1.0), (1, 2.2)):
        tb = _two_node_tables(mesh, shape, stride, 2, combos, combos, flags=flags)
        assert tb.n_entries == len(combos) ** 2
        d, want = _run_and_compare(tb, mesh, rescale, gpu_device)
        comm = d.comm.cpu().numpy().reshape(len(combos), len(combos))
        assert (np.diag(comm) == 0.0).all()  # identical placements cost nothing
        if M <= 2:
            py = po.build_tables(tb.as_dict(), po.make_params(mesh, rescale=rescale))
            assert np.array_equal(d.comm.cpu().numpy(), np.asarray(py["comm"]))
            assert np.array_equal(d.cost.cpu().numpy(), np.asarray(py["cost"]))
            assert np.array_equal(d.transition.cpu().numpy(), np.asarray(py["transition"], dtype=np.uint8))


def test_fused_input_tables_match_the_three_entry_points(gpu_device):
    mesh = (16, 8, 4)
    tb = stress_dag(seed=9, n_nodes=2500, mesh_sizes=mesh, frac_nonspec_nodes=0.03, frac_noncontiguous=0.2)
    p = CostModelParams.from_mesh(mesh, rescale=2.2)
    names = ("tensor_bytes", "tensor_contiguous", "compute_cost", "compute_cost_per_arg", "comm", "transition", "cost",
             "row_min", "row_argmin")
    results = []
    for fused in (False, True):
        d = DeviceCostTables(tb, p, device=gpu_device)
        step = d.prepare_step(row_min=True, fused_inputs=fused, one_launch=False, row_min_in_tiles=False)
        assert ("input_tables" in step) == fused and len(step) == (3 if fused else 5)
        for name in names:
            getattr(d, name).zero_()
        spec = d._step_keepalive[1]
        for v in spec.values():
            v.zero_()
        for launch in step.values():
            launch()
        torch.cuda.synchronize()
        out = {name: getattr(d, name).cpu().numpy() for name in names}
        out.update({f"spec_{k}": v.cpu().numpy() for k, v in spec.items()})
        results.append(out)
    for key in results[0]:
        assert np.array_equal(results[0][key], results[1][key]), key
    enc = tb.as_dict()
    assert np.array_equal(results[1]["tensor_bytes"], c_oracle.tensor_tables(enc)[0])
    assert _same_rows(results[1]["spec_local_shape"], c_oracle.spec_tables(enc, mesh)[1])
    assert (results[1]["cost"] != 0).any()


@pytest.mark.parametrize("mesh,threads", [((32, 8), None), ((16, 8, 4), None), ((16, 8, 4), 64), ((16, 8, 4), 256), ((2, 3, 2, 2), None)])
def test_one_launch_build_matches_the_separate_entry_points(gpu_device, mesh, threads, monkeypatch):
    """apc_build_tables (tiles that derive tensor bytes, contiguity and compute costs themselves,
    beside the workgroups that write those tables) against the launch-by-launch pass and the
    oracle: every output array, bit for bit; with identical edges stored to several copies,
    non-contiguous tensors and specs that are not DTensorSpecs in the mix."""
    from test_abi_and_encoding import twin_graph

    if threads:
        monkeypatch.setenv("APC_TILE_THREADS", str(threads))
    tb = twin_graph(stress_dag(seed=17, n_nodes=900, mesh_sizes=mesh, frac_nonspec_nodes=0.03, frac_noncontiguous=0.2))
    tb.build_tiles(1024, dedupe=True)
    p = CostModelParams.from_mesh(mesh, rescale=2.2)
    names = ("tensor_bytes", "tensor_contiguous", "compute_cost", "compute_cost_per_arg", "comm", "transition", "cost",
             "row_min", "row_argmin")
    results = []
    assert tb.rows_fit_tiles()
    for one_launch, in_tiles in ((False, False), (True, False), (False, True), (True, True)):
        # in_tiles: the launch that writes the matrices takes the row minima as well
        d = DeviceCostTables(tb, p, device=gpu_device)
        step = d.prepare_step(row_min=True, fused_inputs=True, one_launch=one_launch, row_min_in_tiles=in_tiles)
        assert list(step) == (["build_tables"] if one_launch else ["input_tables", "redistribute_tables"]) + \
            ([] if in_tiles else ["segmented_min"])
        for name in names:
            getattr(d, name).zero_()
        spec = d._step_keepalive[1]
        for v in spec.values():
            v.zero_()
        for launch in step.values():
            launch()
        torch.cuda.synchronize()
        out = {name: getattr(d, name).cpu().numpy() for name in names}
        out.update({f"spec_{k}": v.cpu().numpy() for k, v in spec.items()})
        results.append(out)
    for other in results[1:]:
        for key in results[0]:
            assert np.array_equal(results[0][key], other[key]), key
    enc = tb.as_dict()
    op = po.make_params(mesh, rescale=2.2)
    want_cc, want_pa = c_oracle.compute_costs(enc, op)
    want = c_oracle.build_tables(enc, op, per_arg=want_pa)
    _assert_costs(results[1]["cost"], want["cost"], "cost")
    _assert_costs(results[1]["comm"], want["comm"], "comm")
    assert np.array_equal(results[1]["transition"], want["transition"])
    _assert_costs(results[1]["compute_cost"], want_cc, "compute_cost")
    want_min, want_arg = c_oracle.segmented_min(want["cost"], tb.row_ptr())
    assert np.array_equal(results[3]["row_min"], want_min) and np.array_equal(results[3]["row_argmin"], want_arg)


def test_randomized_configurations(gpu_device, monkeypatch):
    """A seeded sweep over what the launchers choose between: mesh rank, strategy counts up to
    130 (column-chunked tiles), tile size, identical-edge copies, wavefronts per tile, one or two
    table launches, gradient rescale; every output against the C oracle, bit for bit."""
    from test_abi_and_encoding import twin_graph

    rng = np.random.default_rng(2024)
    meshes = [(64,), (32, 8), (8, 8, 8), (5, 3, 2), (2, 3, 2, 2), (128, 2)]
    for it in range(48):
        mesh = meshes[it % len(meshes)]
        maxs = int(rng.choice([2, 8, 40, 64, 130]))
        tb = stress_dag(seed=int(rng.integers(1, 10**6)), n_nodes=int(rng.integers(50, 600)), mesh_sizes=mesh,
                        max_strategies=maxs, min_strategies=min(4, maxs) if maxs > 2 else 1,
                        frac_nonspec_nodes=float(rng.choice([0.0, 0.02, 0.1])),
                        frac_noncontiguous=float(rng.choice([0.0, 0.2, 0.6])),
                        frac_grad_nodes=float(rng.choice([0.0, 0.05, 0.3])))
        if rng.random() < 0.5:
            tb = twin_graph(tb)
        copies = int(rng.choice([1, 2, 8]))
        tb.build_tiles(int(rng.choice([64, 300, 1024, 4096])), dedupe=copies > 1, max_copies=copies)
        threads = str(rng.choice(["", "64", "128", "256"]))
        if threads:
            monkeypatch.setenv("APC_TILE_THREADS", threads)
        else:
            monkeypatch.delenv("APC_TILE_THREADS", raising=False)
        one_launch = bool(rng.random() < 0.5)
        rescale = float(rng.choice([1.0, 2.2]))
        d = DeviceCostTables(tb, CostModelParams.from_mesh(mesh, rescale=rescale), device=gpu_device)
        in_tiles = tb.rows_fit_tiles() and bool(rng.random() < 0.7)  # row minima taken by the table launch
        assert tb.rows_fit_tiles() or maxs > 64
        # which per-entry arrays the pass writes: all three, the assembled cost alone (the planner's
        # pass; both are compile-time modes of the kernels on 2-D and 3-D meshes) or another subset
        outputs = [("comm", "transition", "cost"), ("cost",), ("comm", "cost"), ("transition", "cost")][int(rng.integers(0, 4))]
        spec_table = bool(rng.random() < 0.5)
        step = d.prepare_step(row_min=True, fused_inputs=True, one_launch=one_launch, row_min_in_tiles=in_tiles,
                              outputs=outputs, spec_table=spec_table)
        assert ("segmented_min" in step) != in_tiles
        d.row_min.fill_(-1.0)
        d.row_argmin.fill_(-7)
        for launch in step.values():
            launch()
        torch.cuda.synchronize()
        enc, op = tb.as_dict(), po.make_params(mesh, rescale=rescale)
        want_cc, want_pa = c_oracle.compute_costs(enc, op)
        want = c_oracle.build_tables(enc, op, per_arg=want_pa)
        want_min, want_arg = c_oracle.segmented_min(want["cost"], tb.row_ptr())
        what = (f"case {it}: mesh {mesh}, {maxs} strategies, {copies} copies, threads {threads or 'auto'}, one launch "
                f"{one_launch}, row minima in tiles {in_tiles}, outputs {outputs}, spec table {spec_table}")
        assert (d.comm is None) == ("comm" not in outputs) and (d.transition is None) == ("transition" not in outputs)
        if d.comm is not None:
            _assert_costs(d.comm.cpu().numpy(), want["comm"], what + " comm")
        _assert_costs(d.cost.cpu().numpy(), want["cost"], what + " cost")
        if d.transition is not None:
            assert np.array_equal(d.transition.cpu().numpy(), want["transition"]), what
        # an array the pass left out is computed on request, by a launch that writes it alone
        _assert_costs(d.fetch("comm").cpu().numpy(), want["comm"], what + " fetched comm")
        assert np.array_equal(d.fetch("transition").cpu().numpy(), want["transition"]), what + " fetched transition"
        _assert_costs(d.compute_cost.cpu().numpy(), want_cc, what + " compute_cost")
        assert np.array_equal(d.row_min.cpu().numpy(), want_min) and np.array_equal(d.row_argmin.cpu().numpy(), want_arg), what


def test_cpp_consumer_of_the_c_abi(gpu_device):
    """tests/abi_consumer.cpp: a C++ program that includes include/apcost.h, links the library
    and checks the hand-derived known answers itself (no Python, no torch in that process)."""
    import os
    import subprocess

    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "abi_consumer")
    if not os.path.exists(exe):
        pytest.fail(f"{exe} is missing: build it with `python -m autoparallel_amd._build`")
    run = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "abi consumer ok" in run.stdout


@pytest.mark.parametrize("write_through", [0, 1])
def test_measurement_kernels_do_what_they_say(gpu_device, write_through):
    """apc_calibrate_fill writes exactly out[0 .. n) (both kinds of store, an odd count, a
    workgroup that gets a partial run), apc_calibrate_launch runs and touches nothing, and both
    refuse arguments that make no sense."""
    import ctypes

    from autoparallel_amd import _native

    lib = _native.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    n = 100_001
    buf = torch.full((n + 6,), -1.0, dtype=torch.float64, device=gpu_device)
    rc = lib.apc_calibrate_fill(ctypes.c_void_p(buf.data_ptr()), ctypes.c_int64(n), ctypes.c_int64(2048), ctypes.c_double(3.25),
                                ctypes.c_int32(write_through), stream)
    _native.check(rc, "apc_calibrate_fill")
    _native.check(lib.apc_calibrate_launch(ctypes.c_int64(777), ctypes.c_int32(128), stream), "apc_calibrate_launch")
    torch.cuda.synchronize()
    got = buf.cpu().numpy()
    assert (got[:n] == 3.25).all() and (got[n:] == -1.0).all()
    assert lib.apc_calibrate_fill(ctypes.c_void_p(buf.data_ptr()), ctypes.c_int64(n), ctypes.c_int64(7), ctypes.c_double(0.0),
                                  ctypes.c_int32(write_through), stream) != 0
    assert lib.apc_calibrate_fill(ctypes.c_void_p(buf.data_ptr() + 8), ctypes.c_int64(n), ctypes.c_int64(8), ctypes.c_double(0.0),
                                  ctypes.c_int32(write_through), stream) != 0
    assert lib.apc_calibrate_launch(ctypes.c_int64(0), ctypes.c_int32(128), stream) != 0
