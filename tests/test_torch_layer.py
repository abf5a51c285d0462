"""The torch layer over the C ABI (``torch.ops.apcost``, csrc/apcost_torch.cpp): it loads, exports
its operators with named schemas, rejects malformed arguments with RuntimeError before anything
is launched, and its operators give the oracle's bits on the HIP device."""

import numpy as np
import pytest
import torch

from autoparallel_amd import CostModelParams, _native
from autoparallel_amd.device_tables import DeviceCostTables, _to_device
from autoparallel_amd.synthetic import stress_dag
from oracle import c_oracle
from oracle import cost_oracle as po

OPERATORS = (
    "abi_version", "validate_tables", "tensor_tables", "shard_shapes_bytes", "strategy_inputs", "compute_cost", "segmented_min", "cost_objective",
    "redistribute_cost_tables", "strategy_bounds", "diffusion_sweeps_", "bind_tensor_tables", "bind_spec_tables",
    "bind_compute_costs", "bind_segmented_min", "bind_redistribute_tables", "bind_input_tables", "bind_cost_tables",
)


def test_the_extension_loads_and_exports_its_operators():
    ops = _native.torch_ops()
    assert int(ops.abi_version()) == int(_native.lib().apc_version())
    for name in OPERATORS:
        schema = str(getattr(ops, name).default._schema)
        assert schema.startswith(f"apcost::{name}("), schema
        assert "_0" not in schema, f"{name}: arguments are named"
    assert "Tensor(a!) theta" in str(ops.diffusion_sweeps_.default._schema)
    assert "BoundLaunch" in str(ops.bind_cost_tables.default._schema)


def test_arguments_are_checked_before_any_launch():
    ops = _native.torch_ops()
    f64, i64 = torch.zeros(3, dtype=torch.float64), torch.zeros(2, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="must be on the HIP device"):
        ops.segmented_min(f64, i64)
    params = _native.params_tensor(CostModelParams.from_mesh((4, 2)).to_c())
    assert params.dtype == torch.uint8 and params.numel() == 368  # sizeof(struct apc_params)
    i32 = torch.zeros(1, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="struct apc_params"):
        ops.shard_shapes_bytes(params[:-8], i32, i32, i32, i32, i64, i64, 8)
    with pytest.raises(RuntimeError, match="struct apc_params"):
        ops.compute_cost(params.to(torch.float32), i64, i64, i32, i32, i32)
    with pytest.raises(RuntimeError, match="must be on the HIP device"):
        ops.compute_cost(params, i64, i64, i32, i32, i32)


@pytest.fixture(scope="module")
def small_table(gpu_device):
    mesh = (4, 4, 2)
    tb = stress_dag(seed=5, n_nodes=400, mesh_sizes=mesh, frac_nonspec_nodes=0.02, frac_noncontiguous=0.2)
    params = CostModelParams.from_mesh(mesh, rescale=2.2)
    dev = {k: _to_device(getattr(tb, k), gpu_device) for k in (
        "tensor_rank", "tensor_itemsize", "tensor_shape", "tensor_stride", "spec_codes", "spec_tensor", "strat_flops",
        "strat_rw_bytes", "strat_dtype", "strat_zero_cost", "strat_num_args", "pt_values", "tile_records", "dup_entry_begin")}
    want = c_oracle.build_tables(tb.as_dict(), po.make_params(mesh, rescale=2.2))
    return mesh, tb, _native.params_tensor(params.to_c()), dev, want


@pytest.mark.gpu
def test_operators_match_the_oracle(small_table):
    """The operators named by the extension's contract, called directly: shard shapes and byte
    counts, compute costs, the cost matrices and the row minima."""
    mesh, tb, p, d, want = small_table
    ops = _native.torch_ops()
    table = (d["tensor_rank"], d["tensor_itemsize"], d["tensor_shape"], d["tensor_stride"])
    nbytes, contiguous = ops.tensor_tables(*table)
    wb, wc = c_oracle.tensor_tables(tb.as_dict())
    assert np.array_equal(nbytes.cpu().numpy(), wb) and np.array_equal(contiguous.cpu().numpy(), wc)
    got = ops.shard_shapes_bytes(p, d["spec_codes"], d["spec_tensor"], *table, 8)
    for g, w in zip(got, c_oracle.spec_tables(tb.as_dict(), mesh)):
        assert np.array_equal(g.cpu().numpy().reshape(np.asarray(w).shape), w)
    compute, per_arg, err = ops.compute_cost(p, d["strat_flops"], d["strat_rw_bytes"], d["strat_dtype"], d["strat_zero_cost"],
                                             d["strat_num_args"])
    assert int(err.item()) == 0
    want_compute, want_per_arg = c_oracle.compute_costs(tb.as_dict(), po.make_params(mesh, rescale=2.2))[:2]
    assert np.array_equal(compute.cpu().numpy(), want_compute) and np.array_equal(per_arg.cpu().numpy(), want_per_arg)
    comm, transition, cost = ops.redistribute_cost_tables(p, nbytes, contiguous, d["spec_codes"], d["spec_tensor"], d["pt_values"],
                                                          per_arg, d["tile_records"], d["dup_entry_begin"], tb.n_entries)
    assert np.array_equal(comm.cpu().numpy(), want["comm"])
    assert np.array_equal(transition.cpu().numpy(), want["transition"])
    assert np.array_equal(cost.cpu().numpy(), want["cost"])
    mins, args = ops.segmented_min(cost, torch.from_numpy(tb.row_ptr()).to(cost.device))
    wm, wa = c_oracle.segmented_min(want["cost"], tb.row_ptr())
    assert np.array_equal(mins.cpu().numpy(), wm) and np.array_equal(args.cpu().numpy(), wa)


@pytest.mark.gpu
def test_tensor_table_on_shapes_with_empty_and_unit_dims(gpu_device):
    """Bytes and contiguity (torch spec_to_bytes, check_contiguous_sizes_strides) of hand-made
    rows: dims of size 0 (after which the expected stride is 0, or the product with sizes below
    1 counted as 1), dims of size 1 with any stride, rank 0, non-contiguous and permuted strides,
    random rows; against the oracle and, for contiguity, against torch's own function."""
    from torch._prims_common import check_contiguous_sizes_strides

    rows = [((), ()), ((5,), (1,)), ((5,), (2,)), ((4, 3), (3, 1)), ((4, 3), (1, 4)), ((4, 1, 3), (3, 77, 1)),
            ((4, 0, 3), (0, 3, 1)), ((4, 0, 3), (3, 3, 1)), ((4, 0, 3), (0, 0, 1)), ((0,), (1,)), ((0,), (5,)),
            ((2, 0, 0, 3), (0, 0, 3, 1)), ((2, 0, 0, 3), (3, 3, 3, 1)), ((2, 0, 0, 3), (9, 3, 3, 1)),
            ((1, 1, 1), (9, 8, 7)), ((2, 3, 4, 5, 6, 7, 8, 9), (181440, 60480, 15120, 3024, 504, 72, 9, 1)),
            ((2, 3, 4, 5, 6, 7, 8, 9), (181440, 60480, 15120, 3024, 504, 72, 1, 8)), ((3, 1, 0, 1, 2), (0, 5, 2, 9, 1))]
    rng = np.random.default_rng(5)
    for _ in range(300):
        r = int(rng.integers(0, 9))
        shape = [int(x) for x in rng.choice([0, 1, 1, 2, 3, 5, 8], r)]
        stride = []
        z = 1
        for x in reversed(shape):  # contiguous strides, then some of them disturbed
            stride.append(z)
            z *= max(x, 1) if rng.random() < 0.5 else x
        stride = list(reversed(stride))
        for i in range(r):
            if rng.random() < 0.15:
                stride[i] = int(rng.integers(0, 50))
        rows.append((tuple(shape), tuple(stride)))
    n = len(rows)
    rank = np.asarray([len(s) for s, _ in rows], np.int32)
    itemsize = np.asarray([(1, 2, 4, 8)[i % 4] for i in range(n)], np.int32)
    shape = np.zeros((n, 8), np.int64)
    stride = np.zeros((n, 8), np.int64)
    for i, (sh, st) in enumerate(rows):
        shape[i, :len(sh)] = sh
        stride[i, :len(st)] = st
    enc = {"tensor_rank": rank, "tensor_itemsize": itemsize, "tensor_shape": shape, "tensor_stride": stride}
    wb, wc = po.tensor_tables(enc)
    for (sh, st), c in zip(rows, wc):
        assert bool(c) == bool(check_contiguous_sizes_strides(sh, st, False)), (sh, st)
    assert {0, 1} == set(wc) and 0 in wb
    ops = _native.torch_ops()
    nbytes, contiguous = ops.tensor_tables(*(_to_device(a, gpu_device) for a in (rank, itemsize, shape, stride)))
    assert np.array_equal(nbytes.cpu().numpy(), np.asarray(wb, np.int64))
    assert np.array_equal(contiguous.cpu().numpy(), np.asarray(wc, np.uint8))


@pytest.mark.gpu
def test_lengths_that_disagree_are_rejected(small_table):
    mesh, tb, p, d, want = small_table
    ops = _native.torch_ops()
    with pytest.raises(RuntimeError, match="tensor_itemsize has"):
        ops.tensor_tables(d["tensor_rank"], d["tensor_itemsize"][:-1], d["tensor_shape"], d["tensor_stride"])
    with pytest.raises(RuntimeError, match="one row per strategy"):
        ops.compute_cost(p, d["strat_flops"], d["strat_rw_bytes"][:-1], d["strat_dtype"], d["strat_zero_cost"], d["strat_num_args"])
    with pytest.raises(RuntimeError, match="must be Long"):
        ops.segmented_min(torch.zeros(4, dtype=torch.float64, device=d["pt_values"].device),
                          torch.zeros(2, dtype=torch.int32, device=d["pt_values"].device))
    with pytest.raises(RuntimeError, match="must be contiguous"):
        ops.tensor_tables(d["tensor_rank"], d["tensor_itemsize"], d["tensor_shape"].t(), d["tensor_stride"])
    nbytes, contiguous = ops.tensor_tables(d["tensor_rank"], d["tensor_itemsize"], d["tensor_shape"], d["tensor_stride"])
    cost = torch.empty(tb.n_entries + 1, dtype=torch.float64, device=nbytes.device)
    with pytest.raises(RuntimeError, match="a per-entry output has"):
        ops.bind_redistribute_tables(p, nbytes, contiguous, d["spec_codes"], d["spec_tensor"], d["pt_values"], None,
                                     d["tile_records"], d["dup_entry_begin"], tb.n_entries, None, None, cost, None, None, None, None)
    with pytest.raises(RuntimeError, match="cost_out needs compute_cost_per_arg"):  # the library's own check, as RuntimeError
        ops.bind_redistribute_tables(p, nbytes, contiguous, d["spec_codes"], d["spec_tensor"], d["pt_values"], None,
                                     d["tile_records"], d["dup_entry_begin"], tb.n_entries, None, None, cost[:-1], None, None, None,
                                     None).run()


@pytest.mark.gpu
def test_a_bound_launch_follows_the_current_stream(small_table, gpu_device):
    """A bound launch enqueues on whatever stream is current when it runs (and on a given
    stream handle): the same values from a side stream as from the default stream."""
    mesh, tb, p, d, want = small_table
    dev = DeviceCostTables(tb, CostModelParams.from_mesh(mesh, rescale=2.2), device=gpu_device)
    step = dev.planner_pass()
    side = torch.cuda.Stream(device=dev.device)  # default priority
    for name, launch in step.items():
        assert launch.bound.name().startswith("apc_"), name
    with torch.cuda.stream(side):
        for launch in step.values():
            launch()
    side.synchronize()
    assert np.array_equal(dev.cost.cpu().numpy(), want["cost"])
    dev.cost.zero_()
    torch.cuda.synchronize()
    for launch in step.values():
        launch(side)
    side.synchronize()
    assert np.array_equal(dev.cost.cpu().numpy(), want["cost"])


def _host_tables(tb):
    from autoparallel_amd.device_tables import _to_device

    names = ("tensor_rank", "spec_codes", "spec_tensor", "edge_src_begin", "edge_n_src", "edge_tgt_begin", "edge_n_tgt",
             "edge_flags", "edge_pt_begin", "edge_entry_begin", "edge_strat_begin")
    t = [_to_device(np.ascontiguousarray(getattr(tb, k)), "cpu") for k in names]
    return t, _to_device(tb.tile_records, "cpu"), _to_device(np.ascontiguousarray(tb.dup_entry_begin), "cpu")


@pytest.mark.parametrize("mutate, message", [
    (None, None),
    (lambda t: t.tensor_rank.__setitem__(0, 9), "rank"),                                            # rank above the maximum
    (lambda t: t.spec_codes.__setitem__(0, 0xC0), "no meaning"),                                    # placement code out of range
    (lambda t: t.spec_codes.__setitem__(0, 0x800000), "beyond mesh ndim"),
    (lambda t: t.edge_entry_begin.__setitem__(2, int(t.edge_entry_begin[2]) + 1), "entry_begin"),  # pointer that does not follow the sizes
    (lambda t: t.edge_src_begin.__setitem__(1, t.n_specs), "producer spec range"),
])
def test_malformed_tables_raise_runtime_error_through_the_operator(mutate, message):
    """The host-side validator behind ``torch.ops.apcost.validate_tables``: malformed flattened
    tables (rank above the maximum, placement codes without a meaning, pointers that do not
    follow the sizes, ranges outside a table) are RuntimeErrors that name the row."""
    ops = _native.torch_ops()
    tb = stress_dag(seed=3, n_nodes=30, mesh_sizes=(4, 2), max_strategies=6)
    tb.build_tiles()
    if mutate is not None:
        mutate(tb)
        tb.pack_tile_records()
    arrays, tiles, dups = _host_tables(tb)
    params = _native.params_tensor(CostModelParams.from_mesh((4, 2)).to_c())
    call = lambda: ops.validate_tables(params, *arrays, len(tb.pt_values), tb.n_strategies, tiles, dups)  # noqa: E731
    if mutate is None:
        call()
    else:
        with pytest.raises(RuntimeError, match=message):
            call()
