"""The pass the planner issues (`DeviceCostTables.planner_pass`: assembled cost + tensor and
compute-cost tables, row minima where cheap, no spec table, no comm / transition arrays) and the
objective reduction on the device (`apc_cost_objective`), through the C ABI, against the oracle.
Bar: bit-exact."""

import numpy as np
import pytest
import torch

from autoparallel_amd import CostModelParams
from autoparallel_amd.device_tables import DeviceCostTables
from autoparallel_amd.synthetic import stress_dag
from oracle import c_oracle
from oracle import cost_oracle as po
from test_abi_and_encoding import twin_graph


def _groups(tb, rng, link: bool):
    """Variable groups as the planner builds them: every edge on its own, or (``link``) each edge
    of the first half sharing its variables with its twin in the second half.
    -> (n_vars, group_var_begin, group_member_begin, member_entry_begin, var_of_entry)"""
    begin = tb.edge_entry_begin.astype(np.int64)
    sizes = np.diff(begin)
    n = tb.n_edges
    rep = np.arange(n)
    if link:
        half = n // 2
        linked = rng.random(half) < 0.7
        rep[half:][linked] = np.arange(half)[linked]
    live = sizes > 0
    roots = np.nonzero((rep == np.arange(n)) & live)[0]
    base = np.zeros(n, np.int64)
    base[roots] = np.cumsum(sizes[roots]) - sizes[roots]
    n_vars = int(sizes[roots].sum())
    members = np.nonzero(live)[0]
    members = members[np.argsort(rep[members], kind="stable")]
    counts = np.bincount(np.searchsorted(roots, rep[members]), minlength=len(roots))
    gmb = np.zeros(len(roots) + 1, np.int64)
    np.cumsum(counts, out=gmb[1:])
    gvb = np.concatenate([base[roots], [n_vars]]).astype(np.int64)
    var = np.repeat(base[rep] - begin[:-1], sizes) + np.arange(tb.n_entries)
    return n_vars, gvb, gmb, begin[:-1][members], var


def test_cost_objective_oracle_is_the_sequential_accumulation():
    """CPU pin of the oracle's objective: the reference's loop (int 0 start, entries in order)
    equals numpy.bincount's sequential sum bit for bit; hand case with a shared variable, an
    infinite and a NaN cost."""
    inf = float("inf")
    obj, forced = po.cost_objective([1.5, inf, 0.1, 0.2, float("nan"), 0.3], [0, 1, 2, 2, 3, 2], 5)
    assert obj == [1.5, 10000.0, (0.1 + 0.2) + 0.3, 10000.0, 0.0]
    assert forced == [False, True, False, True, False]
    assert (0.1 + 0.2) + 0.3 != 0.1 + (0.2 + 0.3)  # the order of the additions is visible in the bits
    rng = np.random.default_rng(0)
    cost = rng.random(5000) * 10.0 ** rng.integers(-3, 6, 5000)
    cost[rng.random(5000) < 0.02] = inf
    var = rng.integers(0, 700, 5000)
    obj, forced = po.cost_objective(cost, var, 700)
    bad = ~np.isfinite(cost)
    assert np.array_equal(np.asarray(obj), np.bincount(var, weights=np.where(bad, 10000.0, cost), minlength=700))
    assert np.array_equal(np.asarray(forced), np.bincount(var, weights=bad, minlength=700) > 0)


@pytest.mark.gpu
@pytest.mark.parametrize("packed", [True, False])
@pytest.mark.parametrize("mesh,link", [((32, 8), True), ((16, 8, 4), True), ((8, 4), False), ((64,), True), ((6, 10), True),
                                       ((2, 4, 2, 2), False)])
def test_planner_pass_and_objective_match_the_oracle(gpu_device, mesh, link, packed):
    """``packed``: the pass runs over packed tiles (the planner's choice for a table this small:
    every wavefront evaluates whole rows on its own) or over the tile records and tables."""
    rng = np.random.default_rng(hash(mesh) % 1000)
    tb = twin_graph(stress_dag(seed=21, n_nodes=700, mesh_sizes=mesh, frac_nonspec_nodes=0.03, frac_noncontiguous=0.2))
    tb.build_tiles(None, dedupe=True, max_copies=8)
    p = CostModelParams.from_mesh(mesh, rescale=2.2)
    d = DeviceCostTables(tb, p, device=gpu_device)
    assert d.packed_pass_pays()
    step = d.planner_pass(packed=packed)
    assert list(step) == (["build_tables_packed"] if packed else ["build_tables"])
    assert "spec_tables" not in step and d.comm is None and d.transition is None and d.cost is not None
    assert d.row_min is not None, "a table this small has its row minima taken by the table launch"
    d.cost.fill_(-3.0)
    for launch in step.values():
        launch()
    torch.cuda.synchronize()
    d.check_error_flag()
    enc, op = tb.as_dict(), po.make_params(mesh, rescale=2.2)
    want_cc, want_pa = c_oracle.compute_costs(enc, op)
    want = c_oracle.build_tables(enc, op, per_arg=want_pa)
    assert np.array_equal(d.cost.cpu().numpy(), want["cost"])
    assert np.array_equal(d.compute_cost.cpu().numpy(), want_cc)
    assert np.array_equal(d.compute_cost_per_arg.cpu().numpy(), want_pa)
    wm, wa = c_oracle.segmented_min(want["cost"], tb.row_ptr())
    assert np.array_equal(d.row_min.cpu().numpy(), wm) and np.array_equal(d.row_argmin.cpu().numpy(), wa)
    assert np.isinf(want["cost"]).any(), "the case must exercise the forced-to-zero flags"
    # objective: linked edges add up in entry order
    n_vars, gvb, gmb, meb, var = _groups(tb, rng, link)
    obj, forced = d.cost_objective(n_vars, gvb, gmb, meb)
    torch.cuda.synchronize()
    bad = ~np.isfinite(want["cost"])
    want_obj = np.bincount(var, weights=np.where(bad, 10000.0, want["cost"]), minlength=n_vars)
    assert np.array_equal(obj.cpu().numpy(), want_obj)
    assert np.array_equal(forced.cpu().numpy().astype(bool), np.bincount(var, weights=bad, minlength=n_vars) > 0)
    # the scalar Python oracle on a prefix of the variables' entries
    some = np.nonzero(var < 300)[0]
    py_obj, py_forced = po.cost_objective(want["cost"][some], var[some], 300)
    assert np.array_equal(obj.cpu().numpy()[:300], np.asarray(py_obj))
    assert np.array_equal(forced.cpu().numpy()[:300].astype(bool), np.asarray(py_forced))
    # arrays the pass did not write come from a launch of their own, same values
    assert np.array_equal(d.fetch("comm").cpu().numpy(), want["comm"])
    assert np.array_equal(d.fetch("transition").cpu().numpy(), want["transition"])


@pytest.mark.gpu
@pytest.mark.parametrize("n_groups,max_size,max_members", [
    (350_000, 40, 3),     # four variables per thread; groups of a single variable next to larger ones; a three-round search
    (3_000, 5000, 2),     # the same kernel over few, large groups
    (70_000, 30, 9),      # one variable per thread, more members than are in flight at once, a three-round search
    (1, 700, 33),         # one group
    (6, 300, 3000),       # more members than a workgroup stages: their offsets straight from memory
])
def test_cost_objective_on_synthetic_groups(gpu_device, n_groups, max_size, max_members):
    """The objective kernel on its own (``torch.ops.apcost.cost_objective``): both of its forms
    (one / four variables per thread, chosen by the number of variables), groups of one
    variable, members beyond one round of the member loop, as many groups as take the search
    for a workgroup's first group three rounds.  Expected values: numpy.bincount, which adds in
    array order from 0.0 (pinned against the reference's loop in the CPU test above)."""
    from autoparallel_amd import _native

    rng = np.random.default_rng(n_groups)
    sizes = rng.integers(1, max_size + 1, n_groups)
    sizes[rng.random(n_groups) < 0.4] = 1
    members = rng.integers(1, max_members + 1, n_groups)
    members[0] = max_members
    gvb = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    gmb = np.concatenate([[0], np.cumsum(members)]).astype(np.int64)
    n_vars = int(gvb[-1])
    member_size = np.repeat(sizes, members)
    # the members' entry ranges, in a shuffled order of the groups with gaps between them, ascending inside a group
    order = rng.permutation(n_groups)
    group_entries = sizes * members
    start = np.zeros(n_groups, np.int64)
    start[order] = np.cumsum(group_entries[order] + 3) - (group_entries[order] + 3)
    meb = np.repeat(start, members) + (np.arange(gmb[-1]) - np.repeat(gmb[:-1], members)) * member_size
    n_entries = int((group_entries + 3).sum())
    cost = rng.uniform(0, 1e4, n_entries)
    cost[rng.random(n_entries) < 0.01] = np.inf
    cost[rng.random(n_entries) < 0.001] = np.nan
    var = np.full(n_entries, -1, np.int64)
    idx = np.repeat(meb, member_size) + (np.arange(int(member_size.sum())) - np.repeat(np.cumsum(member_size) - member_size, member_size))
    var[idx] = np.repeat(np.repeat(gvb[:-1], members), member_size) + (idx - np.repeat(meb, member_size))
    used = var >= 0
    bad = ~np.isfinite(cost)
    want = np.bincount(var[used], weights=np.where(bad, 10000.0, cost)[used], minlength=n_vars)
    want_forced = np.bincount(var[used], weights=bad[used], minlength=n_vars) > 0
    dev = lambda a: torch.from_numpy(a).to(gpu_device)  # noqa: E731
    obj, forced = _native.torch_ops().cost_objective(n_vars, dev(gvb), dev(gmb), dev(meb), dev(cost), 10000.0)
    torch.cuda.synchronize()
    assert (n_vars >= 1 << 22) == (n_groups == 350_000 or n_groups == 3_000)
    assert np.array_equal(obj.cpu().numpy(), want)
    assert np.array_equal(forced.cpu().numpy().astype(bool), want_forced)


@pytest.mark.gpu
def test_cost_objective_refuses_an_empty_group(gpu_device):
    """The objective kernel takes one workgroup per variable group and never searches for the
    group of a variable: the host wrapper refuses pointers that do not ascend strictly."""
    tb = stress_dag(seed=21, n_nodes=60, mesh_sizes=(4, 2))
    d = DeviceCostTables(tb, CostModelParams.from_mesh((4, 2)), device=gpu_device)
    for launch in d.planner_pass().values():
        launch()
    n_vars, gvb, gmb, meb, _ = _groups(tb, np.random.default_rng(0), False)
    d.cost_objective(n_vars, gvb, gmb, meb)
    bad = gvb.copy()
    bad[3] = bad[2]
    with pytest.raises(ValueError, match="at least one variable"):
        d.cost_objective(n_vars, bad, gmb, meb)


@pytest.mark.gpu
def test_planner_pass_on_a_table_whose_rows_do_not_fit_tiles(gpu_device):
    """Producers with more than 64 strategies: the pass writes the cost alone, the row minima are
    taken on request by a segmented minimum over the distinct rows."""
    mesh = (8, 8, 8)
    tb = twin_graph(stress_dag(seed=4, n_nodes=400, mesh_sizes=mesh, max_strategies=125))
    tb.build_tiles(None, dedupe=True, max_copies=2)
    assert not tb.rows_fit_tiles()
    d = DeviceCostTables(tb, CostModelParams.from_mesh(mesh, rescale=2.2), device=gpu_device)
    step = d.planner_pass()
    assert d.row_min is None
    for launch in step.values():
        launch()
    torch.cuda.synchronize()
    enc, op = tb.as_dict(), po.make_params(mesh, rescale=2.2)
    want = c_oracle.build_tables(enc, op, per_arg=c_oracle.compute_costs(enc, op)[1])
    assert np.array_equal(d.cost.cpu().numpy(), want["cost"])
    mins, args = d.row_minima()
    wm, wa = c_oracle.segmented_min(want["cost"], tb.row_ptr())
    assert np.array_equal(mins.cpu().numpy(), wm) and np.array_equal(args.cpu().numpy(), wa)
    with pytest.raises(RuntimeError, match="producer strategies"):
        d.run_redistribute_tables(row_min=True)
