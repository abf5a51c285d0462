"""Plan-level parity.  The reference's own planner tests hold golden *plans*: the exact
placements its ILP must choose for a two-layer FFN and a transformer block on a 1-D
(256,) and a 2-D (32, 8) mesh (tests/test_optimize_placement.py:141-315).  Reproducing
them pins, end to end, this repository's graph capture, strategy enumeration, cost
arithmetic, cost assembly and ILP formulation against the reference's expectations.

The CPU tests build the tables with the oracle (test backend); the GPU tests build them
with the HIP kernels and additionally require bit-identical tables and the identical
plan and objective from the same solver."""

import math
import warnings

import numpy as np
import pytest
import torch
from torch._functorch._aot_autograd.fx_utils import get_param_nodes
from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

from autoparallel_amd.api import AutoParallelPlanner
from autoparallel_amd.optimize_sharding import ShardingOptimizer
from models import make_model_and_inputs
from oracle_backend import OracleBackend


class OracleOptimizer(ShardingOptimizer):
    backend_cls = OracleBackend


class OraclePlanner(AutoParallelPlanner):
    optimizer_cls = OracleOptimizer


@pytest.fixture(scope="module")
def meshes(fake_pg):
    from torch.distributed.device_mesh import init_device_mesh

    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        return {"1d": init_device_mesh("cpu", (256,), mesh_dim_names=("dp",)),
                "2d": init_device_mesh("cpu", (32, 8), mesh_dim_names=("dp", "tp")),
                "3d": init_device_mesh("cpu", (8, 8, 4), mesh_dim_names=("dp", "tp", "cp"))}


def _plan(planner_cls, mesh, kind, high_mem):
    model_fn, input_fn = make_model_and_inputs(mesh, kind)
    with torch.device("meta"):
        model = model_fn()
    with planner_cls(model, input_fn, mesh) as autop:
        autop.add_parameter_memory_constraint(low=0, high=high_mem)
        placement = autop.optimize_placement()
        return autop, placement


# ---- expectations held by the reference's tests ---------------------------------------------
_mm1 = [(Shard(0), Replicate()), (Replicate(), Shard(1)), (Shard(0), Shard(1))]
_mm2 = [(Shard(0), Shard(1)), (Replicate(), Shard(0)), (Shard(0), Partial("sum"))]
_mm3 = [(Shard(1), Replicate()), (Shard(0), Shard(1)), (Partial("sum"), Shard(1))]
_mm4 = [(Shard(1), Shard(0)), (Shard(0), Replicate()), (Partial("sum"), Shard(0))]
EXPECTED_2D = {
    "ffn": ([(Shard(0), Shard(0)), (Shard(0), Shard(1))], [_mm1, _mm2, _mm3, _mm1, _mm4]),
    "block": ([(Shard(0), Shard(0))] * 3 + [(Shard(0), Shard(1)), (Shard(0), Shard(0)), (Shard(0), Shard(1))],
              [_mm1, _mm1, _mm1, _mm2, _mm1, _mm2, _mm3, _mm1, _mm4, _mm2, _mm3, _mm1, _mm4, _mm2, _mm4, _mm2, _mm4,
               _mm2]),
}


def _check_1d(autop, placement, kind, high_mem):
    want = {None: (Shard(0),), 1.0: (Replicate(),)}[high_mem]
    for node in get_param_nodes(autop.gm.graph):
        assert placement[node].output_specs.placements == want
    mm = autop.gm.graph.find_nodes(op="call_function", target=torch.ops.aten.mm.default)
    n_mm, n_fwd = {"ffn": (5, 2), "block": (18, 6)}[kind]
    assert len(mm) == n_mm
    for node in mm[:n_fwd]:  # forward: batch-sharded activations, replicated weights
        p = placement[node]
        assert (p.input_specs[0].placements, p.input_specs[1].placements, p.output_specs.placements) == \
            ((Shard(0),), (Replicate(),), (Shard(0),))
    for node in mm[n_fwd::2]:  # weight gradients
        p = placement[node]
        assert (p.input_specs[0].placements, p.input_specs[1].placements, p.output_specs.placements) == \
            ((Shard(1),), (Shard(0),), (Partial("sum"),))
    for node in mm[n_fwd + 1::2]:  # input gradients
        p = placement[node]
        assert (p.input_specs[0].placements, p.input_specs[1].placements, p.output_specs.placements) == \
            ((Shard(0),), (Replicate(),), (Shard(0),))


def _check_2d(autop, placement, kind):
    want_params, want_mm = EXPECTED_2D[kind]
    for node, want in zip(get_param_nodes(autop.gm.graph), want_params):
        assert placement[node].output_specs.placements == want
    mm = autop.gm.graph.find_nodes(op="call_function", target=torch.ops.aten.mm.default)
    assert len(mm) == len(want_mm)
    for node, want in zip(mm, want_mm):
        p = placement[node]
        assert [p.input_specs[0].placements, p.input_specs[1].placements, p.output_specs.placements] == want, node
    for node in autop.gm.graph.find_nodes(op="call_function",
                                          target=torch.ops.aten._scaled_dot_product_efficient_attention.default):
        p = placement[node]
        for spec in (p.input_specs[0], p.input_specs[1], p.input_specs[2], p.output_specs[0]):
            assert spec.placements == (Shard(0), Shard(1))


@pytest.mark.parametrize("kind", ["ffn", "block"])
@pytest.mark.parametrize("high_mem", [None, 1.0])
def test_reference_golden_plans_1d_with_oracle_tables(meshes, kind, high_mem):
    autop, placement = _plan(OraclePlanner, meshes["1d"], kind, high_mem)
    _check_1d(autop, placement, kind, high_mem)


@pytest.mark.parametrize("kind", ["ffn", "block"])
def test_reference_golden_plans_2d_with_oracle_tables(meshes, kind):
    autop, placement = _plan(OraclePlanner, meshes["2d"], kind, None)
    _check_2d(autop, placement, kind)
    opt = autop.sharding_optimizer
    # every (node, argument) picked exactly one entry and nothing infinite was chosen
    assert len(opt.res) == opt.encoded.tables.n_edges
    assert np.array_equal(opt.res_entries, np.nonzero(opt.prob.x[opt.var_of_entry] == 1)[0])
    assert np.isfinite(opt.comm_cost[opt.res_entries]).all()
    assert not opt.prob.violated_constraints()
    # ds is a mapping over the flat arrays with the reference's record fields
    key = opt.res[0]
    rec = opt.ds[key]
    assert set(rec) == {"va", "cost", "compute_cost", "comm_cost", "sharding_transition_cost", "full_strat",
                        "out_strat", "inp_strat"}
    assert rec["cost"] == rec["comm_cost"] + rec["compute_cost"] + rec["sharding_transition_cost"]
    assert key in opt.ds and (10**6, 0, 0, 0) not in opt.ds and len(opt.ds) == opt.encoded.tables.n_entries
    # the recomputed costs were written back into OpSpec.redistribute_cost
    s_i, argi, ss, ii = key
    assert opt.strats[opt.nodes[s_i]].strategies[ss].redistribute_cost[argi][ii] == rec["comm_cost"]
    log = opt.get_log()
    assert "total_cost" in log and "Violated constraints: []" in log


def _plan_local_map(planner_cls, mesh):
    """tests/test_optimize_placement.py:425-452"""
    model_fn, input_fn = make_model_and_inputs(mesh, "local_map_block")
    with torch.device("meta"):
        model = model_fn()
    with planner_cls(model, input_fn, mesh, dynamo=True) as autop:
        autop.add_parameter_memory_constraint(low=None, high=None)
        x_sharding = (Shard(0), Replicate(), Shard(1))
        autop.add_input_constraints([x_sharding])
        autop.add_output_constraints([x_sharding])
        placement = autop.optimize_placement()
        return autop, placement


def _check_local_map(autop, placement):
    """The expectations of tests/test_optimize_placement.py:454-493.  The number of
    activations the forward call saves depends on the attention kernel the trace
    dispatches to (the reference counts 7 on a CUDA device); their placement does not."""
    regions = [n for n in autop.gm.graph.nodes if "local_map_kwargs" in n.meta]
    assert len(regions) == 2, "expected a forward and a backward call"
    fw, bw = placement[regions[0]], placement[regions[1]]
    rep = (Replicate(), Replicate(), Replicate())
    q, k, v = fw.input_specs
    assert q.placements == (Shard(0), Shard(1), Shard(2))
    assert k.placements == v.placements == (Shard(0), Shard(1), Replicate())
    out, *saved = fw.output_specs
    assert out.placements == (Shard(0), Shard(1), Shard(2)) and len(saved) >= 3
    assert all(s.placements == rep for s in saved if s is not None)
    *saved_in, grad_out = bw.input_specs
    assert len(saved_in) == len(saved)
    assert grad_out.placements == (Shard(0), Shard(1), Shard(2))
    assert all(s.placements == rep for s in saved_in if s is not None)
    gq, gk, gv = bw.output_specs
    assert gq.placements == (Shard(0), Shard(1), Shard(2))
    assert gk.placements == gv.placements == (Shard(0), Shard(1), Replicate())


def test_local_map_placements_are_respected_with_oracle_tables(meshes):
    autop, placement = _plan_local_map(OraclePlanner, meshes["3d"])
    _check_local_map(autop, placement)
    assert not autop.sharding_optimizer.prob.violated_constraints()
    # the plan honours the pinned input / output placement around the region
    from torch._functorch._aot_autograd.fx_utils import get_plain_input_and_grad_nodes

    ((x, grad_x),) = get_plain_input_and_grad_nodes(autop.gm.graph).values()
    assert placement[x].output_specs.placements == (Shard(0), Replicate(), Shard(1))
    assert placement[grad_x].output_specs.placements == (Shard(0), Replicate(), Shard(1))


def test_parameter_smaller_than_the_mesh_stays_replicated(meshes):
    """tests/test_optimize_placement.py:496-533: a parameter with fewer elements than the
    mesh has ranks is left out of the memory constraint and ends up replicated."""
    mesh = meshes["1d"]
    model_fn, input_fn = make_model_and_inputs(mesh, "small_param")
    with torch.device("meta"):
        model = model_fn()
    with OraclePlanner(model, input_fn, mesh) as autop:
        autop.add_input_constraints([(Shard(0),)])
        autop.add_parameter_memory_constraint()
        placement = autop.optimize_placement()
        params = list(get_param_nodes(autop.gm.graph))
        assert len(params) == 1
        for node in params:
            assert placement[node].output_specs.placements == (Replicate(),)


def test_cost_rows_are_written_into_specs_each_node_owns(meshes):
    """optimize_sharding.py:361-363 on request: ``OpSpec.redistribute_cost[argi][ii]`` of every
    strategy holds the recomputed communication cost.  Nodes enumerated from one memo entry
    share their OpSpec objects until then; the write-back gives each node its own."""
    mesh = meshes["2d"]
    model_fn, input_fn = make_model_and_inputs(mesh, "block")
    with torch.device("meta"):
        model = model_fn()
    with OraclePlanner(model, input_fn, mesh) as autop:
        opt = autop.sharding_optimizer
        nodes = [n for n in opt.nodes if n.op != "output"]
        shared_before = len({id(s) for n in nodes for s in opt.strats[n].strategies})
        total = sum(len(opt.strats[n].strategies) for n in nodes)
        assert shared_before < total  # (some nodes do share: the memo had hits)
        opt.materialize_redistribute_costs()
        assert len({id(s) for n in nodes for s in opt.strats[n].strategies}) == total
        tb, comm = opt.encoded.tables, opt.comm_cost
        for e, (s_i, argi) in enumerate(opt.encoded.edge_keys):
            ns, nt, b = int(tb.edge_n_src[e]), int(tb.edge_n_tgt[e]), int(tb.edge_entry_begin[e])
            rows = [s.redistribute_cost[argi] for s in opt.strats[opt.nodes[s_i]].strategies]
            assert len(rows) == nt and all(len(r) == ns for r in rows)
            assert np.array_equal(np.asarray(rows, np.float64).reshape(-1), comm[b:b + ns * nt])
        # the plan is the same afterwards
        autop.add_parameter_memory_constraint(low=0, high=None)
        placement = autop.optimize_placement()
        _check_2d(autop, placement, "block")


def test_collector_is_paused_while_planning_and_restored_afterwards(meshes):
    """Objects made by capture and construction are frozen out of the cyclic collector's sight
    inside the ``with`` block and handed back at exit; the collector's on / off state is the
    caller's again as soon as ``__enter__`` returns (also when construction raises)."""
    import gc

    mesh = meshes["1d"]
    model_fn, input_fn = make_model_and_inputs(mesh, "small_param")
    with torch.device("meta"):
        model = model_fn()
    assert gc.isenabled() and gc.get_freeze_count() == 0
    with OraclePlanner(model, input_fn, mesh) as autop:
        assert gc.isenabled() and gc.get_freeze_count() > 0
        autop.add_input_constraints([(Shard(0),)])
        autop.optimize_placement()
    assert gc.isenabled() and gc.get_freeze_count() == 0

    class Failing(OraclePlanner):
        def _enter(self):
            raise ValueError("construction failed")

    # `with` does not call __exit__ after a failing __enter__: nothing stays frozen, the
    # collector is in the caller's state
    for on in (False, True):
        (gc.enable if on else gc.disable)()
        try:
            with pytest.raises(ValueError, match="construction failed"):
                with Failing(model, input_fn, mesh):
                    pass
            assert gc.isenabled() == on and gc.get_freeze_count() == 0
        finally:
            gc.enable()

    class FailsAfterCapture(OraclePlanner):
        class optimizer_cls(OracleOptimizer):
            def __init__(self, *a, **k):
                raise ValueError("optimizer failed")

    with pytest.raises(ValueError, match="optimizer failed"):
        with FailsAfterCapture(model, input_fn, mesh):
            pass
    assert gc.isenabled() and gc.get_freeze_count() == 0
    # the capture context was closed: a new planner can enter
    with OraclePlanner(model, input_fn, mesh) as autop:
        assert autop.active is True

    # an application that froze its own objects keeps them frozen: the planner neither adds to
    # the frozen set nor thaws it
    gc.freeze()
    try:
        theirs = gc.get_freeze_count()
        assert theirs > 0
        # (the count only shrinks as frozen objects die: nothing was added, nothing thawed)
        with OraclePlanner(model, input_fn, mesh) as autop:
            assert 0.9 * theirs < gc.get_freeze_count() <= theirs
        assert 0.9 * theirs < gc.get_freeze_count() <= theirs
    finally:
        gc.unfreeze()


def test_unsolvable_problem_raises(meshes):
    model_fn, input_fn = make_model_and_inputs(meshes["2d"], "ffn")
    with torch.device("meta"):
        model = model_fn()
    with OraclePlanner(model, input_fn, meshes["2d"]) as autop:
        node = get_param_nodes(autop.gm.graph)[0]
        autop.sharding_optimizer.add_node_constraint(node, (Replicate(), Replicate()))
        autop.sharding_optimizer.add_node_constraint(node, (Shard(0), Shard(0)))
        with pytest.raises(RuntimeError, match="Unsolvable"):
            autop.optimize_placement()
        with pytest.raises(RuntimeError, match="Couldn't find appropriate constraint"):
            autop.sharding_optimizer.add_node_constraint(node, (Partial("sum"), Replicate()))


@pytest.mark.gpu
@pytest.mark.parametrize("kind,mesh_key,high_mem", [("ffn", "2d", None), ("block", "2d", None), ("block", "1d", 1.0)])
def test_device_tables_give_identical_tables_plan_and_objective(gpu_device, meshes, kind, mesh_key, high_mem):
    dev_autop, dev_plan = _plan(AutoParallelPlanner, meshes[mesh_key], kind, high_mem)
    ora_autop, ora_plan = _plan(OraclePlanner, meshes[mesh_key], kind, high_mem)
    d, o = dev_autop.sharding_optimizer, ora_autop.sharding_optimizer
    assert type(d.backend).__name__ == "DeviceBackend"
    # tables: bit-identical (integer inputs and fp64 outputs)
    for name in ("strat_flops", "strat_rw_bytes", "strat_dtype", "strat_zero_cost", "spec_codes", "spec_tensor"):
        assert np.array_equal(getattr(d.encoded.tables, name), getattr(o.encoded.tables, name)), name
    assert np.array_equal(d.comm_cost, o.comm_cost)
    assert np.array_equal(d.transition_cost, o.transition_cost)
    assert np.array_equal(d.cost, o.cost)
    assert np.array_equal(d.compute_cost_per_arg, o.compute_cost_per_arg)
    # plan and objective: identical
    assert d.res == o.res
    assert d.objective_value() == o.objective_value()
    for (n1, s1), (n2, s2) in zip(dev_plan.items(), ora_plan.items()):
        assert n1.name == n2.name and str(s1) == str(s2)
    if mesh_key == "2d":
        _check_2d(dev_autop, dev_plan, kind)
    else:
        _check_1d(dev_autop, dev_plan, kind, high_mem)
    # row minima from the segmented-min kernel agree with the oracle's
    dm, da = d.row_minima()
    om, oa = o.row_minima()
    assert np.array_equal(dm, om) and np.array_equal(da, oa)
    # so do the greedy strategies and the lower bound built on them, which the optimum respects
    (dc, dlb), (oc, olb) = d.greedy_strategies(), o.greedy_strategies()
    assert dlb == olb and {n.name: k for n, k in dc.items()} == {n.name: k for n, k in oc.items()}
    assert dlb <= d.objective_value() * (1 + 1e-12)


@pytest.mark.parametrize("kind,mesh_key,high_mem", [("ffn", "2d", None), ("block", "2d", None), ("block", "1d", None),
                                                    ("block", "1d", 1.0)])
def test_pruning_before_the_solve_changes_neither_plan_nor_objective(meshes, kind, mesh_key, high_mem):
    """The dual ascent + incumbent + bound-based fixing in front of the solver (pruning.py): on the
    reference's test models the solver receives a fraction of the columns and returns the
    objective of the full program with a plan that is optimal in the full program
    (where several plans tie, e.g. a backward permute that may stay Partial or not at equal cost,
    the two solves may return different ones); the reference's expected placements hold for both."""

    class FullOptimizer(OracleOptimizer):
        prune_before_solve = False

    class FullPlanner(AutoParallelPlanner):
        optimizer_cls = FullOptimizer

    a, plan_a = _plan(OraclePlanner, meshes[mesh_key], kind, high_mem)
    b, plan_b = _plan(FullPlanner, meshes[mesh_key], kind, high_mem)
    oa, ob = a.sharding_optimizer, b.sharding_optimizer
    sa, sb = oa.solve_stats, ob.solve_stats
    assert "columns_after_pruning" in sa and "columns_after_pruning" not in sb
    assert sa["incumbent"] is not None and sa["lower_bound"] <= sa["incumbent"] * (1 + 1e-9)
    assert sa["columns_after_pruning"] < 0.5 * sa["columns"] and sb["columns_solved"] == sb["columns"]
    # (tied plans sum different entries: equal to the last bits, not always bit for bit)
    assert math.isclose(oa.objective_value(), ob.objective_value(), rel_tol=1e-13)
    # the pruned program's plan is a feasible plan of the full program with the full optimum as its cost
    assert not ob.prob.violated_constraints(oa.prob.x)
    assert math.isclose(float(ob.prob.objective @ oa.prob.x), ob.prob.objective_value, rel_tol=1e-12)
    # so is the incumbent the pruning worked with (feasible; no better than the optimum)
    assert not ob.prob.violated_constraints(oa.incumbent)
    assert float(ob.prob.objective @ oa.incumbent) >= ob.prob.objective_value * (1 - 1e-12)
    # no variable of the full program's optimum was fixed to zero unless another optimum was kept
    for autop, plan in ((a, plan_a), (b, plan_b)):
        if mesh_key == "2d":
            _check_2d(autop, plan, kind)
        else:
            _check_1d(autop, plan, kind, high_mem)


def test_a_second_solve_under_more_constraints_starts_from_the_unpruned_program(meshes):
    """What the first solve pruned was ruled out under its constraints only: after a new
    constraint the second solve finds what a fresh planner with both constraints finds."""
    mesh = meshes["2d"]
    model_fn, input_fn = make_model_and_inputs(mesh, "ffn")

    def planner():
        with torch.device("meta"):
            model = model_fn()
        p = OraclePlanner(model, input_fn, mesh)
        p.__enter__()
        p.add_parameter_memory_constraint(low=0, high=None)
        return p

    a = planner()
    first_plan = a.optimize_placement()
    oa = a.sharding_optimizer
    first = oa.objective_value()
    assert oa.solve_stats["columns_after_pruning"] < oa.solve_stats["columns"]
    node = get_param_nodes(a.gm.graph)[0]

    def plan_of(_, n):
        return first_plan[n].output_specs.placements

    assert plan_of(a, node) == (Shard(0), Shard(0))
    forced = (Shard(0), Shard(1))  # not what the first plan chose: its variables were pruned
    oa.add_node_constraint(node, forced)
    plan = a.optimize_placement()
    assert plan[node].output_specs.placements == forced
    second, columns = oa.objective_value(), oa.solve_stats["columns"]
    a.__exit__(None, None, None)
    b = planner()
    b.sharding_optimizer.add_node_constraint(get_param_nodes(b.gm.graph)[0], forced)
    b.optimize_placement()
    assert math.isclose(second, b.sharding_optimizer.objective_value(), rel_tol=1e-13)
    assert second > first
    assert columns == b.sharding_optimizer.solve_stats["columns"]
    b.__exit__(None, None, None)


@pytest.mark.parametrize("kind,mesh_key", [("ffn", "2d"), ("block", "2d"), ("block", "1d")])
def test_solve_near_the_bound_is_the_programs_optimum(meshes, kind, mesh_key):
    """With an ascent cut short the incumbent stays above the bound; the program restricted to
    the variables near the bound is solved for growing slacks and the first restricted optimum
    within its slack is taken: it equals the full program's optimum, and the plan is a feasible
    plan of the full program."""

    class ShortAscent(OracleOptimizer):
        prune_sweep_chunks = (2,)
        prune_max_sweeps = 2
        prune_slacks = (1e-6, 1e-3, 1e-1)

    class ShortAscentPlanner(AutoParallelPlanner):
        optimizer_cls = ShortAscent

    class FullOptimizer(OracleOptimizer):
        prune_before_solve = False

    class FullPlanner(AutoParallelPlanner):
        optimizer_cls = FullOptimizer

    a, plan_a = _plan(ShortAscentPlanner, meshes[mesh_key], kind, None)
    b, plan_b = _plan(FullPlanner, meshes[mesh_key], kind, None)
    oa, ob = a.sharding_optimizer, b.sharding_optimizer
    sa = oa.solve_stats
    assert sa["prune_sweeps"] == 2 and sa["incumbent"] - sa["lower_bound"] > oa.prune_gap * abs(sa["incumbent"]), sa
    tries = sa["near_bound_solves"]
    assert tries and tries[-1]["value"] is not None and tries[-1]["value"] <= sa["lower_bound"] + tries[-1]["slack"]
    assert [t["slack"] for t in tries] == sorted(t["slack"] for t in tries)
    assert all(t["value"] is None or t["value"] > sa["lower_bound"] + t["slack"] for t in tries[:-1])
    assert sa["columns_solved"] < sa["columns"]
    assert math.isclose(oa.objective_value(), ob.objective_value(), rel_tol=1e-13)
    assert not ob.prob.violated_constraints(oa.prob.x)
    assert math.isclose(float(ob.prob.objective @ oa.prob.x), ob.prob.objective_value, rel_tol=1e-12)
    if mesh_key == "2d":
        _check_2d(a, plan_a, kind)
    else:
        _check_1d(a, plan_a, kind, None)


@pytest.mark.parametrize("kind,mesh_key", [("ffn", "2d"), ("block", "1d")])
def test_node_choice_variables_do_not_change_the_optimum(meshes, kind, mesh_key):
    """Declaring only the per-(node, strategy) variables integral is a reformulation: the
    reference's all-binary program has the same optimum."""

    class AllBinaryOptimizer(OracleOptimizer):
        node_choice_variables = False

    class AllBinaryPlanner(AutoParallelPlanner):
        optimizer_cls = AllBinaryOptimizer

    a, plan_a = _plan(OraclePlanner, meshes[mesh_key], kind, None)
    b, plan_b = _plan(AllBinaryPlanner, meshes[mesh_key], kind, None)
    oa, ob = a.sharding_optimizer, b.sharding_optimizer
    assert oa.n_choice_variables > 0 and ob.n_choice_variables == 0
    assert oa.prob.n_vars == oa.n_variables + oa.n_choice_variables and ob.prob.n_vars == ob.n_variables
    assert math.isclose(oa.objective_value(), ob.objective_value(), rel_tol=1e-12)
    assert not oa.prob.violated_constraints() and not ob.prob.violated_constraints()


@pytest.mark.gpu
@pytest.mark.parametrize("kind,mesh_key", [("block", "2d"), ("ffn", "2d")])
def test_solve_near_the_bound_from_device_sweeps(gpu_device, meshes, kind, mesh_key):
    """The ascent cut short on the device as on its CPU restatement: the same bound, the same
    tries near the bound, the same optimum as the full program's."""

    class ShortDevice(ShardingOptimizer):
        prune_sweep_chunks = (2,)
        prune_max_sweeps = 2
        prune_slacks = (1e-6, 1e-3, 1e-1)

    class ShortDevicePlanner(AutoParallelPlanner):
        optimizer_cls = ShortDevice

    class ShortOracle(OracleOptimizer):
        prune_sweep_chunks = (2,)
        prune_max_sweeps = 2
        prune_slacks = (1e-6, 1e-3, 1e-1)

    class ShortOraclePlanner(AutoParallelPlanner):
        optimizer_cls = ShortOracle

    class FullOptimizer(OracleOptimizer):
        prune_before_solve = False

    class FullPlanner(AutoParallelPlanner):
        optimizer_cls = FullOptimizer

    a, plan_a = _plan(ShortDevicePlanner, meshes[mesh_key], kind, None)
    b, _ = _plan(ShortOraclePlanner, meshes[mesh_key], kind, None)
    c, _ = _plan(FullPlanner, meshes[mesh_key], kind, None)
    oa, ob, oc = a.sharding_optimizer, b.sharding_optimizer, c.sharding_optimizer
    assert type(oa.backend).__name__ == "DeviceBackend"
    sa, sb = oa.solve_stats, ob.solve_stats
    assert sa["near_bound_solves"] and len(sa["near_bound_solves"]) == len(sb["near_bound_solves"])
    assert math.isclose(sa["lower_bound"], sb["lower_bound"], rel_tol=1e-12)
    for ta, tb_ in zip(sa["near_bound_solves"], sb["near_bound_solves"]):
        assert ta["columns"] == tb_["columns"] and math.isclose(ta["slack"], tb_["slack"], rel_tol=1e-9)
    assert math.isclose(oa.objective_value(), oc.objective_value(), rel_tol=1e-13)
    assert not oc.prob.violated_constraints(oa.prob.x)
    _check_2d(a, plan_a, kind)


@pytest.mark.gpu
def test_local_map_plan_from_device_tables(gpu_device, meshes):
    dev_autop, dev_plan = _plan_local_map(AutoParallelPlanner, meshes["3d"])
    ora_autop, ora_plan = _plan_local_map(OraclePlanner, meshes["3d"])
    d, o = dev_autop.sharding_optimizer, ora_autop.sharding_optimizer
    assert type(d.backend).__name__ == "DeviceBackend"
    assert np.array_equal(d.comm_cost, o.comm_cost)
    assert np.array_equal(d.transition_cost, o.transition_cost)
    assert np.array_equal(d.cost, o.cost)
    assert d.res == o.res and d.objective_value() == o.objective_value()
    _check_local_map(dev_autop, dev_plan)


def test_reference_entry_point_signature(meshes):
    """``AutoParallel`` with the reference's constructor (api.py:202-253): mixed-precision policy,
    loss function with (inputs, target), context-manager discipline, plan on the (32, 8) mesh."""
    from torch.distributed.fsdp import MixedPrecisionPolicy

    from autoparallel_amd.api import AutoParallel

    class OracleAutoParallel(AutoParallel):
        optimizer_cls = OracleOptimizer

    mesh = meshes["2d"]
    bs, dim = 64 * mesh.shape[0], 1024
    with torch.device("meta"):
        model = torch.nn.Linear(dim, dim)

    def input_fn():
        return torch.randn(bs, dim)

    def with_target():
        return input_fn(), torch.randn(bs, dim)

    autop = OracleAutoParallel(model, with_target, mesh, MixedPrecisionPolicy(param_dtype=torch.bfloat16, reduce_dtype=torch.float32),
                               loss_fn=torch.nn.functional.mse_loss, repeated_subgraphs=True)
    with pytest.raises(RuntimeError, match="context manager"):
        autop.add_parameter_memory_constraint()
    with autop:
        assert autop.sharding_optimizer.rescale_grad_comm_cost_for_mp == pytest.approx(4 / 2 * 1.1)
        autop.add_parameter_memory_constraint(low=None, high=None)
        autop.add_input_constraints([(Shard(0), Replicate())] * 2)
        autop.add_output_constraints([(Replicate(), Replicate())])  # the loss is a scalar: no batch dim to shard
        placement = autop.optimize_placement(verbose=False)
        params = get_param_nodes(autop.gm.graph)
        assert len(params) == 2 and all(placement[n].output_specs.tensor_meta.dtype == torch.float32 for n in params)
        with pytest.raises(NotImplementedError, match="outside this package"):
            autop.apply_placement(placement)
    with pytest.raises(RuntimeError, match="not reentrant"):
        autop.optimize_placement()
    with pytest.raises(ValueError, match="input_fn must return"):
        with OracleAutoParallel(model, input_fn, mesh, loss_fn=torch.nn.functional.mse_loss):
            pass


class _PartlyFrozen(torch.nn.Module):
    """Trainable weights, a frozen weight and a buffer (the planning half of the reference's
    tests/test_ordered_sharding.py:90-188: parameters whose gradient node is None)."""

    def __init__(self, dim, all_frozen=False):
        super().__init__()
        self.first = torch.nn.Linear(dim, dim, bias=False)
        self.frozen = torch.nn.Parameter(torch.randn(dim, dim), requires_grad=False)
        self.register_buffer("offset", torch.randn(dim))
        self.last = torch.nn.Linear(dim, dim, bias=False)
        if all_frozen:
            for p in self.parameters():
                p.requires_grad = False

    def forward(self, x):
        x = self.first(x)
        x = x + torch.mm(x, self.frozen)
        x = x + self.offset
        return self.last(x)


@pytest.mark.parametrize("all_frozen", [False, True])
def test_plans_with_parameters_that_have_no_gradient(meshes, all_frozen):
    from torch._functorch._aot_autograd.fx_utils import get_param_and_grad_nodes

    mesh, dim = meshes["2d"], 128
    with torch.device("meta"):
        model = _PartlyFrozen(dim, all_frozen)
    with OraclePlanner(model, lambda: torch.randn(512, dim, requires_grad=True), mesh) as autop:
        autop.add_parameter_memory_constraint(low=0, high=None)
        placement = autop.optimize_placement()
        pairs = list(get_param_and_grad_nodes(autop.gm.graph).values())
        assert len(pairs) == 3
        assert any(grad is None for _, grad in pairs)
        assert all(grad is None for _, grad in pairs) == all_frozen
        for param, grad in pairs:  # a parameter and its gradient (where it has one) are placed alike
            assert param in placement
            if grad is not None:
                assert placement[param].output_specs.placements == placement[grad].output_specs.placements
        assert not autop.sharding_optimizer.prob.violated_constraints()



def test_print_costs_for_node(meshes, capsys):
    autop, _ = _plan(OraclePlanner, meshes["2d"], "ffn", None)
    opt = autop.sharding_optimizer
    mm = autop.gm.graph.find_nodes(op="call_function", target=torch.ops.aten.mm.default)[0]
    opt.print_costs_for_node(mm, arg=1, floatfmt=".3f")
    out = capsys.readouterr().out.splitlines()
    n_rows = len(opt.strats[mm].strategies)
    n_cols = len(opt.strats[opt._all_input_nodes(mm)[1]].strategies)
    assert len(out) == 2 + n_rows  # header, rule, one line per strategy of the node
    s_i = opt.node_map[mm]
    first = opt.ds[(s_i, 1, 0, 0)]["comm_cost"]
    assert f"{first:.3f}" in out[2]
    assert len(out[0].split("  ")) >= n_cols


def _plan_clustered(planner_cls, mesh, clustering=None):
    model_fn, input_fn = make_model_and_inputs(mesh, "block")
    with torch.device("meta"):
        model = model_fn()

    class Planner(planner_cls):
        pass

    if clustering is not None:
        class Optimizer(planner_cls.optimizer_cls):
            pass

        Optimizer.clustering = clustering
        Planner.optimizer_cls = Optimizer
    with Planner(model, input_fn, mesh, repeated_subgraphs=True) as autop:
        autop.add_parameter_memory_constraint(low=0, high=None)
        placement = autop.optimize_placement()
        return autop, placement


def _reference_links_of_the_block():
    import json
    import os

    with open(os.path.join(os.path.dirname(__file__), "golden", "reference_strategies_and_costs.json")) as f:
        case = json.load(f)["cases"]["block_32x8"]
    assert case["cluster_links_error"] is None and len(case["cluster_links"]) == 50
    return case["cluster_links"]


def test_repeated_subgraphs_take_the_references_links_where_its_algorithm_returns(meshes):
    """``repeated_subgraphs=True`` on the reference's transformer block: the default finds the links
    the reference's own ``get_identical_regions`` + ``create_cluster_links`` produced on this
    graph (held by the fixture), i.e. it solves the reference's program; on a Llama-shaped graph,
    where the reference's function ends in its "Duplicate node" error, the neighbourhood algorithm
    takes over and says so."""
    autop, plan = _plan_clustered(OraclePlanner, meshes["2d"])
    o = autop.sharding_optimizer
    assert o.clustering == "reference" and o.clustering_used.startswith("regions")
    assert {n.name: r.name for n, r in o.node_representative.items()} == _reference_links_of_the_block()
    # the same program as with the reference's algorithm asked for by name; another one than the
    # neighbourhood algorithm's (which links other node sets on this graph)
    by_name, plan_by_name = _plan_clustered(OraclePlanner, meshes["2d"], "regions")
    assert by_name.sharding_optimizer.objective_value() == o.objective_value()
    assert {n.name: str(s) for n, s in plan.items()} == {n.name: str(s) for n, s in plan_by_name.items()}
    other, _ = _plan_clustered(OraclePlanner, meshes["2d"], "neighbourhood")
    assert other.sharding_optimizer.clustering_used.startswith("neighbourhood")
    assert {n.name: r.name for n, r in other.sharding_optimizer.node_representative.items()} != _reference_links_of_the_block()
    # linked nodes take one strategy; the clustered optimum is no better than the free one
    for node, rep in o.node_representative.items():
        assert str(plan[node]) == str(plan[rep]), (node, rep)
    free, _ = _plan(OraclePlanner, meshes["2d"], "block", None)
    assert o.objective_value() >= free.sharding_optimizer.objective_value() * (1 - 1e-12)
    # (the reference's expected placements of this model are those of the free program: its links tie
    # the four attention projections to one strategy, which moves the optimum)


def test_repeated_subgraphs_fall_back_where_the_references_algorithm_raises(fake_pg):
    from autoparallel_amd.graphs import workloads

    mesh = workloads.logical_mesh((32, 8))
    model, input_fn, _, _ = workloads.build_model("llama3_8b", mesh, n_layers=2)
    with OraclePlanner(model, input_fn, mesh, param_dtype=torch.bfloat16, repeated_subgraphs=True) as autop:
        o = autop.sharding_optimizer
        assert o.clustering_used.startswith("neighbourhood (the reference's algorithm raised: Duplicate node")
        assert len(o.node_representative) > 0

    class Small(OracleOptimizer):
        regions_max_nodes = 10

    class Planner(OraclePlanner):
        optimizer_cls = Small

    with Planner(model, input_fn, mesh, param_dtype=torch.bfloat16, repeated_subgraphs=True) as autop:
        assert "regions_max_nodes" in autop.sharding_optimizer.clustering_used


@pytest.mark.gpu
def test_repeated_subgraphs_with_device_tables_solve_the_references_program(gpu_device, meshes):
    """The device tables under the reference's links: the plan and objective of the oracle's tables
    under the same links."""
    dev, dev_plan = _plan_clustered(AutoParallelPlanner, meshes["2d"])
    ora, ora_plan = _plan_clustered(OraclePlanner, meshes["2d"])
    d, o = dev.sharding_optimizer, ora.sharding_optimizer
    assert type(d.backend).__name__ == "DeviceBackend" and d.clustering_used.startswith("regions")
    assert {n.name: r.name for n, r in d.node_representative.items()} == _reference_links_of_the_block()
    assert d.res == o.res and d.objective_value() == o.objective_value()
    assert {n.name: str(s) for n, s in dev_plan.items()} == {n.name: str(s) for n, s in ora_plan.items()}
