"""The per-strategy lower bounds and greedy strategies (no reference counterpart: the
reference hands the full table to the solver, optimize_sharding.py:648-659).  The oracle's
restatement is pinned by brute force over every plan of tiny graphs; the planner's bound is
checked against the solved optimum."""

import itertools
import math

import numpy as np
import pytest

from oracle import cost_oracle as po


def _tiny_graph(seed, n_nodes=5, chain_only=False):
    """Random DAG with 2-3 strategies per node and random cost matrices, in the planner's
    layout: edges ordered by consumer, one matrix [consumer strategies x producer strategies]
    per edge, stored row-major."""
    rng = np.random.default_rng(seed)
    n_strat = rng.integers(2, 4, n_nodes)
    edges = []  # (consumer, producer)
    for c in range(1, n_nodes):
        k = 1 if chain_only else int(rng.integers(1, 3))
        for p in sorted(rng.choice(c, size=min(k, c), replace=False)):
            edges.append((c, int(p)))
    mats = []
    for c, p in edges:
        m = rng.uniform(0.0, 100.0, (n_strat[c], n_strat[p]))
        m[rng.random(m.shape) < 0.1] = math.inf  # banned transitions
        m[:, 0] = np.where(np.isinf(m[:, 0]), 1.0, m[:, 0])  # (keep every row feasible)
        mats.append(m)
    nsb = np.zeros(n_nodes + 1, np.int64)
    np.cumsum(n_strat, out=nsb[1:])
    enc = {"node_strat_begin": nsb, "edge_node": np.array([c for c, _ in edges], np.int32),
           "edge_n_tgt": np.array([n_strat[c] for c, _ in edges], np.int32)}
    return n_strat, edges, mats, enc


def _row_min(mats):
    return [float(m[r].min()) for m in mats for r in range(m.shape[0])]


def _best_plan(n_strat, edges, mats):
    best = math.inf
    for a in itertools.product(*[range(int(s)) for s in n_strat]):
        best = min(best, math.fsum(m[a[c], a[p]] for (c, p), m in zip(edges, mats)))
    return best


@pytest.mark.parametrize("seed", range(12))
def test_bound_never_exceeds_the_best_plan(seed):
    n_strat, edges, mats, enc = _tiny_graph(seed)
    bound, mins, args, lb = po.greedy_strategies(enc, _row_min(mats))
    best = _best_plan(n_strat, edges, mats)
    assert lb <= best * (1 + 1e-12)
    # per-strategy bound, written out: the consumer's row minimum on each of its edges
    for n in range(len(n_strat)):
        for k in range(int(n_strat[n])):
            want = math.fsum(float(m[k].min()) for (c, _), m in zip(edges, mats) if c == n)
            assert math.isclose(bound[int(enc["node_strat_begin"][n]) + k], want, rel_tol=1e-12, abs_tol=0.0)
        seg = bound[int(enc["node_strat_begin"][n]):int(enc["node_strat_begin"][n + 1])]
        assert mins[n] == min(seg) and args[n] == seg.index(min(seg))


@pytest.mark.parametrize("seed", range(6))
def test_bound_is_tight_when_producers_are_free(seed):
    """Consumers whose producers are distinct source nodes: every consumer can take its best
    row and every producer the column that row prefers, so the bound IS the optimum.  (A
    dropped edge, a row/column mix-up or a min over the wrong axis breaks the equality.)"""
    rng = np.random.default_rng(100 + seed)
    n_src, n_cons = 4, 2
    n_strat = rng.integers(2, 4, n_src + n_cons)
    edges = [(n_src + 0, 0), (n_src + 0, 1), (n_src + 1, 2), (n_src + 1, 3)]
    mats = [rng.uniform(1.0, 50.0, (n_strat[c], n_strat[p])) for c, p in edges]
    nsb = np.zeros(len(n_strat) + 1, np.int64)
    np.cumsum(n_strat, out=nsb[1:])
    enc = {"node_strat_begin": nsb, "edge_node": np.array([c for c, _ in edges], np.int32),
           "edge_n_tgt": np.array([n_strat[c] for c, _ in edges], np.int32)}
    _, _, args, lb = po.greedy_strategies(enc, _row_min(mats))
    assert math.isclose(lb, _best_plan(n_strat, edges, mats), rel_tol=1e-12)
    assert all(a == 0 for a in args[:n_src])  # nodes without input edges: every strategy costs 0


def test_a_node_without_strategies_adds_nothing():
    enc = {"node_strat_begin": np.array([0, 2, 2, 4], np.int64), "edge_node": np.array([2], np.int32),
           "edge_n_tgt": np.array([2], np.int32)}
    bound, mins, args, lb = po.greedy_strategies(enc, [3.0, 2.0])
    assert bound == [0.0, 0.0, 3.0, 2.0] and args == [0, -1, 1] and lb == 2.0


def test_planner_bound_and_greedy_choice(fake_pg):
    import torch
    from torch.distributed.device_mesh import init_device_mesh

    from models import make_model_and_inputs
    from test_planner_plans import OraclePlanner

    mesh = init_device_mesh("cpu", (32, 8), mesh_dim_names=("dp", "tp"))
    model_fn, input_fn = make_model_and_inputs(mesh, "ffn")
    with torch.device("meta"):
        model = model_fn()
    with OraclePlanner(model, input_fn, mesh) as autop:
        autop.add_parameter_memory_constraint(low=0, high=None)
        autop.optimize_placement()
        opt = autop.sharding_optimizer
        choice, lb = opt.greedy_strategies()
        assert 0.0 < lb <= opt.objective_value() * (1 + 1e-12)
        assert lb == opt.lower_bound()
        assert set(choice) == {n for n in opt.nodes if n.op != "output"}
        for node, k in choice.items():
            assert 0 <= k < len(opt.strats[node].strategies)
        # edge minima: the minimum of each whole matrix, at the flattened index of its first occurrence
        mins, args = opt.edge_minima()
        eb = opt.encoded.tables.edge_entry_begin
        for e in (0, len(mins) // 2, len(mins) - 1):
            seg = opt.cost[eb[e]:eb[e + 1]]
            assert mins[e] == seg.min() and args[e] == int(np.argmin(seg))
