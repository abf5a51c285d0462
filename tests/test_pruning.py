"""Pruning of the planning program before the solve (no reference counterpart: the reference
hands the whole program to CBC, optimize_sharding.py:648-659).  The dual ascent is pinned by
what the mathematics fixes: a node update leaves the cost of EVERY labelling unchanged and
never lowers the bound (brute force over every labelling of tiny problems), the bound never
exceeds the brute-force optimum, pruning with an incumbent never removes an optimal labelling;
on the reference's test models the pruned program gives the plan and objective of the full one.
GPU: the kernel's sweeps equal the CPU restatement bit for bit."""

import itertools
import math

import numpy as np
import pytest

from autoparallel_amd import pruning
from oracle import cost_oracle as po


def _random_problem(seed, n=6, max_labels=4, p_edge=0.5, p_inf=0.15):
    rng = np.random.default_rng(seed)
    sizes = [int(x) for x in rng.integers(2, max_labels + 1, n)]
    blocks, costs = [], {}
    var = 0
    for i in range(n):
        if rng.random() < 0.5:  # an edge without a producer: only its row minima count
            ns = int(rng.integers(1, 3))
            blocks.append(pruning.Block(var, sizes[i], ns, i, -1))
            costs[var] = rng.uniform(0, 50, (sizes[i], ns))
            var += sizes[i] * ns
        for j in range(i):
            if rng.random() < p_edge:
                m = rng.uniform(0, 100, (sizes[i], sizes[j]))
                m[rng.random(m.shape) < p_inf] = np.inf
                blocks.append(pruning.Block(var, sizes[i], sizes[j], i, j))
                costs[var] = m
                var += m.size
                if rng.random() < 0.3:  # a parallel block, stored the other way round
                    m2 = rng.uniform(0, 10, (sizes[j], sizes[i]))
                    blocks.append(pruning.Block(var, sizes[j], sizes[i], j, i))
                    costs[var] = m2
                    var += m2.size
    masks = {0: rng.random(sizes[0]) < 0.8}
    masks[0][0] = True
    g = pruning.build_label_graph(blocks, sizes, lambda b: costs[b.var_begin], masks, [])
    return g, sizes


def _energy(g, theta, unary, lab):
    e = math.fsum(unary[g.label_begin[c] + lab[c]] for c in range(g.n_classes))
    return e + math.fsum(g.matrix(theta, k)[lab[g.edge_i[k]], lab[g.edge_j[k]]] for k in range(g.n_edges))


def _sweep(g, theta, unary, n):
    theta, unary = theta.copy(), unary.copy()
    po.diffusion_sweeps(n, g.label_begin, g.inc_begin, g.inc_edge, g.inc_side, g.edge_begin, g.edge_i, g.edge_j,
                        g.color_begin, g.color_nodes, theta, unary)
    return theta, unary


@pytest.mark.parametrize("seed", range(10))
def test_sweeps_keep_every_labelling_and_raise_the_bound(seed):
    g, sizes = _random_problem(seed)
    # colours: no two classes of a colour share an edge
    for c0, c1 in zip(g.color_begin[:-1], g.color_begin[1:]):
        group = set(int(x) for x in g.color_nodes[c0:c1])
        assert not any(int(g.edge_i[k]) in group and int(g.edge_j[k]) in group for k in range(g.n_edges))
    labellings = list(itertools.product(*[range(s) for s in sizes]))
    before = np.asarray([_energy(g, g.theta, g.unary, lab) for lab in labellings])
    best = before.min()
    assert np.isfinite(best)
    theta, unary, bound = g.theta, g.unary, -math.inf
    for _ in range(6):
        theta, unary = _sweep(g, theta, unary, 1)
        after = np.asarray([_energy(g, theta, unary, lab) for lab in labellings])
        fin = np.isfinite(before)
        assert np.array_equal(np.isfinite(after), fin)
        assert np.allclose(after[fin], before[fin], rtol=1e-12, atol=1e-9)
        new_bound = pruning.lower_bound(g, theta, unary)[0]
        assert new_bound >= bound - 1e-9 and new_bound <= best + 1e-9
        bound = new_bound
    # an incumbent from the rounding; pruning with it keeps every optimal labelling
    lab = pruning.decode(g, theta, unary)
    ub = _energy(g, g.theta, g.unary, lab)
    if np.isfinite(ub):
        dead_label, dead_pair = pruning.prune_masks(g, theta, unary, ub)
        for opt in (l for l, e in zip(labellings, before) if e <= best + 1e-9):
            assert not any(dead_label[g.label_begin[c] + opt[c]] for c in range(g.n_classes))
            assert not any(g.matrix(dead_pair, k)[opt[g.edge_i[k]], opt[g.edge_j[k]]] for k in range(g.n_edges))
        # and on a chain-like problem this small the bound usually closes: something is pruned
        assert dead_label.sum() + dead_pair.sum() >= 0


def test_chain_bound_is_exact():
    """On a chain the ascent converges to the optimum (dynamic programming in disguise)."""
    rng = np.random.default_rng(3)
    sizes = [3, 4, 2, 5, 3]
    blocks, costs, var = [], {}, 0
    for i in range(1, len(sizes)):
        m = rng.uniform(0, 10, (sizes[i], sizes[i - 1]))
        blocks.append(pruning.Block(var, sizes[i], sizes[i - 1], i, i - 1))
        costs[var] = m
        var += m.size
    g = pruning.build_label_graph(blocks, sizes, lambda b: costs[b.var_begin], {}, [])
    best = min(_energy(g, g.theta, g.unary, lab) for lab in itertools.product(*[range(s) for s in sizes]))
    theta, unary = _sweep(g, g.theta, g.unary, 60)
    assert math.isclose(pruning.lower_bound(g, theta, unary)[0], best, rel_tol=1e-9)
    assert math.isclose(_energy(g, g.theta, g.unary, pruning.decode(g, theta, unary)), best, rel_tol=1e-12)


@pytest.mark.gpu
@pytest.mark.parametrize("seed,n,max_labels", [(0, 8, 5), (1, 40, 70), (2, 25, 130), (3, 150, 24)])
def test_device_sweeps_equal_the_cpu_restatement(gpu_device, seed, n, max_labels):
    from autoparallel_amd import CostModelParams
    from autoparallel_amd.device_tables import DeviceCostTables
    from autoparallel_amd.synthetic import stress_dag

    g, _ = _random_problem(seed, n=n, max_labels=max_labels, p_edge=min(0.5, 4.0 / n))
    dev = DeviceCostTables(stress_dag(seed=1, n_nodes=20, mesh_sizes=(4, 2)), CostModelParams.from_mesh((4, 2)),
                           device=gpu_device)
    theta, unary = g.theta, g.unary
    for chunk in (1, 3, 10):
        want_t, want_u = _sweep(g, theta, unary, chunk)
        theta, unary = dev.diffusion_sweeps(g, theta, unary, chunk)
        assert np.array_equal(theta, want_t) and np.array_equal(unary, want_u), chunk


def _star_problem(seed, centre_labels, leaf_labels, p_inf=0.1):
    """One class joined to every other, the matrices stored either way round."""
    rng = np.random.default_rng(seed)
    sizes = [centre_labels] + list(leaf_labels)
    blocks, costs, var = [], {}, 0
    for j in range(1, len(sizes)):
        rows, cols, ci, cj = (sizes[0], sizes[j], 0, j) if j % 2 else (sizes[j], sizes[0], j, 0)
        m = rng.uniform(0, 100, (rows, cols))
        m[rng.random(m.shape) < p_inf] = np.inf
        blocks.append(pruning.Block(var, rows, cols, ci, cj))
        costs[var] = m
        var += m.size
    return pruning.build_label_graph(blocks, sizes, lambda b: costs[b.var_begin], {}, [])


@pytest.mark.gpu
@pytest.mark.parametrize("name,centre,leaves", [
    ("more labels than threads of a workgroup", 300, [5, 3, 6]),
    ("more incident matrices than are staged", 6, [3] * 70),
    ("as many pairs and elements as are staged", 16, [4] * 64),
    ("one pair of labels more than is staged", 17, [3] * 64),
    ("a few elements more than are staged", 16, [4] * 63 + [5]),
    ("matrices larger than the staging array", 40, [60, 50, 70, 45]),
    ("a planning program's shape", 16, [16, 12, 9, 16, 15, 15, 8, 12, 16, 16, 22, 24, 16, 16, 16, 16]),
])
def test_device_sweeps_on_the_shapes_that_choose_the_kernels_path(gpu_device, name, centre, leaves):
    """The update kernel stages a class's incident matrices in LDS when their number, the pairs
    (matrix, label) and the elements fit, and works on them in memory otherwise: the bits of the
    CPU restatement either way, at the limits and on both sides of them."""
    from autoparallel_amd import CostModelParams
    from autoparallel_amd.device_tables import DeviceCostTables
    from autoparallel_amd.synthetic import stress_dag

    g = _star_problem(7, centre, leaves)
    dev = DeviceCostTables(stress_dag(seed=1, n_nodes=20, mesh_sizes=(4, 2)), CostModelParams.from_mesh((4, 2)),
                           device=gpu_device)
    theta, unary = g.theta, g.unary
    for chunk in (1, 4):
        want_t, want_u = _sweep(g, theta, unary, chunk)
        theta, unary = dev.diffusion_sweeps(g, theta, unary, chunk)
        assert np.array_equal(theta, want_t) and np.array_equal(unary, want_u), (name, chunk)


@pytest.mark.parametrize("seed", range(12))
def test_refine_never_raises_the_cost_and_ends_where_no_single_change_helps(seed):
    g, sizes = _random_problem(100 + seed, n=7, p_inf=0.0)
    theta, unary = _sweep(g, g.theta, g.unary, 2)
    rng = np.random.default_rng(seed)
    start = np.asarray([int(rng.integers(0, s)) for s in sizes], np.int64)
    if not np.isfinite(_energy(g, theta, unary, start)):  # (a masked label of class 0)
        start[0] = 0
    end = pruning.refine(g, theta, unary, start)
    e0, e1 = _energy(g, theta, unary, start), _energy(g, theta, unary, end)
    assert e1 <= e0 + 1e-9
    for c in range(g.n_classes):  # a local optimum: no class alone can do better
        for lab in range(sizes[c]):
            other = end.copy()
            other[c] = lab
            assert _energy(g, theta, unary, other) >= e1 - 1e-9
    # the labelling decode proposes is only ever improved
    d = pruning.decode(g, theta, unary)
    assert _energy(g, theta, unary, pruning.refine(g, theta, unary, d)) <= _energy(g, theta, unary, d) + 1e-9
