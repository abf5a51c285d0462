"""Bound-based pruning of the planning program before it goes to the solver.

No counterpart in the reference, which hands the full program to CBC
(autoparallel/optimize_sharding.py:648-659).  The planning program is a pairwise labelling
problem: every node (every class of linked nodes, optimize_sharding.py:211-231) takes one
strategy, and every edge block charges ``theta[r, c]`` for the pair (consumer strategy r,
producer strategy c).  On that form a dual ascent is cheap and, run on the device, nearly
free:

  * ``LabelGraph`` is the labelling problem read off the planner's variable blocks: classes,
    one unary cost vector per class (edges without a producer, masks of the user constraints)
    and one cost matrix per pair of adjacent classes (+inf for forbidden pairs);
  * the backend runs sweeps of *min-sum diffusion* over it: a node update takes the row / column
    minima of the node's incident matrices into the node (the segmented minimum of the cost
    tables, applied to the reparametrised matrices) and hands the sum back in equal shares.
    Every update leaves the cost of every labelling unchanged and never lowers the bound
    ``LB = sum_classes min unary + sum_edges min matrix``;
  * ``decode`` rounds the reparametrised costs to a labelling and ``refine`` improves it by local
    search; if the labelling satisfies every row of the program it is an incumbent with cost ``UB``;
  * ``prune`` fixes to zero every strategy whose min-marginal bound, and every strategy pair
    whose entry bound, exceeds ``UB``: such a variable is in no optimal plan, so the set of
    optimal plans, and the optimum, are unchanged, and the solver receives a program a tenth
    (Llama-3-8B) of the size.

Where the rounded labelling stays above the bound, the planner solves the program restricted to the
variables whose bound lies within a slack of ``LB`` (``ShardingOptimizer._solve_near_the_bound``): an
optimum of the restricted program that is itself within the slack is an optimum of the program.

Constraints the labelling form does not model are simply left out of the bound (it stays a
valid lower bound of the constrained program); the incumbent is checked against ALL rows.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np

# a variable is fixed only if its bound exceeds the incumbent by more than this relative margin:
# far above the rounding of a few hundred fp64 updates, far below one transition cost unit
RELATIVE_MARGIN = 1e-7
MAX_LABELS = 2048  # labels of one class the device kernel stages in LDS


@dataclass
class Block:
    """One block of entry variables: ``nt x ns`` variables from ``var_begin``, rows = strategies of
    class ``row_class``, columns = strategies of class ``col_class`` (-1: no producer)."""
    var_begin: int
    nt: int
    ns: int
    row_class: int
    col_class: int
    edge: int = -1  # merged edge that carries this block (-1: unary or folded diagonal)
    transposed: bool = False  # the merged edge stores col_class x row_class


@dataclass
class LabelGraph:
    label_begin: np.ndarray  # int64 [n_classes + 1]
    unary: np.ndarray  # f64 [n_labels]
    edge_i: np.ndarray  # int32 [n_edges] class of the rows
    edge_j: np.ndarray  # int32 [n_edges] class of the columns
    edge_begin: np.ndarray  # int64 [n_edges + 1]
    theta: np.ndarray  # f64, matrix of edge k = theta[edge_begin[k]:edge_begin[k + 1]].reshape(n_i, n_j)
    inc_begin: np.ndarray  # int64 [n_classes + 1]
    inc_edge: np.ndarray  # int32
    inc_side: np.ndarray  # uint8: 0 = the class labels the rows of the edge, 1 = the columns
    color_begin: np.ndarray  # int64 [n_colors + 1]
    color_nodes: np.ndarray  # int32: classes grouped by colour (no two of a colour share an edge)
    blocks: list = field(default_factory=list)
    class_of_choice_base: dict = field(default_factory=dict)

    @property
    def n_classes(self) -> int:
        return len(self.label_begin) - 1

    @property
    def n_edges(self) -> int:
        return len(self.edge_i)

    def labels(self, c: int) -> int:
        return int(self.label_begin[c + 1] - self.label_begin[c])

    def matrix(self, theta: np.ndarray, k: int) -> np.ndarray:
        ni, nj = self.labels(int(self.edge_i[k])), self.labels(int(self.edge_j[k]))
        return theta[int(self.edge_begin[k]):int(self.edge_begin[k + 1])].reshape(ni, nj)


def build_label_graph(blocks: list, class_sizes: list, block_costs, masks: dict, ties: list) -> LabelGraph:
    """``blocks``: ``Block`` records over merged class ids; ``class_sizes[c]``: labels of class c;
    ``block_costs(block) -> [nt, ns] matrix`` (+inf = forbidden); ``masks[c]``: allowed labels;
    ``ties``: ``(class_i, class_j, matrix)`` extra pair costs (0 / +inf)."""
    n = len(class_sizes)
    label_begin = np.zeros(n + 1, np.int64)
    np.cumsum(class_sizes, out=label_begin[1:])
    unary = [np.zeros(s) for s in class_sizes]
    merged: dict = {}
    order: list = []

    def add_pair(i, j, m, block=None):
        if i == j:  # both sides are the same class: only the diagonal can be taken
            unary[i] += np.diagonal(m)
            return
        if (i, j) in merged:
            merged[(i, j)] = merged[(i, j)] + m
            key, tr = (i, j), False
        elif (j, i) in merged:
            merged[(j, i)] = merged[(j, i)] + m.T
            key, tr = (j, i), True
        else:
            merged[(i, j)] = m.copy()
            order.append((i, j))
            key, tr = (i, j), False
        if block is not None:
            block.edge, block.transposed = key, tr

    for b in blocks:
        m = block_costs(b)
        if b.col_class < 0:
            unary[b.row_class] += m.min(axis=1)  # the program takes the cheapest column of the row
        else:
            add_pair(b.row_class, b.col_class, m, b)
    for i, j, m in ties:
        add_pair(i, j, m)
    for c, allowed in masks.items():
        unary[c] = np.where(allowed, unary[c], np.inf)
    index = {key: k for k, key in enumerate(order)}
    for b in blocks:
        if isinstance(b.edge, tuple):
            b.edge = index[b.edge]
    edge_i = np.asarray([i for i, _ in order], np.int32)
    edge_j = np.asarray([j for _, j in order], np.int32)
    sizes = np.asarray([class_sizes[i] * class_sizes[j] for i, j in order], np.int64)
    edge_begin = np.zeros(len(order) + 1, np.int64)
    np.cumsum(sizes, out=edge_begin[1:])
    theta = np.concatenate([merged[key].ravel() for key in order]) if order else np.zeros(0)
    # incidence, in edge order
    inc: list = [[] for _ in range(n)]
    for k, (i, j) in enumerate(order):
        inc[i].append((k, 0))
        inc[j].append((k, 1))
    inc_begin = np.zeros(n + 1, np.int64)
    np.cumsum([len(x) for x in inc], out=inc_begin[1:])
    inc_edge = np.asarray([k for x in inc for k, _ in x], np.int32)
    inc_side = np.asarray([s for x in inc for _, s in x], np.uint8)
    # greedy colouring in class order: classes of one colour share no edge and update together
    color = np.full(n, -1, np.int64)
    for c in range(n):
        used = {int(color[int(edge_j[k]) if s == 0 else int(edge_i[k])]) for k, s in inc[c]}
        col = 0
        while col in used:
            col += 1
        color[c] = col
    n_colors = int(color.max()) + 1 if n else 0
    color_nodes = np.argsort(color, kind="stable").astype(np.int32)
    color_begin = np.zeros(n_colors + 1, np.int64)
    np.cumsum(np.bincount(color, minlength=n_colors), out=color_begin[1:])
    return LabelGraph(label_begin=label_begin, unary=np.concatenate(unary) if n else np.zeros(0), edge_i=edge_i,
                      edge_j=edge_j, edge_begin=edge_begin, theta=np.ascontiguousarray(theta, np.float64),
                      inc_begin=inc_begin, inc_edge=inc_edge, inc_side=inc_side, color_begin=color_begin,
                      color_nodes=color_nodes, blocks=blocks)


def lower_bound(g: LabelGraph, theta: np.ndarray, unary: np.ndarray):
    """-> (LB, per-class minimum of the unary vector, per-edge minimum of the matrix)"""
    lb = g.label_begin
    umin = np.asarray([unary[lb[c]:lb[c + 1]].min() if lb[c + 1] > lb[c] else 0.0 for c in range(g.n_classes)])
    emin = np.asarray([theta[g.edge_begin[k]:g.edge_begin[k + 1]].min() for k in range(g.n_edges)])
    return math.fsum(umin) + math.fsum(emin), umin, emin


def decode(g: LabelGraph, theta: np.ndarray, unary: np.ndarray) -> np.ndarray:
    """A labelling from the reparametrised costs: classes in order, each takes the label that is
    cheapest given the labels already taken by its neighbours and the best case for the rest."""
    n = g.n_classes
    lab = np.full(n, -1, np.int64)
    lb = g.label_begin
    for c in range(n):
        score = unary[lb[c]:lb[c + 1]].copy()
        for t in range(int(g.inc_begin[c]), int(g.inc_begin[c + 1])):
            k, side = int(g.inc_edge[t]), int(g.inc_side[t])
            m = g.matrix(theta, k)
            if side == 1:
                m = m.T
            other = int(g.edge_j[k]) if side == 0 else int(g.edge_i[k])
            score = score + (m[:, lab[other]] if lab[other] >= 0 else m.min(axis=1))
        lab[c] = int(np.argmin(score)) if len(score) else -1
    return lab


def refine(g: LabelGraph, theta: np.ndarray, unary: np.ndarray, labels: np.ndarray, max_rounds: int = 10) -> np.ndarray:
    """Local search from a labelling: class by class, the label that is cheapest given the labels
    of all its neighbours, until a round changes nothing (after the first round only classes with
    a changed neighbour are looked at again).  Never raises the labelling's cost."""
    lab = labels.copy()
    lb = g.label_begin
    todo = np.ones(g.n_classes, bool)
    for _ in range(max_rounds):
        again = np.zeros(g.n_classes, bool)
        for c in np.nonzero(todo)[0]:
            if lab[c] < 0:
                continue
            score = unary[lb[c]:lb[c + 1]].copy()
            others = []
            for t in range(int(g.inc_begin[c]), int(g.inc_begin[c + 1])):
                k, side = int(g.inc_edge[t]), int(g.inc_side[t])
                m = g.matrix(theta, k)
                other = int(g.edge_j[k]) if side == 0 else int(g.edge_i[k])
                others.append(other)
                score = score + (m[:, lab[other]] if side == 0 else m[lab[other], :])
            best = int(np.argmin(score))
            if score[best] < score[lab[c]]:
                lab[c] = best
                again[others] = True
        if not again.any():
            break
        todo = again
    return lab


def prune_masks(g: LabelGraph, theta: np.ndarray, unary: np.ndarray, ub: float):
    """-> (dead labels bool[n_labels], dead pairs bool[len(theta)]): labels whose min-marginal
    bound, pairs whose entry bound, exceed ``ub`` by more than the margin; a pair with a dead
    end is dead."""
    bound, umin, emin = lower_bound(g, theta, unary)
    limit = ub + RELATIVE_MARGIN * max(abs(ub), 1.0)
    lb = g.label_begin
    label_bound = np.empty(len(unary))
    for c in range(g.n_classes):
        b = (bound - umin[c]) + unary[lb[c]:lb[c + 1]]
        for t in range(int(g.inc_begin[c]), int(g.inc_begin[c + 1])):
            k, side = int(g.inc_edge[t]), int(g.inc_side[t])
            m = g.matrix(theta, k)
            b = (b - emin[k]) + (m.min(axis=1) if side == 0 else m.min(axis=0))
        label_bound[lb[c]:lb[c + 1]] = b
    dead_label = ~(label_bound <= limit)
    dead_pair = np.zeros(len(theta), bool)
    for k in range(g.n_edges):
        i, j = int(g.edge_i[k]), int(g.edge_j[k])
        m = g.matrix(theta, k)
        d = ~((bound - emin[k]) + m <= limit)
        d |= dead_label[lb[i]:lb[i + 1]][:, None] | dead_label[lb[j]:lb[j + 1]][None, :]
        dead_pair[int(g.edge_begin[k]):int(g.edge_begin[k + 1])] = d.ravel()
    return dead_label, dead_pair
