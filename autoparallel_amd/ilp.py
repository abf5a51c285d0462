"""A small sparse 0/1 linear program container and its solve through HiGHS
(``scipy.optimize.milp``).

It plays the role PuLP + CBC play for the reference planner
(autoparallel/optimize_sharding.py:86, 648-659): named linear constraints over binary
variables and a linear objective.  Constraints are appended as whole index/coefficient
arrays so a planner can emit thousands of rows per numpy call.
"""

from __future__ import annotations

import time

import numpy as np

_NAME_COUNTERS: dict = {}


def preload_solver():
    """Imports what ``BinaryProgram`` takes from scipy on a helper thread and returns at once
    (in a process that has not used scipy yet, reading its libraries in is a third of the solve
    of a pruned program; a planner starts this before it captures the graph)."""
    import threading

    def load():
        try:
            import scipy.optimize  # noqa: F401
            import scipy.sparse  # noqa: F401
        except Exception:  # noqa: BLE001 (the solve's own import reports it)
            pass

    t = threading.Thread(target=load, name="apcost-solver-import", daemon=True)
    t.start()
    return t


def next_name(prefix: str) -> str:
    idx = _NAME_COUNTERS.setdefault(prefix, 0)
    _NAME_COUNTERS[prefix] += 1
    return f"{prefix}_{idx:03}"


class BinaryProgram:
    def __init__(self, n_vars: int, name: str = "AutoParallel"):
        self.name = name
        self.n_vars = int(n_vars)
        self._cols: list = []
        self._vals: list = []
        self._row_len: list = []
        self._lb: list = []
        self._ub: list = []
        self._names: list = []
        self.upper = np.ones(self.n_vars, np.float64)  # variable upper bounds (0 = forced off)
        # 1 = the variable must be integral, 0 = continuous in [0, upper] (a planner may leave
        # variables continuous whose integrality follows from that of others)
        self.integrality = np.ones(self.n_vars, np.float64)
        self.objective = np.zeros(self.n_vars, np.float64)
        self.status = None
        self.x = None
        self.objective_value = None
        self.solve_seconds = None

    @property
    def n_constraints(self) -> int:
        return len(self._names)

    # ---- building ------------------------------------------------------------------------
    def add_row(self, cols, vals, lb, ub, name: str) -> None:
        cols = np.asarray(cols, np.int64)
        vals = np.broadcast_to(np.asarray(vals, np.float64), cols.shape)
        self._cols.append(cols)
        self._vals.append(vals)
        self._row_len.append(len(cols))
        self._lb.append(float(lb))
        self._ub.append(float(ub))
        self._names.append(name)

    def add_rows(self, cols, vals, row_lengths, lb, ub, prefix: str) -> None:
        """Many rows at once: ``cols`` / ``vals`` are the concatenated rows,
        ``row_lengths`` their lengths; every row gets bounds [lb, ub]."""
        cols = np.asarray(cols, np.int64)
        vals = np.broadcast_to(np.asarray(vals, np.float64), cols.shape)
        row_lengths = np.asarray(row_lengths, np.int64)
        assert int(row_lengths.sum()) == len(cols)
        self._cols.append(cols)
        self._vals.append(vals)
        self._row_len.extend(int(x) for x in row_lengths)
        self._lb.extend([float(lb)] * len(row_lengths))
        self._ub.extend([float(ub)] * len(row_lengths))
        self._names.extend(next_name(prefix) for _ in range(len(row_lengths)))

    def force_zero(self, var_ids) -> None:
        self.upper[np.asarray(var_ids, np.int64)] = 0.0

    def matrix(self):
        from scipy.sparse import csr_matrix

        if not self._names:
            return csr_matrix((0, self.n_vars))
        cached = getattr(self, "_matrix_cache", None)
        if cached is not None and cached[0] == len(self._names):  # rows are only ever appended
            return cached[1]
        indptr = np.zeros(len(self._row_len) + 1, np.int64)
        np.cumsum(self._row_len, out=indptr[1:])
        cols = np.concatenate(self._cols) if self._cols else np.zeros(0, np.int64)
        vals = np.concatenate(self._vals) if self._vals else np.zeros(0, np.float64)
        m = csr_matrix((vals, cols, indptr), shape=(len(self._row_len), self.n_vars))
        m.sum_duplicates()
        self._matrix_cache = (len(self._names), m)
        return m

    def deduplicated(self):
        """(matrix, lb, ub) with repeated rows removed.  Variable sharing makes many
        constraints of linked nodes literally identical; rows are compared through two
        independent 64-bit hashes of their (column, coefficient) pairs."""
        a = self.matrix().copy()
        lb, ub = np.asarray(self._lb), np.asarray(self._ub)
        if a.shape[0] == 0:
            return a, lb, ub
        a.sort_indices()
        a.eliminate_zeros()
        indptr = a.indptr.astype(np.int64)
        nnz_rows = np.nonzero(np.diff(indptr) > 0)[0]
        cols = a.indices.astype(np.uint64)
        vals = a.data.view(np.uint64)
        with np.errstate(over="ignore"):
            h1 = (cols * np.uint64(0x9E3779B97F4A7C15) + np.uint64(0x632BE59BD9B4E019)) ^ (vals * np.uint64(0xD6E8FEB86659FD93))
            h2 = (cols * np.uint64(0xC2B2AE3D27D4EB4F) + np.uint64(0x165667B19E3779F9)) ^ (vals * np.uint64(0xFF51AFD7ED558CCD))
            h1 = h1 * (h1 >> np.uint64(29) | np.uint64(1))
            h2 = h2 * (h2 >> np.uint64(31) | np.uint64(1))
            r1 = np.zeros(a.shape[0], np.uint64)
            r2 = np.zeros(a.shape[0], np.uint64)
            r1[nnz_rows] = np.add.reduceat(h1, indptr[nnz_rows])
            r2[nnz_rows] = np.add.reduceat(h2, indptr[nnz_rows])
        sig = np.stack([r1, r2, np.diff(indptr).astype(np.uint64), lb.view(np.uint64), ub.view(np.uint64)], axis=1)
        _, keep = np.unique(sig, axis=0, return_index=True)
        keep.sort()
        self.rows_before_dedupe, self.rows_after_dedupe = a.shape[0], len(keep)
        return a[keep], lb[keep], ub[keep]

    # ---- solving -------------------------------------------------------------------------
    # The planning programs are pairwise labelling problems whose linear relaxation is almost
    # always tight (HiGHS closed every benchmark graph at the root node).  ``solve`` therefore
    # first drops the columns that are fixed to zero, then solves the relaxation as a plain LP
    # (no MIP presolve, no analytic-centre start: about half the time of the MIP call on the
    # Llama graphs) and accepts a vertex that is integral on the integer columns: an integral
    # optimum of the relaxation is an optimum of the program.  Anything else (a fractional
    # vertex, which needs ties between plans; a time limit) goes to the MIP solver as before.
    lp_first = True

    def _reduced(self):
        """(matrix, lb, ub, kept columns) without the columns whose upper bound is 0; rows keep
        their bounds (a row that can no longer be met makes the program infeasible, as it was)."""
        a, lb, ub = self.deduplicated()
        keep = np.nonzero(self.upper > 0)[0]
        if len(keep) < self.n_vars and a.shape[0]:
            a = a.tocsc()[:, keep].tocsr()
        self.cols_after_fixing = len(keep)
        return a, lb, ub, keep

    def _solve_relaxation(self, a, lb, ub, keep, time_limit):
        from scipy.optimize import linprog

        eq = lb == ub
        a_eq, b_eq = (a[eq], lb[eq]) if eq.any() else (None, None)
        a_ub = b_ub = None
        if (~eq).any():
            from scipy.sparse import vstack

            ai, li, ui = a[~eq], lb[~eq], ub[~eq]
            hi, lo = np.isfinite(ui), np.isfinite(li)
            a_ub = vstack([ai[hi], -ai[lo]]).tocsr()
            b_ub = np.concatenate([ui[hi], -li[lo]])
        options = {} if time_limit is None else {"time_limit": float(time_limit)}
        res = linprog(self.objective[keep], A_ub=a_ub, b_ub=b_ub, A_eq=a_eq, b_eq=b_eq,
                      bounds=np.stack([np.zeros(len(keep)), self.upper[keep]], axis=1), method="highs", options=options)
        if res.status != 0 or res.x is None:
            return None
        ints = self.integrality[keep] > 0
        if np.abs(res.x[ints] - np.rint(res.x[ints])).max(initial=0.0) > 1e-7:
            return None
        return res

    def solve(self, verbose: bool = False, time_limit: float | None = None, mip_rel_gap: float | None = None):
        from scipy.optimize import Bounds, LinearConstraint, milp

        a, lb, ub, keep = self._reduced()
        t0 = time.time()
        self.solved_by = None
        res = None
        if self.lp_first and self._names and len(keep):
            res = self._solve_relaxation(a, lb, ub, keep, time_limit)
            if res is not None:
                self.solved_by = "lp relaxation (integral vertex)"
        if res is None:
            options = {"disp": bool(verbose)}
            if time_limit is not None:
                options["time_limit"] = float(time_limit)
            if mip_rel_gap is not None:
                options["mip_rel_gap"] = float(mip_rel_gap)
            constraints = [LinearConstraint(a, lb, ub)] if self._names else []
            res = milp(self.objective[keep], integrality=self.integrality[keep],
                       bounds=Bounds(np.zeros(len(keep)), self.upper[keep]), constraints=constraints, options=options)
            self.solved_by = "milp"
        self.solve_seconds = time.time() - t0
        self.raw = res
        # scipy: 0 optimal, 1 iteration/time limit, 2 infeasible, 3 unbounded, 4 other
        if res.status == 0 or (res.status == 1 and res.x is not None):
            self.status = 1
            x = np.zeros(self.n_vars, np.int8)
            x[keep] = np.rint(res.x).astype(np.int8)
            self.x = x
            self.objective_value = float(res.fun)
        else:
            self.status = -1
            self.x = None
            self.objective_value = None
        return self.status

    # ---- inspection ------------------------------------------------------------------------
    def violated_constraints(self, x=None, tol: float = 1e-6) -> list:
        x = self.x if x is None else x
        if x is None or not self._names:
            return []
        act = self.matrix() @ np.asarray(x, np.float64)
        bad = np.nonzero((act < np.asarray(self._lb) - tol) | (act > np.asarray(self._ub) + tol))[0]
        return [self._names[i] for i in bad]
