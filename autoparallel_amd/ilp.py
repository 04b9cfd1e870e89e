"""Sparse 0/1 integer program: rows as index/coefficient arrays, an LP-file
writer, and the solver hand-off.

The reference builds one ``pulp.LpVariable`` per decision variable and one
``LpAffineExpression`` per constraint and hands the model to CBC through PuLP
(autoparallel/optimize_sharding.py:412-438, 665-820, 887-912).  Here the same
model is kept as arrays: a row is (name, variable indices, coefficients, sense,
rhs).  Names follow the reference: variables
``n={node},s={idx},arg={a},output_p={o},input_p={j}`` (:432-436), rows
``{prefix}_{counter:03}`` (:293-296).  Solvers: HiGHS through SciPy (always
available with the pinned SciPy), or PuLP's CBC when PuLP is importable; both
receive the identical matrix.
"""
from __future__ import annotations

import collections
import re
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

EQ, LE, GE = 0, -1, 1
_SENSE_STR = {EQ: "=", LE: "<=", GE: ">="}

STATUS_OPTIMAL = 1
STATUS_INFEASIBLE = -1
STATUS_NOT_SOLVED = 0


class Row:
    __slots__ = ("name", "idx", "coef", "sense", "rhs")

    def __init__(self, name: str, idx: np.ndarray, coef: np.ndarray, sense: int, rhs: float):
        self.name = name
        self.idx = np.asarray(idx, np.int64)
        self.coef = np.asarray(coef, np.float64)
        self.sense = sense
        self.rhs = float(rhs)

    def valid(self, x: np.ndarray, tol: float = 1e-6) -> bool:
        lhs = float((self.coef * x[self.idx]).sum())
        if self.sense == EQ:
            return abs(lhs - self.rhs) <= tol
        if self.sense == LE:
            return lhs <= self.rhs + tol
        return lhs >= self.rhs - tol


class SparseILP:
    """Minimise c.x over binary x subject to named rows."""

    def __init__(self, n_vars: int):
        self.n_vars = int(n_vars)
        self.objective = np.zeros(self.n_vars, np.float64)
        self.upper = np.ones(self.n_vars, np.float64)  # 0 fixes a variable out of the model
        self.constraints: "collections.OrderedDict[str, Row]" = collections.OrderedDict()
        self._counters: Dict[str, int] = {}
        self.status = STATUS_NOT_SOLVED
        self.x: Optional[np.ndarray] = None
        self.objective_value: Optional[float] = None

    # -- naming ---------------------------------------------------------------
    def next_name(self, prefix: str) -> str:
        i = self._counters.setdefault(prefix, 0)
        self._counters[prefix] = i + 1
        return f"{prefix}_{i:03}"

    # -- rows -----------------------------------------------------------------
    def add_row(self, prefix_or_name: str, idx, coef, sense: int, rhs: float, exact_name: bool = False) -> str:
        name = prefix_or_name if exact_name else self.next_name(prefix_or_name)
        idx = np.asarray(idx, np.int64)
        if np.isscalar(coef):
            coef = np.full(idx.shape[0], float(coef))
        assert idx.shape[0] == len(coef)
        assert idx.size == 0 or (0 <= idx.min() and idx.max() < self.n_vars)
        self.constraints[name] = Row(name, idx, coef, sense, rhs)
        return name

    def remove(self, name: str) -> None:
        del self.constraints[name]

    # -- matrices ---------------------------------------------------------------
    def to_matrix(self):
        """(A csr, lower, upper, var_upper): rows ``var == 0`` become variable
        bounds instead of matrix rows."""
        import scipy.sparse as sp

        ub = self.upper.copy()
        data, cols, ptr, lo, hi = [], [], [0], [], []
        for r in self.constraints.values():
            if r.sense == EQ and r.rhs == 0.0 and r.idx.shape[0] == 1 and r.coef[0] != 0:
                ub[r.idx[0]] = 0.0
                continue
            data.append(r.coef)
            cols.append(r.idx)
            ptr.append(ptr[-1] + r.idx.shape[0])
            if r.sense == EQ:
                lo.append(r.rhs); hi.append(r.rhs)
            elif r.sense == LE:
                lo.append(-np.inf); hi.append(r.rhs)
            else:
                lo.append(r.rhs); hi.append(np.inf)
        n_rows = len(lo)
        A = sp.csr_matrix(
            (np.concatenate(data) if data else np.zeros(0), np.concatenate(cols) if cols else np.zeros(0, np.int64),
             np.asarray(ptr, np.int64)),
            shape=(n_rows, self.n_vars),
        )
        return A, np.asarray(lo), np.asarray(hi), ub

    # -- solve ------------------------------------------------------------------
    def solve(self, backend: str = "auto", time_limit: Optional[float] = None, verbose: bool = False) -> int:
        if backend == "auto":
            backend = "highs"
        if backend == "highs":
            return self._solve_highs(time_limit, verbose)
        if backend == "cbc":
            return self._solve_pulp_cbc(verbose)
        raise ValueError(f"unknown ILP backend {backend!r}")

    def _solve_highs(self, time_limit, verbose) -> int:
        from scipy.optimize import Bounds, LinearConstraint, milp

        A, lo, hi, ub = self.to_matrix()
        cons = [LinearConstraint(A, lo, hi)] if A.shape[0] else []
        opts = {"disp": bool(verbose)}
        if time_limit is not None:
            opts["time_limit"] = float(time_limit)
        res = milp(self.objective, constraints=cons, integrality=np.ones(self.n_vars),
                   bounds=Bounds(np.zeros(self.n_vars), ub), options=opts)
        if res.x is None:
            self.status = STATUS_INFEASIBLE
            self.x = None
            self.objective_value = None
            return self.status
        self.x = np.rint(res.x)
        self.objective_value = float(self.objective @ self.x)
        self.status = STATUS_OPTIMAL
        return self.status

    def _solve_pulp_cbc(self, verbose) -> int:
        import tempfile

        import pulp  # only when the caller asks for it

        prob = pulp.LpProblem("AutoParallel", pulp.LpMinimize)
        xs = [pulp.LpVariable(f"x{i}", cat=pulp.LpBinary) for i in range(self.n_vars)]
        prob += pulp.lpSum(float(c) * v for c, v in zip(self.objective, xs) if c != 0.0)
        for r in self.constraints.values():
            e = pulp.lpSum(float(c) * xs[i] for i, c in zip(r.idx, r.coef))
            prob += ((e == r.rhs) if r.sense == EQ else (e <= r.rhs) if r.sense == LE else (e >= r.rhs), r.name)
        solver = pulp.PULP_CBC_CMD(msg=verbose)
        with tempfile.TemporaryDirectory() as tmp:
            solver.tmpDir = tmp
            prob.solve(solver)
        if prob.status == -1:
            self.status = STATUS_INFEASIBLE
            return self.status
        self.x = np.asarray([round(v.value() or 0.0) for v in xs], np.float64)
        self.objective_value = float(self.objective @ self.x)
        self.status = STATUS_OPTIMAL
        return self.status

    def violated(self) -> List[str]:
        if self.x is None:
            return []
        return [n for n, r in self.constraints.items() if not r.valid(self.x)]

    # -- LP file ------------------------------------------------------------------
    def write_lp(self, path: str, var_names: Optional[Sequence[str]] = None) -> None:
        """CPLEX LP text of the model (what PuLP's ``writeLP`` produces for the
        reference's problem, up to term order)."""
        def vn(i):
            if var_names is None:
                return f"x{i}"
            return re.sub(r"[^A-Za-z0-9_.]", "_", var_names[i])

        def expr(idx, coef):
            parts = []
            for i, c in zip(idx, coef):
                if c == 0:
                    continue
                sign = "-" if c < 0 else "+"
                mag = abs(c)
                parts.append(f"{sign} {vn(i)}" if mag == 1 else f"{sign} {mag!r} {vn(i)}")
            return " ".join(parts) if parts else "0"

        with open(path, "w") as f:
            f.write("\\* AutoParallel *\\\nMinimize\nOBJ: ")
            nz = np.nonzero(self.objective)[0]
            f.write(expr(nz, self.objective[nz]) + "\nSubject To\n")
            for r in self.constraints.values():
                f.write(f"{r.name}: {expr(r.idx, r.coef)} {_SENSE_STR[r.sense]} {r.rhs!r}\n")
            f.write("Binaries\n")
            for i in range(self.n_vars):
                if self.upper[i] > 0:  # variables fixed out of the model are not declared
                    f.write(vn(i) + "\n")
            f.write("End\n")
