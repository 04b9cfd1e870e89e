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

import collections.abc

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


class _Block:
    """Rows added together, as CSR: names ``{prefix}_{first + i:03}`` (or one exact
    name), one sense, a rhs and a liveness flag per row."""

    __slots__ = ("prefix", "first", "exact", "indptr", "idx", "coef", "sense", "rhs", "alive", "n_alive")

    def __init__(self, prefix, first, exact, indptr, idx, coef, sense, rhs):
        self.prefix, self.first, self.exact = prefix, first, exact
        self.indptr, self.idx, self.coef, self.sense, self.rhs = indptr, idx, coef, sense, rhs
        self.alive = np.ones(rhs.shape[0], bool)
        self.n_alive = int(rhs.shape[0])

    def name(self, i: int) -> str:
        return self.exact if self.exact is not None else f"{self.prefix}_{self.first + i:03}"

    def row(self, i: int) -> Row:
        a, b = self.indptr[i], self.indptr[i + 1]
        return Row(self.name(i), self.idx[a:b], self.coef[a:b], self.sense, self.rhs[i])


class _BlockNames(collections.abc.Sequence):
    """The names of a block's rows, made when asked for (a block can hold millions)."""

    def __init__(self, block, n: int):
        self._block, self._n = block, n

    def __len__(self) -> int:
        return self._n

    def __getitem__(self, i):
        if isinstance(i, slice):
            return [self._block.name(k) for k in range(*i.indices(self._n))]
        if i < 0:
            i += self._n
        if not 0 <= i < self._n:
            raise IndexError(i)
        return self._block.name(i)

    def __eq__(self, other) -> bool:
        return list(self) == list(other) if isinstance(other, (list, tuple, _BlockNames)) else NotImplemented

    def __repr__(self) -> str:
        return repr(list(self))


class _Rows:
    """The model's rows as an ordered name -> Row mapping (insertion order) over
    the blocks; Row objects are made on access."""

    def __init__(self):
        self.blocks: List[_Block] = []
        self.by_prefix: Dict[str, List[_Block]] = {}
        self.exact: Dict[str, _Block] = {}

    def _find(self, name: str) -> Optional[Tuple[_Block, int]]:
        b = self.exact.get(name)
        if b is not None:
            return (b, 0) if b.alive[0] else None
        prefix, _, num = name.rpartition("_")
        if not num.isdigit() or name != f"{prefix}_{int(num):03}":
            return None
        k = int(num)
        for b in self.by_prefix.get(prefix, ()):
            if b.first <= k < b.first + b.rhs.shape[0]:
                return (b, k - b.first) if b.alive[k - b.first] else None
        return None

    def __contains__(self, name) -> bool:
        return self._find(name) is not None

    def __getitem__(self, name) -> Row:
        hit = self._find(name)
        if hit is None:
            raise KeyError(name)
        return hit[0].row(hit[1])

    def __delitem__(self, name) -> None:
        hit = self._find(name)
        if hit is None:
            raise KeyError(name)
        b, i = hit
        b.alive[i] = False
        b.n_alive -= 1
        if b.exact is not None:
            del self.exact[name]

    def pop(self, name, default=None):
        hit = self._find(name)
        if hit is None:
            return default
        row = hit[0].row(hit[1])
        del self[name]
        return row

    def __len__(self) -> int:
        return sum(b.n_alive for b in self.blocks)

    def items(self):
        for b in self.blocks:
            if b.n_alive == 0:
                continue
            for i in (range(b.rhs.shape[0]) if b.n_alive == b.rhs.shape[0] else np.nonzero(b.alive)[0]):
                r = b.row(int(i))
                yield r.name, r

    def __iter__(self):
        for b in self.blocks:
            if b.n_alive == 0:
                continue
            for i in (range(b.rhs.shape[0]) if b.n_alive == b.rhs.shape[0] else np.nonzero(b.alive)[0]):
                yield b.name(int(i))

    keys = __iter__

    def values(self):
        for _, r in self.items():
            yield r


class SparseILP:
    """Minimise c.x over binary x subject to named rows."""

    def __init__(self, n_vars: int):
        self.n_vars = int(n_vars)
        self.objective = np.zeros(self.n_vars, np.float64)
        self.upper = np.ones(self.n_vars, np.float64)  # 0 fixes a variable out of the model
        self.constraints = _Rows()
        self._counters: Dict[str, int] = {}
        self.status = STATUS_NOT_SOLVED
        self.x: Optional[np.ndarray] = None
        self.objective_value: Optional[float] = None
        self.mip_rel_gap = 0.0  # relative optimality gap HiGHS may stop at

    # -- naming ---------------------------------------------------------------
    def next_name(self, prefix: str) -> str:
        i = self._counters.setdefault(prefix, 0)
        self._counters[prefix] = i + 1
        return f"{prefix}_{i:03}"

    # -- rows -----------------------------------------------------------------
    def add_rows(self, prefix: str, indptr, idx, coef, sense: int, rhs) -> List[str]:
        """A block of rows at once: row i has variables ``idx[indptr[i]:indptr[i+1]]``
        with coefficients ``coef`` (an array as long as idx, or one value) and
        right-hand side ``rhs`` (an array or one value).  Names continue the
        prefix's counter.  Returns the names."""
        indptr = np.ascontiguousarray(indptr, np.int64)
        idx = np.ascontiguousarray(idx)
        if idx.dtype != np.int32:  # 32-bit indices are kept as they come: half the bytes of a large block
            idx = np.ascontiguousarray(idx, np.int64)
        n = indptr.shape[0] - 1
        if n <= 0:
            return []
        # coefficients that are all small whole numbers (the +-1 of the default rows) are kept
        # as bytes: an eighth of the memory of a block; a row read out of the block is float64
        if np.isscalar(coef):
            small = float(coef) == int(coef) and -128 <= coef <= 127
            coef = np.full(idx.shape[0], coef, np.int8 if small else np.float64)
        else:
            coef = np.ascontiguousarray(coef)
            if coef.dtype != np.int8:
                coef = np.ascontiguousarray(coef, np.float64)
        rhs = np.full(n, float(rhs)) if np.isscalar(rhs) else np.ascontiguousarray(rhs, np.float64)
        assert indptr[0] == 0 and indptr[-1] == idx.shape[0] == coef.shape[0] and (np.diff(indptr) >= 0).all()
        assert idx.size == 0 or (0 <= idx.min() and idx.max() < self.n_vars)
        first = self._counters.get(prefix, 0)
        self._counters[prefix] = first + n
        b = _Block(prefix, first, None, indptr, idx, coef, sense, rhs)
        self.constraints.blocks.append(b)
        self.constraints.by_prefix.setdefault(prefix, []).append(b)
        return _BlockNames(b, n)

    def add_row(self, prefix_or_name: str, idx, coef, sense: int, rhs: float, exact_name: bool = False) -> str:
        idx = np.asarray(idx, np.int64)
        if not exact_name:
            return self.add_rows(prefix_or_name, [0, idx.shape[0]], idx, coef, sense, rhs)[0]
        coef = np.full(idx.shape[0], float(coef)) if np.isscalar(coef) else np.asarray(coef, np.float64)
        assert idx.shape[0] == coef.shape[0]
        assert idx.size == 0 or (0 <= idx.min() and idx.max() < self.n_vars)
        self.constraints.pop(prefix_or_name, None)  # an exact name replaces its row
        b = _Block(None, 0, prefix_or_name, np.asarray([0, idx.shape[0]], np.int64), idx, coef, sense,
                   np.asarray([float(rhs)]))
        self.constraints.blocks.append(b)
        self.constraints.exact[prefix_or_name] = b
        return prefix_or_name

    def remove(self, name: str) -> None:
        del self.constraints[name]

    # -- matrices ---------------------------------------------------------------
    def to_matrix(self):
        """(A csr, lower, upper, var_upper): rows ``var == 0`` become variable
        bounds instead of matrix rows."""
        import scipy.sparse as sp

        ub = self.upper.copy()
        data, cols, lens, lo, hi = [], [], [], [], []
        for b in self.constraints.blocks:
            if b.n_alive == 0:
                continue
            ln = np.diff(b.indptr)
            keep = b.alive.copy()
            if b.sense == EQ:
                # a single variable pinned to zero is a bound, not a row
                pin = keep & (ln == 1) & (b.rhs == 0.0)
                if pin.any():
                    at = b.indptr[:-1][pin]
                    pin[pin] = b.coef[at] != 0
                    ub[b.idx[b.indptr[:-1][pin]]] = 0.0
                    keep &= ~pin
            if not keep.any():
                continue
            if keep.all():
                data.append(b.coef); cols.append(b.idx); lens.append(ln)
            else:
                ent = np.repeat(keep, ln)
                data.append(b.coef[ent]); cols.append(b.idx[ent]); lens.append(ln[keep])
            r = b.rhs[keep]
            lo.append(r if b.sense != LE else np.full(r.shape[0], -np.inf))
            hi.append(r if b.sense != GE else np.full(r.shape[0], np.inf))
        cat = lambda xs, dt: np.concatenate(xs).astype(dt, copy=False) if xs else np.zeros(0, dt)
        lens = cat(lens, np.int64)
        ptr = np.zeros(lens.shape[0] + 1, np.int64)
        np.cumsum(lens, out=ptr[1:])
        A = sp.csr_matrix((cat(data, np.float64), cat(cols, np.int64), ptr), shape=(lens.shape[0], self.n_vars))
        # A row may name a variable twice: with repeated subgraphs sharing variables, the two sides of
        # a difference row can stand for the same ones.  HiGHS takes such a matrix for a model error.
        A.sum_duplicates()
        A.eliminate_zeros()
        return A, cat(lo, np.float64), cat(hi, np.float64), ub

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
        # no optimality gap: the reference's solver (CBC at its defaults) stops at a
        # proven optimum, so a near-tie must not be decided by a tolerance here
        opts = {"disp": bool(verbose), "mip_rel_gap": float(self.mip_rel_gap)}
        if time_limit is not None:
            opts["time_limit"] = float(time_limit)
        try:
            res = milp(self.objective, constraints=cons, integrality=np.ones(self.n_vars),
                       bounds=Bounds(np.zeros(self.n_vars), ub), options=opts)
        except (ValueError, MemoryError) as exc:
            # what the solver's own code raises when it runs out of room part-way (seen at
            # 1.6 M variables and 40 M nonzeros): not an answer about the problem
            raise RuntimeError(
                f"the ILP solver failed inside on {self.n_vars} variables x {A.shape[0]} rows ({exc}); "
                "write_lp() writes the problem for another solver") from exc
        if res.x is None:
            if res.status not in (2, 3):  # scipy's milp: 2 infeasible, 3 unbounded; anything else is not an answer
                raise RuntimeError(f"the ILP solver did not solve the problem: {res.message}")
            if "infeasible" not in str(res.message).lower() and res.status == 2:
                # status 2 also stands for a model HiGHS refuses to read
                raise RuntimeError(f"the ILP solver refused the problem: {res.message}")
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
            self.x = None
            self.objective_value = None
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
                mag = abs(float(c))  # a Python float: numpy scalars print as np.float64(...)
                parts.append(f"{sign} {vn(i)}" if mag == 1 else f"{sign} {mag!r} {vn(i)}")
            return " ".join(parts) if parts else "0"

        with open(path, "w") as f:
            f.write("\\* AutoParallel *\\\nMinimize\nOBJ: ")
            nz = np.nonzero(self.objective)[0]
            f.write(expr(nz, self.objective[nz]) + "\nSubject To\n")
            for r in self.constraints.values():
                f.write(f"{r.name}: {expr(r.idx, r.coef)} {_SENSE_STR[r.sense]} {float(r.rhs)!r}\n")
            f.write("Binaries\n")
            for i in range(self.n_vars):
                if self.upper[i] > 0:  # variables fixed out of the model are not declared
                    f.write(vn(i) + "\n")
            f.write("End\n")
