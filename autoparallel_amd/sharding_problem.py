"""ILP formulation of the sharding search over a packed graph.

Mirrors the reference's ``ShardingOptimizer`` below the FX layer
(autoparallel/optimize_sharding.py): coefficients come from the HIP engine,
constraint rows are assembled from index arithmetic on the packed layout, and
the model is handed to a MILP solver.  Decision variable (node v, arg a, out o,
inp j) is column ``var_start[e(v, a)] + o * S_src + j``.

Constraint families and their reference counterparts:
  unique_decision          add_unique_decision_constraint            :665-688
  same_across_args         add_same_output_across_args_constraint     :690-721
  output_input_consistent  add_output_input_consistent_constraint     :723-801
  inf_cases                add_inf_cost_constraint                    :803-812
  grad_*_constraint        add_forward_backward_consistency_constraints :1463-1485
  fwd_param_dtype / grad_reduce_dtype  add_grad_reduce_dtype_constraints  :1487-1606
  memory_constraint_*      _apply_memory_constraint                   :1629-1671
  user constraints         add_node_constraint / _add_node_constraint :1401-1417, 1673-1718
"""
from __future__ import annotations

import collections.abc
import dataclasses
import logging
import math
import time
import types
from typing import Dict, Iterable, List, Optional, Sequence, Set, Tuple, Union

import numpy as np

from . import ilp
from .packed import MAX_TUPLES, SPEC_NONE, PackedGraph, plc_str

logger = logging.getLogger(__name__)


@dataclasses.dataclass
class GraphRoles:
    """What the reference reads off the AOT graph descriptors
    (torch._functorch._aot_autograd.fx_utils): forward/backward pairs and the
    dtype-cast chains of parameters and gradients."""

    param_grad: List[Tuple[int, int]] = dataclasses.field(default_factory=list)  # grad -1 if none
    input_grad: List[Tuple[int, int]] = dataclasses.field(default_factory=list)
    output_tangent: List[Tuple[int, int]] = dataclasses.field(default_factory=list)
    fwd_pre_cast: Set[int] = dataclasses.field(default_factory=set)
    bwd_pre_cast: Set[int] = dataclasses.field(default_factory=set)


class Coefficients:
    """Host copy of the coefficient arrays, one element per decision variable
    (padding slots removed), plus the per-(node, out_idx) compute vectors."""

    def __init__(self, g: PackedGraph, comm, cost, flags, compute, per_arg):
        """comm, cost, flags: per slot of the entry arrays (padding is dropped here),
        or already per decision variable."""
        if len(comm) != g.num_entries:
            slots = g.entry_slots()
            comm, cost, flags = comm[slots], cost[slots], flags[slots]
        self.comm = np.ascontiguousarray(comm)
        self.cost = np.ascontiguousarray(cost)
        self.flags = np.ascontiguousarray(flags)
        self.compute = np.asarray(compute)
        self.per_arg = np.asarray(per_arg)

    def subset(self, keep: np.ndarray) -> "Coefficients":
        """The coefficients of the variables ``keep`` marks (bool per variable),
        in order: what is left when some edges lose their entry blocks."""
        out = object.__new__(Coefficients)
        out.comm, out.cost, out.flags = self.comm[keep].copy(), self.cost[keep].copy(), self.flags[keep].copy()
        out.compute, out.per_arg = self.compute, self.per_arg
        return out

    @classmethod
    def from_engine(cls, eng) -> "Coefficients":
        r = eng.results(compact=True)  # padding taken out on the device: 17 B per variable cross the link
        return cls(eng.g, r["comm"], r["cost"], r["flags"], r["compute"], r["per_arg"])

    @classmethod
    def from_decision_var_arrays(cls, g: PackedGraph, keys, vals, compute, per_arg) -> "Coefficients":
        """From the saved twin (keys int32[E, 4], vals float64[E, 3] =
        compute, comm, transition per variable, any row order).  cost is
        rebuilt as the reference's loader does
        (autoparallel/serialization.py:313, then add_inf_cost_constraint)."""
        keys = np.asarray(keys, np.int64)
        e = g.node_edge_off[:-1].astype(np.int64)[keys[:, 0]] + keys[:, 1]
        if (e >= g.node_edge_off[1:].astype(np.int64)[keys[:, 0]]).any():
            raise RuntimeError("saved key names an argument its node does not have")
        if (keys[:, 2] >= g.edge_sdst[e]).any() or (keys[:, 3] >= g.edge_ssrc[e]).any() or (keys < 0).any():
            raise RuntimeError("saved key outside its edge block")
        slot = g.edge_off[:-1][e] + keys[:, 2] * g.edge_ssrc[e].astype(np.int64) + keys[:, 3]
        n = g.num_slots
        comm, cost, flags = np.zeros(n), np.zeros(n), np.zeros(n, np.uint8)
        seen = np.zeros(n, bool)
        seen[slot] = True
        if int(seen.sum()) != g.num_entries or keys.shape[0] != g.num_entries:
            raise RuntimeError("saved keys do not cover every decision variable exactly once")
        comm[slot] = vals[:, 1]
        c = vals[:, 0] + vals[:, 1] + vals[:, 2]
        bad = ~np.isfinite(c)
        cost[slot] = np.where(bad, 10000.0, c)
        flags[slot] = (vals[:, 2] != 0).astype(np.uint8) | (bad.astype(np.uint8) << 1)
        out = cls(g, comm, cost, flags, compute, per_arg)
        out.saved_arrays = (np.asarray(keys, np.int32), np.asarray(vals, np.float64))
        out.slot_arrays = (comm, cost, flags)
        return out


class MeshPlaceholder:
    """What a plan needs of a DeviceMesh when none exists (a problem reopened
    without a process group): shape, dim names, ndim, size()
    (autoparallel/serialization.py:25-42)."""

    def __init__(self, shape, dim_names=None):
        self.shape = tuple(int(x) for x in shape)
        self.mesh_dim_names = tuple(dim_names) if dim_names else None
        self.ndim = len(self.shape)

    def size(self) -> int:
        return int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1


class PackedDecisionVars(collections.abc.Mapping):
    """(node, arg, out_idx, inp_idx) -> the variable's coefficients, in the
    reference's key order, over the packed arrays."""

    def __init__(self, core: "PackedShardingOptimizer"):
        self._core = core
        self._keys = None

    def _all(self) -> np.ndarray:
        if self._keys is None:
            self._keys = self._core.g.entry_keys()[self._core.g.decision_var_order()]
        return self._keys

    def __len__(self) -> int:
        return self._core.n_vars

    def __iter__(self):
        return (tuple(int(x) for x in k) for k in self._all())

    def __getitem__(self, key):
        core, g = self._core, self._core.g
        try:
            v, a, o, j = (int(x) for x in key)
        except (TypeError, ValueError):
            raise KeyError(key) from None
        if not (0 <= v < g.num_nodes and 0 <= a < int(g.node_edge_off[v + 1]) - int(g.node_edge_off[v])):
            raise KeyError(key)
        e = int(g.node_edge_off[v]) + a
        # a linked node has no variables of its own: its root's stand for it
        if core.linked[v] or not (0 <= o < int(g.edge_sdst[e]) and 0 <= j < int(g.edge_ssrc[e])):
            raise KeyError(key)
        i = int(core.var_start[e]) + o * int(g.edge_ssrc[e]) + j
        x = core.prob.x
        return types.SimpleNamespace(
            var=i, cost=float(core.coef.cost[i]), comm_cost=float(core.coef.comm[i]),
            compute_cost=float(core.coef.per_arg[int(core.g.node_comp_off[v]) + o]),
            sharding_transition_cost=int(core.coef.flags[i] & 1), value=None if x is None else float(x[i]))


class PackedShardingOptimizer:
    def __init__(
        self,
        g: PackedGraph,
        roles: Optional[GraphRoles] = None,
        force_grad_reduce_in_higher_precision: bool = False,
        coefficients: Optional[Coefficients] = None,
        device: str = "cuda",
        device_name: Optional[str] = None,
        nccl_config=None,
        repeated_subgraphs: Union[bool, str] = False,  # True: the reference's pass; "extended": see below
        cluster_root: Optional[np.ndarray] = None,
        topo_config=None,
    ):
        """repeated_subgraphs: cluster identical regions (node hashes from the
        device) and let every repeated node share the decision variables of its
        root (autoparallel/optimize_sharding.py:261-266, 356-378).  The string
        "extended" also clusters the duplicates that the reference's pass leaves
        out because an earlier region took one of their siblings.
        cluster_root: the same link table given explicitly (int[N], root[v] = v
        for unlinked nodes), e.g. from a saved file."""
        self.g = g
        self.roles = roles or getattr(g, "roles", None) or GraphRoles()
        self.force_grad_reduce_in_higher_precision = force_grad_reduce_in_higher_precision
        self.engine = None
        self.phase_s: Dict[str, float] = {}  # seconds per phase of the construction
        self._memory_ratio_cache: Dict[int, np.ndarray] = {}  # parameter node -> local/global size per strategy
        # The reference writes the flow rows of every edge from an unlinked producer to a linked
        # consumer, although they are the rows of the edge to that consumer's root over again
        # (one copy per repeated layer for a tensor every layer reads).  The extended mode, which
        # has no row numbering of the reference to keep, writes each distinct row once.
        self._distinct_flow_rows_only = repeated_subgraphs == "extended"
        self.region_groups: List[List[List[int]]] = []
        engine_kw = dict(device=device, device_name=device_name, nccl_config=nccl_config, topo_config=topo_config)
        # Repeated subgraphs are found before anything is priced: the hashes need the
        # problem on the device, not its coefficients.  The nodes of a repeat then get
        # no entries of their own: their edges read the entry blocks of their root
        # (autoparallel/optimize_sharding.py:501-507, 554-577).
        t0 = time.perf_counter()
        if cluster_root is None and repeated_subgraphs:
            from . import clustering
            from .engine import CostEngine

            assert g.edge_alias is None, "the graph already carries a clustering"
            key = g.node_cluster_key if g.node_cluster_key is not None else g.node_phase
            hashes = CostEngine(g, allocate_results=False, **engine_kw).node_hashes(key)
            self.region_groups = clustering.identical_regions(
                g, hashes, keep_unclaimed=repeated_subgraphs == "extended")
            cluster_root = clustering.cluster_roots(g, self.region_groups)
        g_in = g
        self._set_cluster_root(cluster_root)
        g = self.g  # with the entry blocks of linked nodes dropped, if any are linked
        if coefficients is not None and g is not g_in and coefficients.cost.shape[0] == g_in.num_entries:
            # coefficients of every node were handed in: keep those of the edges that still own a block
            coefficients = coefficients.subset(np.repeat(g.priced, g_in.block_sizes()))
        self.phase_s["clustering"] = time.perf_counter() - t0
        if coefficients is None:
            from .engine import CostEngine  # the HIP path; raises without the library / a GPU

            t0 = time.perf_counter()
            self.engine = CostEngine(g, **engine_kw)
            t1 = time.perf_counter()
            self.engine.build(clamp_inf=True)
            self.engine.synchronize()
            t2 = time.perf_counter()
            coefficients = Coefficients.from_engine(self.engine)
            self.phase_s.update(engine_construct=t1 - t0, device_build=t2 - t1, readback=time.perf_counter() - t2)
        self.coef = coefficients
        t0 = time.perf_counter()
        self.var_start = np.concatenate([[0], np.cumsum(g.block_sizes())]).astype(np.int64)
        self.n_vars = int(self.var_start[-1])
        assert self.coef.cost.shape[0] == self.n_vars, "coefficients do not match the graph's decision variables"
        self.prob = ilp.SparseILP(self.n_vars)
        self._memory_constraint: Optional[Tuple[float, float]] = None
        self._node_constraint_names: Dict[str, int] = {}
        self._constraint_log: List[Tuple[str, dict]] = []  # replayed by load (serialization.py)
        self.mesh_dim_names: Optional[List[str]] = None
        self.selected: Optional[np.ndarray] = None
        self.add_default_constraints()
        self.phase_s["ilp_rows"] = time.perf_counter() - t0

    # -- clusters ---------------------------------------------------------------
    def _set_cluster_root(self, root: Optional[np.ndarray]) -> None:
        g = self.g
        n = g.num_nodes
        self.root = np.arange(n, dtype=np.int64) if root is None else np.asarray(root, np.int64)
        assert self.root.shape == (n,) and (self.root[self.root] == self.root).all(), "roots must be unlinked"
        self.linked = self.root != np.arange(n)
        # edge of the root node that stands in for edge e (same argument position)
        v = g.edge_node.astype(np.int64)
        first = g.node_edge_off[:-1].astype(np.int64)
        self.edge_alias = first[self.root[v]] + (np.arange(g.num_edges) - first[v])
        if self.linked.any():
            from . import clustering

            if g.edge_alias is None:
                g = self.g = g.with_edge_alias(self.edge_alias)
            else:  # a graph saved with its clustering
                assert np.array_equal(g.edge_alias, self.edge_alias), "the graph's aliases are not this clustering's"
            g.node_multiplier = clustering.multipliers(self.root)
        else:
            assert g.edge_alias is None, "the graph aliases edges but no node is linked"

    @property
    def cluster_links(self) -> Dict[int, int]:
        """linked node -> root node (the node-level form of the reference's
        per-variable cluster_links, as its save file stores it)."""
        return {int(v): int(self.root[v]) for v in np.nonzero(self.linked)[0]}

    # -- indexing ---------------------------------------------------------------
    def edge_of(self, v: int, a: int) -> int:
        """Edge whose variables stand for (node v, argument a): the root's for a linked node."""
        e = int(self.g.node_edge_off[v]) + a
        assert e < int(self.g.node_edge_off[v + 1])
        return int(self.edge_alias[e])

    def var(self, v: int, a: int, o: int, j: int) -> int:
        e = self.edge_of(v, a)
        return int(self.var_start[e]) + o * int(self.g.edge_ssrc[e]) + j

    def _row_vars(self, e: int, o: int) -> np.ndarray:
        """Variables of edge e with output strategy o (all inp_idx)."""
        e = int(self.edge_alias[e])
        s = int(self.g.edge_ssrc[e])
        b = int(self.var_start[e]) + o * s
        return np.arange(b, b + s, dtype=np.int64)

    def _col_vars(self, e: int, j: int) -> np.ndarray:
        """Variables of edge e with input strategy j (all out_idx)."""
        e = int(self.edge_alias[e])
        s = int(self.g.edge_ssrc[e])
        return int(self.var_start[e]) + np.arange(int(self.g.edge_sdst[e]), dtype=np.int64) * s + j

    def var_names(self) -> List[str]:
        g = self.g
        keys = g.entry_keys()
        names = g.node_names or [f"node{i}" for i in range(g.num_nodes)]
        return [f"n={names[v]},s={v},arg={a},output_p={o},input_p={j}" for v, a, o, j in keys]

    # -- default constraints ------------------------------------------------------
    def add_default_constraints(self) -> None:
        self.add_unique_decision_constraint()
        self.add_same_output_across_args_constraint()
        self.add_output_input_consistent_constraint()
        self.add_inf_cost_constraint()
        self.add_forward_backward_consistency_constraints()
        self.add_grad_reduce_dtype_constraints()

    @staticmethod
    def _segments(start, count, stride=None, dtype=np.int64):
        """Concatenation of start[k] + stride[k] * arange(count[k]) over k, and
        the offsets of the pieces.  ``dtype``: of the concatenation (int32 halves the
        bytes the passes below move when every value fits)."""
        start = np.asarray(start, np.int64)
        count = np.asarray(count, np.int64)
        ptr = np.zeros(count.shape[0] + 1, np.int64)
        np.cumsum(count, out=ptr[1:])
        total = int(ptr[-1])
        if total == 0:
            return np.zeros(0, dtype), ptr
        # as a running sum of steps: the stride inside a piece, and at the first element of a
        # piece the jump from the last element of the piece before (three passes over the
        # output instead of six)
        step = np.ones(total, dtype) if stride is None else np.repeat(np.asarray(stride, dtype), count)
        some = count > 0
        first, st, cn = ptr[:-1][some], start[some], count[some]
        last = st + (cn - 1 if stride is None else (cn - 1) * np.asarray(stride, np.int64)[some])
        step[first[0]] = st[0]
        step[first[1:]] = st[1:] - last[:-1]
        return np.cumsum(step, dtype=dtype), ptr

    @property
    def _idx_dtype(self):
        """Variable indices of the row blocks: 32 bits while they fit."""
        return np.int32 if self.n_vars < 2**31 - 1 else np.int64

    def _add_difference_rows(self, prefix, plus_start, plus_count, minus_start, minus_count, minus_stride) -> None:
        """Rows  sum(plus piece) - sum(minus piece) = 0, one per pair of pieces."""
        n = len(plus_start)
        if n == 0:
            return
        start = np.empty(2 * n, np.int64); start[0::2] = plus_start; start[1::2] = minus_start
        count = np.empty(2 * n, np.int64); count[0::2] = plus_count; count[1::2] = minus_count
        stride = np.ones(2 * n, np.int64); stride[1::2] = minus_stride
        idx, ptr = self._segments(start, count, stride, self._idx_dtype)
        sign = np.ones(2 * n, np.int8); sign[1::2] = -1
        self.prob.add_rows(prefix, ptr[0::2], idx, np.repeat(sign, count), ilp.EQ, 0.0)

    def add_unique_decision_constraint(self) -> None:
        # for every (node, arg): exactly one (out, inp) pair
        g = self.g
        e = np.nonzero(~self.linked[g.edge_node])[0]
        idx, ptr = self._segments(self.var_start[e], self.var_start[e + 1] - self.var_start[e], None, self._idx_dtype)
        self.prob.add_rows("unique_decision", ptr, idx, 1.0, ilp.EQ, 1.0)

    def _num_input_nodes(self, v: int) -> int:
        g = self.g
        e0, e1 = int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])
        return int((g.edge_src_node[e0:e1] >= 0).sum())

    def add_same_output_across_args_constraint(self) -> None:
        # all arguments of a node pick the same output strategy: for every later
        # argument e and output strategy o, row o of argument 0 minus row o of e
        g = self.g
        first = g.node_edge_off[:-1].astype(np.int64)
        n_in = np.add.reduceat(np.concatenate([(g.edge_src_node >= 0).astype(np.int64), [0]]),
                               np.minimum(first, g.num_edges))[: g.num_nodes]
        n_in[np.diff(g.node_edge_off) == 0] = 0
        v = g.edge_node.astype(np.int64)
        later = np.nonzero((np.arange(g.num_edges) != first[v]) & ~self.linked[v] & (n_in[v] > 1))[0]
        if later.size == 0:
            return
        S = g.node_nstrat[v[later]].astype(np.int64)
        o = np.arange(int(S.sum()), dtype=np.int64) - np.repeat(np.cumsum(S) - S, S)
        # per edge first, then one value per (edge, strategy)
        e0 = self.edge_alias[first[v[later]]]
        ek = self.edge_alias[later]
        s0, sk = g.edge_ssrc[e0].astype(np.int64), g.edge_ssrc[ek].astype(np.int64)
        s0r, skr = np.repeat(s0, S), np.repeat(sk, S)
        self._add_difference_rows("same_across_args", np.repeat(self.var_start[e0], S) + o * s0r, s0r,
                                  np.repeat(self.var_start[ek], S) + o * skr, skr, np.ones_like(skr))

    def add_output_input_consistent_constraint(self) -> None:
        # producer's chosen output strategy == the input strategy its consumer assumes:
        # for the first edge of every (producer u, consumer v) pair and every strategy k
        # of u, row k of u's argument 0 minus column k of the edge; producers in order
        g = self.g
        u = g.edge_src_node.astype(np.int64)
        v = g.edge_node.astype(np.int64)
        has = np.nonzero(u >= 0)[0]
        # an edge between two linked nodes is covered by the edge between their roots
        # (autoparallel/optimize_sharding.py:743-746) -- when the roots are joined by one: regions of
        # different groups can meet so that the producer's root is not what the consumer's root
        # reads at that argument, and then the edge needs its own rows
        both = self.linked[u[has]] & self.linked[v[has]]
        covered = both & (g.edge_src_node[self.edge_alias[has]].astype(np.int64) == self.root[u[has]])
        has = has[~covered]
        if has.size == 0:
            return
        _, firsts = np.unique(u[has] * g.num_nodes + v[has], return_index=True)  # first matching argument only
        edges = has[np.sort(firsts)]
        edges = edges[np.argsort(u[edges], kind="stable")]
        if self._distinct_flow_rows_only:
            # the rows of an edge are a function of the two blocks they name
            pair = self.edge_alias[g.node_edge_off[u[edges]].astype(np.int64)] * g.num_edges + self.edge_alias[edges]
            _, firsts = np.unique(pair, return_index=True)
            edges = edges[np.sort(firsts)]
        assert (g.edge_ssrc[edges] == g.node_nstrat[u[edges]]).all()
        S = g.node_nstrat[u[edges]].astype(np.int64)
        k = np.arange(int(S.sum()), dtype=np.int64) - np.repeat(np.cumsum(S) - S, S)
        # per edge first, then one value per (edge, strategy of the producer)
        eu = self.edge_alias[g.node_edge_off[u[edges]].astype(np.int64)]  # argument 0 of the producer
        ev = self.edge_alias[edges]
        su = np.repeat(g.edge_ssrc[eu].astype(np.int64), S)
        sv = np.repeat(g.edge_ssrc[ev].astype(np.int64), S)
        self._add_difference_rows("output_input_consistent", np.repeat(self.var_start[eu], S) + k * su, su,
                                  np.repeat(self.var_start[ev], S) + k,
                                  np.repeat(g.edge_sdst[ev].astype(np.int64), S), sv)

    def add_inf_cost_constraint(self) -> None:
        # the engine already wrote 10000.0 into cost; pin those variables to 0
        # (linked nodes have no variables of their own)
        i = np.nonzero(((self.coef.flags & 2) != 0) & (self.prob.upper > 0))[0]
        self.prob.add_rows("inf_cases", np.arange(i.shape[0] + 1), i, 1.0, ilp.EQ, 0.0)

    def _out_placements(self, v: int) -> List[Optional[int]]:
        """Placement-tuple id of output 0 of each strategy of node v (None for
        a missing spec): what ``str(output_specs)`` distinguishes."""
        g = self.g
        run = int(g.node_out_list[v])
        words = g.lists[run : run + int(g.node_nstrat[v])]
        return [None if int(w) == SPEC_NONE else int(w) & (MAX_TUPLES - 1) for w in words]

    def _first_out_placements(self, v: int) -> List[Optional[int]]:
        """Per strategy of node v, the placement-tuple id of its first output
        that has a spec (None if none has): what a node constraint is matched
        against for a tuple-valued node (autoparallel/optimize_sharding.py:1696-1706)."""
        g = self.g
        runs = None if g.node_out_runs is None else [int(r) for r in g.node_out_runs[v] if r >= 0]
        if not runs or len(runs) == 1:
            return self._out_placements(v)
        out: List[Optional[int]] = []
        for o in range(int(g.node_nstrat[v])):
            words = [int(g.lists[r + o]) for r in runs]
            first = next((w for w in words if w != SPEC_NONE), None)
            out.append(None if first is None else first & (MAX_TUPLES - 1))
        return out

    def _add_paired_output_constraint(self, a: int, b: int, name: str) -> None:
        pa, pb = self._out_placements(a), self._out_placements(b)
        ea, eb = int(self.g.node_edge_off[a]), int(self.g.node_edge_off[b])
        # rows in strategy order; consecutive rows of one kind go in as one block (the names
        # and their order are those of a row-by-row loop: a counter per prefix)
        run_prefix, ptr, idx, coef = None, [0], [], []

        def flush():
            if run_prefix is not None and len(ptr) > 1:
                self.prob.add_rows(run_prefix, np.asarray(ptr, np.int64), np.concatenate(idx), np.concatenate(coef),
                                   ilp.EQ, 0.0)

        for o, t in enumerate(pa):
            va = self._row_vars(ea, o)
            if t not in pb:
                prefix, row_idx, row_coef = name + "_disable", [va], [np.ones(len(va))]
            else:
                vb = self._row_vars(eb, pb.index(t))
                prefix, row_idx, row_coef = name, [vb, va], [np.ones(len(vb)), -np.ones(len(va))]
            if prefix != run_prefix:
                flush()
                run_prefix, ptr, idx, coef = prefix, [0], [], []
            idx += row_idx
            coef += row_coef
            ptr.append(ptr[-1] + sum(len(x) for x in row_idx))
        flush()

    def add_forward_backward_consistency_constraints(self) -> None:
        for p, gnode in self.roles.param_grad:
            if gnode >= 0:
                self._add_paired_output_constraint(p, gnode, "grad_param_constraint")
        for n, gnode in self.roles.input_grad:
            if gnode >= 0:
                self._add_paired_output_constraint(n, gnode, "grad_input_constraint")
        for n, t in self.roles.output_tangent:
            if t >= 0:
                self._add_paired_output_constraint(n, t, "grad_output_constraint")

    def add_grad_reduce_dtype_constraints(self) -> None:
        g = self.g
        for nodes, name, enabled in (
            (self.roles.fwd_pre_cast, "fwd_param_dtype", True),
            (self.roles.bwd_pre_cast, "grad_reduce_dtype", self.force_grad_reduce_in_higher_precision),
        ):
            if not enabled or not nodes:
                continue
            # the variables of those nodes: the blocks their edges own, in variable order
            marked = np.zeros(g.num_nodes, bool)
            marked[np.fromiter(nodes, np.int64)] = True
            e = np.nonzero(marked[g.edge_node] & (self.var_start[1:] > self.var_start[:-1]))[0]
            i, _ = self._segments(self.var_start[e], self.var_start[e + 1] - self.var_start[e])
            i = i[(self.coef.comm[i] > 0) & (self.prob.upper[i] > 0)]
            self.prob.add_rows(name, np.arange(i.shape[0] + 1), i, 1.0, ilp.EQ, 0.0)

    # -- user constraints -----------------------------------------------------------
    def add_node_constraint(self, v: int, placement: Optional[Sequence[int]] = None,
                            constraint_name: Optional[str] = None) -> List[str]:
        """Force node v's output placement (placement bytes per mesh dim;
        default Shard(0) on the first mesh dim, Replicate elsewhere)."""
        g = self.g
        if placement is None:
            placement = (0x40,) + (0x00,) * (g.ndim - 1)
        want = tuple(int(p) for p in placement)
        allowed = [o for o, t in enumerate(self._first_out_placements(v))
                   if t is not None and tuple(int(x) for x in g.tuple_plc[t, : g.ndim]) == want]
        if not allowed:
            raise RuntimeError(
                f"Couldn't find appropriate constraint {g.node_names[v] if g.node_names else v} "
                f"{constraint_name} {[plc_str(p) for p in want]}")
        # A node of a repeated subgraph has no variables of its own: the rows go on
        # its root's (edge_alias), as the reference's variable lookup resolves a
        # linked key to its root (autoparallel/optimize_sharding.py:1401-1417).
        names = []
        for e in range(int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])):
            idx = np.concatenate([self._row_vars(e, o) for o in allowed])
            name = self.prob.add_row(constraint_name or "user_constraint", idx, 1.0, ilp.EQ, 1.0)
            names.append(name)
            self._node_constraint_names[name] = v
        # logged once the rows exist: a refused constraint is not replayed by load()
        self._constraint_log.append(("add_node_constraint", {
            "v": int(v), "placement": [int(p) for p in want], "constraint_name": constraint_name}))
        return names

    def add_parameter_memory_constraint(self, memory_factor_low: float, memory_factor_high: float) -> None:
        self._memory_constraint = (memory_factor_low, memory_factor_high)
        self._constraint_log.append(("add_parameter_memory_constraint", {
            "memory_factor_low": memory_factor_low, "memory_factor_high": memory_factor_high}))

    def _memory_ratios(self, params: List[int]) -> List[np.ndarray]:
        """prod(local shape) / prod(global shape) of every strategy of every
        parameter, local shapes from the device (apc_local_shapes)."""
        import ctypes as C

        import torch

        from . import _lib
        from .engine import make_model

        g = self.g
        cache = self._memory_ratio_cache
        wanted, params = params, [p for p in params if p not in cache]
        if not params:  # computed before, or carried by the file this problem was read from
            return [cache[p] for p in wanted]
        lib = _lib.load()
        rows = []
        for p in params:
            run = int(g.edge_dst_list[int(g.node_edge_off[p])])
            for w in g.lists[run : run + int(g.node_nstrat[p])]:
                rows.append((int(w) >> 12, int(w) & (MAX_TUPLES - 1)))
        mids = np.asarray([r[0] for r in rows], np.int64)
        tids = np.asarray([r[1] for r in rows], np.int64)
        dev = self.engine.device if self.engine is not None else torch.device("cuda")
        up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
        rank, shape, stride = up(g.meta_rank[mids]), up(g.meta_shape[mids]), up(g.meta_stride[mids])
        plc = up(g.tuple_plc[tids])
        out_shape, out_stride = torch.empty_like(shape), torch.empty_like(stride)
        name = self.engine.device_name if self.engine is not None else "AMD Instinct MI355X"
        model = make_model([int(x) for x in g.mesh_shape], g.devices_per_host, name)
        _lib.check(lib.apc_local_shapes(C.byref(model), len(rows), rank.data_ptr(), shape.data_ptr(),
                                        stride.data_ptr(), plc.data_ptr(), out_shape.data_ptr(),
                                        out_stride.data_ptr(), None), "apc_local_shapes")
        torch.cuda.synchronize(dev)
        local = out_shape.cpu().numpy()
        k = 0
        for p in params:
            S = int(g.node_nstrat[p])
            r = []
            for i in range(S):
                rk = int(g.meta_rank[mids[k + i]])
                new = math.prod(int(x) for x in local[k + i, :rk])
                old = math.prod(int(x) for x in g.meta_shape[mids[k + i], :rk])
                r.append(new / old)
            cache[p] = np.asarray(r)
            k += S
        return [cache[p] for p in wanted]

    def _apply_memory_constraint(self) -> None:
        if self._memory_constraint is None:
            return
        low, high = self._memory_constraint
        for name in ("memory_constraint_high", "memory_constraint_low"):
            self.prob.constraints.pop(name, None)
        constrained = set(self._node_constraint_names.values())
        params = [p for p, _ in self.roles.param_grad if p not in constrained]
        if not params:
            return
        idx, coef = [], []
        budget_low = budget_high = 0.0
        for p, ratios in zip(params, self._memory_ratios(params)):
            for o, r in enumerate(ratios):
                idx.append(self.var(p, 0, o, 0))
                coef.append(r)
            best = float(ratios.min())
            budget_low += max(best, low)
            budget_high += max(best, high)
        self.prob.add_row("memory_constraint_high", idx, coef, ilp.LE, budget_high, exact_name=True)
        self.prob.add_row("memory_constraint_low", idx, coef, ilp.GE, budget_low, exact_name=True)

    def reset_problem(self, prob: Optional[ilp.SparseILP] = None) -> None:
        """An empty problem over the same decision variables (or ``prob``): no rows,
        no variable fixed, no memory budget, no logged constraint."""
        assert prob is None or prob.n_vars == self.n_vars
        self.prob = prob if prob is not None else ilp.SparseILP(self.n_vars)
        self._memory_constraint = None
        self._node_constraint_names = {}
        self._constraint_log = []
        self.selected = None

    def remove_constraints(self, names: Iterable[str]) -> None:
        for name in names:
            self.prob.remove(name)
            self._node_constraint_names.pop(name, None)
            if name in ("memory_constraint_high", "memory_constraint_low"):
                self._memory_constraint = None

    # -- coefficient post-passes ---------------------------------------------------
    def apply_prefetch_discount(self, scale: float = 0.0) -> int:
        """Needs the engine (runs on the device arrays), then refreshes the host copy."""
        assert self.engine is not None, "coefficients were injected: no engine to run the discount on"
        n = self.engine.apply_prefetch_discount(scale)
        self.coef = Coefficients.from_engine(self.engine)
        return n

    # -- solve ------------------------------------------------------------------------
    def _set_objective(self) -> None:
        keys = self.g.entry_keys()
        mult = self.g.node_multiplier[keys[:, 0]] if self.g.node_multiplier is not None else 1
        self.prob.objective = self.coef.cost * mult

    def _solve(self, backend: str = "auto", verbose: bool = False) -> None:
        self._apply_memory_constraint()
        status = self.prob.solve(backend=backend, verbose=verbose)
        if status == ilp.STATUS_INFEASIBLE:
            logger.warning(self.get_violated_constraints_log())
            raise RuntimeError(
                "The sharding optimizer could not find a feasible solution. This typically means "
                "the user-specified constraints are contradictory or the device mesh is too small "
                "for the requested sharding. Check the WARNING log above for the list of violated "
                "constraints, and consider relaxing input/output constraints or using a larger mesh.")
        self.selected = np.nonzero(self.prob.x > 0.5)[0]

    def _extract(self) -> np.ndarray:
        """out_idx per node from the selected variables; checks that each
        (node, arg) has exactly one selection and that all args agree."""
        keys = self.g.entry_keys()[self.selected]
        sol = np.full(self.g.num_nodes, -1, np.int64)
        if self.linked.any():  # linked nodes follow their root (optimize_sharding.py:902-903)
            k = keys[~self.linked[keys[:, 0]]]
            for v, a, o, j in k:
                sol[v] = o
            sol[self.linked] = sol[self.root[self.linked]]

        seen = set()
        for v, a, o, j in keys:
            if (v, a) in seen:
                raise RuntimeError(f"Multiple solutions for node {v}, arg {a}")
            seen.add((int(v), int(a)))
            if sol[v] >= 0 and sol[v] != o:
                raise AssertionError(f"arguments of node {v} disagree on the output strategy")
            sol[v] = o
        return sol

    def get_solution(self, backend: str = "auto", verbose: bool = False) -> np.ndarray:
        self._set_objective()
        self._solve(backend, verbose)
        return self._extract()

    def resolve(self, backend: str = "auto", verbose: bool = False) -> np.ndarray:
        self._solve(backend, verbose)
        return self._extract()

    @property
    def objective_value(self) -> float:
        return self.prob.objective_value

    def solution_placements(self, sol: np.ndarray) -> List[Optional[Tuple[str, ...]]]:
        out = []
        for v in range(self.g.num_nodes):
            t = self._out_placements(v)[int(sol[v])]
            out.append(None if t is None else tuple(plc_str(int(c)) for c in self.g.tuple_plc[t, : self.g.ndim]))
        return out

    # -- device access for an optimizer whose coefficients were injected ---------------
    def _ensure_engine(self):
        """The CostEngine holding the coefficients; for a loaded optimizer the
        saved arrays are uploaded on first use (no cost is recomputed)."""
        if self.engine is None:
            from .engine import CostEngine

            slot_arrays = getattr(self.coef, "slot_arrays", None)
            if slot_arrays is None:
                raise RuntimeError("coefficients were injected without their slot arrays: no device copy to use")
            self.engine = CostEngine(self.g)
            self.engine.load_results(*slot_arrays, self.coef.compute, self.coef.per_arg)
        return self.engine

    def vars_of_keys(self, keys) -> np.ndarray:
        keys = np.asarray(keys, np.int64).reshape(-1, 4)
        e = self.g.node_edge_off[:-1].astype(np.int64)[keys[:, 0]] + keys[:, 1]
        return self.var_start[e] + keys[:, 2] * self.g.edge_ssrc[e].astype(np.int64) + keys[:, 3]

    def decision_var_arrays(self):
        """(keys int32[E, 4], vals float64[E, 3]) in the reference's
        decision_vars order, written by the device from the resident results."""
        saved = getattr(self.coef, "saved_arrays", None)
        if self.engine is None and saved is not None:
            return saved  # loaded and untouched since
        keys, vals = self._ensure_engine().export_decision_vars()
        return keys.cpu().numpy(), vals.cpu().numpy()

    def _spec_str(self, word: int) -> Optional[str]:
        if int(word) == SPEC_NONE:
            return None
        t = int(word) & (MAX_TUPLES - 1)
        return "".join(plc_str(int(c)) for c in self.g.tuple_plc[t, : self.g.ndim])

    def output_placement_str(self, v: int, o: int) -> Optional[str]:
        return self._spec_str(self.g.lists[int(self.g.node_out_list[v]) + o])

    def input_placement_strs(self, v: int, o: int) -> List[Optional[str]]:
        g = self.g
        return [self._spec_str(g.lists[int(g.edge_dst_list[e]) + o])
                for e in range(int(g.node_edge_off[v]), int(g.node_edge_off[v + 1]))]

    def solution_terms(self, sol: np.ndarray):
        """(terms float64[n_edge, 4] = compute, comm, transition, cost of the
        selected entry of every edge; slot int64[n_edge]) from the device."""
        import torch

        eng = self._ensure_engine()
        a = torch.from_numpy(np.ascontiguousarray(sol.astype(np.int16))).to(eng.device)
        terms, slot = eng.solution_terms(a)
        return terms.cpu().numpy(), slot.cpu().numpy()

    # -- what code written for the reference reads on an optimizer it loaded (serialization.py:25-42,
    #    tests/test_serialization.py:119-260): nodes, decision variables by key, the mesh's shape, the
    #    selected keys
    @property
    def nodes(self) -> List[str]:
        """Node names in graph order (the reference holds fx nodes there; a reloaded packed problem has their names)."""
        return list(self.g.node_names) if self.g.node_names else [f"node{i}" for i in range(self.g.num_nodes)]

    @property
    def mesh(self) -> "MeshPlaceholder":
        return MeshPlaceholder([int(x) for x in self.g.mesh_shape], self.mesh_dim_names)

    @property
    def selected_keys(self) -> List[Tuple[int, int, int, int]]:
        """(node, arg, out_idx, inp_idx) of every selected variable, the expanded ones of linked nodes
        included (optimize_sharding.py:896-905)."""
        if self.selected is None:
            return []
        sol = self._extract()
        keys = [tuple(int(x) for x in k) for k in self.g.entry_keys()[self.selected]]
        g = self.g
        for v in np.nonzero(self.linked)[0]:
            for a, e in enumerate(range(int(g.node_edge_off[v]), int(g.node_edge_off[v + 1]))):
                u = int(g.edge_src_node[e])
                keys.append((int(v), a, int(sol[v]), int(sol[u]) if u >= 0 else 0))
        return keys

    @property
    def decision_vars(self) -> "PackedDecisionVars":
        return PackedDecisionVars(self)

    def save(self, path: str) -> None:
        from . import serialization

        serialization.save_optimizer(self, path, self.mesh_dim_names)

    @classmethod
    def load(cls, path: str) -> "PackedShardingOptimizer":
        from . import serialization

        return serialization.load_optimizer(path, cls)

    def get_json(self, sol: Optional[np.ndarray] = None) -> dict:
        from . import export_json

        return export_json.export_sharding_json(self, self._extract() if sol is None else sol)

    def get_violated_constraints_log(self) -> str:
        """The rows the current solution violates, with their terms, in the
        reference's layout (optimize_sharding.py:1115-1124)."""
        x = self.prob.x
        violated = [(n, r) for n, r in self.prob.constraints.items() if x is not None and not r.valid(x)]
        out = f"Violated constraints: {[n for n, _ in violated]}"
        names = self.var_names() if violated else []
        for name, r in violated:
            out += f"\n========= {name} ============="
            for i, c in zip(r.idx, r.coef):
                out += f"\n{names[int(i)]}, coeff={c}, value={x[int(i)]}"
        return out

    def get_log(self, sol: Optional[np.ndarray] = None) -> str:
        from . import log_formatting

        return log_formatting.format_packed_log(self, self._extract() if sol is None else sol,
                                                self.get_violated_constraints_log() if sol is None else "")

    def compute_solution_cost(self, sol: np.ndarray) -> Dict[str, float]:
        """The reference's _compute_solution_cost for one assignment, on the device."""
        self._ensure_engine()
        import torch

        a = torch.from_numpy(np.ascontiguousarray(sol.astype(np.int16).reshape(-1, 1))).to(self.engine.device)
        r = self.engine.score(a).cpu().numpy()[0]
        return {"total": r[0], "compute": r[1], "comm": r[2], "transition": r[3]}
