"""``ShardingOptimizer`` with the reference's constructor and public surface
(autoparallel/optimize_sharding.py:220-291, 955-979 and the constraint adders),
over the HIP cost engine.

What happens where:
  * strategies per node: host, torch DTensor (``shardings.placement_options``)
  * packing of ``{node: OpStrategy}`` into SoA arrays: host (``_pack``)
  * every coefficient (compute, comm, transition, cost, inf flags): device
  * ILP rows and the solver hand-off: ``sharding_problem`` / ``ilp``
``decision_vars`` is a mapping view over the coefficient arrays in the
reference's insertion order (node, out_idx, argi, inp_idx; :511-520).
"""
from __future__ import annotations

import collections.abc
import contextlib
import dataclasses
import gc
import logging
import time
import operator
import weakref
from typing import Any, Dict, Iterator, List, Optional, Tuple, Union

import numpy as np
import torch
from torch.distributed.tensor._dtensor_spec import DTensorSpec
from torch.distributed.tensor._op_schema import OpSpec, OpStrategy
from torch.utils._pytree import tree_flatten, tree_map_only

from . import fx_programs
from .cost_models import collective_runtime_estimation as _cre
from .dtensor_bridge import devices_per_host as _mesh_dph
from .dtensor_bridge import placement_codes
from .engine import detect_device_name
from .packed import GraphBuilder, NodeDesc, PackedGraph
from .sharding_problem import GraphRoles, PackedShardingOptimizer
from .shardings.placement_options import _create_all_options, get_placement_options_for_node

logger = logging.getLogger(__name__)


def _produces_tensor(val) -> bool:
    if isinstance(val, torch.Tensor):
        return True
    if isinstance(val, (tuple, list)):
        return any(_produces_tensor(v) for v in val)
    return False


class DecisionVar:
    """One (node, arg, out, inp) choice.  Made by the optimizer it is a view:
    attribute reads and writes go to the coefficient arrays.  Made from the
    fields of the reference's dataclass (``DecisionVar(var=..., cost=...,
    compute_cost=..., comm_cost=..., sharding_transition_cost=..., strategy=...,
    output_spec=..., input_spec=...)``, autoparallel/optimize_sharding.py:191-203)
    it is a record of its own that holds them."""

    __slots__ = ("_opt", "_i", "key", "_own")
    _FIELDS = ("var", "cost", "compute_cost", "comm_cost", "sharding_transition_cost", "strategy",
               "output_spec", "input_spec")

    def __init__(self, opt: Optional["ShardingOptimizer"] = None, i: Optional[int] = None, key: Optional[tuple] = None,
                 **fields):
        if opt is None:
            unknown = set(fields) - set(self._FIELDS)
            if unknown:
                raise TypeError(f"DecisionVar got unexpected fields {sorted(unknown)}")
            missing = [f for f in self._FIELDS if f not in fields]
            if missing:
                raise TypeError(f"DecisionVar is missing fields {missing}")
            self._opt, self._i, self.key, self._own = None, None, key, dict(fields)
        else:
            assert not fields, "a view takes its fields from the optimizer"
            self._opt, self._i, self.key, self._own = opt, i, key, None

    @property
    def var(self):
        return self._i if self._own is None else self._own["var"]  # column of the ILP

    @property
    def cost(self) -> float:
        return float(self._opt._core.coef.cost[self._i]) if self._own is None else self._own["cost"]

    @cost.setter
    def cost(self, v: float) -> None:
        if self._own is None:
            self._opt._core.coef.cost[self._i] = v
        else:
            self._own["cost"] = v

    @property
    def comm_cost(self) -> float:
        return float(self._opt._core.coef.comm[self._i]) if self._own is None else self._own["comm_cost"]

    @comm_cost.setter
    def comm_cost(self, v: float) -> None:
        if self._own is None:
            self._opt._core.coef.comm[self._i] = v
        else:
            self._own["comm_cost"] = v

    @property
    def sharding_transition_cost(self):
        if self._own is not None:
            return self._own["sharding_transition_cost"]
        return int(self._opt._core.coef.flags[self._i] & 1)

    @property
    def compute_cost(self) -> float:
        if self._own is not None:
            return self._own["compute_cost"]
        v, _, o, _ = self.key
        return float(self._opt._core.coef.per_arg[int(self._opt._packed.node_comp_off[v]) + o])

    @property
    def strategy(self):
        if self._own is not None:
            return self._own["strategy"]
        v, _, o, _ = self.key
        return self._opt.strats[self._opt.nodes[v]].strategies[o]

    @property
    def output_spec(self):
        return self.strategy.output_specs if self._own is None else self._own["output_spec"]

    @property
    def input_spec(self):
        if self._own is not None:
            return self._own["input_spec"]
        ins = self.strategy.input_specs
        a = self.key[1]
        return ins[a] if ins is not None and a < len(ins) else None

    def value(self) -> Optional[float]:
        if self._own is not None:
            v = self._own["var"]
            return v.value() if hasattr(v, "value") else None
        x = self._opt._core.prob.x
        return None if x is None else float(x[self._i])

    def __repr__(self) -> str:
        return "DecisionVar(" + ", ".join(f"{f}={getattr(self, f)!r}" for f in self._FIELDS) + ")"


class _OwnedByOptimizer:
    """A view that the optimizer itself holds: it refers back weakly, so that the
    optimizer and its million strategy objects are freed when the last reference to
    it goes, not when the cyclic collector next walks the heap.  (The DecisionVar
    views handed out to callers hold the optimizer strongly.)"""

    def _bind(self, opt: "ShardingOptimizer") -> None:
        self._opt_ref = weakref.ref(opt)

    @property
    def _opt(self) -> "ShardingOptimizer":
        opt = self._opt_ref()
        if opt is None:
            raise ReferenceError("the ShardingOptimizer behind this mapping no longer exists")
        return opt


class DecisionVars(_OwnedByOptimizer, collections.abc.Mapping):
    def __init__(self, opt: "ShardingOptimizer"):
        self._bind(opt)
        self._ordered_keys: Optional[np.ndarray] = None  # made when the mapping is first iterated

    def _col(self, key) -> int:
        v, a, o, j = key
        try:
            return self._opt._core.var(int(v), int(a), int(o), int(j))
        except AssertionError:
            raise KeyError(key)

    def __getitem__(self, key) -> DecisionVar:
        g = self._opt._packed
        v, a, o, j = key
        if not (0 <= v < g.num_nodes) or not (0 <= o < g.node_nstrat[v]):
            raise KeyError(key)
        # a repeated (linked) node owns no variables, as in the reference, where decision_vars
        # holds the keys of cluster roots and cluster_links maps a linked key to its root's
        if self._opt._core.linked[v]:
            raise KeyError(key)
        e = int(g.node_edge_off[v]) + a
        if a < 0 or e >= int(g.node_edge_off[v + 1]) or not (0 <= j < g.edge_ssrc[e]):
            raise KeyError(key)
        return DecisionVar(self._opt, self._col(key), (int(v), int(a), int(o), int(j)))

    def __iter__(self) -> Iterator[tuple]:
        if self._ordered_keys is None:
            g = self._opt._packed
            self._ordered_keys = g.entry_keys()[g.decision_var_order()]
        for k in self._ordered_keys:
            yield tuple(int(x) for x in k)

    def __len__(self) -> int:
        return int(self._opt._packed.num_entries)


class _ClusterLinks(_OwnedByOptimizer, collections.abc.Mapping):
    """The reference's per-variable link table (linked key -> root key,
    autoparallel/optimize_sharding.py:356-378) as a view over the node-level
    links: a repeated node's key maps to the same (arg, out, inp) of its root.
    Keys are produced on iteration, not stored (a 32-layer model has millions)."""

    def __init__(self, opt: "ShardingOptimizer", node_links: Dict[int, int]):
        self._bind(opt)
        self._nodes = dict(node_links)

    def __getitem__(self, key):
        v, a, o, j = key
        r = self._nodes.get(int(v))
        if r is None or (r, int(a), int(o), int(j)) not in self._opt.decision_vars:
            raise KeyError(key)
        return (r, int(a), int(o), int(j))

    def __iter__(self):
        for v in self._nodes:
            for a, o, j in self._opt.walk_over_options(self._opt.nodes[v]):
                yield (v, a, o, j)

    def __len__(self) -> int:
        g = self._opt._packed
        sizes = g.edge_sdst.astype(np.int64) * g.edge_ssrc
        linked = np.zeros(g.num_nodes, bool)
        linked[list(self._nodes)] = True
        return int(sizes[linked[g.edge_node]].sum())

    def __bool__(self) -> bool:
        return bool(self._nodes)


def concretize_symint(val):
    """A SymInt becomes its hint; one without a hint (unbacked) and anything
    else pass through (autoparallel/optimize_sharding.py:111-120)."""
    if isinstance(val, torch.SymInt):
        hint = val.node.hint
        return val if hint is None else hint
    return val


def concretize_args(args):
    """The same tree with SymInts replaced by their hints and fake tensors of
    symbolic shape replaced by fake tensors of the hinted shape and stride (left
    alone when a size has no hint) (:123-150)."""
    from torch._subclasses.fake_tensor import FakeTensor

    def one(x):
        if isinstance(x, torch.SymInt):
            return concretize_symint(x)
        if isinstance(x, FakeTensor) and any(isinstance(d, torch.SymInt) for d in x.shape):
            shape = [concretize_symint(d) for d in x.shape]
            stride = [concretize_symint(d) for d in x.stride()]
            if not all(isinstance(d, int) for d in shape):
                return x
            with x.fake_mode:
                return torch.empty_strided(shape, stride, dtype=x.dtype, device=x.device)
        return x

    return tree_map_only((torch.SymInt, FakeTensor), one, args)


def concretize_gm(gm):
    """(copy of gm with every ``meta['val']`` made concrete, original -> copy,
    copy -> original).  The planner works on the copy; the caller keeps the
    symbolic graph (:162-189)."""
    graph = torch.fx.Graph()
    to_concrete: Dict[torch.fx.Node, torch.fx.Node] = {}
    for node in gm.graph.nodes:
        twin = graph.node_copy(node, lambda n: to_concrete[n])
        to_concrete[node] = twin
        if twin.meta.get("val") is not None:  # node_copy made a shallow copy of meta
            twin.meta["val"] = concretize_args(twin.meta["val"])
    return torch.fx.GraphModule(gm, graph), to_concrete, {v: k for k, v in to_concrete.items()}


def _has_symbolic_sizes(gm) -> bool:
    for node in gm.graph.nodes:
        val = node.meta.get("val")
        # a node's value is a tensor, a number or a flat tuple/list of them nearly always
        leaves = (val,) if isinstance(val, torch.Tensor) or not isinstance(val, (tuple, list, dict)) \
            else tree_flatten(val)[0]
        for x in leaves:
            if isinstance(x, torch.SymInt):
                return True
            if isinstance(x, torch.Tensor) and any(isinstance(d, torch.SymInt) for d in tuple(x.shape) + tuple(x.stride())):
                return True
    return False


class _Variables(collections.abc.Mapping):
    """``pulp_variables`` of the reference (autoparallel/optimize_sharding.py:412-444):
    key -> an object with the variable's name and, after a solve, ``varValue``.
    The variables themselves are columns of the packed problem."""

    class _Var:
        __slots__ = ("name", "index", "_prob")

        def __init__(self, name, index, prob):
            self.name, self.index, self._prob = name, index, prob

        @property
        def varValue(self):
            x = self._prob.x
            return None if x is None else float(x[self.index])

        def value(self):
            return self.varValue

    def __init__(self, opt: "ShardingOptimizer"):
        self._opt = opt

    def __getitem__(self, key):
        opt = self._opt
        root_key = opt.cluster_links.get(key, key)  # a repeated node's variable is its root's
        if root_key not in opt.decision_vars:
            raise KeyError(key)
        col = opt.decision_vars._col(root_key)
        v, a, o, j = key
        return self._Var(f"n={opt.nodes[v]},s={v},arg={a},output_p={o},input_p={j}", col, opt.prob)

    def __iter__(self):
        return iter(self._opt.decision_vars)

    def __len__(self):
        return len(self._opt.decision_vars)


def _flat_args(a, out: list) -> list:
    """Leaves of an FX argument structure in pytree order (tuples, lists and
    dicts are the only containers FX arguments have); tree_flatten gives the
    same list at twenty times the cost."""
    if isinstance(a, (tuple, list)):
        for x in a:
            _flat_args(x, out)
    elif isinstance(a, dict):
        for x in a.values():
            _flat_args(x, out)
    else:
        out.append(a)
    return out


def _map_nodes(a, fn):
    """tree_map_only(torch.fx.Node, fn, a) for FX argument structures."""
    if isinstance(a, torch.fx.Node):
        return fn(a)
    if isinstance(a, tuple):
        return tuple(_map_nodes(x, fn) for x in a)
    if isinstance(a, list):
        return [_map_nodes(x, fn) for x in a]
    if isinstance(a, dict):
        return {k: _map_nodes(v, fn) for k, v in a.items()}
    return a


def enumerate_strategies(graph, mesh, input_nodes: Optional[dict] = None) -> Dict[torch.fx.Node, Any]:
    """Placement strategies of every node that carries a tensor, in graph order
    (build_sharding_metadata, autoparallel/optimize_sharding.py:306-354).
    ``input_nodes``: a dict that receives, per call_function node, the
    tensor-carrying nodes among its flattened args (what the packer asks for again)."""
    strats: Dict[torch.fx.Node, Any] = {}
    for node in graph.nodes:
        if node.op in ("placeholder", "get_attr"):
            val = node.meta.get("val")
            if isinstance(val, torch.Tensor):
                strats[node] = _create_all_options(mesh, val.shape, tensor=val)
            elif node.op == "placeholder":
                strats[node] = _create_all_options(mesh, ())
        elif node.op == "call_function":
            if not _produces_tensor(node.meta.get("val")):
                continue
            in_nodes = [x for x in _flat_args(node.args, [])
                        if isinstance(x, torch.fx.Node) and x in strats]
            if input_nodes is not None:
                input_nodes[node] = in_nodes
            producers = [strats[x] for x in in_nodes]
            arg_vals = [x.meta["val"] for x in in_nodes]
            schema_args = _map_nodes(node.args, lambda x: strats.get(x, x.meta.get("val")))
            strats[node] = get_placement_options_for_node(mesh, node, producers, arg_vals, schema_args)
        elif node.op == "output":
            strats[node] = tree_map_only(torch.fx.Node, lambda x: strats[x], node.args)
        else:
            raise ValueError(f"Unexpected node op: {node.op}")
    return strats


@contextlib.contextmanager
def _gc_paused():
    """The cyclic collector off for the duration.  Building strategies, the packed
    problem and the rows allocates millions of small objects that all stay alive,
    next to a traced graph of tens of thousands; every threshold crossing made the
    collector walk all of it again (measured on the Llama-3-8B graph: 1.5-1.7 s for
    the constructor with it, 0.73 s without; strategy enumeration alone 0.94 s
    against 0.22 s).  Reference counting frees as usual; the collector resumes on
    exit, if it was on.

    What was allocated meanwhile and is still alive (the strategies and their cost
    rows: 0.6 M tracked objects for that graph) lives as long as the optimizer.  Left
    in the youngest generation, all of it is walked at the first allocation after the
    collector resumes (0.1 s, a quarter of the constructor).  freeze() followed by
    unfreeze() hands every tracked object to the oldest generation without walking it
    (two list splices), where the next full collection finds it as it finds every other
    long-lived object.  Not done when the caller keeps a frozen generation of its own,
    which unfreeze() would release."""
    was = gc.isenabled()
    gc.disable()
    try:
        yield
    finally:
        if was:
            if gc.get_freeze_count() == 0:
                gc.freeze()
                gc.unfreeze()
            gc.enable()


class ShardingOptimizer:
    def __init__(self, gm, mesh, force_grad_reduce_in_higher_precision: bool = False,
                 repeated_subgraphs: Union[bool, str] = False, devices_per_host: Optional[int] = None,
                 device_name: Optional[str] = None):
        with _gc_paused():
            self._construct(gm, mesh, force_grad_reduce_in_higher_precision, repeated_subgraphs,
                            devices_per_host, device_name)

    def _construct(self, gm, mesh, force_grad_reduce_in_higher_precision, repeated_subgraphs, devices_per_host,
                   device_name):
        self.orig_gm = gm
        # planning needs concrete sizes: a graph with symbolic ones is planned on a
        # copy at their hints, and plans are handed back on the caller's nodes
        # (autoparallel/optimize_sharding.py:228-237); a static graph is planned as it is
        if _has_symbolic_sizes(gm):
            gm, self._orig_to_concrete, self._concrete_to_orig = concretize_gm(gm)
        else:
            self._orig_to_concrete = {n: n for n in gm.graph.nodes}
            self._concrete_to_orig = dict(self._orig_to_concrete)
        self.gm = gm
        self.graph = gm.graph
        self.mesh = mesh
        self.force_grad_reduce_in_higher_precision = force_grad_reduce_in_higher_precision
        self.repeated_subgraphs = bool(repeated_subgraphs)
        # "extended": also cluster what the reference's pass leaves out (see
        # clustering.identical_regions); any other true value is the reference's pass
        self._cluster_mode = "extended" if repeated_subgraphs == "extended" else self.repeated_subgraphs
        self.cluster_links: Dict[tuple, tuple] = {}
        self._devices_per_host = devices_per_host if devices_per_host is not None else _mesh_dph(mesh)
        self._device_name = device_name or detect_device_name()
        _cre.configure(self._devices_per_host, self._device_name)
        self._constraint_log: List[Tuple[str, dict]] = []
        # seconds per phase, the split the reference logs at DEBUG
        # (autoparallel/optimize_sharding.py:249-291, 579-587)
        self.phase_s: Dict[str, float] = {}
        t0 = time.perf_counter()
        self.strats = self.build_sharding_metadata()
        self.phase_s["strategy_enumeration"] = time.perf_counter() - t0
        self.nodes = list(self.strats.keys())
        self.node_map = {n: i for i, n in enumerate(self.nodes)}
        self.decision_vars = self._build_decision_vars()
        t0 = time.perf_counter()
        self.validate()
        self.phase_s["validate"] = time.perf_counter() - t0
        logger.debug("ShardingOptimizer phases (s): %s", self.phase_s)

    # -- accessors of the reference's class ----------------------------------------
    @property
    def pulp_variables(self) -> _Variables:
        return _Variables(self)

    def _normalize_node(self, node):
        """The planner's node for a node of either graph (:298-304)."""
        return self._orig_to_concrete.get(node, node)

    def _to_orig_solution(self, solution):
        return {self._concrete_to_orig.get(n, n): spec for n, spec in solution.items()}

    def _to_concrete_solution(self, solution):
        return {self._orig_to_concrete.get(n, n): spec for n, spec in solution.items()}

    def get_strategy(self, node):
        return self.strats[self._normalize_node(node)]

    def _get_pulp_variable(self, key):
        return self.pulp_variables[key]

    def _resolve_decision_var(self, key) -> DecisionVar:
        """The variable that stands for a key: its own, or its cluster root's (:446-460)."""
        return self.decision_vars[self.cluster_links.get(key, key)]

    @classmethod
    def load(cls, path: str):
        """A saved optimizer, reopened without the model, mesh or process group
        (the packed form: PackedShardingOptimizer)."""
        return PackedShardingOptimizer.load(path)

    # -- strategies ---------------------------------------------------------------
    def build_sharding_metadata(self) -> Dict[torch.fx.Node, Any]:
        self._input_nodes_of: Dict[torch.fx.Node, List[torch.fx.Node]] = {}
        return enumerate_strategies(self.graph, self.mesh, self._input_nodes_of)

    def _all_input_nodes(self, node) -> List[torch.fx.Node]:
        """The tensor-carrying nodes among a node's flattened args, duplicates kept
        (autoparallel/optimize_sharding.py:522); asked several times per node, so kept."""
        cache = self.__dict__.setdefault("_input_nodes_of", {})
        got = cache.get(node)
        if got is None:
            got = cache[node] = [x for x in _flat_args(node.args, [])
                                 if isinstance(x, torch.fx.Node) and x in self.strats]
        return got

    def walk_over_options(self, node, constrain_arg=None):
        if node not in self.strats or node.op == "output":
            return
        st = self.strats[node]
        for argi in range(len(st.strategies[0].input_specs)):
            if constrain_arg is not None and argi != constrain_arg:
                continue
            for out_idx, s in enumerate(st.strategies):
                for inp_idx in range(len(s.redistribute_cost[argi])):
                    yield argi, out_idx, inp_idx

    # -- packing -------------------------------------------------------------------
    def _has_aot_descriptors(self) -> bool:
        """Whether the graph is an AOT joint graph with input/output descriptors
        (meta['desc'] on its placeholders): the source of the forward/backward
        pairs.  A hand-built graph has none, and then no such pairs exist."""
        phs = [n for n in self.graph.nodes if n.op == "placeholder"]
        return bool(phs) and all("desc" in n.meta for n in phs)

    def _roles(self) -> GraphRoles:
        from torch._functorch._aot_autograd import fx_utils

        self._input_idx, self._output_idx = [], []
        if not self._has_aot_descriptors():
            logger.debug("no AOT descriptors on the graph: no forward/backward constraints")
            return GraphRoles()
        # With descriptors, anything that goes wrong below is an error, as in the
        # reference: a plan without the parameter/gradient rows would be wrong silently.
        r = GraphRoles()
        nm = self.node_map
        input_idx, output_idx = [], []
        for p, g in fx_utils.get_param_and_grad_nodes(self.graph).values():
            r.param_grad.append((nm[p], nm[g] if g is not None and g in nm else -1))
        # position of each plain input / output among the traced function's own
        # (an input without a placeholder of its own, e.g. an alias, leaves a gap)
        for desc, (n, g) in fx_utils.get_plain_input_and_grad_nodes(self.graph).items():
            r.input_grad.append((nm[n], nm[g] if g is not None and g in nm else -1))
            input_idx.append(getattr(desc, "idx", len(input_idx)))
        for desc, (n, t) in fx_utils.get_plain_output_and_tangent_nodes(self.graph).items():
            r.output_tangent.append((nm[n], nm[t] if t is not None and t in nm else -1))
            output_idx.append(getattr(desc, "idx", len(output_idx)))
        self._mark_pre_cast_nodes(r)
        self._input_idx, self._output_idx = input_idx, output_idx
        return r

    # operators that stand for the mixed-precision cast of a parameter or its gradient
    # (the reference's parametrization inserts torch.ops.autoparallel.dtype_cast)
    dtype_cast_targets: set = set()

    def _mark_pre_cast_nodes(self, r: GraphRoles) -> None:
        """Nodes before the mixed-precision cast, on which a redistribution would
        run in the larger dtype (autoparallel/optimize_sharding.py:1487-1606).
        Forward: from a parameter along single-user, single-input nodes to a cast
        that narrows the dtype, cast included.  Backward: from a gradient back
        along single-input nodes, the cast and everything before it in that
        chain except the first producer with more than one input."""
        from torch._functorch._aot_autograd import fx_utils

        casts = set(self.dtype_cast_targets)
        ns = getattr(torch.ops, "autoparallel", None)
        if ns is not None and hasattr(ns, "dtype_cast"):
            casts.add(ns.dtype_cast.default)
        if not casts:
            return
        nm = self.node_map
        for param, grad in fx_utils.get_param_and_grad_nodes(self.graph).values():
            n = param
            while n.target not in casts:
                users = list(n.users)
                if len(users) != 1 or len(users[0].all_input_nodes) != 1:
                    break
                n = users[0]
            if n.target in casts and n.meta["val"].dtype.itemsize < param.meta["val"].dtype.itemsize:
                node = n
                while node is not param:
                    if node in nm:
                        r.fwd_pre_cast.add(nm[node])
                    node = node.all_input_nodes[0]
            if grad is None:
                continue
            chain, n = [grad], grad
            while len(n.all_input_nodes) == 1:
                parent = n.all_input_nodes[0]
                if len(parent.all_input_nodes) != 1:
                    break
                chain.append(parent)
                n = parent
            at = next((i for i, node in enumerate(chain) if node.target in casts), None)
            if at is not None:
                r.bwd_pre_cast.update(nm[node] for node in chain[at:] if node in nm)

    def _prefetchable(self, g: PackedGraph, packed_nodes) -> np.ndarray:
        """uint8 per edge: 1 where the producer is parameter-derived or the consumer
        terminal-derived (autoparallel/graph_passes/graph_utils.py:447-484)."""
        from .graph_utils import build_param_derived_set, build_terminal_derived_set

        if not self._has_aot_descriptors():  # a graph without AOT descriptors has no parameters to prefetch
            return np.zeros(g.num_edges, np.uint8)
        derived_set = build_param_derived_set(self.graph)
        terminal_set = build_terminal_derived_set(self.graph)
        derived = np.fromiter((n in derived_set for n in packed_nodes), bool, len(packed_nodes))
        terminal = np.fromiter((n in terminal_set for n in packed_nodes), bool, len(packed_nodes))
        # an argument row counts when it has a producer among the node's inputs (named or not)
        src = g.edge_src_node.astype(np.int64)
        return ((src >= 0) & (derived[np.maximum(src, 0)] | terminal[g.edge_node])).astype(np.uint8)

    def _pack(self) -> PackedGraph:
        b = GraphBuilder(tuple(self.mesh.shape), self._devices_per_host)
        index_of: Dict[torch.fx.Node, int] = {}
        memo: Dict[str, dict] = {}
        # One template per strategy query: the repeated layers of a model ask the same
        # queries (same operator, arguments and candidates: same specs and program), and
        # a node then only adds its producers.  Everything else is array work in pack().
        template_of: Dict[tuple, int] = {}
        strats, input_nodes_of = self.strats, self._all_input_nodes
        packed_nodes: List[torch.fx.Node] = []
        kinds: List[int] = []   # 1 placeholder, 2 get_attr, 0 anything else
        phases: List[int] = []  # 1: tagged as backward by the partitioner
        getitem_target = operator.getitem
        for node in self.nodes:
            op = node.op
            if op == "output":
                continue
            st: OpStrategy = strats[node]
            qkey = getattr(st, "_apc_query_id", None)
            if qkey is not None:
                # the answer of a query as it was handed out: a caller may have dropped or
                # replaced strategies since (the specs of an answer are shared by its copies)
                sts = st.strategies
                qkey = (qkey, len(sts), id(sts[0].output_specs), id(sts[-1].output_specs))
            t = template_of.get(qkey) if qkey is not None else None
            if t is None:
                desc = fx_programs.describe_node(node, st.strategies, b, name=node.name, memo=memo)
                # rows of the strategies as they stand (their number per strategy is the
                # number of arguments; the values are read below, where an edge keeps them)
                desc.default_rows = [s.redistribute_cost for s in st.strategies]
                desc.nargs = len(st.strategies[0].input_specs)
                t = b.add_template(desc)
                if qkey is not None:
                    template_of[qkey] = t
            getitem = int(node.args[1]) if op == "call_function" and node.target is getitem_target else None
            index_of[node] = b.add_instance(t, [index_of[x] for x in input_nodes_of(node)], getitem, node.name)
            packed_nodes.append(node)
            kinds.append(1 if op == "placeholder" else (2 if op == "get_attr" else 0))
            phases.append(1 if node.meta.get("partitioner_tag") == "is_backward" else 0)
        # default rows: what a strategy carried before the engine ran; the packer reads them
        # where an edge has no producer or a spec is missing
        g = b.pack(default_rows_of=lambda v: [s.redistribute_cost for s in strats[packed_nodes[v]].strategies])
        assert self.nodes[:len(packed_nodes)] == packed_nodes, "node order must be preserved"
        g.roles = self._roles()
        g.edge_prefetchable = self._prefetchable(g, packed_nodes)
        g.node_kind = np.asarray(kinds, np.uint8)
        g.node_phase = np.asarray(phases, np.int32)
        if self.repeated_subgraphs:
            g.node_cluster_key = self._cluster_keys(packed_nodes)
        return g

    @staticmethod
    def _cluster_keys(nodes) -> np.ndarray:
        """int32 per node: an id of the parts of the reference's clustering key that
        the packed arrays do not hold: the operator's name, the forward/backward
        tag, the source position, and the arguments (tensor arguments by their
        metadata, integers by value, anything else as absent)
        (autoparallel/graph_passes/graph_clustering.py:35-52, 68-73).  Nodes with
        different ids never fall into one group of duplicates."""
        of_node: Dict[torch.fx.Node, object] = {}  # a producer is described once

        def arg_key(a):
            if isinstance(a, torch.fx.Node):
                k = of_node.get(a, of_node)
                if k is of_node:
                    v = a.meta.get("val")
                    if isinstance(v, torch.Tensor):
                        shape, stride = v.shape, v.stride()
                        try:  # plain integers: the tuples themselves (equal exactly when their texts are)
                            hash(shape), hash(stride)
                            k = (tuple(shape), stride, v.dtype)
                        except TypeError:  # a symbolic size has no hash: by its text
                            k = (tuple(str(d) for d in shape), tuple(str(d) for d in stride), v.dtype)
                    else:
                        k = None if v is None else str(v)
                    of_node[a] = k
                return k
            return a if isinstance(a, int) else None

        ids: Dict[tuple, int] = {}
        names: Dict[object, str] = {}  # an operator's name is asked once
        out = np.empty(len(nodes), np.int32)
        for i, n in enumerate(nodes):
            kwargs = n.kwargs
            kw = sorted(kwargs.items(), key=lambda kv: kv[0]) if kwargs else ()
            flat = _flat_args(kw, _flat_args(n.args, [])) if kw else _flat_args(n.args, [])
            target = n.target
            name = names.get(target)
            if name is None:
                name = names[target] = str(target)
            meta = n.meta
            key = (name, meta.get("partitioner_tag"), meta.get("stack_trace"),
                   tuple(k for k, _ in kw), tuple([arg_key(a) for a in flat]))
            out[i] = ids.setdefault(key, len(ids))
        return out

    # -- coefficients ----------------------------------------------------------------
    def _build_decision_vars(self) -> DecisionVars:
        t0 = time.perf_counter()
        self._packed = self._pack()
        self.phase_s["pack"] = time.perf_counter() - t0
        self._core = PackedShardingOptimizer(
            self._packed, roles=self._packed.roles,
            force_grad_reduce_in_higher_precision=self.force_grad_reduce_in_higher_precision,
            device_name=self._device_name, nccl_config=_cre.get_nccl_topo_config(),
            topo_config=_cre.get_mesh_topo_config(),
            repeated_subgraphs=self._cluster_mode)
        self._packed = self._core.g  # with the entry blocks of repeated nodes dropped, if any
        # per-variable link table of the reference (:356-378): linked key -> root key
        self.cluster_links = _ClusterLinks(self, self._core.cluster_links)
        self._cluster_linked_node_idxs = set(self._core.cluster_links)
        self.phase_s.update(self._core.phase_s)
        t0 = time.perf_counter()
        self._write_back_redistribute_costs()
        self.phase_s["write_back_redistribute_cost"] = time.perf_counter() - t0
        return DecisionVars(self)

    def _write_back_redistribute_costs(self, as_built: bool = True) -> None:
        """strategy.redistribute_cost[argi][inp_idx] = comm, as the reference's
        loop does in place (:540)."""
        g, comm = self._packed, self._core.coef.comm
        vs, alias = self._core.var_start, self._core.edge_alias
        nodes, strats = self.nodes, self.strats
        edge_node, edge_arg, edge_ssrc = g.edge_node.tolist(), g.edge_arg.tolist(), g.edge_ssrc.tolist()
        vs, alias = np.asarray(vs).tolist(), np.asarray(alias).tolist()
        # Edges that read one matrix of the block table have the same block of comm values
        # while the arrays are as the build wrote them (the entry kernel copies the matrix): the
        # floats are made once per matrix, and an edge gets lists of its own over them.  Without a
        # block table, or after a pass that changed comm edge by edge, every edge converts its own.
        engine = getattr(self._core, "engine", None)
        if as_built and engine is not None and engine.table_mode != "direct":
            matrix_of = g.block_table(engine.table_mode == "compressed")[3].tolist()
        else:
            matrix_of = [-1] * g.num_edges
        by_matrix: Dict[int, list] = {}
        made: Dict[int, list] = {}  # rows of the edges that own a block, as lists
        for e in range(g.num_edges):
            r = alias[e]  # a repeated node's rows are its root's (:554-571)
            block = made.get(r)
            if block is None:
                m = matrix_of[r]
                shared = by_matrix.get(m) if m >= 0 else None
                if shared is None:
                    block = comm[vs[r] : vs[r + 1]].reshape(-1, edge_ssrc[e]).tolist()
                    if m >= 0:
                        by_matrix[m] = block
                else:
                    block = [row[:] for row in shared]
                made[r] = block
                rows = block
            else:  # lists of its own over the same numbers (:569-571)
                rows = [row[:] for row in block]
            a = edge_arg[e]
            for s, row in zip(strats[nodes[edge_node[e]]].strategies, rows):
                s.redistribute_cost[a] = row

    def validate(self) -> None:
        for node in self.graph.nodes:
            if node.op != "call_function" or node not in self.strats:
                continue
            s0 = self.strats[node].strategies[0]
            ins = self._all_input_nodes(node)
            assert len(s0.redistribute_cost) == len(ins) or (len(ins) == 0 and len(s0.redistribute_cost) == 1), \
                f"{node}, {len(s0.redistribute_cost)}, {len(ins)}"
            # every spec the first strategy carries knows its tensor (:205-218, 651-654)
            for label, specs in (("output_specs", s0.output_specs), ("input_spec", tuple(s0.input_specs))):
                for spec in (specs if isinstance(specs, (list, tuple)) else (specs,)):
                    assert not spec or spec.tensor_meta is not None, f"{node} {label} doesn't have a tensor_meta"
            for i, arg in enumerate(ins):
                assert len(s0.redistribute_cost[i]) == len(self.strats[arg].strategies), \
                    f"{node}, {len(s0.redistribute_cost[i])}, {len(self.strats[arg].strategies)}"

    # -- constraints (delegated to the packed formulation) ------------------------------
    @property
    def prob(self):
        """The ILP of the current decision variables (``ilp.SparseILP``)."""
        return self._core.prob

    @prob.setter
    def prob(self, value):
        """The reference's rebuild sequence assigns a new problem before it adds the
        default rows again (``opt.prob = pulp.LpProblem(...)``,
        tests/test_paired_output_constraint.py:58-62, serialization.py:330-337): an
        assignment starts an empty problem over the current decision variables.  A
        SparseILP of that size is taken as it is; anything else only marks the restart."""
        from . import ilp

        core = self._core
        if value is core.prob:
            return
        core.reset_problem(value if isinstance(value, ilp.SparseILP) and value.n_vars == core.n_vars else None)
        self._constraint_log.clear()  # the rows it would replay are gone

    @property
    def _name_counters(self) -> Dict[str, int]:
        """Next index per constraint-name prefix (autoparallel/optimize_sharding.py:248, 293-296)."""
        return self._core.prob._counters

    @_name_counters.setter
    def _name_counters(self, value) -> None:
        counters = self._core.prob._counters
        counters.clear()
        counters.update(value)

    def add_default_constraints(self):
        """The six groups of rows every problem has (autoparallel/optimize_sharding.py:814-822).
        ``_build_decision_vars`` leaves them in place; a caller that assigned ``prob`` adds them here."""
        self._core.add_default_constraints()

    def add_unique_decision_constraint(self):  # :665-688
        self._core.add_unique_decision_constraint()

    def add_same_output_across_args_constraint(self):  # :690-721
        self._core.add_same_output_across_args_constraint()

    def add_output_input_consistent_constraint(self):  # :723-801
        self._core.add_output_input_consistent_constraint()

    def add_inf_cost_constraint(self):  # :803-812
        self._core.add_inf_cost_constraint()

    def add_forward_backward_consistency_constraints(self):  # :1460-1485
        self._core.add_forward_backward_consistency_constraints()

    def add_grad_reduce_dtype_constraints(self):  # :1487-1627
        self._core.add_grad_reduce_dtype_constraints()

    def add_node_constraint(self, node, placement=None, constraint_name=None):
        node = self._normalize_node(node)
        assert node in self.strats, node
        codes = None if placement is None else placement_codes(placement)
        names = self._core.add_node_constraint(self.node_map[node], codes, constraint_name)
        # logged once the rows exist: a refused constraint must not be replayed from a saved file
        self._constraint_log.append(("add_node_constraint", {"node_name": node.name, "placement": placement,
                                                             "constraint_name": constraint_name}))
        return names

    def add_sharded_input_constraint(self, input_placements=None):
        self._io_constraints(self._packed.roles.input_grad, input_placements, "input_constraint",
                             getattr(self, "_input_idx", None), "inputs")

    def add_sharded_output_constraint(self, output_placements=None):
        self._io_constraints(self._packed.roles.output_tangent, output_placements, "output_constraint",
                             getattr(self, "_output_idx", None), "outputs")

    def _io_constraints(self, pairs, placements, name, idx=None, what="inputs"):
        """Forward-side nodes only; their gradients / tangents follow through the
        forward-backward rows (autoparallel/optimize_sharding.py:1720-1752)."""
        remaining = None if placements is None else dict(enumerate(placements))
        for i, (n, _) in enumerate(pairs):
            plc = None if remaining is None else remaining.pop(i if not idx else idx[i])
            codes = None if plc is None else placement_codes(plc)
            self._core.add_node_constraint(n, codes, name)
        ignored = [] if not remaining else [i for i, p in remaining.items() if p is not None]
        if ignored:
            raise RuntimeError(
                f"We were unable to respect placements for {what} at indices {ignored}.  This is because the "
                f"traced joint graph did not actually have a dedicated node for them, typically because some "
                f"{what} aliased each other.  Replace the placement with None, or clone the tensors.")

    def add_parameter_memory_constraint(self, memory_factor_low: float, memory_factor_high: float):
        self._core.add_parameter_memory_constraint(memory_factor_low, memory_factor_high)

    def remove_constraints(self, names):
        self._core.remove_constraints(names)

    def apply_prefetch_discount(self, scale: float = 0.0) -> int:
        n = self._core.apply_prefetch_discount(scale)
        self._write_back_redistribute_costs(as_built=False)  # the discount is per edge, not per matrix
        return n

    # -- solve ------------------------------------------------------------------------------
    def _solution_dict(self, sol: np.ndarray) -> Dict[torch.fx.Node, OpSpec]:
        self.selected_keys = [tuple(int(x) for x in k) for k in self._packed.entry_keys()[self._core.selected]]
        g = self._packed
        for v in np.nonzero(self._core.linked)[0]:  # linked nodes repeat their root's choice (:902-903)
            for a, e in enumerate(range(int(g.node_edge_off[v]), int(g.node_edge_off[v + 1]))):
                u = int(g.edge_src_node[e])
                self.selected_keys.append((int(v), a, int(sol[v]), int(sol[u]) if u >= 0 else 0))
        return self._to_orig_solution({self.nodes[v]: self.strats[self.nodes[v]].strategies[int(sol[v])]
                                       for v in range(self._packed.num_nodes)})

    def get_solution(self, verbose: bool = False) -> Dict[torch.fx.Node, OpSpec]:
        return self._solution_dict(self._core.get_solution(verbose=verbose))

    def resolve(self, verbose: bool = False) -> Dict[torch.fx.Node, OpSpec]:
        return self._solution_dict(self._core.resolve(verbose=verbose))

    def _out_indices(self, solution: Dict[torch.fx.Node, OpSpec]) -> np.ndarray:
        sol = np.zeros(self._packed.num_nodes, np.int64)
        for node, spec in self._to_concrete_solution(solution).items():
            if node not in self.node_map or node.op == "output":
                continue
            for i, s in enumerate(self.strats[node].strategies):
                if s is spec:
                    sol[self.node_map[node]] = i
                    break
        return sol

    def _compute_solution_cost(self, solution: Dict[torch.fx.Node, OpSpec]) -> Dict[str, float]:
        return self._core.compute_solution_cost(self._out_indices(solution))

    def diff_solutions(self, solution_a, solution_b) -> str:
        a, b = self._compute_solution_cost(solution_a), self._compute_solution_cost(solution_b)
        changed = sum(1 for n in solution_a if n in solution_b
                      and isinstance(solution_a[n].output_specs, DTensorSpec)
                      and isinstance(solution_b[n].output_specs, DTensorSpec)
                      and solution_a[n].output_specs.placements != solution_b[n].output_specs.placements)
        lines = [f"Objective: {a['total']:.1f} -> {b['total']:.1f} ({b['total'] - a['total']:+.1f})"]
        for k, label in (("compute", "compute"), ("comm", "comm:   "), ("transition", "trans:  ")):
            lines.append(f"  {label} {a[k]:.1f} -> {b[k]:.1f} ({b[k] - a[k]:+.1f})")
        lines.append(f"Placement changes: {changed} nodes changed")
        out = "\n".join(lines)
        print(out)
        return out

    def print_costs_for_node(self, node, arg: int = 0) -> str:
        v = self.node_map[self._normalize_node(node)]
        e = self._core.edge_of(v, arg)
        g = self._packed
        block = self._core.coef.cost[self._core.var_start[e] : self._core.var_start[e + 1]]
        text = f"{node} arg {arg}: cost[out_idx][inp_idx]\n{block.reshape(-1, int(g.edge_ssrc[e]))}"
        print(text)
        return text

    # -- export / persistence ------------------------------------------------------------------
    def _node_info(self) -> List[Dict[str, Any]]:
        """Per-node fields only the FX graph carries (export_json.py:362-407 of the
        reference), and the cluster of every repeated node."""
        from . import export_json

        linked = {self.nodes[v]: self.nodes[r] for v, r in self._core.cluster_links.items()}
        return export_json.fx_node_info(self.nodes, linked)

    def get_json(self) -> Dict[str, Any]:
        from . import export_json

        self._core.mesh_dim_names = list(self.mesh.mesh_dim_names) if self.mesh.mesh_dim_names else None
        data = export_json.export_sharding_json(self._core, self._core._extract(), self._node_info())
        out_node = next((n for n in self.graph.nodes if n.op == "output"), None)
        if out_node is not None:  # completes the DAG; the optimizer does not solve for it
            data["nodes"].append({"name": out_node.name, "op": "output",
                                  "inputs": [{"name": n.name} for n in out_node.all_input_nodes]})
        return data

    def get_log(self, colored: bool = False, verbose: bool = False) -> str:
        from . import log_formatting

        sol = self._core._extract()
        by_node: Dict[torch.fx.Node, List[DecisionVar]] = {}
        for key in self.selected_keys:
            by_node.setdefault(self.nodes[key[0]], []).append(self._resolve_decision_var(key))
        del sol
        return log_formatting.format_sharding_log(self.graph, by_node, colored, verbose,
                                                  self.get_violated_constraints_log())

    def get_violated_constraints_log(self) -> str:
        return self._core.get_violated_constraints_log()

    def save(self, path: str) -> None:
        """Packed state (graph arrays, coefficient twin, constraint log,
        solution).  ``PackedShardingOptimizer.load(path)`` reopens it without
        the model, mesh or process group."""
        self._core.mesh_dim_names = list(self.mesh.mesh_dim_names) if self.mesh.mesh_dim_names else None
        self._core.save(path)

    def save_placements(self, path: str) -> None:
        from . import serialization

        names = list(self.mesh.mesh_dim_names) if self.mesh.mesh_dim_names else None
        serialization.save_placements(self._core, self._core._extract(), path, names)

    def load_placements(self, path: str) -> Dict[torch.fx.Node, OpSpec]:
        from . import serialization

        names = list(self.mesh.mesh_dim_names) if self.mesh.mesh_dim_names else None
        sol = serialization.load_placements(self._core, path, names)
        return self._to_orig_solution({self.nodes[v]: self.strats[self.nodes[v]].strategies[int(sol[v])]
                                       for v in range(self._packed.num_nodes)})

    def explain_placement(self, target_placement, start_node=None, max_nodes=None) -> str:
        """Why the optimizer did not choose ``target_placement``: per node, the
        chosen placement with its compute and communication cost next to the
        cost the target would have if every node that offers it used it (a node
        that does not keeps its chosen strategy), as the reference's
        explain_placement (:1227-1397).  The two plans' per-edge terms come from
        the device (apc_solution_terms).  Call after get_solution()."""
        from tabulate import tabulate
        from torch.distributed.tensor._op_schema import _pretty_print_spec

        g, core = self._packed, self._core
        target = tuple(target_placement)
        chosen = core._extract()
        tgt_idx = np.full(g.num_nodes, -1, np.int64)
        for v in range(g.num_nodes):
            for i, s in enumerate(self.strats[self.nodes[v]].strategies):
                if isinstance(s.output_specs, DTensorSpec) and s.output_specs.placements == target:
                    tgt_idx[v] = i
                    break
        what_if = np.where(tgt_idx >= 0, tgt_idx, chosen)
        terms_c, _ = core.solution_terms(chosen)
        terms_t, _ = core.solution_terms(what_if)
        start_node = None if start_node is None else self._normalize_node(start_node)
        rows, started = [], start_node is None
        for v in range(g.num_nodes):
            node = self.nodes[v]
            if not started:
                if node is not start_node:
                    continue
                started = True
            if max_nodes is not None and len(rows) >= max_nodes:
                break
            spec = self.strats[node].strategies[int(chosen[v])].output_specs
            if not isinstance(spec, DTensorSpec):
                continue  # tuple-output nodes are skipped
            e0, e1 = int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])
            prod = g.edge_src_node[e0:e1] >= 0
            c_comp, c_comm = float(terms_c[e0:e1, 0].sum()), float(terms_c[e0:e1, 1][prod].sum())
            shape = str(list(spec.tensor_meta.shape)) if spec.tensor_meta is not None else "?"
            if tgt_idx[v] >= 0:
                t_comp, t_comm = float(terms_t[e0:e1, 0].sum()), float(terms_t[e0:e1, 1][prod].sum())
                if spec.placements == target:
                    status = "CHOSEN"
                elif abs((c_comp + c_comm) - (t_comp + t_comm)) < 0.01:
                    status = "TIE"
                elif t_comp + t_comm < c_comp + c_comm:
                    status = "TARGET CHEAPER"
                else:
                    status = "CHOSEN CHEAPER"
                if abs(t_comp - 7.0) < 0.01 and abs(c_comp - 7.0) < 0.01:
                    status += " [floor]"
                t_comp_s, t_comm_s = f"{t_comp:.1f}", f"{t_comm:.1f}"
            else:
                t_comp_s = t_comm_s = "N/A"
                status = "UNAVAILABLE"
            rows.append([str(node), shape, _pretty_print_spec(spec), f"{c_comp:.1f}", f"{c_comm:.1f}", t_comp_s,
                         t_comm_s, status])
        text = f"explain_placement: target={_pretty_print_spec(DTensorSpec(self.mesh, target))}\n\n"
        text += tabulate(rows, headers=["Node", "Shape", "Chosen", "Ch.Comp", "Ch.Comm", "Tgt.Comp", "Tgt.Comm",
                                        "Status"])
        print(text)
        return text
