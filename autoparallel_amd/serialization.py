"""Save / load of the sharding optimizer's state on the packed layout, and the
lightweight placement file.

The reference pickles the FX graph, the strategy objects and two compact arrays
(autoparallel/serialization.py:104-211): ``dv_costs_keys int32[E, 4]`` and
``dv_costs_vals float64[E, 3]``.  Here the whole state is arrays: the packed
graph (its arrays are the strategies), the same two coefficient arrays — written
by the device from the resident results (apc_export_decision_vars) in the
reference's ``decision_vars`` order —, the per-(node, out_idx) compute vectors,
the constraint log and the selected keys.  The container is an ``.npz`` without
pickled objects, so loading executes nothing from the file.

Loading (reference :214-372) rebuilds the ILP from the saved coefficients and
replays the user constraints; it needs no mesh, process group or GPU to re-solve.
Entry points that evaluate on the device (scoring, JSON export) upload the saved
coefficients into a CostEngine on first use.
"""
from __future__ import annotations

import dataclasses
import json
from typing import Dict, List, Optional

import numpy as np

from .packed import PackedGraph

FORMAT_VERSION = 1

_ARRAY_FIELDS = [
    f.name for f in dataclasses.fields(PackedGraph)
    if f.name not in ("devices_per_host", "n_compute", "node_names", "roles")
]


def graph_to_arrays(g: PackedGraph) -> Dict[str, np.ndarray]:
    out: Dict[str, np.ndarray] = {}
    for name in _ARRAY_FIELDS:
        v = getattr(g, name)
        if v is not None:
            out["g_" + name] = np.asarray(v)
    out["g_scalars"] = np.asarray([g.devices_per_host, g.n_compute], np.int64)
    out["g_node_names"] = np.frombuffer(json.dumps(g.node_names).encode(), np.uint8)
    roles = g.roles
    if roles is not None:
        d = {k: sorted(v) if isinstance(v, set) else [list(x) for x in v] for k, v in dataclasses.asdict(roles).items()}
        out["g_roles"] = np.frombuffer(json.dumps(d).encode(), np.uint8)
    return out


def graph_from_arrays(d) -> PackedGraph:
    from .sharding_problem import GraphRoles

    kw = {name: (d["g_" + name] if "g_" + name in d else None) for name in _ARRAY_FIELDS}
    dph, n_compute = (int(x) for x in d["g_scalars"])
    names = json.loads(bytes(d["g_node_names"]).decode())
    roles = None
    if "g_roles" in d:
        r = json.loads(bytes(d["g_roles"]).decode())
        roles = GraphRoles(
            param_grad=[tuple(x) for x in r["param_grad"]], input_grad=[tuple(x) for x in r["input_grad"]],
            output_tangent=[tuple(x) for x in r["output_tangent"]], fwd_pre_cast=set(r["fwd_pre_cast"]),
            bwd_pre_cast=set(r["bwd_pre_cast"]))
    g = PackedGraph(devices_per_host=dph, n_compute=n_compute, node_names=names, roles=roles, **kw)
    g.validate()
    return g


def _json_arr(obj) -> np.ndarray:
    return np.frombuffer(json.dumps(obj).encode(), np.uint8)


def save_optimizer(core, path: str, mesh_dim_names: Optional[List[str]] = None) -> None:
    """core: a PackedShardingOptimizer (solved or not), or the ShardingOptimizer that holds one
    (the reference's call, ``save_optimizer(opt, path)``, autoparallel/serialization.py:145)."""
    if hasattr(core, "_core"):
        if mesh_dim_names is None and getattr(core.mesh, "mesh_dim_names", None):
            mesh_dim_names = list(core.mesh.mesh_dim_names)
        core = core._core
    g = core.g
    keys, vals = core.decision_var_arrays()
    names = g.node_names or [f"node{i}" for i in range(g.num_nodes)]
    selected = np.zeros((0, 4), np.int32)
    if core.selected is not None:
        selected = g.entry_keys()[core.selected].astype(np.int32)
    # local/global size of every parameter's strategies: what the memory budget
    # rows weigh with.  They come from the device, so the file carries them and a
    # problem read back can be solved under a memory budget where there is no GPU.
    params = [int(p) for p, _ in core.roles.param_grad]
    if core.engine is not None and params:
        core._memory_ratios(params)
    kept = [p for p in params if p in core._memory_ratio_cache]
    ratio_vals = [core._memory_ratio_cache[p] for p in kept]
    arrays = graph_to_arrays(g)
    arrays.update(
        memory_ratio_node=np.asarray(kept, np.int32),
        memory_ratio_off=np.cumsum([0] + [len(r) for r in ratio_vals]).astype(np.int64),
        memory_ratio_val=np.concatenate(ratio_vals) if ratio_vals else np.zeros(0),
    )
    arrays.update(
        version=np.asarray(FORMAT_VERSION),
        mesh_shape=np.asarray(g.mesh_shape, np.int64),
        mesh_dim_names=_json_arr(mesh_dim_names),
        force_grad_reduce_in_higher_precision=np.asarray(bool(core.force_grad_reduce_in_higher_precision)),
        dv_costs_node_names=_json_arr(names),
        dv_costs_keys=keys,
        dv_costs_vals=vals,
        compute=np.asarray(core.coef.compute, np.float64),
        per_arg=np.asarray(core.coef.per_arg, np.float64),
        constraint_log=_json_arr(core._constraint_log),
        cluster_root=np.asarray(core.root, np.int32),
        selected_keys=selected,
    )
    with open(path, "wb") as f:
        np.savez_compressed(f, **arrays)


def load_optimizer(path: str, cls=None):
    """Returns a PackedShardingOptimizer (or ``cls``) with the saved
    coefficients, default constraints, replayed user constraints and, if the
    file holds one, the saved solution."""
    from .sharding_problem import Coefficients, PackedShardingOptimizer

    if isinstance(path, type) or (cls is not None and not isinstance(cls, type)):
        path, cls = cls, path  # the reference's order: load_optimizer(cls, path) (autoparallel/serialization.py:298)
    if cls is None or not issubclass(cls, PackedShardingOptimizer):
        cls = PackedShardingOptimizer  # a file holds the packed problem, whichever class asked for it
    with np.load(path, allow_pickle=False) as d:
        version = int(d["version"])
        if version != FORMAT_VERSION:
            raise RuntimeError(f"Unsupported save file version: {version}")
        g = graph_from_arrays(d)
        keys, vals = d["dv_costs_keys"], d["dv_costs_vals"]
        compute, per_arg = d["compute"], d["per_arg"]
        log = json.loads(bytes(d["constraint_log"]).decode())
        selected = d["selected_keys"]
        force = bool(d["force_grad_reduce_in_higher_precision"])
        dim_names = json.loads(bytes(d["mesh_dim_names"]).decode())
        cluster_root = d["cluster_root"] if "cluster_root" in d else None
        ratios = {}
        if "memory_ratio_node" in d:
            off, val = d["memory_ratio_off"], d["memory_ratio_val"]
            ratios = {int(p): val[off[i]:off[i + 1]].copy() for i, p in enumerate(d["memory_ratio_node"])}
    if keys.shape != (g.num_entries, 4) or vals.shape != (g.num_entries, 3):
        raise RuntimeError("coefficient arrays do not match the packed graph")
    coef = Coefficients.from_decision_var_arrays(g, keys, vals, compute, per_arg)
    core = cls(g, roles=g.roles, force_grad_reduce_in_higher_precision=force, coefficients=coef,
               cluster_root=cluster_root)
    core.mesh_dim_names = dim_names
    core._memory_ratio_cache = ratios
    for method, kwargs in log:
        getattr(core, method)(**kwargs)
    core._constraint_log = [(m, k) for m, k in log]
    core._set_objective()
    if selected.shape[0]:
        core.selected = core.vars_of_keys(selected)
        core.prob.x = np.zeros(core.n_vars)
        core.prob.x[core.selected] = 1.0
        core.prob.objective_value = float(core.prob.objective @ core.prob.x)
    return core


def save_placements(core, sol: np.ndarray, path: str, mesh_dim_names: Optional[List[str]] = None) -> None:
    """Chosen placements per node name as JSON (reference :392-412)."""
    g = core.g
    names = g.node_names or [f"node{i}" for i in range(g.num_nodes)]
    placements = {}
    for v in range(g.num_nodes):
        placements[names[v]] = {"output": core.output_placement_str(v, int(sol[v])),
                                "inputs": core.input_placement_strs(v, int(sol[v]))}
    with open(path, "w") as f:
        json.dump({"version": 1, "mesh_shape": [int(x) for x in g.mesh_shape], "mesh_dim_names": mesh_dim_names,
                   "placements": placements}, f, indent=2)


def load_placements(core, path: str, mesh_dim_names: Optional[List[str]] = None) -> np.ndarray:
    """out_idx per node matching the saved placement strings against the
    strategies of ``core`` (reference :415-475, same error behaviour)."""
    with open(path) as f:
        d = json.load(f)
    if d["version"] != 1:
        raise RuntimeError(f"Unsupported placements file version: {d['version']}")
    g = core.g
    if [int(x) for x in g.mesh_shape] != list(d["mesh_shape"]):
        raise RuntimeError(f"Mesh shape mismatch: saved {list(d['mesh_shape'])}, current {[int(x) for x in g.mesh_shape]}")
    saved_names = tuple(d["mesh_dim_names"]) if d.get("mesh_dim_names") else None
    cur_names = tuple(mesh_dim_names) if mesh_dim_names else None
    if saved_names != cur_names:
        raise RuntimeError(f"Mesh dim names mismatch: saved {list(saved_names or [])}, current {list(cur_names or [])}")
    names = g.node_names or [f"node{i}" for i in range(g.num_nodes)]
    index = {n: i for i, n in enumerate(names)}
    sol = np.full(g.num_nodes, -1, np.int64)
    for name, entry in d["placements"].items():
        if name not in index:
            raise RuntimeError(f"Node '{name}' from saved placements not found in current graph. "
                               "The model may have changed since the placements were saved.")
        v = index[name]
        for o in range(int(g.node_nstrat[v])):
            if core.output_placement_str(v, o) == entry["output"] and core.input_placement_strs(v, o) == entry["inputs"]:
                sol[v] = o
                break
        else:
            raise RuntimeError(f"Placement '{entry['output']}' for node '{name}' not found in available strategies. "
                               "The model or mesh may have changed.")
    return sol
