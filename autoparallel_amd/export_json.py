"""Structured export of a solved plan from the packed layout.

Counterpart of the reference's ``export_sharding_json``
(autoparallel/export_json.py:240-424): one record per node with its chosen
placement, its input edges (producer placement, placement the consumer asked
for, communication and transition cost of the selected variable) and its
compute cost, plus the summary totals.  The selected variables' terms are
gathered on the device (apc_solution_terms); fields that only an FX graph
carries (source location, module path, AC region, clusters) come from
``fx_node_info`` below, which the FX facade hands in.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional

import numpy as np

from .packed import SPEC_NONE

_DTYPE_NAMES = {0: "float64", 1: "float32", 2: "float16", 3: "bfloat16", 4: "int8"}


def _shape_dtype(g, word: int):
    if int(word) == SPEC_NONE:
        return None, None
    m = int(word) >> 12
    r = int(g.meta_rank[m])
    return [int(x) for x in g.meta_shape[m, :r]], _DTYPE_NAMES.get(int(g.meta_dtype[m]), "other")


# ---------------------------------------------------------------------------
# Fields that only the FX graph carries (autoparallel/export_json.py:23-215).
# The functions take anything with ``meta`` / ``op`` / ``name`` attributes.
# ---------------------------------------------------------------------------
_PLACEHOLDER_KINDS = {"ParamAOTInput": "param", "BufferAOTInput": "buffer", "TangentAOTInput": "tangent",
                      "PlainAOTInput": "input"}


def placeholder_kind(node) -> Optional[str]:
    desc = node.meta.get("desc")
    return _PLACEHOLDER_KINDS.get(type(desc).__name__) if desc is not None else None


def source_info(node) -> Optional[Dict[str, Any]]:
    """Innermost frame of the node's recorded stack trace (:23-37)."""
    import re

    trace = node.meta.get("stack_trace")
    frames = re.findall(r'File "([^"]+)", line (\d+), in (\w+)\n\s+(.*)', trace) if trace else []
    if not frames:
        return None
    file, line, func, code = frames[-1]
    return {"file": file, "line": int(line), "func": func, "code": code.strip()}


def _module_stack(node):
    return node.meta.get("nn_module_stack") or node.meta.get("fwd_nn_module_stack")


def _own_module_path(node) -> Optional[str]:
    path = node.meta.get("module_path")  # written into graphs that were saved
    if path is not None:
        return path
    if getattr(node, "op", None) == "placeholder":
        target = getattr(node.meta.get("desc"), "target", None)
        if isinstance(target, str) and target:
            return target
    stack = _module_stack(node)
    if not stack:
        return None
    innermost = list(stack.values())[-1]  # name -> (qualified name, class), outermost first
    return innermost[0] if innermost else None


def module_path(node) -> Optional[str]:
    """Qualified name of the innermost module the node was traced in (:40-110).  A
    node that lost its module stack (backward helpers) gets what its producers and
    users agree on: the common prefix of their paths, parameters counted by their
    module (``...weight`` / ``...bias`` dropped), the bare root excluded."""
    own = _own_module_path(node)
    if own is not None:
        return own
    around = [_own_module_path(n) for n in list(node.all_input_nodes) + list(node.users)]
    parts = []
    for path in around:
        if path:
            p = path.split(".")
            p = p[:-1] if p[-1] in ("weight", "bias") else p
            if p:
                parts.append(p)
    if not parts:
        return None
    common = parts[0]
    for p in parts[1:]:
        n = 0
        while n < min(len(common), len(p)) and common[n] == p[n]:
            n += 1
        common = common[:n]
    if not common or common in (["L['self']"], ["_export_root"]):
        return None
    return ".".join(common)


def phase(node) -> str:
    """"forward" or "backward" (:113-146): from the placeholder's role, the
    partitioner's tag, which of the two module stacks the node carries, and last
    its position relative to the first tangent input."""
    if node.meta.get("phase") is not None:
        return node.meta["phase"]
    kind = placeholder_kind(node)
    if kind is not None:
        return "backward" if kind == "tangent" else "forward"
    tag = node.meta.get("partitioner_tag")
    if tag in ("is_forward", "is_backward"):
        return tag[3:]
    if node.op == "placeholder":
        return "backward" if node.name.startswith("tangents") else "forward"
    if "nn_module_stack" in node.meta:
        return "forward"
    if "fwd_nn_module_stack" in node.meta:
        return "backward"
    after_tangent = False
    for n in node.graph.nodes:
        after_tangent = after_tangent or (n.op == "placeholder" and n.name.startswith("tangents"))
        if n is node:
            break
    return "backward" if after_tangent else "forward"


def layer_index(node) -> Optional[int]:
    """Index of the repeated layer the node belongs to (``layers.<i>`` anywhere
    in its module stack), or None (:149-162)."""
    import re

    for value in (_module_stack(node) or {}).values():
        found = re.search(r"layers\.(\d+)", value[0])
        if found:
            return int(found.group(1))
    return None


def normalize_cluster_layer(cluster_roots: Dict[Any, Any]) -> None:
    """``cluster_roots`` maps a linked node to its root.  Forward clusters root in the
    first layer and backward ones in the last (topological order); for a steadier
    picture every cluster whose root is outside the lowest layer that holds a root
    is re-rooted, in place, at its member nearest to that layer (:165-215)."""
    members: Dict[Any, List[Any]] = {}
    for linked, root in cluster_roots.items():
        members.setdefault(root, []).append(linked)
    layers = {layer_index(root) for root in members} - {None}
    if not layers:
        return
    lowest = min(layers)
    for root in list(members):
        at = layer_index(root)
        if at is None or at == lowest:
            continue
        ranked = [(abs(layer_index(n) - lowest), i) for i, n in enumerate(members[root]) if layer_index(n) is not None]
        if not ranked:
            continue
        new_root = members[root][min(ranked)[1]]
        if layer_index(new_root) == at:
            continue
        rest = [n for n in members.pop(root) if n is not new_root] + [root]
        del cluster_roots[new_root]
        for n in rest:
            cluster_roots[n] = new_root
        members[new_root] = rest


def fx_node_info(nodes, cluster_root_of: Optional[Dict[Any, Any]] = None) -> List[Dict[str, Any]]:
    """The per-node fields of the reference's export that come from the FX graph
    (:362-407): op, phase, placeholder kind, source line, module path, activation
    checkpointing region, and the cluster a repeated node belongs to (``cluster_root_of``:
    linked node -> root node; re-rooted as ``normalize_cluster_layer`` does)."""
    roots = dict(cluster_root_of or {})
    normalize_cluster_layer(roots)
    cluster_id: Dict[Any, int] = {}
    for root in roots.values():
        cluster_id.setdefault(root, len(cluster_id))
    out = []
    for node in nodes:
        info: Dict[str, Any] = {"op": str(node.target) if node.op == "call_function" else node.op, "phase": phase(node)}
        kind = placeholder_kind(node) if node.op == "placeholder" else None
        if kind:
            info["placeholder_kind"] = kind
        src = source_info(node)
        if src is not None:
            info["source"] = src
        path = module_path(node)
        if path is not None:
            info["module_path"] = path
        if node.meta.get("ac_graph_id") is not None:
            recompute = node.meta.get("recompute")
            info["ac_region"] = {"id": node.meta["ac_graph_id"], "type": recompute.name if recompute is not None else None}
        if node in roots:
            info["cluster_id"], info["cluster_root"] = cluster_id[roots[node]], roots[node].name
        elif node in cluster_id:
            info["cluster_id"] = cluster_id[node]
        out.append(info)
    return out


def export_sharding_json(core, sol: np.ndarray, node_info: Optional[List[Dict[str, Any]]] = None) -> Dict[str, Any]:
    """node_info: optional per-node extra fields (op, phase, source, ...)
    merged into each record."""
    g = core.g
    terms, _ = core.solution_terms(sol)
    names = g.node_names or [f"node{i}" for i in range(g.num_nodes)]
    clusters = g.node_multiplier
    nodes_list = []
    total_compute = total_comm = total_transition = 0.0
    for v in range(g.num_nodes):
        o = int(sol[v])
        e0, e1 = int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])
        inputs = []
        node_comm = node_transition = compute = 0.0
        for e in range(e0, e1):
            compute += float(terms[e, 0])  # split across args in the ILP: the sum is the op's cost
            u = int(g.edge_src_node[e])
            if u < 0:
                continue
            comm, trans = float(terms[e, 1]), float(terms[e, 2])
            node_comm += comm
            node_transition += trans
            src_word = g.lists[int(g.edge_src_list[e]) + int(sol[u])]
            inputs.append({
                "name": names[u],
                "src_placement": core._spec_str(src_word),
                "dst_placement": core._spec_str(g.lists[int(g.edge_dst_list[e]) + o]),
                "comm_cost": comm,
                "transition_cost": trans,
            })
        total_compute += compute
        total_comm += node_comm
        total_transition += node_transition
        entry: Dict[str, Any] = {
            "name": names[v],
            "op": "node",
            "placement": core.output_placement_str(v, o),
            "inputs": inputs,
            "compute_cost": compute,
            "transition_cost": node_transition,
        }
        shape, dtype = _shape_dtype(g, g.lists[int(g.node_out_list[v]) + o])
        if dtype is not None:
            entry["dtype"] = dtype
        if shape is not None:
            entry["shape"] = shape
        if clusters is not None and int(clusters[v]) > 1:
            entry["cluster_multiplicity"] = int(clusters[v])
        if node_info is not None:
            entry.update(node_info[v])
        nodes_list.append(entry)
    return {
        "mesh": {"shape": [int(x) for x in g.mesh_shape], "dim_names": core.mesh_dim_names},
        "nodes": nodes_list,
        "summary": {
            "total": total_compute + total_comm + total_transition,
            "comm": total_comm,
            "compute": total_compute,
            "transition": total_transition,
        },
    }
