"""Structured export of a solved plan from the packed layout.

Counterpart of the reference's ``export_sharding_json``
(autoparallel/export_json.py:240-424): one record per node with its chosen
placement, its input edges (producer placement, placement the consumer asked
for, communication and transition cost of the selected variable) and its
compute cost, plus the summary totals.  The selected variables' terms are
gathered on the device (apc_solution_terms); fields that only an FX graph
carries (source location, module path, AC region) are added by the FX facade.
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
