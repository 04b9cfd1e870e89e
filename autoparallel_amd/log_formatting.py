"""Human-readable log of a solved plan.

``format_sharding_log`` has the reference's signature and output contract
(autoparallel/log_formatting.py:19-210): the FX graph's Python code with, on the
line that assigns each node, ``# placement=<strategy> , cost=[(comm, compute,
transition), ...]``, placeholders that share a line listed as comments under the
``def``, and the four totals at the end.  ``format_packed_log`` is the same
report for a packed graph without FX code.
"""
from __future__ import annotations

import re
from typing import Any, Dict, List

import numpy as np


def _totals_block(total, comm, compute, transition, violated: str = "") -> str:
    out = (f"\ntotal_cost: {total:.2f}\n  comm_cost: {comm:.2f}\n  compute_cost: {compute:.2f}"
           f"\n  transition_cost: {transition:.2f}")
    if violated:
        out += "\n" + violated
    return out


def format_sharding_log(graph, opt: Dict[Any, List[Any]], colored: bool = False, verbose: bool = False,
                        violated_constraints_log: str = "") -> str:
    from torch.fx.graph import _color_fns, _identity

    src = graph.python_code("self", colored=colored, verbose=verbose).src
    lines = src.split("\n")
    blue = _color_fns["blue"] if colored else _identity
    red = _color_fns["red"] if colored else _identity
    # first non-comment line on which each name is the assignment target
    assigned: Dict[str, int] = {}
    for i, line in enumerate(lines):
        s = line.lstrip()
        if s.startswith("#") or s.startswith("def "):
            continue
        m = re.match(r"([A-Za-z_][A-Za-z_0-9]*)\s*(:|=|,|$)", s)
        if m and m.group(1) not in assigned:
            assigned[m.group(1)] = i
    total = comm = compute = transition = 0.0
    used = set()
    loose: List[str] = []
    for node in graph.nodes:
        if node.op == "output" or node not in opt:
            continue
        d = opt[node]
        for e in d:
            total += e.cost
            comm += e.comm_cost
            compute += e.compute_cost
            transition += e.sharding_transition_cost
        costs = [(x.comm_cost, x.compute_cost, x.sharding_transition_cost) for x in d]
        order = node.meta.get("shard_order")
        mid = f" shard_order={order!r} " if order else " "
        note = f"  {blue('# placement=')}{red(str(d[0].strategy))}{mid}{blue(', cost=')}{red(str(costs))}"
        i = assigned.get(repr(node))
        if i is not None and i not in used:
            lines[i] += note
            used.add(i)
        elif node.op == "placeholder":
            loose.append(f"    # {node.name}:{note}")
    if loose:
        at = next((i + 1 for i, line in enumerate(lines) if line.lstrip().startswith("def ")), 1)
        lines[at:at] = loose
    return "\n".join(lines) + _totals_block(total, comm, compute, transition, violated_constraints_log)


def format_packed_log(core, sol: np.ndarray, violated_constraints_log: str = "") -> str:
    g = core.g
    terms, _ = core.solution_terms(sol)
    names = g.node_names or [f"node{i}" for i in range(g.num_nodes)]
    out = []
    total = comm = compute = transition = 0.0
    for v in range(g.num_nodes):
        o = int(sol[v])
        e0, e1 = int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])
        costs = [(float(terms[e, 1]), float(terms[e, 0]), float(terms[e, 2])) for e in range(e0, e1)]
        for e in range(e0, e1):
            total += float(terms[e, 3])
            comm += float(terms[e, 1])
            compute += float(terms[e, 0])
            transition += float(terms[e, 2])
        args = ", ".join(names[int(u)] for u in g.edge_src_node[e0:e1] if u >= 0)
        ins = ", ".join(str(s) for s in core.input_placement_strs(v, o))
        out.append(f"{names[v]} = node({args})  # placement=({ins}) -> {core.output_placement_str(v, o)} , cost={costs}")
    return "\n".join(out) + _totals_block(total, comm, compute, transition, violated_constraints_log)
