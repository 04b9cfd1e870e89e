"""Graph sets that decide which edges the prefetch discount applies to
(counterparts of build_param_derived_set / build_terminal_derived_set,
autoparallel/graph_passes/graph_utils.py:442-484): host index work on the FX
graph, feeding the APC_EDGE_PREFETCHABLE flag of the packed edges."""
from __future__ import annotations

from typing import Set

import torch.fx
from torch._functorch._aot_autograd import fx_utils


def build_param_derived_set(graph: torch.fx.Graph) -> Set[torch.fx.Node]:
    """Parameters and every node all of whose inputs are parameter-derived
    (dtype casts, views, aliases of parameters: all-gatherable ahead of time)."""
    derived = set(fx_utils.get_param_nodes(graph))
    for node in graph.nodes:
        ins = node.all_input_nodes
        if ins and all(i in derived for i in ins):
            derived.add(node)
    return derived


def build_terminal_derived_set(graph: torch.fx.Graph) -> Set[torch.fx.Node]:
    """Parameter-gradient nodes and every node all of whose users are in the
    set: the tail of each gradient chain, whose reduce-scatter can overlap."""
    terminal = {g for _, g in fx_utils.get_param_and_grad_nodes(graph).values() if g is not None}
    for node in reversed(list(graph.nodes)):
        if node.op == "output":
            continue
        if node.users and all(u in terminal for u in node.users):
            terminal.add(node)
    return terminal


def add_alias_nodes(gm: torch.fx.GraphModule) -> torch.fx.GraphModule:
    """Gives the planner a place to change placement where a value fans out and
    where it leaves the graph, as the reference prepares its joint graph
    (autoparallel/graph_passes/graph_utils.py:99-183, the "v2" form): an
    ``aten.alias`` after every tensor-valued node with two or more users (its
    users then read the alias), and one after every node the output returns.
    An alias has every placement of its tensor as a candidate, so the edge into
    it can carry a redistribution that the producer's own strategies cannot."""
    graph = gm.graph
    order = {n: i for i, n in enumerate(graph.nodes)}

    def alias_of(node: torch.fx.Node, before: torch.fx.Node = None) -> torch.fx.Node:
        ctx = graph.inserting_before(before) if before is not None else graph.inserting_after(node)
        with ctx:
            a = graph.call_function(torch.ops.aten.alias.default, args=(node,))
        meta = dict(node.meta)
        if "tangents" in node.name:  # tangents carry a forward tag that would mislead the partitioner
            meta.pop("partitioner_tag", None)
        a.meta.update(meta)
        return a

    for node in list(order):
        if len(node.users) < 2 or not isinstance(node.meta.get("val"), torch.Tensor):
            continue
        first_user = min(node.users, key=order.__getitem__)
        a = alias_of(node, before=first_user)
        node.replace_all_uses_with(a, delete_user_cb=lambda user, a=a: user is not a)
    out = next(n for n in graph.nodes if n.op == "output")
    for node in list(out.all_input_nodes):
        a = alias_of(node)
        node.replace_all_uses_with(a, delete_user_cb=lambda user, a=a: user is not a)
    gm.recompile()
    return gm
