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
