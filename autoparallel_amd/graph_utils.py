"""What the planner's input graph needs before it is planned, host index work on
the FX graph: the node sets that decide which edges the prefetch discount
applies to (build_param_derived_set / build_terminal_derived_set,
autoparallel/graph_passes/graph_utils.py:442-484; they feed the
APC_EDGE_PREFETCHABLE flag of the packed edges), alias nodes where values fan out
(:99-183), and linear layers rewritten as einsums (:270-439)."""
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
        if ins and derived.issuperset(ins):
            derived.add(node)
    return derived


def build_terminal_derived_set(graph: torch.fx.Graph) -> Set[torch.fx.Node]:
    """Parameter-gradient nodes and every node all of whose users are in the
    set: the tail of each gradient chain, whose reduce-scatter can overlap."""
    terminal = {g for _, g in fx_utils.get_param_and_grad_nodes(graph).values() if g is not None}
    for node in reversed(list(graph.nodes)):
        if node.op == "output":
            continue
        if node.users and terminal.issuperset(node.users):
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


# ---------------------------------------------------------------------------
# Linear layers as einsums
# ---------------------------------------------------------------------------
# A linear layer on an input of three or more dims is traced as "flatten the
# leading dims, mm, unflatten"; the flattened 2-D matmul has no strategy that
# keeps batch and sequence sharded separately, so the planner would never be
# offered sequence parallelism.  The reference rewrites the two shapes this takes
# (the layer itself, and the weight gradient in the backward) into einsums before
# planning (autoparallel/graph_passes/graph_utils.py:270-439, called from
# api.py:208); this is that rewrite.
_VIEWS = (torch.ops.aten.view.default, torch.ops.aten._unsafe_view.default)
_AUTOGRAD_KEYS = ("seq_nr", "recompute", "ac_graph_id")  # what the mm carried and the einsum must keep


def _shape(node) -> tuple:
    return tuple(node.meta["val"].shape)


def _flattens_leading_dims(full: tuple, flat: tuple) -> bool:
    """flat == [prod(full[:-1]), full[-1]] with at least two leading dims."""
    if len(full) < 3 or len(flat) != 2:
        return False
    lead = 1
    for d in full[:-1]:
        lead *= d
    return flat == (lead, full[-1])


def _is_transpose(node) -> bool:
    """permute(x, [1, 0]), or aten.t, which is what torch 2.10 traces for it."""
    if node.op != "call_function":
        return False
    if node.target is torch.ops.aten.t.default:
        return len(_shape(node)) == 2
    return node.target is torch.ops.aten.permute.default and list(node.args[1]) == [1, 0]


def _flattened_source(node):
    """x if node is view(x) flattening x's leading dims, else None."""
    if node.op != "call_function" or node.target not in _VIEWS:
        return None
    src = node.all_input_nodes[0]
    return src if _flattens_leading_dims(_shape(src), _shape(node)) else None


def _letters(n: int) -> str:
    assert 0 < n <= 23  # 'a'.. ; k and n are taken by the contraction and the output feature
    return "abcdefghijlmopqrstuvwxyz"[:n]


def _linear_as_einsum(mm):
    """(equation, operands, node to replace) if mm is the matmul of a traced
    linear layer or of its weight gradient, else None."""
    if len(mm.args) != 2 or not all(isinstance(a, torch.fx.Node) for a in mm.args) or len(mm.users) != 1:
        return None
    lhs, rhs = mm.args
    (user,) = mm.users
    # forward: view(x [*b, K] -> [B, K]) @ w [K, N] -> view([B, N] -> [*b, N])
    x = _flattened_source(lhs)
    if x is not None and user.target in _VIEWS:
        xs, ws, ys = _shape(x), _shape(rhs), _shape(user)
        if (len(ws) == 2 and all(d != 0 for d in xs) and _flattens_leading_dims(ys, _shape(mm))
                and ys[:-1] == xs[:-1] and ws == (xs[-1], ys[-1])):
            b = _letters(len(xs) - 1)
            return f"{b}k,kn->{b}n", [x, rhs], user
    # weight gradient: view(g [*b, N])^T @ view(x [*b, K]) -> [N, K], then ^T -> [K, N]
    if _is_transpose(lhs) and _is_transpose(user) and len(_shape(mm)) == 2:
        g, x = _flattened_source(lhs.all_input_nodes[0]), _flattened_source(rhs)
        if g is not None and x is not None and _shape(g)[:-1] == _shape(x)[:-1]:
            b = _letters(len(_shape(g)) - 1)
            return f"{b}n,{b}k->kn", [g, x], user
    return None


def replace_view_mm_view_with_einsum(gm: torch.fx.GraphModule) -> int:
    """Rewrites every traced linear layer (and weight-gradient matmul) of the
    graph into ``aten.einsum`` over the unflattened tensors; what the rewrite
    leaves without users is removed.  Returns the number of einsums made.
    ``aten._unsafe_view`` and ``aten.t``, which torch 2.10 traces for the unflatten
    and the transposes, count as view and permute here (the reference matches
    ``aten.view`` and ``aten.permute`` only)."""
    graph = gm.graph
    made = 0
    for mm in graph.find_nodes(op="call_function", target=torch.ops.aten.mm.default):
        found = _linear_as_einsum(mm)
        if found is None:
            continue
        equation, operands, replaced = found
        with graph.inserting_before(mm):
            ein = graph.call_function(torch.ops.aten.einsum.default, args=(equation, operands))
        ein.meta.update(replaced.meta)
        for key in _AUTOGRAD_KEYS:
            if key in mm.meta:
                ein.meta[key] = mm.meta[key]
        replaced.replace_all_uses_with(ein)
        made += 1
    if made:
        graph.eliminate_dead_code()
        graph.lint()
        gm.recompile()
    return made


_replace_view_mm_view_with_einsum = replace_view_mm_view_with_einsum  # the reference's name
