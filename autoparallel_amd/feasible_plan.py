"""Row filters that let a walk in graph order end without a forbidden entry.

``CostEngine.sample_feasible`` gives every node one of the strategies whose
entries against its producers' choices are finite.  On a graph whose strategies
are arbitrary spec lists (the planner stress DAG) a node now and then has none:
all of its strategies ask some producer for a Partial placement, and the
producer, drawn earlier and without regard to it, did not choose one.  A walk in
graph order cannot take that choice back.

What it can do is keep the producers from choosing wrongly in the first place.
The rule that forbids an entry is local to a mesh dim
(``redistribute_cost``, autoparallel/cost_models/collective_runtime_estimation.py:
134-140 and 215-222): the entry (consumer strategy o, producer strategy j) of an
argument is infinite exactly when the consumer's input spec has a Partial on a
mesh dim where the producer's output spec has none.  So a strategy whose input
specs hold no Partial is finite against anything (a *safe* strategy), a node
that has one never runs out, and only the few nodes without one need help: for
each of them, going through the graph backwards, one strategy is fixed as its
way out and its producers are confined to the strategies that serve it; a
producer that is left without a safe strategy by that is treated the same way.
The result is one boolean filter per confined node, the same for every
assignment: the walk draws uniformly among the allowed strategies that pass the
node's filter, and then always finds one.

Everything here is host work on the spec words of the packed graphs (a byte per
strategy and argument); the draw itself stays on the device.
"""
from __future__ import annotations

import heapq
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np

from .packed import PLC_KIND_MASK, PLC_PARTIAL, SPEC_NONE, TUPLE_BITS, PackedGraph

_TUPLE_MASK = (1 << TUPLE_BITS) - 1


def _partial_masks(g: PackedGraph, words: np.ndarray, missing: int) -> np.ndarray:
    """uint8 per spec word: bit i set where the placement on mesh dim i is a
    Partial (of any reduction); ``missing`` for SPEC_NONE."""
    nd = g.ndim
    plc = g.tuple_plc[(words & _TUPLE_MASK).astype(np.int64) % max(g.tuple_plc.shape[0], 1), :nd]
    m = (((plc & PLC_KIND_MASK) == PLC_PARTIAL) << np.arange(nd, dtype=np.uint8)).sum(axis=1).astype(np.uint8)
    return np.where(words == SPEC_NONE, np.uint8(missing), m)


@dataclass
class NodeMasks:
    """What the plan needs to know about one node."""
    out: np.ndarray  # uint8[S] Partial dims of the output spec of every strategy
    producers: List[int] = field(default_factory=list)  # global node id per argument with a producer
    wants: List[np.ndarray] = field(default_factory=list)  # uint8[S] per such argument: Partial dims of its input spec

    def safe(self) -> np.ndarray:
        """bool[S]: the strategies that ask no producer for a Partial."""
        s = np.ones(self.out.shape[0], bool)
        for w in self.wants:
            s &= w == 0
        return s

    def __post_init__(self):
        self.has_safe = None  # filled by finish(): made where the masks are made, read where the plan is

    def finish(self) -> "NodeMasks":
        self.has_safe = bool(self.safe().any())
        return self


def window_masks(g: PackedGraph, gid: Optional[np.ndarray] = None, first_node: int = 0) -> Dict[int, NodeMasks]:
    """NodeMasks of the nodes [first_node, N) of a packed graph, keyed by their
    global id (``gid[i]``, or i).  The stand-ins of a window (the nodes below
    first_node) belong to the window that owns them."""
    if g.node_out_runs is not None and g.node_out_runs.shape[1] > 1 and (g.node_out_runs[:, 1:] >= 0).any():
        raise NotImplementedError("feasible_plan: nodes with several outputs")
    full = (1 << g.ndim) - 1
    out: Dict[int, NodeMasks] = {}
    for v in range(first_node, g.num_nodes):
        S = int(g.node_nstrat[v])
        o0 = int(g.node_out_list[v])
        # a strategy without an output spec prices its consumers' entries from default rows: finite
        nm = NodeMasks(out=_partial_masks(g, g.lists[o0:o0 + S], full) if o0 >= 0 else np.full(S, full, np.uint8))
        for e in range(int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])):
            u = int(g.edge_src_node[e])
            if u < 0:
                continue
            d0 = int(g.edge_dst_list[e])
            nm.producers.append(int(gid[u]) if gid is not None else u)
            nm.wants.append(_partial_masks(g, g.lists[d0:d0 + S], 0))
        out[int(gid[v]) if gid is not None else v] = nm.finish()
    return out


def _plan_once(nodes: Dict[int, NodeMasks], banned):
    """One pass from the last node to the first.  Returns (filters, stuck, culprits):
    ``culprits`` the (node, strategy) ways out chosen earlier in the pass that confined a
    stuck node or one of its producers."""
    filters: Dict[int, np.ndarray] = {}
    owners: Dict[int, list] = {}
    stuck: List[int] = []
    culprits = set()

    def allowed(v):
        f = filters.get(v)
        return f if f is not None else np.ones(nodes[v].out.shape[0], bool)

    # nodes without a safe strategy, largest id first; confined producers join as the plan goes
    heap = [-v for v, nm in nodes.items()
            if nm.wants and not (nm.has_safe if nm.has_safe is not None else nm.safe().any())]
    heapq.heapify(heap)
    queued = {-x for x in heap}
    while heap:
        v = -heapq.heappop(heap)
        nm = nodes[v]
        rows = allowed(v)
        if (rows & nm.safe()).any():
            continue  # whatever the producers choose, one of these is allowed
        best = None
        for o in np.flatnonzero(rows):
            if (v, int(o)) in banned:
                continue
            after: Dict[int, np.ndarray] = {}
            ok = True
            for u, w in zip(nm.producers, nm.wants):
                need = int(w[o])
                left = after.get(u)
                if left is None:
                    left = allowed(u)
                if need:
                    left = left & ((nodes[u].out & need) == need)
                if not left.any():
                    ok = False
                    break
                after[u] = left
            if not ok:
                continue
            # prefer a way out that leaves every producer a safe strategy, then one that asks for least
            unsafe = sum(1 for u, left in after.items() if nodes[u].wants and not (left & nodes[u].safe()).any())
            asks = sum(bin(int(w[o])).count("1") for w in nm.wants)
            key = (unsafe, asks, int(o))
            if best is None or key < best[0]:
                best = (key, after)
        if best is None:
            stuck.append(v)
            for u in [v] + list(nm.producers):
                culprits.update(owners.get(u, ()))
            continue
        for u, left in best[1].items():
            if not np.array_equal(left, allowed(u)):
                filters[u] = left
                owners.setdefault(u, []).append((v, best[0][2]))
                if u not in queued:
                    queued.add(u)
                    heapq.heappush(heap, -u)
    return filters, stuck, culprits


def plan_filters(nodes: Dict[int, NodeMasks], rounds: int = 32):
    """(filters, stuck): ``filters[v]`` bool[S_v] for every node the plan confines,
    ``stuck`` the nodes for which it found no way out (the walk may fall back
    there).  Producers have smaller ids than their consumers.  A pass that leaves a
    node stuck is repeated without the ways out that confined that node or its
    producers, so that the nodes that chose them choose again."""
    banned = set()
    best = None
    for _ in range(rounds):
        filters, stuck, culprits = _plan_once(nodes, banned)
        if best is None or len(stuck) < len(best[1]):
            best = (filters, stuck)
        if not stuck or not culprits - banned:
            break
        banned |= culprits
    return best


def unservable(nodes: Dict[int, NodeMasks], v: int) -> bool:
    """True if every strategy of node v asks some producer for Partial placements that no
    strategy of that producer offers: v then selects a forbidden entry in every assignment
    of the graph, whatever the others choose (the ILP of such a graph has no solution)."""
    nm = nodes[v]
    for o in range(nm.out.shape[0]):
        if all(((nodes[u].out & int(w[o])) == int(w[o])).any() for u, w in zip(nm.producers, nm.wants)):
            return False
    return bool(nm.wants)
