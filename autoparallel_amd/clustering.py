"""Repeated-subgraph clustering on the packed graph.

The reference groups nodes by a hash of (op, forward/backward tag, own
strategies, producers' strategies) and grows, from the latest group backwards,
the largest position-wise identical regions
(autoparallel/graph_passes/graph_clustering.py:85-206, with torch's
``fully_expand_region_group``, torch:_dynamo/graph_region_tracker.py); every
node of a later region is then linked to the node at the same position of the
group's first region and shares its decision variables
(autoparallel/optimize_sharding.py:356-378).

Here the hash of every node comes from the device (apc_node_hashes over the
packed arrays); grouping, the backward breadth-first region growth and the link
table are host index work on the packed graph.
"""
from __future__ import annotations

from collections import deque
from typing import Dict, List, Optional, Sequence

import numpy as np

from .packed import PackedGraph


def _unique_args(g: PackedGraph) -> List[List[int]]:
    out: List[List[int]] = []
    for v in range(g.num_nodes):
        e0, e1 = int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])
        out.append(list(dict.fromkeys(int(u) for u in g.edge_src_node[e0:e1] if u >= 0)))
    return out


def placeholder_mask(g: PackedGraph) -> np.ndarray:
    if g.node_kind is not None:
        return np.asarray(g.node_kind) == 1
    has_producer = np.zeros(g.num_nodes, bool)
    has_producer[g.edge_node[g.edge_src_node >= 0]] = True
    return ~has_producer & (np.asarray(g.node_op) == 0)


class _Region:
    """One region under growth: its nodes, the breadth-first queue of argument
    nodes still to consider, and the ancestors of everything in it."""

    def __init__(self, root: int, args: List[List[int]], anc: List[int]):
        self.nodes = [root]
        self.member = {root}
        self.queue = deque(args[root])
        self.ancestors = anc[root]
        self._args, self._anc = args, anc

    def next(self) -> Optional[int]:
        return self.queue.popleft() if self.queue else None

    def closes_cycle(self, v: int, users: List[List[int]]) -> bool:
        # a user outside the region that the region depends on
        return any(u not in self.member and (self.ancestors >> u) & 1 for u in users[v])

    def add(self, v: int) -> None:
        self.nodes.append(v)
        self.member.add(v)
        self.queue.extend(self._args[v])
        self.ancestors |= self._anc[v]


def identical_regions(g: PackedGraph, hashes: Sequence[int], check_cycles: bool = True,
                      keep_unclaimed: bool = False) -> List[List[List[int]]]:
    """Region groups, each a list of regions (node lists in graph order) that
    are identical position by position; groups and regions in graph order.

    keep_unclaimed: the reference drops a whole list of duplicates as soon as an
    earlier region has taken one of them (graph_clustering.py:169-176), which
    leaves e.g. the second normalisation of every transformer layer outside any
    region when the first one was taken.  With this set, the duplicates that are
    still free are grown into regions of their own when two or more remain, and
    duplicates that end up in no region at all form regions of one node each."""
    n = g.num_nodes
    args = _unique_args(g)
    users: List[List[int]] = [[] for _ in range(n)]
    for v in range(n):
        for u in args[v]:
            users[u].append(v)
    anc = [0] * n
    if check_cycles:  # bit u of anc[v]: u is an ancestor of v
        for v in range(n):
            a = 0
            for u in args[v]:
                a |= anc[u] | (1 << u)
            anc[v] = a
    is_ph = placeholder_mask(g)
    phase = np.asarray(g.node_phase) if g.node_phase is not None else np.zeros(n, np.int32)
    klass: Dict[int, int] = {}  # node -> id of its duplicate list
    groups: Dict[int, List[int]] = {}
    for v in range(n):
        if is_ph[v]:
            continue
        h = int(hashes[v])
        groups.setdefault(h, []).append(v)
        klass[v] = h
    cand = [grp for grp in groups.values() if len(grp) > 1]
    cand.sort(key=lambda grp: -min(grp))  # latest first: the largest regions form first
    seen: set = set()
    result = []
    for grp in cand:
        if any(r in seen for r in grp):
            if not keep_unclaimed:
                continue
            grp = [r for r in grp if r not in seen]
            if len(grp) < 2:
                continue
        ph = int(phase[grp[0]])
        regions = [_Region(r, args, anc) for r in grp]
        cur = regions[0].next()
        while cur is not None:
            ok = not regions[0].closes_cycle(cur, users)
            picked = [cur]
            for reg in regions[1:]:
                c = reg.next()
                if c is None or not ok:
                    ok = False
                    continue
                ok = (c not in seen and c not in picked and not is_ph[c] and klass.get(c) is not None
                      and klass.get(c) == klass.get(cur) and c != cur and int(phase[c]) == ph
                      and int(phase[cur]) == ph and not reg.closes_cycle(c, users))
                picked.append(c)
            if ok:
                for reg, v in zip(regions, picked):
                    reg.add(v)
                    seen.add(v)
            cur = regions[0].next()
        if len(regions[0].nodes) > 1:
            result.append([sorted(reg.nodes) for reg in regions])
            if keep_unclaimed:  # the roots of a kept region are taken too
                seen.update(grp)
    if keep_unclaimed:
        # what no region took: duplicates of each other still share variables, as
        # regions of one node (the reference keeps no such region, :188-190)
        for grp in cand:
            free = [r for r in grp if r not in seen]
            if len(free) > 1:
                result.append([[r] for r in free])
                seen.update(free)
    for grp in result:
        grp.sort(key=lambda r: r[0])
    result.sort(key=lambda grp: grp[0][0])
    used: set = set()
    for grp in result:
        for reg in grp:
            for v in reg:
                if v in used:
                    raise RuntimeError(f"Duplicate node {v} in region group")
                used.add(v)
    return result


def cluster_roots(g: PackedGraph, region_groups: List[List[List[int]]]) -> np.ndarray:
    """int32[N]: root[v] = node whose decision variables v shares (v itself for
    roots and unclustered nodes).  Checks that linked nodes offer the same
    options as their root (the reference asserts it, optimize_sharding.py:366-371)."""
    root = np.arange(g.num_nodes, dtype=np.int32)
    for grp in region_groups:
        first = grp[0]
        for reg in grp[1:]:
            if len(reg) != len(first):
                raise RuntimeError("regions of one group differ in length")
            for a, b in zip(first, reg):
                ea, eb = int(g.node_edge_off[a]), int(g.node_edge_off[b])
                na, nb = int(g.node_edge_off[a + 1]) - ea, int(g.node_edge_off[b + 1]) - eb
                same = (na == nb and int(g.node_nstrat[a]) == int(g.node_nstrat[b])
                        and np.array_equal(g.edge_ssrc[ea:ea + na], g.edge_ssrc[eb:eb + nb]))
                if not same:
                    raise RuntimeError(
                        f"Problem with graph clustering: nodes {a} and {b} don't have the same number "
                        "of input/output placements. Please report a bug")
                root[b] = a
    return root


def multipliers(root: np.ndarray) -> np.ndarray:
    """1 + number of linked copies for roots, as _set_objective weighs them
    (optimize_sharding.py:879-885); 0 for linked nodes (their variables are the
    root's)."""
    mult = np.bincount(root, minlength=root.shape[0]).astype(np.int32)
    return mult
