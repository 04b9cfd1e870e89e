"""CPU oracle for the node clustering key.  TEST INFRASTRUCTURE ONLY.

Nothing under ``autoparallel_amd/`` may import this module.

``node_key`` is the exact content the reference hashes per node
(autoparallel/graph_passes/graph_clustering.py:68-82: op, forward/backward tag,
the node's own strategies, its producers' strategies), read from the packed
arrays; ``node_hash`` restates the device's 64-bit hash of that content word by
word on Python ints.

Pinning: the hash is this repository's own function (the reference uses SHA-256
of a pickle, any collision-free key gives the same groups), so what is pinned is
the grouping: tests assert that two nodes share a hash exactly when their
``node_key`` tuples are equal, and that the repeated layers of the benchmark
graphs fall into one group per layer position.
"""
from __future__ import annotations

import struct
from typing import List, Optional, Sequence

M64 = (1 << 64) - 1


def mix64(z: int) -> int:
    z &= M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    return z ^ (z >> 31)


def term(section: int, pos: int, w: int) -> int:
    return mix64((w & M64) ^ mix64(((section << 40) + pos + 0x9E3779B97F4A7C15) & M64))


def _sections(g, v: int, phase: Optional[Sequence[int]]):
    """[(section, [words...])] of node v: the content of the key."""
    S = int(g.node_nstrat[v])
    e0, e1 = int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])
    op = int(g.node_op[v])
    out = [(0, [op, int(g.node_nargs[v]), S, int(phase[v]) if phase is not None else 0, e1 - e0])]
    po, pl = int(g.node_prog_off[v]), int(g.node_prog_len[v])
    out.append((1, [int(x) for x in g.prog[po:po + pl]] if pl else []))
    ol = int(g.node_out_list[v])
    out.append((2, [int(x) for x in g.lists[ol:ol + S]]))
    if op == 2:
        b = int(g.node_comp_off[v])
        out.append((3, [int(x) for x in g.explicit_flops[b:b + S]]))
        out.append((4, [int(x) for x in g.explicit_bytes[b:b + S]]))
    for e in range(e0, e1):
        sec = 16 + 4 * (e - e0)
        ssrc, sdst = int(g.edge_ssrc[e]), int(g.edge_sdst[e])
        d_off = int(g.edge_default_off[e])
        out.append((sec, [ssrc, sdst, int(g.edge_flags[e]) & 3, int(d_off >= 0)]))
        dl = int(g.edge_dst_list[e])
        out.append((sec + 1, [int(x) for x in g.lists[dl:dl + sdst]]))
        if int(g.edge_src_node[e]) >= 0:
            sl = int(g.edge_src_list[e])
            out.append((sec + 2, [int(x) for x in g.lists[sl:sl + ssrc]]))
        if d_off >= 0:
            vals = g.default_vals[d_off:d_off + ssrc * sdst]
            out.append((sec + 3, [struct.unpack("<q", struct.pack("<d", float(x)))[0] for x in vals]))
    return out


def node_key(g, v: int, phase: Optional[Sequence[int]] = None) -> tuple:
    return tuple((sec, tuple(words)) for sec, words in _sections(g, v, phase) if words)


def node_hash(g, v: int, phase: Optional[Sequence[int]] = None) -> int:
    acc = 0
    for sec, words in _sections(g, v, phase):
        for i, w in enumerate(words):
            acc = (acc + term(sec, i, w)) & M64
    return mix64(acc)


def node_hashes(g, phase: Optional[Sequence[int]] = None) -> List[int]:
    return [node_hash(g, v, phase) for v in range(g.num_nodes)]
