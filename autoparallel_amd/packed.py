"""Packed structure-of-arrays form of a sharding-search problem.

This is the data format on both sides of the cost engine: the HIP kernels read
it from HBM, the host builds it from ``{node: OpStrategy}`` (or directly from
a shape-level generator).  It flattens what the reference keeps as Python
objects:

* ``DTensorSpec.placements``          -> a row of the interned placement-tuple
                                         table (``tuple_plc``, one byte per mesh dim)
* ``DTensorSpec.tensor_meta``         -> a row of the tensor-meta table
* a ``DTensorSpec``                   -> one 32-bit word ``meta_id << 12 | tuple_id``
                                         (``SPEC_NONE`` where the reference has ``None``)
* ``OpSpec.input_specs / output_specs`` -> runs of spec words in ``lists``
* ``strats[node]`` / ``_all_input_nodes(node)[argi]`` -> the edge table
  (reference: autoparallel/optimize_sharding.py:306-354, 380-398, 481-552)

Placement byte (equality of bytes == Python equality of placements, which is
what the reference's ``current == target`` test needs,
autoparallel/cost_models/collective_runtime_estimation.py:157):

    0x00          Replicate
    0x40 | dim    Shard(dim)                 dim < 64
    0x80 | id     Partial; id 0 = "sum" (the default ``Partial()``), 1 = "avg",
                  2 = "min", 3 = "max", 4 = "product", >= 8 interned others
    0xC0 | id     any other placement class (is_shard/is_replicate/is_partial
                  all False, e.g. _StridedShard)

Entry layout: edge e owns ``sdst[e] * ssrc[e]`` consecutive slots starting at
``edge_off[e]``, row-major ``[out_idx][inp_idx]``; edges are ordered by
(node, argi), the order of the reference's ``walk_over_options``
(optimize_sharding.py:400-410).  Every block starts on a multiple of 16 slots
(aligned vector stores, exact 16-slot edge index), so the entry arrays have
``num_slots >= num_entries`` elements; ``entry_slots()`` lists the real ones and
``decision_var_order`` permutes them to the ``decision_vars`` dict order (node,
out_idx, argi, inp_idx; :511-520).
"""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

MAX_MESH_DIMS = 4
MAX_RANK = 8
TUPLE_BITS = 12
MAX_TUPLES = 1 << TUPLE_BITS
MAX_METAS = 1 << (32 - TUPLE_BITS)
SPEC_NONE = 0xFFFFFFFF
CHUNK_SHIFT = 4  # edge blocks start on multiples of 1 << CHUNK_SHIFT slots
ITEM_ENTRIES = 256  # entries of one edge per work item of the entry kernel
# A block table is built when it is at most this many times the entry count (and
# small in absolute terms); otherwise every entry is evaluated directly.
TABLE_MAX_RATIO = 0.5
TABLE_MAX_DOUBLES = 1 << 28
WIDE_ITEMS_FROM = 32_000_000  # entries: from here on work items of 512 entries and, if smaller, the compressed table


def spec_word(meta_id: int, tuple_id: int) -> int:
    return (int(meta_id) << TUPLE_BITS) | int(tuple_id)

# ---- placement codes -------------------------------------------------------
PLC_R = 0x00
PLC_SHARD = 0x40
PLC_PARTIAL = 0x80
PLC_OTHER = 0xC0
PLC_KIND_MASK = 0xC0
PLC_ARG_MASK = 0x3F

PARTIAL_SUM = PLC_PARTIAL | 0
PARTIAL_AVG = PLC_PARTIAL | 1
_REDUCE_OP_IDS = {"sum": 0, "avg": 1, "min": 2, "max": 3, "product": 4}


def shard(dim: int) -> int:
    assert 0 <= dim < 64
    return PLC_SHARD | dim


def partial(reduce_op: str = "sum") -> int:
    return PLC_PARTIAL | _REDUCE_OP_IDS[reduce_op]


def is_shard(code: int) -> bool:
    return (code & PLC_KIND_MASK) == PLC_SHARD


def is_partial(code: int) -> bool:
    return (code & PLC_KIND_MASK) == PLC_PARTIAL


def is_replicate(code: int) -> bool:
    return code == PLC_R


def plc_str(code: int) -> str:
    if code == PLC_R:
        return "R"
    if is_shard(code):
        return f"S({code & PLC_ARG_MASK})"
    if is_partial(code):
        names = {v: k for k, v in _REDUCE_OP_IDS.items()}
        return f"P({names.get(code & PLC_ARG_MASK, code & PLC_ARG_MASK)})"
    return f"X({code & PLC_ARG_MASK})"


# ---- dtype codes -----------------------------------------------------------
# Codes 0..4 are the dtypes the reference's device table prices GEMMs in
# (autoparallel/cost_models/compute_estimation.py:226-239); anything else has
# no tflops entry and is only legal on zero-flop nodes.
DT_F64, DT_F32, DT_F16, DT_BF16, DT_I8, DT_OTHER = 0, 1, 2, 3, 4, 5
DTYPE_ITEMSIZE = {DT_F64: 8, DT_F32: 4, DT_F16: 2, DT_BF16: 2, DT_I8: 1}

# ---- edge flags ------------------------------------------------------------
EDGE_HAS_PRODUCER = 1  # comm is computed from specs (else default row kept)
EDGE_SCORE_TRANSITION = 2  # producer output is a single spec: the plan scorer
#                            counts a transition (optimize_sharding.py:1097-1104)
EDGE_PREFETCHABLE = 4  # set in the device records from ``edge_prefetchable``
EDGE_COMPRESSED = 8  # device records only: the edge's matrix in the block table has one
#                      row / column per distinct spec word; its row length is in
#                      flags >> EDGE_USRC_SHIFT
EDGE_USRC_SHIFT = 8

# ---- compute programs ------------------------------------------------------
# A node's compute estimate needs flops and bytes of the op run on the sharded
# inputs (compute_estimation.py:438-493).  Both are written as small programs
# over the local (sharded) sizes of the tensor args:
#   flops  = sum_t coeff_t * prod_j size(arg a_tj, dim d_tj)
#   out[k] = shape whose dims are each: a constant, size(arg, dim), the
#            broadcast of all tensor args at a right-aligned position, or the
#            whole element count of an argument
OP_ZERO = 0  # placeholder / get_attr / view / non-OpOverload: cost is int 0
OP_PROGRAM = 1  # flops and output shapes from the program
OP_EXPLICIT = 2  # host supplies flops[o], bytes[o] (ops without a closed form)

DIM_CONST = 0  # value
DIM_ARG = 1  # (arg, dim)
DIM_BCAST = 2  # right-aligned position (0 = last dim)
DIM_ARGNUMEL = 3  # (arg): all of an argument's local sizes as one factor (an output shaped like it)


@dataclasses.dataclass
class PackedGraph:
    # mesh
    mesh_shape: np.ndarray  # int32[ndim]
    devices_per_host: int
    # tensor metas
    meta_rank: np.ndarray  # int32[M]
    meta_shape: np.ndarray  # int64[M, MAX_RANK]
    meta_stride: np.ndarray  # int64[M, MAX_RANK]
    meta_itemsize: np.ndarray  # int32[M]
    meta_dtype: np.ndarray  # int32[M]
    # interned placement tuples
    tuple_plc: np.ndarray  # uint8[NT, MAX_MESH_DIMS]
    # runs of spec words (SPEC_NONE = no DTensorSpec at that position)
    lists: np.ndarray  # uint32[L]
    # nodes
    node_nstrat: np.ndarray  # int32[N]
    node_nargs: np.ndarray  # int32[N]   len(strategies[0].input_specs)
    node_comp_off: np.ndarray  # int64[N] slot of (v, out 0) in the compute vector;
    #                            nodes with identical program and input specs share one
    n_compute: int  # length of the compute vector
    comp_nodes: np.ndarray  # int32[...] one representative node per distinct slot
    node_edge_off: np.ndarray  # int32[N+1] edges of node v, ordered by argi
    node_op: np.ndarray  # int32[N]   OP_*
    node_prog_off: np.ndarray  # int64[N]   offset into prog (-1 if none)
    node_prog_len: np.ndarray  # int32[N]   words of the node's program (0 if none)
    node_out_list: np.ndarray  # int64[N]   run of the node's (first) output spec words
    prog: np.ndarray  # int64[...] compute programs
    # explicit flops/bytes (OP_EXPLICIT), indexed like the compute vector
    explicit_flops: Optional[np.ndarray] = None  # int64[sum S]
    explicit_bytes: Optional[np.ndarray] = None  # int64[sum S]
    # edges
    edge_node: np.ndarray = None  # int32[NE] consumer
    edge_arg: np.ndarray = None  # int32[NE]
    edge_src_node: np.ndarray = None  # int32[NE] producer or -1
    edge_sdst: np.ndarray = None  # int32[NE]
    edge_ssrc: np.ndarray = None  # int32[NE]
    edge_dst_list: np.ndarray = None  # int64[NE] offset into lists (sdst words)
    edge_src_list: np.ndarray = None  # int64[NE] offset into lists (ssrc words) or -1
    edge_off: np.ndarray = None  # int64[NE+1] first slot of each block; [-1] = num_slots
    edge_flags: np.ndarray = None  # int32[NE]
    edge_default_off: np.ndarray = None  # int64[NE] offset into default_vals or -1
    default_vals: np.ndarray = None  # float64[...]
    # prefetch-discount mask per edge (producer param-derived or consumer
    # terminal-derived; optimize_sharding.py:853-860)
    edge_prefetchable: Optional[np.ndarray] = None  # uint8[NE]
    # cluster multiplicity per node: 1 + number of linked copies (:883)
    node_multiplier: Optional[np.ndarray] = None  # int32[N]
    node_names: Optional[List[str]] = None
    roles: Optional[object] = None  # sharding_problem.GraphRoles (fwd/bwd pairs, cast chains)
    # clustering inputs: 1 for placeholders (never clustered), and the
    # forward (0) / backward (1) tag regions must not cross
    node_kind: Optional[np.ndarray] = None  # uint8[N]
    node_phase: Optional[np.ndarray] = None  # int32[N]
    # optional id per node of whatever else must agree before two nodes may be
    # duplicates of each other (the packer of a traced graph sets it from the
    # operator's name, source position and arguments); hashed in place of the tag
    node_cluster_key: Optional[np.ndarray] = None  # int32[N]
    # runs of every output of a tuple-valued node (column k: output k, -1 past the
    # node's outputs); column 0 is node_out_list
    node_out_runs: Optional[np.ndarray] = None  # int64[N, max outputs]
    # Repeated subgraphs: edge_alias[e] is the edge whose entry block stands for e
    # (e itself for an edge that owns one).  An aliased edge owns no slots: its
    # edge_off is its alias's, and only owning ("priced") edges count in
    # num_entries, entry_slots, entry_keys and the work items.  None: every edge
    # owns its block.  Set through with_edge_alias().
    edge_alias: Optional[np.ndarray] = None  # int64[NE]

    # -- derived sizes -------------------------------------------------------
    @property
    def ndim(self) -> int:
        return int(self.mesh_shape.shape[0])

    @property
    def num_nodes(self) -> int:
        return int(self.node_nstrat.shape[0])

    @property
    def num_edges(self) -> int:
        return int(self.edge_node.shape[0])

    @property
    def priced(self) -> np.ndarray:
        """bool[NE]: the edge owns an entry block (is not an alias of another)."""
        if self.edge_alias is None:
            return np.ones(self.num_edges, bool)
        return self.edge_alias == np.arange(self.num_edges)

    def block_sizes(self) -> np.ndarray:
        """int64[NE]: entries of each edge's own block (0 for an aliased edge)."""
        sizes = self.edge_sdst.astype(np.int64) * self.edge_ssrc
        return sizes if self.edge_alias is None else np.where(self.priced, sizes, 0)

    @property
    def num_entries(self) -> int:
        """Real entries (decision variables): those of the edges that own a block."""
        return int(self.block_sizes().sum())

    def with_edge_alias(self, alias: np.ndarray) -> "PackedGraph":
        """The same graph with the entry blocks of aliased edges dropped: edge e
        reads the block of edge alias[e], which must have the same strategies on
        both sides (same spec words, same default rows).  Blocks of the owning
        edges are laid out compactly, in edge order."""
        NE = self.num_edges
        alias = np.asarray(alias, np.int64)
        assert alias.shape == (NE,) and (alias[alias] == alias).all(), "an alias must own its block"
        own = alias == np.arange(NE)
        sizes = self.edge_sdst.astype(np.int64) * self.edge_ssrc
        a = alias[~own]
        e = np.nonzero(~own)[0]
        assert (self.edge_sdst[e] == self.edge_sdst[a]).all() and (self.edge_ssrc[e] == self.edge_ssrc[a]).all()
        assert ((self.edge_flags[e] & EDGE_HAS_PRODUCER) == (self.edge_flags[a] & EDGE_HAS_PRODUCER)).all()
        for x, y in zip(e, a):  # same words on both sides, same default rows
            n_d, n_s = int(self.edge_sdst[x]), int(self.edge_ssrc[x])
            if self.edge_dst_list[x] != self.edge_dst_list[y]:
                assert np.array_equal(self.lists[self.edge_dst_list[x]:self.edge_dst_list[x] + n_d],
                                      self.lists[self.edge_dst_list[y]:self.edge_dst_list[y] + n_d])
            if self.edge_src_list[x] != self.edge_src_list[y]:
                assert self.edge_src_list[x] >= 0 and self.edge_src_list[y] >= 0
                assert np.array_equal(self.lists[self.edge_src_list[x]:self.edge_src_list[x] + n_s],
                                      self.lists[self.edge_src_list[y]:self.edge_src_list[y] + n_s])
            dx, dy = int(self.edge_default_off[x]), int(self.edge_default_off[y])
            assert (dx < 0) == (dy < 0)
            if dx >= 0:
                assert np.array_equal(self.default_vals[dx:dx + n_d * n_s], self.default_vals[dy:dy + n_d * n_s])
        pad = (1 << CHUNK_SHIFT) - 1
        padded = np.where(own, (sizes + pad) & ~pad, 0)
        edge_off = np.zeros(NE + 1, np.int64)
        np.cumsum(padded, out=edge_off[1:])
        total = int(edge_off[-1])
        edge_off[:-1][~own] = edge_off[:-1][a]
        edge_off[-1] = total
        return dataclasses.replace(self, edge_off=edge_off, edge_alias=alias)

    @property
    def num_slots(self) -> int:
        """Length of the entry arrays, padding included."""
        return int(self.edge_off[-1])

    def entry_slots(self) -> np.ndarray:
        """int64[E]: slot of every real entry, in (edge, out_idx, inp_idx) order."""
        sizes = self.block_sizes()
        eid = np.repeat(np.arange(self.num_edges, dtype=np.int64), sizes)
        start = np.concatenate([[0], np.cumsum(sizes)[:-1]])
        local = np.arange(int(sizes.sum()), dtype=np.int64) - start[eid]
        return self.edge_off[:-1][eid] + local

    @property
    def num_compute(self) -> int:
        return int(self.n_compute)

    def entry_keys(self) -> np.ndarray:
        """int32[E, 4] keys (node_idx, argi, out_idx, inp_idx) in entry order
        (the key layout of autoparallel/serialization.py:150-157)."""
        E = self.num_entries
        sizes = self.block_sizes()
        eid = np.repeat(np.arange(self.num_edges, dtype=np.int64), sizes)
        start = np.concatenate([[0], np.cumsum(sizes)[:-1]])
        local = np.arange(E, dtype=np.int64) - start[eid]
        ssrc = self.edge_ssrc[eid].astype(np.int64)
        keys = np.empty((E, 4), dtype=np.int32)
        keys[:, 0] = self.edge_node[eid]
        keys[:, 1] = self.edge_arg[eid]
        keys[:, 2] = local // ssrc
        keys[:, 3] = local % ssrc
        return keys

    def decision_var_order(self) -> np.ndarray:
        """Permutation p such that entries[p] is in the reference's
        ``decision_vars`` insertion order: node, out_idx, argi, inp_idx
        (optimize_sharding.py:511-520)."""
        # Without sorting: the order visits, per node and per out_idx, the row of every argument's
        # block in turn, and a row is S_src consecutive entries.  Runs = (node, out_idx, arg).
        sizes = self.block_sizes()
        entry_start = np.concatenate([[0], np.cumsum(sizes)[:-1]]) if self.num_edges else np.zeros(0, np.int64)
        own = np.nonzero(sizes > 0)[0]  # edges that own a block, in (node, arg) order
        if own.size == 0:
            return np.zeros(0, np.int64)
        node = self.edge_node[own].astype(np.int64)
        S = self.edge_sdst[own].astype(np.int64)           # rows of the block = strategies of its node
        ssrc = self.edge_ssrc[own].astype(np.int64)
        # position of each owning edge among its node's owning edges, and how many the node has
        first_of_node = np.ones(own.size, bool)
        first_of_node[1:] = node[1:] != node[:-1]
        group = np.cumsum(first_of_node) - 1
        group_start = np.nonzero(first_of_node)[0]
        n_args = np.diff(np.append(group_start, own.size))
        rank = np.arange(own.size) - group_start[group]
        # runs in order: for each node group, for o in range(S), for each of its edges
        runs_per_group = S[group_start] * n_args
        run_group = np.repeat(np.arange(group_start.size), runs_per_group)
        within = np.arange(int(runs_per_group.sum())) - np.repeat(np.cumsum(runs_per_group) - runs_per_group, runs_per_group)
        o = within // n_args[run_group]
        edge = group_start[run_group] + within % n_args[run_group]  # index into `own`
        start = entry_start[own[edge]] + o * ssrc[edge]
        count = ssrc[edge]
        total = int(count.sum())
        return np.repeat(start - (np.cumsum(count) - count), count) + np.arange(total, dtype=np.int64)

    def export_rows(self):
        """(row_base int64[n_edge], row_stride int32[n_edge]): the row of entry
        (e, out_idx, inp_idx) in ``decision_vars`` insertion order is
        ``row_base[e] + out_idx * row_stride[e] + inp_idx``."""
        ssrc = np.where(self.priced, self.edge_ssrc, 0).astype(np.int64)  # an aliased edge has no rows
        node = self.edge_node.astype(np.int64)
        per_node = np.zeros(self.num_nodes, np.int64)  # sum of S_src over the node's arguments
        np.add.at(per_node, node, ssrc)
        node_rows = per_node * self.node_nstrat.astype(np.int64)
        node_base = np.concatenate([[0], np.cumsum(node_rows)[:-1]]) if self.num_nodes else np.zeros(0, np.int64)
        first = self.node_edge_off[:-1].astype(np.int64)[node]  # first edge of e's node
        csum = np.concatenate([[0], np.cumsum(ssrc)])
        before = csum[np.arange(self.num_edges)] - csum[first]  # S_src of the node's earlier arguments
        return (node_base[node] + before).astype(np.int64), per_node[node].astype(np.int32)

    # -- device-side views ----------------------------------------------------
    EDGE_DTYPE = np.dtype(
        [
            ("off", "<i8"),
            ("default_off", "<i8"),
            ("src_list", "<u4"),
            ("dst_list", "<u4"),
            ("ssrc", "<i4"),
            ("sdst", "<i4"),
            ("comp_base", "<i4"),
            ("flags", "<i4"),
            ("node", "<i4"),
            ("src_node", "<i4"),
            ("table_off", "<i8"),
            ("magic", "<u4"),
            ("local0", "<u4"),
        ]
    )

    def edge_records(self, compressed: bool = False) -> np.ndarray:
        """Edges as 64-byte records (the ``apc_edge`` struct of include/apc.h).
        ``compressed``: records for the compressed block table (``table_off``
        of that layout; EDGE_COMPRESSED and the matrix's row length in
        ``flags`` for the edges whose matrix is stored by distinct spec word)."""
        cache = self.__dict__.setdefault("_edge_records", {})  # made once per layout, like the block table
        if compressed in cache:
            return cache[compressed]
        NE = self.num_edges
        rec = np.zeros(NE, self.EDGE_DTYPE)
        assert rec.dtype.itemsize == 64
        rec["table_off"] = self.block_table(compressed)[3]
        # division by ssrc as a multiply-high (exact while local * ssrc < 2**32)
        ssrc = self.edge_ssrc.astype(np.int64)
        ok = (ssrc > 1) & (ssrc * ssrc * self.edge_sdst < 2**32)
        rec["magic"] = np.where(ok, (2**32) // np.maximum(ssrc, 1) + 1, 0).astype(np.uint32)
        rec["off"] = self.edge_off[:-1]
        rec["default_off"] = self.edge_default_off
        rec["src_list"] = np.where(self.edge_src_list >= 0, self.edge_src_list, 0).astype(np.uint32)
        rec["dst_list"] = self.edge_dst_list.astype(np.uint32)
        rec["ssrc"] = self.edge_ssrc
        rec["sdst"] = self.edge_sdst
        rec["comp_base"] = self.node_comp_off[self.edge_node].astype(np.int32)
        flags = self.edge_flags.astype(np.int32).copy()
        if self.edge_prefetchable is not None:
            flags |= (self.edge_prefetchable.astype(np.int32) != 0) * EDGE_PREFETCHABLE
        if compressed:
            usrc = self.block_table(True)[4]
            flags |= np.where(usrc > 0, EDGE_COMPRESSED | (usrc << EDGE_USRC_SHIFT), 0).astype(np.int32)
        rec["flags"] = flags
        rec["node"] = self.edge_node
        rec["src_node"] = self.edge_src_node
        cache[compressed] = rec
        return rec

    REC_ARGS = 14
    COMP_REC_DTYPE = np.dtype([
        ("node", "<i4"), ("nstrat", "<i4"), ("nargs", "<i4"), ("op", "<i4"), ("comp_off", "<i8"),
        ("prog_off", "<i8"), ("prog_len", "<i4"), ("n_edge", "<i4"), ("dst_list", "<u4", (14,)),
        ("term_off", "<i4"), ("n_term", "<i4"), ("term_flags", "<i4"), ("arg_meta", "<u2", (16,)),
        ("reserved", "<i4", (5,)),
    ])
    PROG_TERM_DTYPE = np.dtype([("coeff", "<i8"), ("idx", "u1", (7,)), ("to_bytes", "u1")])
    SPEC_REC_DTYPE = np.dtype([("word", "<u4"), ("plc", "<u4"), ("nbytes2", "<i8")])
    TABLE_UNIT_DTYPE = np.dtype([
        ("default_off", "<i8"), ("src_list", "<u4"), ("dst_list", "<u4"), ("ncol", "<u4"), ("nrow", "<u4"),
        ("first", "<u4"), ("flags", "<u4"),
    ])
    TERMS_BCAST = 1
    TERMS_MAX = 64

    def comp_records(self) -> np.ndarray:
        """One 160-byte record per evaluated node (``apc_comp_rec`` of
        include/apc.h): what the node kernel reads about the node, gathered,
        and where its program stands as product terms (``program_terms``)."""
        v = self.comp_nodes.astype(np.int64)
        rec = np.zeros(v.shape[0], self.COMP_REC_DTYPE)
        assert rec.dtype.itemsize == 160
        rec["arg_meta"] = 0xFFFF
        e0 = self.node_edge_off[:-1].astype(np.int64)[v]
        n_edge = (self.node_edge_off[1:].astype(np.int64)[v] - e0)
        rec["node"], rec["nstrat"], rec["nargs"] = v, self.node_nstrat[v], self.node_nargs[v]
        rec["op"], rec["comp_off"] = self.node_op[v], self.node_comp_off[v]
        rec["prog_off"], rec["prog_len"], rec["n_edge"] = self.node_prog_off[v], self.node_prog_len[v], n_edge
        for a in range(self.REC_ARGS):
            has = n_edge > a
            rec["dst_list"][has, a] = self.edge_dst_list[(e0 + a)[has]].astype(np.uint32)
            # meta of the argument's first spec, if it has one and it fits the field
            first = self.lists[self.edge_dst_list[(e0 + a)[has]]].astype(np.int64)
            mid = first >> TUPLE_BITS
            rec["arg_meta"][np.nonzero(has)[0], a] = np.where((first != SPEC_NONE) & (mid < 0xFFFF), mid, 0xFFFF)
        _, where = self.program_terms()
        R = self.max_rank
        # a node with more arguments than rows of the value table can name keeps the interpreter
        as_terms = (self.node_op[v] == OP_PROGRAM) & (n_edge <= self.REC_ARGS) & (R + n_edge * (R + 2) <= 0xFF)
        prog_off = self.node_prog_off[v]
        for i in np.nonzero(as_terms)[0].tolist():
            hit = where.get(int(prog_off[i]))
            if hit is not None:
                rec["term_off"][i], rec["n_term"][i], rec["term_flags"][i] = hit
        return rec

    def program_terms(self):
        """Every distinct compute program as product terms (``apc_prog_term`` of
        include/apc.h).  Returns (terms, where): ``where[prog_off] = (term_off,
        n_term, flags)`` for the programs that have this form; one with a term
        of more than 7 factors or more than TERMS_MAX terms has none and is
        interpreted word by word."""
        cached = self.__dict__.get("_program_terms")
        if cached is not None:
            return cached
        R = self.max_rank
        slots = R + 2
        out: List[tuple] = []
        where: Dict[int, Tuple[int, int, int]] = {}
        has_prog = self.node_op == OP_PROGRAM
        if has_prog.any():
            offs, at = np.unique(self.node_prog_off[has_prog], return_index=True)
            lens = dict(zip(offs.tolist(), self.node_prog_len[has_prog][at].tolist()))
        else:
            offs, lens = np.zeros(0, np.int64), {}
        for off in offs:
            off = int(off)
            pr = [int(x) for x in self.prog[off:off + lens[off]]]
            terms, flags, ok = [], 0, True
            q = 2
            for _ in range(pr[0]):
                coeff, nfac = pr[q], pr[q + 1]
                q += 2
                idx = []
                for _ in range(nfac):
                    a, d = pr[q], pr[q + 1]
                    q += 2
                    if d < R:  # no tensor of the graph has that dim otherwise: its size is 1
                        idx.append(R + a * slots + d)
                terms.append((coeff, idx, 0))
            for _ in range(pr[1]):
                coeff, rank = pr[q], pr[q + 1]
                q += 2
                idx = []
                for _ in range(rank):
                    kind, x, y = pr[q], pr[q + 1], pr[q + 2]
                    q += 3
                    if kind == DIM_CONST:
                        coeff *= x
                    elif kind == DIM_ARG:
                        if y < R:
                            idx.append(R + x * slots + y)
                    elif kind == DIM_ARGNUMEL:
                        idx.append(R + x * slots + R + 1)
                    else:  # DIM_BCAST: no tensor reaches a position past the largest rank
                        if x < R:
                            idx.append(x)
                            flags |= self.TERMS_BCAST
                terms.append((coeff, idx, 1))
            assert q == len(pr)
            if len(terms) > self.TERMS_MAX or any(len(t[1]) > 7 or max(t[1], default=0) > 0xFE for t in terms):
                ok = False
            if not (-(2**63) <= min((t[0] for t in terms), default=0) and max((t[0] for t in terms), default=0) < 2**63):
                ok = False
            if ok and terms:
                where[off] = (len(out), len(terms), flags)
                out.extend(terms)
        arr = np.zeros(len(out), self.PROG_TERM_DTYPE)
        assert arr.dtype.itemsize == 16
        for i, (coeff, idx, to_bytes) in enumerate(out):
            arr["coeff"][i] = coeff
            arr["idx"][i] = idx + [0xFF] * (7 - len(idx))
            arr["to_bytes"][i] = to_bytes
        object.__setattr__(self, "_program_terms", (arr, where))
        return arr, where

    def meta_bytes_contiguous(self):
        """(nbytes int64[M], contiguous bool[M]) per tensor meta: itemsize *
        prod(shape), and whether its strides are those of a contiguous tensor
        (torch ``check_contiguous_sizes_strides``,
        _prims_common/__init__.py:252-293: dims of size 1 are skipped, the others
        must have the running product of the sizes to their right as stride)."""
        M = self.meta_rank.shape[0]
        nbytes = self.meta_itemsize.astype(np.int64).copy()
        expected = np.ones(M, np.int64)
        expected_max = np.ones(M, np.int64)
        ok = np.ones(M, bool)
        with np.errstate(over="ignore"):
            for d in range(MAX_RANK - 1, -1, -1):
                live = d < self.meta_rank
                x, y = self.meta_shape[:, d], self.meta_stride[:, d]
                nbytes = np.where(live, nbytes * x, nbytes)
                check = live & (x != 1)
                ok &= ~(check & (y != expected) & (y != expected_max))
                expected_max = np.where(check, expected_max * np.maximum(x, 1), expected_max)
                expected = np.where(check, expected * x, expected)
        return nbytes, ok

    def spec_records(self) -> np.ndarray:
        """One ``apc_spec_rec`` per position of ``lists``: the spec word, its
        placement bytes and its tensor's byte count and contiguity."""
        L = self.lists.shape[0]
        rec = np.zeros(L, self.SPEC_REC_DTYPE)
        assert rec.dtype.itemsize == 16
        rec["word"] = self.lists
        if L == 0:
            return rec
        none = self.lists == SPEC_NONE
        any_none = bool(none.any())
        w = self.lists.astype(np.int64)
        if any_none:
            w[none] = 0
        plc = np.ascontiguousarray(self.tuple_plc).view("<u4").reshape(-1)
        nbytes, contig = self.meta_bytes_contiguous()
        per_meta = (nbytes << 1) | contig  # whole-array gathers: masked ones cost three times as much
        rec["plc"] = plc[w & (MAX_TUPLES - 1)] if plc.shape[0] else 0
        rec["nbytes2"] = per_meta[w >> TUPLE_BITS] if per_meta.shape[0] else 0
        if any_none:
            rec["plc"][none] = 0
            rec["nbytes2"][none] = 0
        return rec

    LUT_TILE_DTYPE = np.dtype([
        ("out", "<i8"), ("default_off", "<i8"), ("src_list", "<u4"), ("dst_list", "<u4"), ("ncol", "<u4"),
        ("nrow", "<u4"), ("col0", "<u4"), ("ncols", "<u4"), ("row0", "<u4"), ("nrows", "<u4"), ("flags", "<u4"),
        ("comp_base", "<i4"), ("magic", "<u4"), ("reserved", "<u4"),
    ])
    LUT_COLS = 64
    LUT_ROWS = 1024
    LUT_TILE_ELEMENTS = 16384

    def lut_tiles(self, compressed: bool = False, entries: bool = False) -> np.ndarray:
        """Tiles (``apc_lut_tile`` of include/apc.h) for the lookup-table kernels:
        of every matrix of the block table (``entries=False``; ``compressed`` as
        for block_table), or of every edge block that owns entries
        (``entries=True``: direct evaluation, edges without a producer included).
        A tile has at most LUT_COLS source columns and LUT_ROWS target rows, and
        about LUT_TILE_ELEMENTS elements, more when there is work for more than a
        few thousand tiles."""
        if entries:
            e = np.nonzero(self.priced & (self.block_sizes() > 0))[0].astype(np.int64)
            ncol, nrow = self.edge_ssrc[e].astype(np.int64), self.edge_sdst[e].astype(np.int64)
            out = self.edge_off[:-1][e]
            flags = (self.edge_flags[e] & EDGE_HAS_PRODUCER).astype(np.int64)
            comp_base = self.node_comp_off[self.edge_node[e]].astype(np.int64)
        else:
            block_edge, block_off, _, _, edge_usrc, block_udst = self.block_table(compressed)
            e = block_edge.astype(np.int64)
            squeezed = edge_usrc[e] > 0
            ncol = np.where(squeezed, edge_usrc[e], self.edge_ssrc[e]).astype(np.int64)
            nrow = np.where(squeezed, block_udst, self.edge_sdst[e]).astype(np.int64)
            out = block_off[:-1]
            flags = EDGE_HAS_PRODUCER | np.where(squeezed, EDGE_COMPRESSED, 0).astype(np.int64)
            comp_base = np.full(e.shape[0], -1, np.int64)
        n_ct = (ncol + self.LUT_COLS - 1) // self.LUT_COLS
        # a tile's lookup tables are made once per tile: tiles as tall as the work allows
        # while there are still a few thousand of them to spread over the chip
        total = int((ncol * nrow).sum())
        tile_elements = int(min(self.LUT_COLS * self.LUT_ROWS, max(self.LUT_TILE_ELEMENTS, total // 3072)))
        rows_per = np.minimum(np.minimum(nrow, self.LUT_ROWS),
                              np.maximum(1, tile_elements // np.minimum(ncol, self.LUT_COLS)))
        n_rt = (nrow + rows_per - 1) // np.maximum(rows_per, 1)
        per = n_ct * n_rt
        k = np.repeat(np.arange(e.shape[0], dtype=np.int64), per)
        start = np.concatenate([[0], np.cumsum(per)[:-1]]) if e.shape[0] else np.zeros(0, np.int64)
        local = np.arange(int(per.sum()), dtype=np.int64) - start[k]
        ct, rt = local % n_ct[k], local // n_ct[k]
        rec = np.zeros(k.shape[0], self.LUT_TILE_DTYPE)
        assert rec.dtype.itemsize == 64
        rec["out"], rec["default_off"] = out[k], self.edge_default_off[e[k]]
        rec["src_list"] = np.maximum(self.edge_src_list[e[k]], 0).astype(np.uint32)
        rec["dst_list"] = self.edge_dst_list[e[k]].astype(np.uint32)
        rec["ncol"], rec["nrow"] = ncol[k], nrow[k]
        rec["col0"] = ct * self.LUT_COLS
        rec["ncols"] = np.minimum(self.LUT_COLS, ncol[k] - ct * self.LUT_COLS)
        rec["row0"] = rt * rows_per[k]
        rec["nrows"] = np.minimum(rows_per[k], nrow[k] - rt * rows_per[k])
        rec["flags"], rec["comp_base"] = flags[k], comp_base[k]
        nc = rec["ncols"].astype(np.int64)
        rec["magic"] = np.where(nc > 1, (2**32) // np.maximum(nc, 1) + 1, 0)  # one column: the row is the index
        assert (rec["nrows"].astype(np.int64) * rec["ncols"] < 2**20).all() and (rec["nrows"] <= self.LUT_ROWS).all()
        return rec

    def table_unit_records(self, compressed: bool = False) -> np.ndarray:
        """One ``apc_table_unit`` per 256 elements of the block table: the two
        runs, the matrix extent and the unit's first element, so that a
        workgroup of the table build starts from one load."""
        block_edge, block_off, unit_block, _, edge_usrc, block_udst = self.block_table(compressed)
        rec = np.zeros(unit_block.shape[0], self.TABLE_UNIT_DTYPE)
        assert rec.dtype.itemsize == 32
        if unit_block.shape[0] == 0:
            return rec
        e = block_edge[unit_block].astype(np.int64)
        squeezed = edge_usrc[e] > 0
        rec["default_off"] = self.edge_default_off[e]
        rec["src_list"] = self.edge_src_list[e].astype(np.uint32)
        rec["dst_list"] = self.edge_dst_list[e].astype(np.uint32)
        rec["ncol"] = np.where(squeezed, edge_usrc[e], self.edge_ssrc[e])
        rec["nrow"] = np.where(squeezed, block_udst[unit_block], self.edge_sdst[e])
        rec["first"] = np.arange(unit_block.shape[0], dtype=np.int64) * 256 - block_off[:-1][unit_block]
        rec["flags"] = np.where(squeezed, EDGE_COMPRESSED, 0)
        return rec

    @property
    def max_node_args(self) -> int:
        return int(np.diff(self.node_edge_off).max()) if self.num_nodes else 0

    @property
    def max_rank(self) -> int:
        return int(self.meta_rank.max()) if self.meta_rank.shape[0] else 0

    def run_unique_index(self):
        """Distinct spec words of every run an edge names (producer runs and
        consumer runs).  Returns (uidx int32[L], ufirst int32[L], nuniq
        int32[L]): ``uidx[p]`` is the rank of ``lists[p]`` among the distinct
        words of its run, ``ufirst[run + k]`` the position inside the run of an
        occurrence of the run's k-th distinct word, ``nuniq[run]`` their number
        (at the run's first position).  None if two runs of different extent
        overlap: a position then has no single rank."""
        cached = getattr(self, "_run_unique", False)
        if cached is not False:
            return cached
        L = self.lists.shape[0]
        hp = (self.edge_flags & EDGE_HAS_PRODUCER) != 0
        runs = np.concatenate([
            np.stack([self.edge_src_list[hp].astype(np.int64), self.edge_ssrc[hp].astype(np.int64)], 1),
            np.stack([self.edge_dst_list.astype(np.int64), self.edge_sdst.astype(np.int64)], 1)])
        runs = np.unique(runs, axis=0)  # sorted by offset, then length
        off, ln = runs[:, 0], runs[:, 1]
        out = None
        if runs.shape[0] == 0 or (off[:-1] + ln[:-1] <= off[1:]).all():
            rid = np.repeat(np.arange(runs.shape[0], dtype=np.int64), ln)
            start = np.concatenate([[0], np.cumsum(ln)[:-1]]) if runs.shape[0] else np.zeros(0, np.int64)
            pos = off[rid] + (np.arange(int(ln.sum()), dtype=np.int64) - start[rid])
            words = self.lists[pos].astype(np.int64)
            # by run, then word, then position: positions already ascend within a run, so a
            # stable sort on (run, word) in one 64-bit key does it (words are 32-bit)
            order = np.argsort((rid << 32) | (words & 0xFFFFFFFF), kind="stable")
            rs, ws, ps = rid[order], words[order], pos[order]
            new = np.ones(rs.shape[0], bool)
            new[1:] = (rs[1:] != rs[:-1]) | (ws[1:] != ws[:-1])
            gid = np.cumsum(new) - 1
            run_first = np.zeros(runs.shape[0], np.int64)
            first_of_run = np.ones(rs.shape[0], bool)
            first_of_run[1:] = rs[1:] != rs[:-1]
            run_first[rs[first_of_run]] = gid[first_of_run]
            rank = gid - run_first[rs]
            uidx = np.zeros(L, np.int32)
            uidx[ps] = rank
            ufirst = np.zeros(L, np.int32)
            ufirst[off[rs[new]] + rank[new]] = ps[new] - off[rs[new]]
            nuniq = np.zeros(L, np.int32)
            last_of_run = np.ones(rs.shape[0], bool)  # ranks ascend within a run: its last one is the largest
            last_of_run[:-1] = rs[1:] != rs[:-1]
            nuniq[off[rs[last_of_run]]] = (rank[last_of_run] + 1).astype(np.int32)
            out = (uidx, ufirst, nuniq)
        object.__setattr__(self, "_run_unique", out)
        return out

    def block_table(self, compressed: bool = False):
        """Layout of the block table: one S_dst x S_src cost matrix per distinct
        (producer run, consumer run) pair among the edges that have a producer
        and no missing spec on either side (runs are identified by their offset
        in ``lists``: identical runs are stored once), and a matrix of its own
        for every edge with a producer and a missing spec.  Every matrix is
        padded to a multiple of 256 elements so that a 256-thread block of the
        table kernel works on one matrix.  Edges without a producer need no
        matrix: their costs are their rows of ``default_vals``, already in
        entry order.

        ``compressed``: the matrices of the first kind keep one row per distinct
        consumer spec word and one column per distinct producer spec word of
        their runs (``run_unique_index``); strategies that differ elsewhere
        (other arguments, other outputs) repeat spec words, and the cost depends
        on the two words only.

        Returns (block_edge int32[B] one edge per matrix, block_off int64[B+1],
        unit_block int32[table_size / 256], edge_table_off int64[NE] (-1 for
        edges without a producer and for empty edges), edge_usrc int32[NE] row
        length of the edge's compressed matrix (0: not compressed), block_udst
        int32[B] rows of every matrix)."""
        cache = self.__dict__.setdefault("_block_tables", {})
        if compressed in cache:
            return cache[compressed]
        NE = self.num_edges
        edge_table_off = np.full(NE, -1, np.int64)
        edge_usrc = np.zeros(NE, np.int32)
        none_before = np.concatenate([[0], np.cumsum(self.lists == SPEC_NONE)])
        hp = (self.edge_flags & EDGE_HAS_PRODUCER) != 0
        src = np.where(hp, self.edge_src_list, 0).astype(np.int64)
        dst = self.edge_dst_list.astype(np.int64)
        ssrc, sdst = self.edge_ssrc.astype(np.int64), self.edge_sdst.astype(np.int64)
        has_none = (none_before[src + ssrc] - none_before[src] > 0) | (none_before[dst + sdst] - none_before[dst] > 0)
        cols, rows = ssrc.copy(), sdst.copy()
        if compressed:
            ru = self.run_unique_index()
            if ru is None:
                raise ValueError("runs of spec words overlap: no compressed block table for this graph")
            squeeze = hp & ~has_none
            cols[squeeze] = ru[2][src[squeeze]]
            rows[squeeze] = ru[2][dst[squeeze]]
            edge_usrc[squeeze] = cols[squeeze]
            assert (cols < (1 << (31 - EDGE_USRC_SHIFT))).all()
        ok = np.nonzero(hp & (ssrc * sdst > 0) & self.priced)[0]  # an aliased edge reads its alias's matrix
        if ok.shape[0] == 0:
            out = (np.zeros(0, np.int32), np.zeros(1, np.int64), np.zeros(0, np.int32), edge_table_off,
                   edge_usrc, np.zeros(0, np.int32))
        else:
            # an edge with a missing spec reads its own default rows: its key is its own index
            own = np.where(has_none[ok], ok, -1)
            # distinct (src, dst, ssrc, sdst, own) rows in lexicographic order, each named by
            # its first edge: a stable sort on three 64-bit keys (np.unique over rows sorts
            # them as structured records, twenty times slower)
            k_runs = src[ok] * (self.lists.shape[0] + 1) + dst[ok]
            k_size = (ssrc[ok] << 31) | sdst[ok]
            order = np.argsort(k_runs, kind="stable")
            kr, ks, ko = k_runs[order], k_size[order], own[order]
            new = np.ones(order.shape[0], bool)
            new[1:] = (kr[1:] != kr[:-1]) | (ks[1:] != ks[:-1]) | (ko[1:] != ko[:-1])
            if (new[1:] & (kr[1:] == kr[:-1])).any():
                # one pair of runs at two extents, or with and without rows of its own: the
                # sort on the runs alone does not group those, the full one does
                order = np.lexsort((own, k_size, k_runs))
                kr, ks, ko = k_runs[order], k_size[order], own[order]
                new[1:] = (kr[1:] != kr[:-1]) | (ks[1:] != ks[:-1]) | (ko[1:] != ko[:-1])
            first = order[new]
            inv = np.empty(order.shape[0], np.int64)
            inv[order] = np.cumsum(new) - 1
            block_edge = ok[first].astype(np.int32)
            size = cols[block_edge] * rows[block_edge]
            block_off = np.zeros(block_edge.shape[0] + 1, np.int64)
            np.cumsum((size + 255) & ~255, out=block_off[1:])
            edge_table_off[ok] = block_off[:-1][inv]
            if self.edge_alias is not None:
                edge_table_off[~self.priced] = edge_table_off[self.edge_alias[~self.priced]]
                edge_usrc[~self.priced] = edge_usrc[self.edge_alias[~self.priced]]
            unit_block = np.repeat(np.arange(block_edge.shape[0], dtype=np.int32), np.diff(block_off) // 256)
            out = (block_edge, block_off, unit_block, edge_table_off, edge_usrc, rows[block_edge].astype(np.int32))
        cache[compressed] = out
        return out

    def chunk_edge_index(self) -> np.ndarray:
        """int32[num_slots / 16]: the edge that owns each 16-slot chunk (blocks
        are 16-slot aligned, so a chunk never spans two edges)."""
        pad = (1 << CHUNK_SHIFT) - 1
        # an edge that owns a block owns ceil(size / 16) consecutive chunks, in edge order
        # (the order the blocks are laid out in); an aliased edge owns none
        chunks = (self.block_sizes() + pad) >> CHUNK_SHIFT
        out = np.repeat(np.arange(self.num_edges, dtype=np.int32), chunks)
        assert out.shape[0] == self.num_slots >> CHUNK_SHIFT
        return out

    def work_items(self, compressed: bool = False, item_entries: int = ITEM_ENTRIES) -> np.ndarray:
        """Work items of the entry kernel: copies of the edge record with ``local0``
        set, in slot order, each covering ``item_entries`` (256 or 512) slots.
        An item starts at a multiple of 64 slots of the entry arrays, so that
        every store instruction of a wave writes whole aligned 512-byte (costs)
        and 64-byte (flags) pieces; blocks start at multiples of 16 slots, so the
        first item of a block may start up to 48 slots before it: its ``local0``
        is then negative modulo 2**32, and the kernel's ``entry < size`` test
        switches those lanes off like the ones past the block's end."""
        assert item_entries in (ITEM_ENTRIES, 2 * ITEM_ENTRIES)
        cache = self.__dict__.setdefault("_work_items", {})  # as the block table: made once per layout
        if (compressed, item_entries) in cache:
            return cache[(compressed, item_entries)]
        sizes = self.block_sizes()
        lead = np.where(sizes > 0, self.edge_off[:-1] % 64, 0).astype(np.int64)
        n = (sizes + lead + item_entries - 1) // item_entries
        eid = np.repeat(np.arange(self.num_edges, dtype=np.int64), n)
        start = np.concatenate([[0], np.cumsum(n)[:-1]])
        k = np.arange(int(n.sum()), dtype=np.int64) - start[eid]
        # rows of eight 64-bit words: gathering structured records field by field is ten times slower
        words = np.take(self.edge_records(compressed).view(np.uint64).reshape(-1, 8), eid, axis=0)
        items = words.reshape(-1).view(self.EDGE_DTYPE)
        items["local0"] = ((k * item_entries - lead[eid]) & 0xFFFFFFFF).astype(np.uint32)
        cache[(compressed, item_entries)] = items
        return items

    def default_table_mode(self) -> str:
        """The block-table layout the engine uses unless told otherwise: "full",
        "compressed" (matrices by distinct spec word) or "direct" (no table)."""
        def small(t):
            return t <= TABLE_MAX_DOUBLES and t <= max(TABLE_MAX_RATIO * self.num_entries, 1 << 16)

        # the table path carries the transition flag in the sign bit of a cost and
        # reads default rows the same way: a default value with its sign bit set
        # (nothing the reference produces) is only exact on the direct path
        if bool(np.signbit(self.default_vals).any()):
            return "direct"
        if small(int(self.block_table(False)[1][-1])):
            # once the outputs stream past every cache, the smaller compressed
            # table costs less than its gathers (measured at 84 M and 418 M entries)
            big = self.num_entries >= WIDE_ITEMS_FROM and self.run_unique_index() is not None
            return "compressed" if big and self.block_table(True)[1][-1] < self.block_table(False)[1][-1] else "full"
        if self.run_unique_index() is not None and small(int(self.block_table(True)[1][-1])):
            return "compressed"
        return "direct"

    def default_item_entries(self, table_mode: str) -> int:
        """Work items of 512 entries pay off from some tens of millions of entries on."""
        return 2 * ITEM_ENTRIES if table_mode != "direct" and self.num_entries >= WIDE_ITEMS_FROM else ITEM_ENTRIES

    def warm_host_layout(self) -> None:
        """Makes, and caches on the graph, the layouts the engine would derive for
        its default choices (they travel with the graph when it is pickled): for
        graphs packed in worker processes."""
        mode = self.default_table_mode()
        if mode != "direct":
            self.block_table(mode == "compressed")
        self.work_items(mode == "compressed", self.default_item_entries(mode))

    def validate(self) -> None:
        """Host-side shape checks run before any kernel launch: every index a
        kernel dereferences must be in range.  A graph that passed is marked, and
        not checked again (its arrays are not meant to be written to)."""
        if self.__dict__.get("_validated"):
            return
        self._validate()
        object.__setattr__(self, "_validated", True)

    def _validate(self) -> None:
        nd = self.ndim
        assert 1 <= nd <= MAX_MESH_DIMS
        assert (self.mesh_shape >= 1).all()
        M = self.meta_rank.shape[0]
        assert self.meta_shape.shape == (M, MAX_RANK)
        assert self.meta_stride.shape == (M, MAX_RANK)
        assert ((self.meta_rank >= 0) & (self.meta_rank <= MAX_RANK)).all()
        if M:
            # The kernels hold a tensor's byte count in int64 (the reference in a
            # Python int), and the block table keeps the transition flag in the sign
            # of a cost: a tensor of 2**62 bytes or more would wrap and turn costs
            # negative.  (Beyond 2**53 bytes the two also round differently.)
            dims = np.where(np.arange(MAX_RANK)[None, :] < self.meta_rank[:, None], np.maximum(self.meta_shape, 1), 1)
            log2_bytes = np.log2(dims.astype(np.float64)).sum(axis=1) + np.log2(np.maximum(self.meta_itemsize, 1))
            if not (log2_bytes < 62).all():
                raise ValueError(f"tensor meta {int(np.argmax(log2_bytes))} has 2**{log2_bytes.max():.1f} bytes: "
                                 "beyond the int64 range of the cost engine")
        NT = self.tuple_plc.shape[0]
        assert self.tuple_plc.shape == (NT, MAX_MESH_DIMS) and NT <= MAX_TUPLES
        assert M <= MAX_METAS
        assert (self.tuple_plc[:, nd:] == 0).all()
        L = self.lists.shape[0]
        assert self.lists.dtype == np.uint32
        if L:
            words = np.unique(self.lists)
            words = words[words != SPEC_NONE]
            wm = (words >> TUPLE_BITS).astype(np.int64)
            wt = (words & (MAX_TUPLES - 1)).astype(np.int64)
            assert (wm < M).all() and (wt < NT).all()
            plc = self.tuple_plc[wt]
            sh = (plc & PLC_KIND_MASK) == PLC_SHARD
            dims = (plc & PLC_ARG_MASK).astype(np.int32)
            rank = self.meta_rank[wm][:, None]
            assert (~sh | (dims < rank)).all(), "Shard(dim) out of tensor rank"
        N, NE = self.num_nodes, self.num_edges
        assert self.node_comp_off.shape == (N,)
        if N:
            assert (self.node_comp_off >= 0).all()
            assert (self.node_comp_off + self.node_nstrat <= self.n_compute).all()
            # every slot is written by exactly one evaluated node
            lo = self.node_comp_off[self.comp_nodes]
            hi = lo + self.node_nstrat[self.comp_nodes]
            covered = (np.bincount(lo, minlength=self.n_compute + 1) - np.bincount(hi, minlength=self.n_compute + 1))
            assert (np.cumsum(covered)[:-1] == 1).all(), "compute slots not covered exactly once"
            assert np.isin(self.node_comp_off, self.node_comp_off[self.comp_nodes]).all()
        assert self.node_edge_off.shape == (N + 1,)
        assert int(self.node_edge_off[-1]) == NE
        assert self.edge_off.shape == (NE + 1,)
        if NE:
            assert (self.edge_sdst >= 1).all() and (self.edge_ssrc >= 1).all()
            assert (self.node_nargs >= 1).all(), "per-arg compute divides by num_args"
            sizes = self.edge_sdst.astype(np.int64) * self.edge_ssrc
            pad = (1 << CHUNK_SHIFT) - 1
            assert (self.edge_off & pad == 0).all(), "edge blocks must be 16-slot aligned"
            if self.edge_alias is None:
                assert (np.diff(self.edge_off) == ((sizes + pad) & ~pad)).all()
            else:
                own = self.priced
                assert self.edge_alias.shape == (NE,) and own[self.edge_alias].all()
                ends = np.concatenate([self.edge_off[:-1][own][1:], self.edge_off[-1:]])
                assert (ends - self.edge_off[:-1][own] == ((sizes[own] + pad) & ~pad)).all()
                assert (self.edge_off[:-1][~own] == self.edge_off[:-1][self.edge_alias[~own]]).all()
            assert (self.edge_dst_list >= 0).all()
            assert (self.edge_dst_list + self.edge_sdst <= L).all()
            hp = (self.edge_flags & EDGE_HAS_PRODUCER) != 0
            assert (self.edge_src_list[hp] >= 0).all()
            assert (self.edge_src_list[hp] + self.edge_ssrc[hp] <= L).all()
            assert (self.edge_sdst == self.node_nstrat[self.edge_node]).all()
            src = self.edge_src_node[hp]
            assert (src >= 0).all() and (src < N).all()
            assert (self.edge_ssrc[hp] == self.node_nstrat[src]).all()
            # inp_idx counts the producer's strategies on every edge that names one
            # (the scorers draw the producer's choice from ssrc)
            named = self.edge_src_node >= 0
            assert (self.edge_ssrc[named] == self.node_nstrat[self.edge_src_node[named]]).all()
            # entries whose spec is missing need a default value
            need_default = ~hp
            assert (self.edge_default_off[need_default] >= 0).all()
            d = self.edge_default_off >= 0
            assert (
                self.edge_default_off[d] + sizes[d] <= self.default_vals.shape[0]
            ).all()
            # a missing spec inside a run is only legal with a default row
            none_csum = np.concatenate([[0], np.cumsum(self.lists == SPEC_NONE)])
            nd_run = none_csum[self.edge_dst_list + self.edge_sdst] - none_csum[self.edge_dst_list]
            ns_run = np.zeros(NE, np.int64)
            ns_run[hp] = (
                none_csum[self.edge_src_list[hp] + self.edge_ssrc[hp]] - none_csum[self.edge_src_list[hp]]
            )
            assert (((nd_run == 0) & (ns_run == 0)) | d).all()
        hasp = self.node_op == OP_PROGRAM
        assert (self.node_prog_off[hasp] >= 0).all() and (self.node_prog_len[hasp] >= 2).all()
        assert (self.node_prog_off[hasp] + self.node_prog_len[hasp] <= self.prog.shape[0]).all()
        if (self.node_op == OP_EXPLICIT).any():
            assert self.explicit_flops is not None and self.explicit_bytes is not None


def check_program(prog: Sequence[int], n_args: int) -> None:
    """Every (arg, dim) a compute program names must exist: the kernel indexes
    the node's argument list and a MAX_RANK-wide shape row with them."""
    p = 2
    n_terms, n_outs = int(prog[0]), int(prog[1])
    for _ in range(n_terms):
        nfac = int(prog[p + 1])
        p += 2
        for _ in range(nfac):
            assert 0 <= prog[p] < n_args and 0 <= prog[p + 1] < MAX_RANK, "program factor out of range"
            p += 2
    for _ in range(n_outs):
        rank = int(prog[p + 1])
        assert prog[p] >= 0 and 0 <= rank <= 64
        p += 2
        for _ in range(rank):
            kind = int(prog[p])
            assert kind in (DIM_CONST, DIM_ARG, DIM_BCAST, DIM_ARGNUMEL)
            if kind == DIM_ARGNUMEL:
                assert 0 <= prog[p + 1] < n_args, "program dim out of range"
            elif kind == DIM_ARG:
                assert 0 <= prog[p + 1] < n_args and 0 <= prog[p + 2] < MAX_RANK, "program dim out of range"
            elif kind == DIM_BCAST:
                assert 0 <= prog[p + 1] < MAX_RANK
            p += 3
    assert p == len(prog), "program length mismatch"


# ---------------------------------------------------------------------------
# Builder: strategy-level description -> PackedGraph
# ---------------------------------------------------------------------------
TensorMetaT = Tuple[Tuple[int, ...], Tuple[int, ...], int, int]  # shape, stride, itemsize, dtype


@dataclasses.dataclass
class NodeDesc:
    """One graph node with its strategies, as the packer consumes it.

    ``in_specs[o][a]`` / ``out_specs[o][k]`` are spec words from
    :meth:`GraphBuilder.spec` (or -1 where the reference has ``None`` or a
    non-``DTensorSpec``).  ``inputs[a]`` is the producer node index of arg a
    (what ``_all_input_nodes(node)[a]`` returns), ``out_index`` the element of
    a tuple-producing producer that ``operator.getitem`` selects.
    """

    name: str
    in_specs: List[List[int]]
    out_specs: List[List[int]]
    inputs: List[int]
    getitem_index: Optional[int] = None
    op: int = OP_ZERO
    program: Optional[List[int]] = None
    default_rows: Optional[List[List[List[float]]]] = None  # [o][a][j]
    flops: Optional[List[int]] = None
    nbytes: Optional[List[int]] = None
    tuple_output: bool = False  # output_specs is a tuple (not a single spec)
    nargs: Optional[int] = None


class GraphBuilder:
    def __init__(self, mesh_shape: Sequence[int], devices_per_host: int = 8):
        self.mesh_shape = tuple(int(x) for x in mesh_shape)
        assert 1 <= len(self.mesh_shape) <= MAX_MESH_DIMS
        self.devices_per_host = int(devices_per_host)
        self._metas: Dict[TensorMetaT, int] = {}
        self._meta_rows: List[TensorMetaT] = []
        self._tuples: Dict[Tuple[int, ...], int] = {}
        self._tuple_rows: List[Tuple[int, ...]] = []
        self.nodes: List[NodeDesc] = []
        self.share_compute_slots = True
        self.prefetchable_edges: set = set()  # (node_idx, argi)
        self.multiplier: Dict[int, int] = {}
        self._reset_templates()

    def meta(self, shape, stride, itemsize: int, dtype: int) -> int:
        key = (tuple(int(s) for s in shape), tuple(int(s) for s in stride), int(itemsize), int(dtype))
        assert len(key[0]) == len(key[1]) <= MAX_RANK
        i = self._metas.get(key)
        if i is None:
            i = len(self._meta_rows)
            self._metas[key] = i
            self._meta_rows.append(key)
        return i

    def tuple_id(self, placements: Sequence[int]) -> int:
        key = tuple(int(p) for p in placements)
        assert len(key) == len(self.mesh_shape)
        i = self._tuples.get(key)
        if i is None:
            i = len(self._tuple_rows)
            assert i < MAX_TUPLES, "too many distinct placement tuples"
            self._tuples[key] = i
            self._tuple_rows.append(key)
        return i

    def spec(self, meta_id: int, placements: Sequence[int]) -> int:
        """Spec word of (tensor meta, placements); -1 stands for None."""
        return spec_word(meta_id, self.tuple_id(placements))

    def specs(self, meta_id: int, placements) -> List[int]:
        """Spec words of one tensor meta under many placement tuples
        (``placements``: int array [n, mesh dims]): the same words, and the same
        tuple ids in the same order, as ``spec`` called row by row."""
        rows = np.ascontiguousarray(placements, dtype=np.int64).reshape(-1, len(self.mesh_shape))
        if rows.shape[0] == 0:
            return []
        assert ((rows >= 0) & (rows < 256)).all()
        key = rows @ (256 ** np.arange(rows.shape[1], dtype=np.int64))
        uniq, first, inverse = np.unique(key, return_index=True, return_inverse=True)
        known = self.__dict__.setdefault("_tuple_of_key", {})  # packed placements -> tuple id
        ids = [known.get(k) for k in uniq.tolist()]
        if None in ids:
            for i in np.argsort(first, kind="stable").tolist():  # new tuples get their ids in order of first use
                if ids[i] is None:
                    ids[i] = known[int(uniq[i])] = self.tuple_id(rows[first[i]].tolist())
        return ((int(meta_id) << TUPLE_BITS) | np.asarray(ids, np.int64)[inverse.reshape(-1)]).tolist()

    def spec_placements(self, word: int) -> Tuple[int, ...]:
        return self._tuple_rows[word & (MAX_TUPLES - 1)]

    def spec_meta_row(self, word: int) -> TensorMetaT:
        return self._meta_rows[word >> TUPLE_BITS]

    def add_node(self, node: NodeDesc) -> int:
        """A node described on its own.  It is read when ``pack`` runs (so its fields
        may still change until then)."""
        assert not self._inst_tmpl, "a builder takes either nodes or template instances"
        self.nodes.append(node)
        return len(self.nodes) - 1

    # -- templates: one description for all the nodes that share it ------------------
    def _add_run(self, words) -> int:
        """Offset of a run of spec words; identical runs are stored once, which also
        makes a producer's run offset the identity of its row table."""
        key = tuple(map(int, words))
        off = self._run_cache.get(key)
        if off is None:
            off = len(self._lists)
            self._run_cache[key] = off
            self._lists.extend(key)
        return off

    def add_template(self, desc: NodeDesc) -> int:
        """Registers everything about a node that does not depend on where it sits in
        the graph: strategy count, runs of output and input spec words, program,
        compute-slot class.  ``desc.inputs`` and ``desc.getitem_index`` are not read;
        ``desc.default_rows`` only for the number of argument rows.  The repeated
        layers of a model share their templates (add_instance)."""
        S = len(desc.in_specs)
        assert S == len(desc.out_specs) and S >= 1
        t = len(self._t_S)
        nargs = desc.nargs if desc.nargs is not None else len(desc.in_specs[0])
        prog_off, prog_len = -1, 0
        if desc.program is not None:
            key = tuple(int(x) for x in desc.program)
            check_program(key, len(desc.in_specs[0]))
            prog_off = self._prog_cache.get(key)
            if prog_off is None:  # identical programs are stored once
                prog_off = len(self._prog)
                self._prog_cache[key] = prog_off
                self._prog.extend(key)
            prog_len = len(key)
        nout = len(desc.out_specs[0])
        out_runs = [self._add_run([row[k] for row in desc.out_specs]) for k in range(nout)]
        # edges: one per row of redistribute_cost (== per arg)
        n_rows = len(desc.in_specs[0]) if desc.default_rows is None else len(desc.default_rows[0])
        dst_runs, dst_none = [], []
        for a in range(n_rows):
            words = [int(row[a]) if a < len(row) else -1 for row in desc.in_specs]
            dst_runs.append(self._add_run(words))
            dst_none.append(min(words) < 0)
        # compute slots: nodes with the same op class, program, arg count and input spec
        # words produce the same estimate (the reference's memo key,
        # compute_estimation.py:449-467) and share one slot; explicit counts are per node
        if desc.op == OP_EXPLICIT:
            comp_class = -1
        else:
            if desc.op == OP_ZERO:
                key = (OP_ZERO, S, int(nargs))
            else:
                key = (desc.op, tuple(int(x) for x in desc.program), int(nargs), tuple(tuple(r) for r in desc.in_specs))
            comp_class = self._comp_classes.setdefault(key, len(self._comp_classes))
        self._t_S.append(S)
        self._t_nargs.append(int(nargs))
        self._t_op.append(int(desc.op))
        self._t_prog.append((prog_off, prog_len))
        self._t_out_runs.append(out_runs)
        self._t_dst_runs.append(dst_runs)
        self._t_dst_none.append(dst_none)
        self._t_tuple_out.append(bool(desc.tuple_output))
        self._t_comp_class.append(comp_class)
        self._t_desc.append(desc)
        return t

    def add_instance(self, template: int, inputs: Sequence[Optional[int]], getitem_index: Optional[int] = None,
                     name: Optional[str] = None, default_rows=None) -> int:
        """A node of the graph: a template at a place.  ``inputs[a]``: the producer of
        argument a (None or negative: none); ``default_rows``: the node's
        ``[o][a][j]`` default costs, or None to ask ``pack``'s callback (or zeros)."""
        assert not self.nodes, "a builder takes either nodes or template instances"
        v = len(self._inst_tmpl)
        self._inst_tmpl.append(template)
        self._inst_inputs.append(inputs)
        self._inst_getitem.append(-1 if getitem_index is None else int(getitem_index))
        self._inst_name.append(name)
        if default_rows is not None:
            self._inst_defaults[v] = default_rows
        return v

    def pack(self, default_rows_of=None) -> PackedGraph:
        """``default_rows_of(v)``: the ``[o][a][j]`` default costs of node v, asked only
        for the arguments that keep them (no producer, or a missing spec)."""
        if self.nodes:  # nodes described on their own: a template each, in node order
            for nd_ in self.nodes:
                v = len(self._inst_tmpl)
                self._inst_tmpl.append(self.add_template(nd_))
                self._inst_inputs.append(nd_.inputs)
                self._inst_getitem.append(-1 if nd_.getitem_index is None else int(nd_.getitem_index))
                self._inst_name.append(nd_.name)
                if nd_.default_rows is not None:
                    self._inst_defaults[v] = nd_.default_rows
            try:
                return self._pack(default_rows_of)
            finally:  # the builder stays what it was: a list of nodes, packed again on the next call
                self._reset_templates()
        return self._pack(default_rows_of)

    def _reset_templates(self) -> None:
        self._lists: List[int] = []
        self._run_cache: Dict[Tuple[int, ...], int] = {}
        self._prog: List[int] = []
        self._prog_cache: Dict[Tuple[int, ...], int] = {}
        self._comp_classes: Dict[tuple, int] = {}
        self._t_S: List[int] = []
        self._t_nargs: List[int] = []
        self._t_op: List[int] = []
        self._t_prog: List[Tuple[int, int]] = []
        self._t_out_runs: List[List[int]] = []
        self._t_dst_runs: List[List[int]] = []
        self._t_dst_none: List[List[bool]] = []
        self._t_tuple_out: List[bool] = []
        self._t_comp_class: List[int] = []
        self._t_desc: List[NodeDesc] = []
        self._inst_tmpl: List[int] = []
        self._inst_inputs: List[Sequence[Optional[int]]] = []
        self._inst_getitem: List[int] = []
        self._inst_name: List[Optional[str]] = []
        self._inst_defaults: Dict[int, object] = {}

    def _pack(self, default_rows_of=None) -> PackedGraph:
        nd = len(self.mesh_shape)
        M = len(self._meta_rows)
        meta_rank = np.zeros(M, np.int32)
        meta_shape = np.ones((M, MAX_RANK), np.int64)
        meta_stride = np.zeros((M, MAX_RANK), np.int64)
        meta_itemsize = np.zeros(M, np.int32)
        meta_dtype = np.zeros(M, np.int32)
        for i, (shape, stride, itemsize, dtype) in enumerate(self._meta_rows):
            r = len(shape)
            meta_rank[i] = r
            meta_shape[i, :r] = shape
            meta_stride[i, :r] = stride
            meta_itemsize[i] = itemsize
            meta_dtype[i] = dtype
        assert M <= MAX_METAS
        nt = len(self._tuple_rows)
        tuple_plc = np.zeros((nt, MAX_MESH_DIMS), np.uint8)
        for i, plc in enumerate(self._tuple_rows):
            tuple_plc[i, :nd] = plc

        def ragged(rows, dtype=np.int64):
            """(flat, first position of every row)"""
            cnt = np.fromiter((len(r) for r in rows), np.int64, len(rows))
            off = np.zeros(len(rows) + 1, np.int64)
            np.cumsum(cnt, out=off[1:])
            flat = np.fromiter((x for r in rows for x in r), dtype, int(off[-1]))
            return flat, off[:-1], cnt

        # per template
        T = len(self._t_S)
        t_S = np.asarray(self._t_S, np.int64)
        t_nargs = np.asarray(self._t_nargs, np.int32)
        t_op = np.asarray(self._t_op, np.int32)
        t_prog = np.asarray(self._t_prog, np.int64).reshape(T, 2)
        t_tuple = np.asarray(self._t_tuple_out, bool)
        t_class = np.asarray(self._t_comp_class, np.int64)
        out_flat, t_out_off, t_nout = ragged(self._t_out_runs)
        dst_flat, t_dst_off, t_nrows = ragged(self._t_dst_runs)
        dst_none_flat = np.fromiter((x for r in self._t_dst_none for x in r), bool, dst_flat.shape[0])
        lists = (np.asarray(self._lists, np.int64) & 0xFFFFFFFF).astype(np.uint32)
        none_csum = np.concatenate([[0], np.cumsum(lists == SPEC_NONE)])

        # per node
        N = len(self._inst_tmpl)
        tm = np.asarray(self._inst_tmpl, np.int64)
        assert N == 0 or ((tm >= 0) & (tm < T)).all()
        node_nstrat = t_S[tm].astype(np.int32)
        node_nargs = t_nargs[tm]
        node_op = t_op[tm]
        node_prog_off = t_prog[tm, 0]
        node_prog_len = t_prog[tm, 1].astype(np.int32)
        getitem = np.asarray(self._inst_getitem, np.int64)
        nrows = t_nrows[tm]
        node_edge_off = np.zeros(N + 1, np.int32)
        np.cumsum(nrows, out=node_edge_off[1:])
        NE = int(node_edge_off[-1])
        in_flat, in_off, in_cnt = ragged([[-1 if u is None else u for u in r] for r in self._inst_inputs])

        # edges: one per argument row
        e_node = np.repeat(np.arange(N, dtype=np.int64), nrows)
        e_arg = np.arange(NE, dtype=np.int64) - node_edge_off[:-1].astype(np.int64)[e_node]
        et = tm[e_node]
        edge_sdst = t_S[et].astype(np.int32)
        e_dst_list = dst_flat[t_dst_off[et] + e_arg]
        has_in = e_arg < in_cnt[e_node]
        u = np.full(NE, -1, np.int64)
        u[has_in] = in_flat[(in_off[e_node] + e_arg)[has_in]]
        has_prod = u >= 0
        assert (u[has_prod] < e_node[has_prod]).all(), "producers must precede consumers"
        ut = tm[np.maximum(u, 0)]
        k = np.maximum(getitem[e_node], 0)
        # a tuple-valued producer consumed directly is not a DTensorSpec: default row kept (:473)
        named = has_prod & ~(t_tuple[ut] & (getitem[e_node] < 0))
        assert (k[named] < t_nout[ut[named]]).all(), "getitem index past the producer's outputs"
        e_src_list = np.full(NE, -1, np.int64)
        e_src_list[named] = out_flat[(t_out_off[ut] + k)[named]]
        edge_ssrc = np.where(has_prod, t_S[ut], 1).astype(np.int32)
        e_flags = np.where(named, EDGE_HAS_PRODUCER, 0) | np.where(has_prod & ~t_tuple[ut], EDGE_SCORE_TRANSITION, 0)
        # a missing spec on either side keeps the default row
        src_none = np.zeros(NE, bool)
        sl = e_src_list[named]
        src_none[named] = none_csum[sl + edge_ssrc[named]] - none_csum[sl] > 0
        need_default = ~named | dst_none_flat[t_dst_off[et] + e_arg] | src_none
        e_def = np.full(NE, -1, np.int64)
        defaults: List[float] = []
        rows_of: Dict[int, object] = {}

        def node_rows(v):
            if v not in rows_of:
                r = self._inst_defaults.get(v)
                if r is None and default_rows_of is not None:
                    r = default_rows_of(v)
                rows_of[v] = r
            return rows_of[v]

        for e in np.nonzero(need_default)[0].tolist():
            v, a = int(e_node[e]), int(e_arg[e])
            rows = node_rows(v)
            if not has_prod[e]:
                edge_ssrc[e] = len(rows[0][a]) if rows is not None else 1
            n_s = int(edge_ssrc[e])
            e_def[e] = len(defaults)
            if rows is None:
                defaults.extend([0.0] * (n_s * int(edge_sdst[e])))
            else:
                assert len(rows) == int(edge_sdst[e]) and len(rows[0]) == int(nrows[v])
                for o in range(int(edge_sdst[e])):
                    row = rows[o][a]
                    assert len(row) == n_s
                    defaults.extend(float(x) for x in row)
        edge_off = np.zeros(NE + 1, np.int64)
        pad = (1 << CHUNK_SHIFT) - 1
        np.cumsum((edge_sdst.astype(np.int64) * edge_ssrc + pad) & ~pad, out=edge_off[1:])

        # compute slots, in the order their first nodes appear
        own_slot = (t_class[tm] < 0) | (not self.share_compute_slots)
        slot_key = np.where(own_slot, -1 - np.arange(N, dtype=np.int64), t_class[tm])
        _, first, inverse = np.unique(slot_key, return_index=True, return_inverse=True)
        order = np.argsort(first, kind="stable")
        comp_nodes = first[order]
        slot_off = np.zeros(comp_nodes.shape[0] + 1, np.int64)
        np.cumsum(node_nstrat[comp_nodes], out=slot_off[1:])
        n_compute = int(slot_off[-1])
        rank_of = np.empty(order.shape[0], np.int64)
        rank_of[order] = np.arange(order.shape[0])
        node_comp_off = slot_off[:-1][rank_of[inverse.reshape(-1)]] if N else np.zeros(0, np.int64)

        pref = np.zeros(NE, np.uint8)
        if self.prefetchable_edges:
            pv = np.asarray(sorted(self.prefetchable_edges), np.int64).reshape(-1, 2)
            pv = pv[(pv[:, 0] >= 0) & (pv[:, 0] < N)]
            pv = pv[(pv[:, 1] >= 0) & (pv[:, 1] < nrows[pv[:, 0]])]
            pref[node_edge_off[:-1].astype(np.int64)[pv[:, 0]] + pv[:, 1]] = 1
        mult = np.ones(N, np.int32)
        for v, m in self.multiplier.items():
            mult[v] = m
        ef = eb = None
        explicit = np.nonzero(node_op == OP_EXPLICIT)[0]
        if explicit.shape[0]:
            ef = np.zeros(n_compute, np.int64)
            eb = np.zeros(n_compute, np.int64)
            for v in explicit.tolist():
                d = self._t_desc[int(tm[v])]
                o0 = int(node_comp_off[v])
                ef[o0 : o0 + len(d.flops)] = d.flops
                eb[o0 : o0 + len(d.nbytes)] = d.nbytes
        max_outs = int(t_nout.max()) if T else 1
        t_out_pad = np.full((T, max(max_outs, 1)), -1, np.int64)
        for t, runs in enumerate(self._t_out_runs):
            t_out_pad[t, : len(runs)] = runs
        names = self._inst_name
        g = PackedGraph(
            mesh_shape=np.asarray(self.mesh_shape, np.int32),
            devices_per_host=self.devices_per_host,
            meta_rank=meta_rank,
            meta_shape=meta_shape,
            meta_stride=meta_stride,
            meta_itemsize=meta_itemsize,
            meta_dtype=meta_dtype,
            tuple_plc=tuple_plc,
            lists=lists,
            node_nstrat=node_nstrat,
            node_nargs=node_nargs,
            node_comp_off=node_comp_off,
            n_compute=n_compute,
            comp_nodes=comp_nodes.astype(np.int32),
            node_edge_off=node_edge_off,
            node_op=node_op,
            node_prog_off=node_prog_off,
            node_prog_len=node_prog_len,
            node_out_list=t_out_pad[tm, 0] if N else np.zeros(0, np.int64),
            prog=np.asarray(self._prog, np.int64),
            explicit_flops=ef,
            explicit_bytes=eb,
            edge_node=e_node.astype(np.int32),
            edge_arg=e_arg.astype(np.int32),
            edge_src_node=u.astype(np.int32),
            edge_sdst=edge_sdst,
            edge_ssrc=edge_ssrc,
            edge_dst_list=e_dst_list,
            edge_src_list=e_src_list,
            edge_off=edge_off,
            edge_flags=e_flags.astype(np.int32),
            edge_default_off=e_def,
            default_vals=np.asarray(defaults, np.float64),
            edge_prefetchable=pref,
            node_multiplier=mult,
            node_names=[n if n is not None else f"node{v}" for v, n in enumerate(names)],
            node_out_runs=t_out_pad[tm] if N else np.zeros((0, max(max_outs, 1)), np.int64),
        )
        g.validate()
        return g
