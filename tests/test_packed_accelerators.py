"""The records the host derives from a packed problem for the prepare launch
(product terms of compute programs, per-position spec records, table units):
each against the definition it stands for, on the CPU."""
import math

import numpy as np
import pytest

from autoparallel_amd import graphgen, packed
from autoparallel_amd.packed import DT_BF16, DT_F32, GraphBuilder, NodeDesc
from oracle import cost_oracle as O

GRAPHS = {
    "llama": lambda: graphgen.llama_graph((8, 8), 1, 1024, 8, 4, 2048, 8192, 512, 16),
    "llama_3d": lambda: graphgen.llama_graph((2, 2, 4), 1, 64, 4, 2, 128, 256, 32, 16),
    "moe": lambda: graphgen.moe_graph((2, 4), 2, 64, 4, 8, 2, 32, 256, 32, 8),
    "stress": lambda: graphgen.stress_graph(60, (4, 8, 8), seed=2, s_max=40),
}


@pytest.mark.parametrize("name", list(GRAPHS))
def test_program_terms_equal_the_interpreter(name):
    """flops and bytes from the product terms, evaluated on the rows of the
    value table the kernel builds, equal run_program on the same local shapes."""
    g = GRAPHS[name]()
    orc = O.GraphOracle(g)
    terms, where = g.program_terms()
    recs = g.comp_records()
    R, slots = g.max_rank, g.max_rank + 2
    checked = 0
    for rec in recs:
        if rec["n_term"] == 0:
            continue
        v = int(rec["node"])
        e0, e1 = int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])
        po = int(g.node_prog_off[v])
        prog = [int(x) for x in g.prog[po:po + int(g.node_prog_len[v])]]
        for o in range(0, int(g.node_nstrat[v]), max(1, int(g.node_nstrat[v]) // 7)):
            words = [int(g.lists[int(g.edge_dst_list[e]) + o]) for e in range(e0, e1)]
            shapes, isz, rows = [], [], {}
            for a, w in enumerate(words):
                if w == packed.SPEC_NONE:
                    shapes.append(None)
                    isz.append(0)
                    local = []
                else:
                    m = w >> packed.TUPLE_BITS
                    r = int(g.meta_rank[m])
                    local, _ = O.sharded_shape_stride(
                        [int(x) for x in g.meta_shape[m, :r]], [int(x) for x in g.meta_stride[m, :r]],
                        [int(x) for x in g.tuple_plc[w & 0xFFF, :g.ndim]], [int(x) for x in g.mesh_shape])
                    shapes.append(list(local))
                    isz.append(int(g.meta_itemsize[m]))
                for d in range(R):
                    rows[R + a * slots + d] = local[d] if d < len(local) else 1
                rows[R + a * slots + R + 1] = math.prod(local)
            for pos in range(R):  # broadcast rows
                size = 1
                for shp in shapes:
                    if shp is None or pos >= len(shp):
                        continue
                    if shp[len(shp) - 1 - pos] != 1:
                        size = shp[len(shp) - 1 - pos]
                rows[pos] = size
            flops = nbytes = 0
            for t in terms[int(rec["term_off"]):int(rec["term_off"]) + int(rec["n_term"])]:
                val = int(t["coeff"])
                for i in t["idx"]:
                    if i != 0xFF:
                        val *= rows[int(i)]
                if t["to_bytes"]:
                    nbytes += val
                else:
                    flops += val
            nbytes += sum(math.prod(s) * z for s, z in zip(shapes, isz) if s is not None)
            assert (flops, nbytes) == O.run_program(prog, shapes, isz), (name, v, o)
            checked += 1
    assert checked > 0
    # every program has the term form on these graphs
    prog_nodes = g.comp_nodes[g.node_op[g.comp_nodes] == packed.OP_PROGRAM]
    assert (recs["n_term"][g.node_op[g.comp_nodes] == packed.OP_PROGRAM] > 0).all(), len(prog_nodes)


def test_program_without_term_form_keeps_the_interpreter():
    b = GraphBuilder((2, 2))
    m = b.meta((4,) * 8, tuple(4 ** (7 - i) for i in range(8)), 2, DT_BF16)
    s = b.spec(m, (0, 0))
    b.add_node(NodeDesc("x", [[s]], [[s]], inputs=[], default_rows=[[[0.0]]]))
    # a term over eight factors: more than a 16-byte term record names
    prog = [1, 0, 2, 8] + [v for d in range(8) for v in (0, d)]
    b.add_node(NodeDesc("y", [[s]], [[s]], inputs=[0], op=packed.OP_PROGRAM, program=prog))
    g = b.pack()
    rec = g.comp_records()
    y = rec[rec["node"] == 1][0]
    assert y["n_term"] == 0 and g.program_terms()[0].shape[0] == 0


def test_spec_records():
    b = GraphBuilder((2, 4))
    metas = [
        b.meta((8, 16, 4), (64, 4, 1), 4, DT_F32),  # contiguous
        b.meta((8, 16, 4), (4, 32, 1), 2, DT_BF16),  # transposed
        b.meta((8, 1, 4), (4, 999, 1), 4, DT_F32),  # size-1 dim: its stride does not count
        b.meta((), (), 8, packed.DT_F64),  # scalar
        b.meta((5, 0, 3), (3, 3, 1), 4, DT_F32),  # no elements
    ]
    specs = [b.spec(m, plc) for m in metas for plc in ((0, 0), (packed.PARTIAL_SUM, 0))]
    b.add_node(NodeDesc("p", [[s] for s in specs], [[s] for s in specs], inputs=[],
                        default_rows=[[[0.0]] for _ in specs]))
    b.add_node(NodeDesc("c", [[specs[0], -1]], [[specs[0]]], inputs=[0, None],
                        default_rows=[[[0.0] * len(specs), [0.0]]]))
    g = b.pack()
    rec = g.spec_records()
    assert rec.shape[0] == g.lists.shape[0] and (rec["word"] == g.lists).all()
    assert (g.lists == packed.SPEC_NONE).any()
    for k, w in enumerate(g.lists):
        if w == packed.SPEC_NONE:
            assert rec["plc"][k] == 0 and rec["nbytes2"][k] == 0
            continue
        m, t = int(w) >> packed.TUPLE_BITS, int(w) & 0xFFF
        r = int(g.meta_rank[m])
        shape, stride = [int(x) for x in g.meta_shape[m, :r]], [int(x) for x in g.meta_stride[m, :r]]
        assert int(rec["plc"][k]) == int.from_bytes(bytes(g.tuple_plc[t]), "little")
        assert int(rec["nbytes2"][k]) >> 1 == int(g.meta_itemsize[m]) * math.prod(shape)
        assert bool(int(rec["nbytes2"][k]) & 1) == O.check_contiguous(shape, stride)
    contig = {int(w) >> packed.TUPLE_BITS: bool(int(n) & 1) for w, n in zip(g.lists, rec["nbytes2"]) if w != packed.SPEC_NONE}
    assert contig == {0: True, 1: False, 2: True, 3: True, 4: True}


@pytest.mark.parametrize("name", list(GRAPHS))
@pytest.mark.parametrize("compressed", [False, True])
def test_table_units_tile_every_matrix(name, compressed):
    g = GRAPHS[name]()
    block_edge, block_off, unit_block, _, edge_usrc, block_udst = g.block_table(compressed)
    units = g.table_unit_records(compressed)
    assert units.shape[0] == unit_block.shape[0] == block_off[-1] // 256
    for b in range(block_edge.shape[0]):
        e = int(block_edge[b])
        mine = units[unit_block == b]
        squeezed = compressed and edge_usrc[e] > 0
        ncol = int(edge_usrc[e]) if squeezed else int(g.edge_ssrc[e])
        nrow = int(block_udst[b]) if squeezed else int(g.edge_sdst[e])
        assert (mine["ncol"] == ncol).all() and (mine["nrow"] == nrow).all()
        assert (mine["src_list"] == g.edge_src_list[e]).all() and (mine["dst_list"] == g.edge_dst_list[e]).all()
        assert (mine["default_off"] == g.edge_default_off[e]).all()
        assert (mine["flags"] == (packed.EDGE_COMPRESSED if squeezed else 0)).all()
        # the units of a matrix start every 256 elements and reach past its last one
        assert (mine["first"] == np.arange(mine.shape[0]) * 256).all()
        assert mine.shape[0] * 256 >= ncol * nrow > (mine.shape[0] - 1) * 256


def test_edge_alias_layout():
    """with_edge_alias: aliased edges own no slots, the owning edges' blocks are
    laid out compactly, and every index structure covers exactly those."""
    from autoparallel_amd import clustering
    from oracle import cluster_oracle as CO

    g = graphgen.llama_graph((2, 4), 3, 64, 4, 2, 128, 256, 32, 8)
    groups = clustering.identical_regions(g, CO.node_hashes(g, g.node_phase))
    root = clustering.cluster_roots(g, groups).astype(np.int64)
    first = g.node_edge_off[:-1].astype(np.int64)
    v = g.edge_node.astype(np.int64)
    alias = first[root[v]] + (np.arange(g.num_edges) - first[v])
    ga = g.with_edge_alias(alias)
    ga.validate()
    own = ga.priced
    assert own.sum() < g.num_edges and (own == (root[v] == v)).all()
    sizes = g.edge_sdst.astype(np.int64) * g.edge_ssrc
    assert ga.num_entries == int(sizes[own].sum()) and ga.num_slots == int(((sizes[own] + 15) & ~15).sum())
    assert (ga.edge_off[:-1][~own] == ga.edge_off[:-1][alias[~own]]).all()
    slots, keys = ga.entry_slots(), ga.entry_keys()
    assert slots.shape[0] == keys.shape[0] == ga.num_entries and len(np.unique(slots)) == ga.num_entries
    assert (root[keys[:, 0]] == keys[:, 0]).all()  # keys of owning nodes only
    eid = np.repeat(np.arange(g.num_edges), ga.block_sizes())
    assert (ga.chunk_edge_index()[slots >> 4] == eid).all()
    items = ga.work_items()
    lead = ga.edge_off[:-1][own] % 64  # items start at multiples of 64 slots
    assert items.shape[0] == int(((sizes[own] + lead + 255) // 256).sum())
    assert set(items["off"].tolist()) == set(ga.edge_off[:-1][own].tolist())
    base, stride = ga.export_rows()
    rows = base[eid] + keys[:, 2] * stride[eid] + keys[:, 3]
    assert np.array_equal(np.sort(rows), np.arange(ga.num_entries))
    assert np.array_equal(np.argsort(rows), ga.decision_var_order())
    # edge records: an aliased edge points at its alias's block and matrix
    rec = ga.edge_records()
    assert (rec["off"][~own] == rec["off"][alias[~own]]).all()
    assert (rec["table_off"][~own] == rec["table_off"][alias[~own]]).all()
    # the oracle over the aliased graph writes each owning block once and the same
    # values again for its aliases: equal to the owning blocks of the plain build
    a, b = O.GraphOracle(ga).build(), O.GraphOracle(g).build()
    assert np.array_equal(a["comm"][slots], b["comm"][g.entry_slots()[np.repeat(own, sizes)]])
    # an alias between edges with different strategies is refused
    bad = np.arange(g.num_edges)
    x = int(np.nonzero(g.edge_ssrc != g.edge_ssrc[0])[0][0])
    bad[x] = 0
    with pytest.raises(AssertionError):
        g.with_edge_alias(bad)


def test_regions_from_the_duplicates_an_earlier_region_left():
    """Three layers of a = A(prev), b = N(a), c = C(b), e = E(input), d = N(c, e): the region grown
    from the C nodes takes a, b and c of every layer.  b and d are duplicates of each other, so the
    reference's pass then drops their whole list (graph_clustering.py:169-176) and d stays alone;
    with keep_unclaimed the d nodes still grow a region of their own, through e, and the f nodes
    (f = F(input), used by nothing), which no region can reach, become regions of one node."""
    from types import SimpleNamespace

    from autoparallel_amd import clustering

    A, N, C, E, F = 11, 12, 13, 14, 15
    args, hashes = [[]], [0]  # node 0: the input
    prev = 0
    for _ in range(3):
        base = len(args)
        args += [[prev], [base], [base + 1], [0], [base + 2, base + 3], [0]]
        hashes += [A, N, C, E, N, F]
        prev = base + 4
    off = np.cumsum([0] + [len(a) for a in args])
    n = len(args)
    g = SimpleNamespace(num_nodes=n, node_edge_off=off, edge_src_node=np.asarray([u for a in args for u in a]),
                        node_kind=np.asarray([1] + [0] * (n - 1)), node_op=np.zeros(n, np.int32), node_phase=None)
    layers = [[1 + 6 * i + k for k in range(6)] for i in range(3)]
    abc = [[lay[0], lay[1], lay[2]] for lay in layers]
    assert clustering.identical_regions(g, hashes) == [abc]
    ext = clustering.identical_regions(g, hashes, keep_unclaimed=True)
    assert ext == [abc, [[lay[3], lay[4]] for lay in layers], [[lay[5]] for lay in layers]]


def test_region_growth_equals_torchs_own():
    """The reference grows its regions with torch's fully_expand_region_group and
    _populate_recursive_ancestor_map (graph_clustering.py:17-27, 103, 178-183) around a few lines
    of its own (:141-206: lists of duplicates, latest first, skip a list whose root is taken, keep
    regions of more than one node, sort).  Here those few lines are restated around torch's two
    functions on FX graphs made of repeated random layers plus stray nodes, and
    clustering.identical_regions must return the same regions on the same graph and classes."""
    nonempty = sum(_regions_mine_and_torchs(seed) for seed in range(40))
    assert nonempty >= 20  # most of the graphs have regions to find


def _regions_mine_and_torchs(seed) -> bool:
    import operator
    from types import SimpleNamespace

    import torch.fx
    from torch._dynamo.graph_region_tracker import _populate_recursive_ancestor_map, fully_expand_region_group

    from autoparallel_amd import clustering

    rng = np.random.default_rng(seed)
    n_layers, width = int(rng.integers(2, 5)), int(rng.integers(5, 12))
    # one random layer: node k reads one or two of (the layer's input, earlier nodes of the layer)
    layer = []
    for k in range(width):
        srcs = sorted(set(int(x) for x in rng.integers(-1, k, size=int(rng.integers(1, 3)))))
        layer.append((int(rng.integers(0, 4)), srcs))  # (class within the layer, sources; -1: the input)
    graph = torch.fx.Graph()
    x = graph.placeholder("x")
    nodes, klass, args = [x], [None], [[]]
    prev = 0
    for _ in range(n_layers):
        base = len(nodes)
        for c, srcs in layer:
            a = [prev if s < 0 else base + s for s in srcs]
            nodes.append(graph.call_function(operator.add if len(a) == 2 else operator.neg, tuple(nodes[i] for i in a)))
            klass.append((c, len(a)))
            args.append(a)
        prev = len(nodes) - 1
        for _ in range(int(rng.integers(0, 3))):  # stray nodes between the layers, of the layers' classes too
            a = [int(rng.integers(0, len(nodes)))]
            nodes.append(graph.call_function(operator.neg, (nodes[a[0]],)))
            klass.append((int(rng.integers(0, 4)), 1))
            args.append(a)
    graph.output(nodes[-1])
    rank = {n: i for i, n in enumerate(nodes)}
    # a forward/backward tag: part of the key, and a barrier for the growth (:123-139, 177)
    cut = int(rng.integers(1, len(nodes) + 1))
    phase = [0 if i < cut else 1 for i in range(len(nodes))]
    klass = [None] + [c + (phase[i],) for i, c in enumerate(klass) if i > 0]

    # the reference's lines around torch's functions
    dup = {}
    for n, c in zip(nodes[1:], klass[1:]):
        dup.setdefault(c, []).append(n)
    of = {n: lst for lst in dup.values() for n in lst}
    anc = _populate_recursive_ancestor_map(graph)
    groups = sorted(([[n] for n in lst] for lst in dup.values() if len(lst) > 1),
                    key=lambda rg: -min(rank[r[0]] for r in rg))
    seen = set()
    for rg in groups:
        if any(r[0] in seen for r in rg):
            continue
        expanding = phase[rank[rg[0][0]]]
        fully_expand_region_group(
            rg, seen, anc,
            lambda a, b: a in of and b in of and of[a] is of[b] and a is not b and phase[rank[a]] == expanding)
        for r in rg:
            r.sort(key=rank.__getitem__)
    groups = [rg for rg in groups if len(rg[0]) > 1]
    for rg in groups:
        rg.sort(key=lambda r: rank[r[0]])
    groups.sort(key=lambda rg: rank[rg[0][0]])
    want = [[[rank[n] for n in r] for r in rg] for rg in groups]

    n = len(nodes)
    ids = {c: i + 1 for i, c in enumerate(dict.fromkeys(klass[1:]))}
    g = SimpleNamespace(num_nodes=n, node_edge_off=np.cumsum([0] + [len(a) for a in args]),
                        edge_src_node=np.asarray([u for a in args for u in a], np.int64),
                        node_kind=np.asarray([1] + [0] * (n - 1)), node_op=np.zeros(n, np.int32),
                        node_phase=np.asarray(phase, np.int32))
    flat = [i for rg in want for r in rg for i in r]
    if len(set(flat)) != len(flat):
        # a root of one list taken into a region of another, later, list: the reference ends with
        # "Duplicate node ... in region group" (:198-205), and so does this
        with pytest.raises(RuntimeError, match="Duplicate node"):
            clustering.identical_regions(g, [0] + [ids[c] for c in klass[1:]])
        return False
    got = clustering.identical_regions(g, [0] + [ids[c] for c in klass[1:]])
    assert got == want, seed
    return len(want) > 0
