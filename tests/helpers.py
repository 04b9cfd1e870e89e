"""Shared helpers for the parity tests."""
import numpy as np

from autoparallel_amd.packed import DT_F32, GraphBuilder, NodeDesc


def bits_equal(a: np.ndarray, b: np.ndarray) -> bool:
    """Bit-for-bit equality of float64 arrays (inf == inf, -0.0 != 0.0)."""
    a = np.ascontiguousarray(a, np.float64).view(np.uint64)
    b = np.ascontiguousarray(b, np.float64).view(np.uint64)
    return a.shape == b.shape and bool((a == b).all())


def first_mismatch(a, b):
    a64 = np.ascontiguousarray(a, np.float64).view(np.uint64)
    b64 = np.ascontiguousarray(b, np.float64).view(np.uint64)
    bad = np.nonzero(a64 != b64)[0]
    if bad.size == 0:
        return None
    i = int(bad[0])
    return i, float(a[i]), float(b[i]), int(bad.size)


def graph_from_pairs(mesh, dph, shape, stride, itemsize, src_tuples, tgt_tuples, dtype=DT_F32):
    """Two-node graph: a producer whose strategies output ``src_tuples`` and a
    consumer whose strategies take ``tgt_tuples``: the single edge's matrix is
    every (tgt, src) pair."""
    b = GraphBuilder(mesh, dph)
    m = b.meta(shape, stride, itemsize, dtype)
    src_specs = [b.spec(m, t) for t in src_tuples]
    tgt_specs = [b.spec(m, t) for t in tgt_tuples]
    b.add_node(NodeDesc("producer", in_specs=[[s] for s in src_specs], out_specs=[[s] for s in src_specs],
                        inputs=[], default_rows=[[[0.0]] for _ in src_specs]))
    b.add_node(NodeDesc("consumer", in_specs=[[s] for s in tgt_specs], out_specs=[[s] for s in tgt_specs],
                        inputs=[0]))
    return b.pack()


def hand_made_plan():
    """A five-node graph, entry arrays filled with literal numbers, one plan, and the
    totals the reference's _compute_solution_cost (optimize_sharding.py:1056-1111) gives
    for it, worked out by hand from that function's text:

        P, Q  placeholders, strategies [Replicate, Shard(0)]
        C     = op(P, Q), two arguments
        T     = op(C) with a tuple of two outputs
        G     = T[0]

    plan: P -> Shard(0), Q -> Replicate, C -> strategy 1 (Shard(0), Shard(0)), T -> 0, G -> 1.
      compute:     every node adds compute_cost * num_args = its whole estimate:
                   P 2 + Q 4 + C 32 (two arguments of 16) + T 64 + G 256            = 358
      comm:        C<-P 0.5, C<-Q inf (not finite: skipped), T<-C 0.25, G<-T 0.125  = 0.875
      transition:  C<-P same placement 0; C<-Q differs 1 (though its comm is inf);
                   T<-C differs 1; G<-T differs, but the producer's output is a tuple
                   of specs, not a spec: not counted                                = 2
      total                                                                         = 360.875
    Returns (graph, comm, transition, compute, assignment, (total, compute, comm, transition))."""
    b = GraphBuilder((2,), 8)
    m = b.meta((8,), (1,), 4, DT_F32)
    R, S = b.spec(m, (0x00,)), b.spec(m, (0x40,))
    for name in ("P", "Q"):
        b.add_node(NodeDesc(name, in_specs=[[R], [S]], out_specs=[[R], [S]], inputs=[],
                            default_rows=[[[0.0]], [[0.0]]]))
    b.add_node(NodeDesc("C", in_specs=[[R, R], [S, S]], out_specs=[[R], [S]], inputs=[0, 1]))
    b.add_node(NodeDesc("T", in_specs=[[R], [S]], out_specs=[[R, R], [S, S]], inputs=[2], tuple_output=True))
    b.add_node(NodeDesc("G", in_specs=[[R], [S]], out_specs=[[R], [S]], inputs=[3], getitem_index=0))
    b.share_compute_slots = False
    g = b.pack()
    comm = np.zeros(g.num_slots)
    transition = np.zeros(g.num_slots, np.uint8)
    edge = {(int(g.edge_node[e]), int(g.edge_arg[e])): e for e in range(g.num_edges)}

    def put(node, arg, rows):
        e = edge[(node, arg)]
        off, ssrc = int(g.edge_off[e]), int(g.edge_ssrc[e])
        for o, row in enumerate(rows):
            for j, val in enumerate(row):
                comm[off + o * ssrc + j] = val
                transition[off + o * ssrc + j] = int(o != j)

    inf = float("inf")
    put(2, 0, [[0.0, 3.0], [5.0, 0.5]])      # C <- P
    put(2, 1, [[0.0, 7.0], [inf, 0.0]])      # C <- Q
    put(3, 0, [[0.0, 0.25], [9.0, 0.0]])     # T <- C
    put(4, 0, [[0.0, 11.0], [0.125, 0.0]])   # G <- T
    compute = np.zeros(g.num_compute)
    for v, vals in enumerate([[1.0, 2.0], [4.0, 8.0], [16.0, 32.0], [64.0, 100.0], [128.0, 256.0]]):
        compute[int(g.node_comp_off[v]): int(g.node_comp_off[v]) + 2] = vals
    assign = [1, 0, 1, 0, 1]
    return g, comm, transition, compute, assign, (360.875, 358.0, 0.875, 2.0)
