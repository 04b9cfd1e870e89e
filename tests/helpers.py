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
