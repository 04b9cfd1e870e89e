"""The C restatement (oracle/cost_oracle.c) against the Python oracle, which the
reference's golden vectors pin: bit-identical on whole graphs, one thread and
several."""
import numpy as np
import pytest

from autoparallel_amd import graphgen
from helpers import bits_equal, graph_from_pairs
from oracle import c_oracle
from oracle import cost_oracle as O

GRAPHS = {
    "llama_2d": lambda: graphgen.llama_graph((8, 8), 1, 1024, 8, 4, 2048, 8192, 512, 16),
    "gpt2_1d": lambda: graphgen.gpt2_graph((8,), n_layers=1),
    "llama_odd_mesh": lambda: graphgen.llama_graph((3, 5), 1, 960, 15, 5, 1920, 3000, 240, 30),
    "stress_3d": lambda: graphgen.stress_graph(60, (4, 8, 8), seed=1, s_max=32),
    "moe_tiny": lambda: graphgen.moe_graph((2, 4), 1, 64, 4, 8, 2, 32, 256, 32, 8),
}


@pytest.mark.parametrize("name", list(GRAPHS))
def test_c_oracle_matches_python_oracle(name):
    g = GRAPHS[name]()
    ref = O.GraphOracle(g).build()
    co = c_oracle.COracle(g)
    for threads in (1, 4):
        got = co.build(threads=threads)
        for k in ("compute", "comm", "cost"):
            assert bits_equal(got[k], ref[k]), (name, k, threads)
        assert np.array_equal(got["transition"], ref["transition"])


def test_c_oracle_golden_vectors(golden):
    """The reference's own redistribution costs, through the C restatement."""
    co = None
    for k in range(int(golden["comm_ncases"][0])):
        mesh = [int(x) for x in golden[f"comm_{k}_mesh"]]
        shape = [int(x) for x in golden[f"comm_{k}_shape"]]
        stride = [int(x) for x in golden[f"comm_{k}_stride"]]
        src, tgt, want = golden[f"comm_{k}_src"], golden[f"comm_{k}_tgt"], golden[f"comm_{k}_cost"]
        src_t = sorted({tuple(int(x) for x in r) for r in src})
        tgt_t = sorted({tuple(int(x) for x in r) for r in tgt})
        g = graph_from_pairs(mesh, 8, shape, stride, int(golden[f"comm_{k}_itemsize"][0]), src_t, tgt_t)
        comm = c_oracle.COracle(g).build()["comm"]
        base, ssrc = int(g.edge_off[1]), int(g.edge_ssrc[1])
        si = {t: i for i, t in enumerate(src_t)}
        ti = {t: i for i, t in enumerate(tgt_t)}
        idx = np.asarray([base + ti[tuple(int(x) for x in t)] * ssrc + si[tuple(int(x) for x in s)]
                          for s, t in zip(src, tgt)])
        assert bits_equal(comm[idx], want), k
