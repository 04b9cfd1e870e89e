"""apc_sample_feasible through the C ABI: the device's assignments equal the
oracle's node by node, none selects a forbidden variable unless a node is counted
as a fallback, and their scores are the oracle's bit for bit."""
import numpy as np
import pytest
import torch

from autoparallel_amd import graphgen
from oracle import cost_oracle as O

pytestmark = pytest.mark.gpu

GRAPHS = {
    "llama_1layer_2x4": lambda: graphgen.llama_graph((2, 4), 1, 64, 4, 2, 128, 256, 32, 16),
    "llama_1layer_8x8": lambda: graphgen.llama_graph((8, 8), 1, 1024, 8, 4, 2048, 8192, 512, 16),
    "moe_tiny": lambda: graphgen.moe_graph((2, 4), 2, 64, 4, 8, 2, 32, 256, 32, 8),
    "stress_3d": lambda: graphgen.stress_graph(150, (2, 2, 4), seed=4, s_min=2, s_max=60),
}


@pytest.fixture(scope="module")
def CostEngine():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from autoparallel_amd.engine import CostEngine

    return CostEngine


@pytest.mark.parametrize("name", list(GRAPHS))
def test_sampled_assignments_equal_the_oracles(CostEngine, name):
    g = GRAPHS[name]()
    print(f"  sampler: {name} nodes={g.num_nodes} E={g.num_entries}", flush=True)
    eng = CostEngine(g).build(clamp_inf=True)
    ref = O.GraphOracle(g).build()
    clamped, forbidden = O.clamp_inf(ref["cost"])
    n = 96
    assign, fallback = eng.sample_feasible(seed=9, first=1000, count=n)
    assign, fallback = assign.cpu().numpy(), fallback.cpu().numpy()
    # uint16 has no signed twin in numpy < 2; the tensor came back as uint16
    scores = eng.score(torch.from_numpy(assign).to(eng.device)).cpu().numpy()
    some_clean = False
    for a in list(range(12)) + [n - 1]:
        want, want_fb = O.sample_feasible(g, forbidden, 9, 1000 + a)
        assert assign[:, a].tolist() == want, (name, a)
        assert int(fallback[a]) == want_fb
        tot = O.score_assignment(g, ref["comm"], ref["transition"], ref["compute"], want)
        obj, viol = O.ilp_objective(g, clamped, forbidden, want)
        assert tuple(scores[a, :4]) == tuple(float(x) for x in tot), (name, a)
        assert scores[a, 4] == obj and scores[a, 5] == viol
        if want_fb == 0:
            assert viol == 0
            some_clean = True
    # over the whole batch: no fallback, nothing forbidden selected
    assert ((fallback == 0) <= (scores[:, 5] == 0)).all()
    if name != "stress_3d":
        assert some_clean and (fallback == 0).any()
    # and the plain draws of the same counters do select forbidden variables on these graphs
    plain = eng.score_random(9, 1000, n).cpu().numpy()
    assert (plain[:, 5] > 0).mean() > (scores[:, 5] > 0).mean()
    # a large batch: the same choices for the same counters
    big, big_fb = eng.sample_feasible(seed=9, first=1000, count=65536)
    assert np.array_equal(big[:, :n].cpu().numpy(), assign) and np.array_equal(big_fb[:n].cpu().numpy(), fallback)
    a = 65535
    want, want_fb = O.sample_feasible(g, forbidden, 9, 1000 + a)
    assert big[:, a].cpu().numpy().tolist() == want and int(big_fb[a]) == want_fb


def test_sampler_continues_from_given_rows(CostEngine):
    """Rows below first_node are taken as given (the stand-in nodes of a window):
    sampling the tail of a graph from the head's choices gives the whole-graph
    sample back."""
    g = GRAPHS["llama_1layer_2x4"]()
    eng = CostEngine(g).build(clamp_inf=True)
    n, cut = 64, g.num_nodes // 2
    whole, fb_whole = eng.sample_feasible(seed=3, first=0, count=n)
    part = whole.clone()
    part[cut:] = 0xFFFF
    gid = np.arange(g.num_nodes, dtype=np.int32)
    part, fb_part = eng.sample_feasible(seed=3, first=0, count=n, node_gid=gid, first_node=cut, assign=part)
    assert torch.equal(part, whole)
    # the tail's fallbacks are a part of the whole's
    assert bool((fb_part <= fb_whole).all())


def _wide_graph():
    """A consumer with 700 strategies (more than a lane keeps in registers: the words are
    formed twice), one with eight argument rows (more than the six a lane keeps), and a
    small one, over producers of a few strategies each."""
    import itertools

    from autoparallel_amd import packed
    from autoparallel_amd.packed import GraphBuilder, NodeDesc

    b = GraphBuilder((2, 2, 2, 2), 8)
    m = b.meta((8, 16, 32, 64), (32768, 2048, 64, 1), 4, packed.DT_F32)
    codes = [0x00, 0x40, 0x41, 0x42, 0x43, 0x80]
    tuples = list(itertools.product(codes, repeat=4))
    rng = np.random.default_rng(3)

    def specs(n):
        return [b.spec(m, tuples[i]) for i in rng.choice(len(tuples), n, replace=False)]

    prods = []
    for k in range(8):
        s = specs(5 + k)
        prods.append(b.add_node(NodeDesc(f"p{k}", in_specs=[[x] for x in s], out_specs=[[x] for x in s], inputs=[],
                                         default_rows=[[[0.0]] for _ in s])))
    wide = specs(700)
    b.add_node(NodeDesc("wide", in_specs=[[x] for x in wide], out_specs=[[x] for x in wide], inputs=[prods[0]]))
    many = specs(40)
    b.add_node(NodeDesc("many_args", in_specs=[[x] * 8 for x in many], out_specs=[[x] for x in many], inputs=prods))
    small = specs(9)
    b.add_node(NodeDesc("small", in_specs=[[x, x] for x in small], out_specs=[[x] for x in small],
                        inputs=[len(prods), len(prods) + 1]))
    return b.pack()


def test_bit_columns_are_the_flags_and_wide_nodes_sample_like_the_oracle(CostEngine):
    g = _wide_graph()
    eng = CostEngine(g).build(clamp_inf=True)
    ref = O.GraphOracle(g).build()
    _, forbidden = O.clamp_inf(ref["cost"])
    assert forbidden.any() and not forbidden.all()
    # the packed columns, bit by bit, against the flags they were made from
    colbits, d_off, max_words = eng._allowed_columns()
    torch.cuda.synchronize()
    bits, off = colbits.cpu().numpy().view(np.uint64), d_off.cpu().numpy()
    flags = eng.results()["flags"]
    assert max_words == (700 + 63) // 64
    for e in range(g.num_edges):
        sdst, ssrc, base = int(g.edge_sdst[e]), int(g.edge_ssrc[e]), int(g.edge_off[e])
        W = (sdst + 63) // 64
        Wc = (W + 1) & ~1  # a column is whole pairs of words
        assert off[e] % 2 == 0
        block = (flags[base: base + sdst * ssrc].reshape(sdst, ssrc) & 2) == 0  # [o][j]: allowed
        for j in range(ssrc):
            words = bits[off[e] + j * Wc: off[e] + j * Wc + W]
            got = np.unpackbits(words.view(np.uint8), bitorder="little")[: W * 64].astype(bool)
            assert np.array_equal(got[:sdst], block[:, j]) and not got[sdst:].any(), (e, j)
    # and the draws
    n = 200
    assign, fallback = eng.sample_feasible(seed=21, first=7, count=n)
    assign, fallback = assign.cpu().numpy(), fallback.cpu().numpy()
    picked_high = False
    for a in range(n):
        want, want_fb = O.sample_feasible(g, forbidden, 21, 7 + a)
        assert assign[:, a].tolist() == want and int(fallback[a]) == want_fb, a
        picked_high |= want[8] >= 512  # the 700-strategy node reaches its last words
    assert picked_high


def test_filtered_draws_equal_the_oracle_and_never_fall_back(CostEngine):
    """Row filters from the plan (feasible_plan): the device's draws equal the oracle's
    with the same filters, no node falls back and no forbidden entry is selected, where
    the walk without filters falls back several times per assignment."""
    from autoparallel_amd import feasible_plan as FP
    from autoparallel_amd import graphgen

    g, _, _ = graphgen.stress_dag_window(600, 0, 600, (4, 8, 8), 0, 4, 48)
    filters, stuck = FP.plan_filters(FP.window_masks(g))
    assert filters and not stuck
    eng = CostEngine(g).build(clamp_inf=True)
    ref = O.GraphOracle(g).build()
    _, forbidden = O.clamp_inf(ref["cost"])
    n = 300
    plain, plain_fb = eng.sample_feasible(seed=4, first=0, count=n)
    assign, fallback = eng.sample_feasible(seed=4, first=0, count=n, row_filter=filters)
    assert int(plain_fb.sum().item()) > n and int(fallback.sum().item()) == 0
    assert (eng.sample_feasible(seed=4, first=0, count=n, row_filter="plan")[0] == assign).all()
    scores = eng.score(assign).cpu().numpy()
    assert (scores[:, 5] == 0).all()
    assign = assign.cpu().numpy()
    for a in range(0, n, 7):
        want, want_fb = O.sample_feasible(g, forbidden, 4, a, row_filter=filters)
        assert assign[:, a].tolist() == want and want_fb == 0, a
    # the launch that fills the chip (another instance of the kernel): the same draws
    big, big_fb = eng.sample_feasible(seed=4, first=0, count=65536, row_filter=filters)
    assert int(big_fb.sum().item()) == 0 and (big[:, :n].cpu().numpy() == assign).all()
