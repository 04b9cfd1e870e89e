"""Scoring of graphs with large edge blocks: from the block table through LDS
(apc_score_table), from compact records (apc_score_compact) and from the
32-byte records (apc_score_packed), each against the scorer that reads the
three entry arrays, bit for bit; and that one against the oracle."""
import numpy as np
import pytest
import torch

from autoparallel_amd import graphgen
from oracle import cost_oracle as O

pytestmark = pytest.mark.gpu

N = 40000


@pytest.fixture(scope="module")
def E():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from autoparallel_amd import engine

    return engine


@pytest.fixture()
def knobs(E):
    saved = (E._SCORE_FROM_TABLE, E._SCORE_COMPACT, E._SCORE_STAGE_TILES, E._SCORE_PER_LANE, E._SCORE_TABLE_FROM,
             E._SCORE_LANES_FROM)
    # the table scorer and the record walks whatever the batch size, where a test asks for them
    E._SCORE_TABLE_FROM = 0
    yield E
    (E._SCORE_FROM_TABLE, E._SCORE_COMPACT, E._SCORE_STAGE_TILES, E._SCORE_PER_LANE, E._SCORE_TABLE_FROM,
     E._SCORE_LANES_FROM) = saved


def _same(a, b):
    return torch.equal(a.view(torch.int64), b.view(torch.int64))


def _calls(eng, g, assign, half):
    gid = np.arange(g.num_nodes, dtype=np.int32) + 1000
    return [eng.score(assign), eng.score_random(3, 5, N), eng.score_random_window(3, 0, N, gid, min(7, g.num_nodes // 2), init=half)]


GRAPHS = {
    # matrices of distinct words of up to a few tiles; blocks of 50 000 entries on average
    "stress": lambda: graphgen.stress_graph(40, (4, 8, 8), seed=3, s_min=64, s_max=400),
    # more strategies than an index list in LDS holds (1024)
    "stress_long_lists": lambda: graphgen.stress_graph(6, (4, 8, 8), seed=4, s_min=1030, s_max=1100),
    # small blocks: nothing about the scorers depends on the blocks being large
    "llama": lambda: graphgen.llama_graph((8, 8), 1, 1024, 8, 4, 2048, 8192, 512, 16),
}


@pytest.mark.parametrize("name", list(GRAPHS))
@pytest.mark.parametrize("table_mode", ["compressed", "full"])
def test_every_backend_gives_the_sums_of_the_entry_arrays(knobs, name, table_mode):
    E = knobs
    g = GRAPHS[name]()
    if name == "stress_long_lists" and table_mode == "full":
        pytest.skip("covered by the compressed table: the lists only matter there")
    rng = np.random.default_rng(2)
    cols = np.stack([rng.integers(0, g.node_nstrat) for _ in range(64)], axis=1).astype(np.int16)
    assign = torch.from_numpy(np.ascontiguousarray(np.tile(cols, (1, N // 64 + 1))[:, :N])).cuda()
    half = torch.rand(N, 6, dtype=torch.float64, device="cuda")
    for clamp in (True, False):
        eng = E.CostEngine(g, table_mode=table_mode).build(clamp_inf=clamp)
        eng.packed_scoring = False
        want = _calls(eng, g, assign, half)
        eng.packed_scoring = True
        eng.large_blocks = True  # the table scorer also for the graph with small blocks
        assert eng._table_clamp == int(clamp)
        # the table, its matrices through LDS (one tile, several tiles) or read in place
        E._SCORE_FROM_TABLE = True
        for tiles, per in ((8, 0), (0, 4), (1, 2), (64, 4), (8, 1)):
            E._SCORE_STAGE_TILES, E._SCORE_PER_LANE = tiles, per
            eng._keep.pop("score_edge_aux", None)
            msize = eng._score_msize()
            if name == "stress" and tiles in (8, 64):
                tile = int(eng.lib.apc_score_table_tile())
                assert (msize > tile).any() and (msize > 0).any()  # several tiles do occur
            for got, ref in zip(_calls(eng, g, assign, half), want):
                assert _same(got, ref), (name, table_mode, clamp, "table", tiles, per)
        # compact records, then the 32-byte ones
        E._SCORE_FROM_TABLE = False
        for per in (0, 1, 2, 4, 8):
            E._SCORE_PER_LANE = per
            for got, ref in zip(_calls(eng, g, assign, half), want):
                assert _same(got, ref), (name, table_mode, clamp, "compact", per)
            assert eng._recs_compact and eng._recs.numel() == 2 * g.num_slots
        E._SCORE_COMPACT, E._SCORE_PER_LANE = False, 0
        eng._recs_valid = False
        for got, ref in zip(_calls(eng, g, assign, half), want):
            assert _same(got, ref), (name, table_mode, clamp, "records")
        assert not eng._recs_compact and eng._recs.numel() == 4 * g.num_slots
        E._SCORE_COMPACT = True


def test_against_the_oracle(E):
    g = GRAPHS["stress"]()
    eng = E.CostEngine(g).build(clamp_inf=True)
    assert eng.packed_scoring and eng.table_mode == "compressed"
    out = eng.score_random(seed=11, first=5, count=N).cpu().numpy()
    ref = O.GraphOracle(g).build()
    cost, bad = O.clamp_inf(ref["cost"])
    for i in (0, 1, 1023, 1024, N - 1):
        asg = eng.random_assignment(11, 5 + i)
        want = O.score_assignment(g, ref["comm"], ref["transition"], ref["compute"], asg)
        obj, viol = O.ilp_objective(g, cost, bad, asg)
        assert tuple(out[i, :4]) == tuple(float(x) for x in want)
        assert out[i, 4] == obj and out[i, 5] == viol


def test_arrays_changed_after_the_build(knobs):
    """The table stands for the entry arrays only as long as the build's own
    kernels wrote them; compact records only while every cost is the sum of its
    parts.  Otherwise the next backend takes over, and the sums follow the
    arrays."""
    E = knobs
    g = GRAPHS["stress"]()
    eng = E.CostEngine(g).build(clamp_inf=True)
    before = eng.score_random(3, 5, N)
    # comm scaled on some edges and their cost remade from it: the table is out, compact records still do
    g2 = graphgen.llama_graph((8, 8), 1, 1024, 8, 4, 2048, 8192, 512, 16)
    eng2 = E.CostEngine(g2).build(clamp_inf=True)
    eng2.packed_scoring = True
    assert eng2.apply_prefetch_discount(0.25) > 0 and eng2._table_clamp is None
    got = eng2.score_random(3, 5, N)
    assert eng2._recs_compact
    eng2.packed_scoring = False
    assert _same(got, eng2.score_random(3, 5, N))
    # one cost overwritten by hand
    slot = int(g.entry_slots()[12345])
    eng.cost[slot] += 1.0
    eng._table_clamp, eng._recs_valid = None, False
    got = eng.score_random(3, 5, N)
    assert not eng._recs_compact
    eng.packed_scoring = False
    assert _same(got, eng.score_random(3, 5, N)) and not _same(got, before)
    # edge_costs on its own (a caller may pass fewer arrays): the table is not trusted either
    eng.edge_costs(clamp_inf=True)
    assert eng._table_clamp is None
    eng.packed_scoring = True
    assert _same(eng.score_random(3, 5, N), before) and eng._recs_compact


def test_batches_beyond_one_launch(knobs):
    """More than 2^20 assignments (table) or 2^21 (compact records) go in several
    launches; a batch that is not a multiple of anything."""
    E = knobs
    g = graphgen.stress_graph(12, (4, 8, 8), seed=5, s_min=100, s_max=200)
    n = (1 << 21) + 1237
    eng = E.CostEngine(g).build(clamp_inf=True)
    eng.packed_scoring = False
    want = eng.score_random(9, 0, n)
    eng.packed_scoring = True
    assert _same(eng.score_random(9, 0, n), want)
    E._SCORE_FROM_TABLE = False
    assert _same(eng.score_random(9, 0, n), want) and eng._recs_compact


def test_twelve_thousand_nodes_in_four_windows():
    """A DAG large enough for four windows of the production size (3000 nodes),
    small enough for one pass: the windows' running sums are the one pass's, bit
    for bit; both read the block table."""
    from autoparallel_amd import windowed
    from autoparallel_amd.engine import CostEngine

    n_total, n_assign, s_min, s_max = 12000, 1 << 18, 32, 256
    got, st = windowed.score_in_windows(n_total, 3000, n_assign, seed=0, assign_seed=1, s_min=s_min, s_max=s_max,
                                        workers=4)
    assert st["windows"] == 4 and st["nodes"] == n_total and st["standin_nodes"] > 3000
    print(f"  windows: {st['entries']:.3g} entries, scoring {st['score_device_s'] * 1e3:.1f} ms", flush=True)
    g, gid, n_standin = graphgen.stress_dag_window(n_total, 0, n_total, (4, 8, 8), 0, s_min, s_max)
    assert n_standin == 0 and st["edges"] == g.num_edges and st["entries"] == g.num_entries
    eng = CostEngine(g).build(clamp_inf=True)
    assert eng.packed_scoring and eng._table_clamp == 1
    whole = eng.score_random(seed=1, first=0, count=n_assign).cpu().numpy()
    assert (got.view(np.uint64) == whole.view(np.uint64)).all()
    eng.packed_scoring = False  # and the one pass over the entry arrays themselves
    plain = eng.score_random(seed=1, first=0, count=n_assign).cpu().numpy()
    assert (plain.view(np.uint64) == whole.view(np.uint64)).all()


def test_small_batches_and_node_ranges(knobs):
    """A batch smaller than a workgroup, and the walk cut into node ranges through
    the C entry points (sums continued from the previous range's result): the
    sums of one walk, bit for bit."""
    import ctypes as C

    from autoparallel_amd import _lib

    E = knobs
    g = GRAPHS["stress"]()
    eng = E.CostEngine(g).build(clamp_inf=True)
    gid = np.arange(g.num_nodes, dtype=np.int32) * 3 + 5
    E._SCORE_LANES_FROM = 0  # the batch scorers for these small batches too
    for n in (1, 7, 1000):
        eng.packed_scoring = False
        want = eng.score_random_window(3, 11, n, gid, 0)
        eng.packed_scoring = True
        for from_table in (True, False):
            E._SCORE_FROM_TABLE = from_table
            assert _same(eng.score_random_window(3, 11, n, gid, 0), want), (n, from_table)
            assert eng.last_score_backend == ("block_table" if from_table else "compact_records")
    # node ranges [0, a), [a, b), [b, N) chained through init
    n = 5000
    eng.packed_scoring = False
    want = eng.score_random_window(3, 0, n, gid, 0)
    d_gid = torch.from_numpy(gid).cuda()
    aux = eng._score_edge_aux(d_gid)
    cuts = [0, g.num_nodes // 3, g.num_nodes // 3 + 1, 2 * g.num_nodes // 3, g.num_nodes]
    out = torch.empty(n, 6, dtype=torch.float64, device="cuda")
    prev = None
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        _lib.check(eng.lib.apc_score_table(
            C.byref(eng.problem), eng._ptr(eng.per_arg), eng._ptr(eng.table), C.c_void_p(aux.data_ptr()), None,
            3, 0, n, eng._ptr(d_gid), lo, hi, 1, 0, eng._ptr(prev), eng._ptr(out), eng._stream()), "apc_score_table")
        prev = out
    assert _same(out, want)
    E._SCORE_FROM_TABLE = False
    eng.packed_scoring = True
    eng.score_random(1, 0, 40000)  # makes the compact records
    assert eng._recs_compact
    prev = None
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        _lib.check(eng.lib.apc_score_compact(
            C.byref(eng.problem), eng._ptr(eng.per_arg), eng._ptr(eng._recs), None, 3, 0, n, eng._ptr(d_gid), lo, hi,
            2, eng._ptr(prev), eng._ptr(out), eng._stream()), "apc_score_compact")
        prev = out
    assert _same(out, want)
    # argument checks
    rc = eng.lib.apc_score_table(C.byref(eng.problem), eng._ptr(eng.per_arg), eng._ptr(eng.table),
                                 C.c_void_p(aux.data_ptr()), None, 3, 0, n, None, 5, 4, 1, 0, None, eng._ptr(out),
                                 eng._stream())
    assert rc == -1 and b"first_node" in eng.lib.apc_last_error()
    rc = eng.lib.apc_score_table(C.byref(eng.problem), eng._ptr(eng.per_arg), eng._ptr(eng.table),
                                 C.c_void_p(aux.data_ptr()), None, 3, 0, n, None, 0, g.num_nodes, 1, 3, None,
                                 eng._ptr(out), eng._stream())
    assert rc == -1 and b"per_lane" in eng.lib.apc_last_error()
