"""Node hashing on the device (the clustering key) and the clustered ILP."""
import numpy as np
import pytest
import torch

from autoparallel_amd import clustering, graphgen
from oracle import cluster_oracle as CO

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def engine_mod():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from autoparallel_amd import engine

    return engine


GRAPHS = {
    "llama_3layer_2x4": lambda: graphgen.llama_graph((2, 4), 3, 64, 4, 2, 128, 256, 32, 8),
    "gpt2_2layer_4": lambda: graphgen.gpt2_graph((4,), n_layers=2, dim=64, n_heads=2, ffn_dim=128, vocab=256, seq=32, batch=8),
    "stress_2d": lambda: graphgen.stress_graph(150, (2, 4), seed=9, s_min=2, s_max=70),
}


@pytest.mark.parametrize("name", list(GRAPHS))
def test_node_hashes_match_oracle(engine_mod, name):
    g = GRAPHS[name]()
    eng = engine_mod.CostEngine(g)
    for phase in (None, g.node_phase):
        got = eng.node_hashes(phase)
        want = np.asarray(CO.node_hashes(g, phase), np.uint64)
        assert np.array_equal(got, want), int(np.nonzero(got != want)[0][0])
    # a changed tag changes the hash of that node only
    if g.node_phase is not None:
        ph = np.asarray(g.node_phase).copy()
        ph[5] ^= 1
        changed = np.nonzero(eng.node_hashes(ph) != eng.node_hashes(g.node_phase))[0]
        assert list(changed) == [5]


def test_full_size_grouping(engine_mod):
    """Llama-3-8B, 32 layers: every per-layer node falls into a group of 32."""
    g = graphgen.config_llama3_8b()
    eng = engine_mod.CostEngine(g)
    h = eng.node_hashes(g.node_phase)
    _, inv, counts = np.unique(h, return_inverse=True, return_counts=True)
    per_node = counts[inv]
    assert (per_node >= 32).sum() > 0.9 * g.num_nodes
    groups = clustering.identical_regions(g, h, check_cycles=False)
    root = clustering.cluster_roots(g, groups)
    linked = root != np.arange(g.num_nodes)
    assert linked.sum() > 0.9 * g.num_nodes * 31 / 32 * 0.9
    assert clustering.multipliers(root).max() >= 32  # 65 for the norm blocks: two per layer and the final one


def _clustered(g, engine_mod):
    eng = engine_mod.CostEngine(g, allocate_results=False)  # the problem alone is enough for the hashes
    groups = clustering.identical_regions(g, eng.node_hashes(g.node_phase))
    root = clustering.cluster_roots(g, groups).astype(np.int64)
    first = g.node_edge_off[:-1].astype(np.int64)
    v = g.edge_node.astype(np.int64)
    return root, first[root[v]] + (np.arange(g.num_edges) - first[v])


@pytest.mark.parametrize("mode", ["full", "compressed", "direct"])
def test_only_cluster_roots_are_priced(engine_mod, mode):
    """With the edges of repeated nodes aliased to their root's, the build
    writes the roots' entries only, bit-equal to the same entries of the build of
    every node; and in that build every repeated edge's block equals its
    root's, which is what makes reading the root's block for it exact."""
    from helpers import bits_equal
    from oracle import cost_oracle as O

    g = GRAPHS["llama_3layer_2x4"]()
    root, alias = _clustered(g, engine_mod)
    ga = g.with_edge_alias(alias)
    assert 0 < ga.num_entries < 0.6 * g.num_entries and ga.num_slots < 0.6 * g.num_slots
    full = engine_mod.CostEngine(g, table_mode=mode).build(clamp_inf=False).results()
    part = engine_mod.CostEngine(ga, table_mode=mode).build(clamp_inf=False).results()
    sizes = g.edge_sdst.astype(np.int64) * g.edge_ssrc
    for e in range(g.num_edges):
        a = int(alias[e])
        lo, n = int(g.edge_off[e]), int(sizes[e])
        ro, po = int(g.edge_off[a]), int(ga.edge_off[e])
        assert po == int(ga.edge_off[a])
        for k in ("comm", "cost"):
            assert bits_equal(full[k][lo:lo + n], full[k][ro:ro + n]), (k, e, a)  # the premise
            assert bits_equal(part[k][po:po + n], full[k][lo:lo + n]), (k, e, a)
        assert (part["flags"][po:po + n] == full["flags"][lo:lo + n]).all()
    assert bits_equal(part["compute"], full["compute"])
    # and the oracle, run over the aliased graph, fills the same arrays
    ref = O.GraphOracle(ga).build()
    assert bits_equal(part["comm"], ref["comm"]) and bits_equal(part["cost"], ref["cost"])
    # the exported twin holds the roots' variables only, in decision_vars order
    eng = engine_mod.CostEngine(ga).build(clamp_inf=False)
    keys, vals = (t.cpu().numpy() for t in eng.export_decision_vars())
    assert keys.shape == (ga.num_entries, 4) and not (root[keys[:, 0]] != keys[:, 0]).any()
    order = ga.decision_var_order()
    assert np.array_equal(keys, ga.entry_keys()[order])
    assert bits_equal(vals[:, 1], part["comm"][ga.entry_slots()][order])


def test_clustered_optimizer_end_to_end(engine_mod):
    from autoparallel_amd.sharding_problem import PackedShardingOptimizer

    plain = PackedShardingOptimizer(GRAPHS["llama_3layer_2x4"]())
    sol_plain = plain.get_solution()
    g = GRAPHS["llama_3layer_2x4"]()
    opt = PackedShardingOptimizer(g, repeated_subgraphs=True)
    assert opt.region_groups and opt.linked.sum() > g.num_nodes // 4
    # linked nodes have no variables of their own, and no entries were built for them
    assert opt.n_vars == opt.g.num_entries < 0.6 * plain.n_vars
    assert opt.engine.comm.numel() == opt.g.num_slots < 0.6 * g.num_slots
    assert not opt.linked[opt.g.entry_keys()[:, 0]].any()
    sol = opt.get_solution()
    assert (sol[opt.linked] == sol[opt.root[opt.linked]]).all()
    # objective (root cost x multiplicity) == the device's objective of the expanded plan
    a = torch.from_numpy(sol.astype(np.int16).reshape(-1, 1)).cuda()
    r = opt.engine.score(a).cpu().numpy()[0]
    assert r[5] == 0
    assert np.isclose(r[4], opt.objective_value, rtol=1e-9)
    assert np.isclose(opt.objective_value, plain.objective_value, rtol=1e-6)
    # the expanded plan scores the same on the engine that priced every node: sums of the
    # reference's _compute_solution_cost, bit for bit (linked rows are read from the root)
    r_plain = plain.engine.score(a).cpu().numpy()[0]
    assert (r[:4] == r_plain[:4]).all()
    # the identical layers make the free optimum a clustered plan too: same placements
    assert plain.solution_placements(sol_plain) == opt.solution_placements(sol)
    # per-edge terms of the plan: a linked edge reports its root's entry
    terms, slot = opt.solution_terms(sol)
    terms_plain, _ = plain.solution_terms(sol)
    assert np.array_equal(terms, terms_plain) and (slot >= 0).all()
    linked_e = np.nonzero(opt.linked[g.edge_node])[0]
    assert linked_e.size and (slot[linked_e] == slot[opt.edge_alias[linked_e]]).all()
    # save / load keeps the links
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        opt.save(tmp + "/c.npz")
        back = PackedShardingOptimizer.load(tmp + "/c.npz")
    assert back.cluster_links == opt.cluster_links and back.n_vars == opt.n_vars
    assert np.array_equal(back._extract(), sol)
    assert set(back.prob.constraints) == set(opt.prob.constraints)


@pytest.mark.parametrize("name", ["llama_3layer_2x4", "gpt2_2layer_4"])
def test_extended_pass_on_the_packed_graphs(engine_mod, name):
    """repeated_subgraphs="extended" keeps every region of the first pass, links at least as many
    nodes, and its objective is the device's objective of the expanded plan, scored both on its
    own engine (linked rows read from the root) and on the engine that priced every node."""
    from autoparallel_amd.sharding_problem import PackedShardingOptimizer

    plain = PackedShardingOptimizer(GRAPHS[name]())
    plain.get_solution()
    first = PackedShardingOptimizer(GRAPHS[name](), repeated_subgraphs=True)
    ext = PackedShardingOptimizer(GRAPHS[name](), repeated_subgraphs="extended")
    taken = {tuple(reg) for grp in ext.region_groups for reg in grp}
    assert all(tuple(reg) in taken for grp in first.region_groups for reg in grp)
    assert ext.linked.sum() >= first.linked.sum() > 0 and ext.n_vars <= first.n_vars
    # regions of one node only ever hold nodes that no larger region took
    seen = [v for grp in ext.region_groups for reg in grp for v in reg]
    assert len(seen) == len(set(seen))
    sol = ext.get_solution()
    first.get_solution()
    assert (sol[ext.linked] == sol[ext.root[ext.linked]]).all()
    a = torch.from_numpy(sol.astype(np.int16).reshape(-1, 1)).cuda()
    for eng in (ext.engine, plain.engine):
        r = eng.score(a).cpu().numpy()[0]
        assert r[5] == 0 and np.isclose(r[4], ext.objective_value, rtol=1e-9)
    assert ext.objective_value >= first.objective_value * (1 - 1e-9) >= plain.objective_value * (1 - 1e-9) ** 2
    # each distinct flow row once; the first pass, like the reference, repeats the rows of a
    # producer outside the regions for every repeated consumer

    def flow_rows(opt):
        return [(r.idx.tobytes(), r.coef.tobytes()) for n, r in opt.prob.constraints.items()
                if n.startswith("output_input_consistent")]

    mine, theirs = flow_rows(ext), flow_rows(first)
    assert len(set(mine)) == len(mine) > 0 and len(set(theirs)) < len(theirs)
