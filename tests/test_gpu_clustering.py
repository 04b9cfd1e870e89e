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


def test_clustered_optimizer_end_to_end(engine_mod):
    from autoparallel_amd.sharding_problem import PackedShardingOptimizer

    plain = PackedShardingOptimizer(GRAPHS["llama_3layer_2x4"]())
    plain.get_solution()
    g = GRAPHS["llama_3layer_2x4"]()
    opt = PackedShardingOptimizer(g, repeated_subgraphs=True)
    assert opt.region_groups and opt.linked.sum() > g.num_nodes // 4
    n_free = int((opt.prob.upper > 0).sum())
    assert n_free < 0.8 * opt.n_vars  # linked nodes have no variables of their own
    sol = opt.get_solution()
    assert (sol[opt.linked] == sol[opt.root[opt.linked]]).all()
    # objective (root cost x multiplicity) == the device's objective of the expanded plan
    a = torch.from_numpy(sol.astype(np.int16).reshape(-1, 1)).cuda()
    r = opt.engine.score(a).cpu().numpy()[0]
    assert r[5] == 0
    assert np.isclose(r[4], opt.objective_value, rtol=1e-9)
    assert np.isclose(opt.objective_value, plain.objective_value, rtol=1e-6)
    # save / load keeps the links
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        opt.save(tmp + "/c.npz")
        back = PackedShardingOptimizer.load(tmp + "/c.npz")
    assert back.cluster_links == opt.cluster_links
    assert np.array_equal(back._extract(), sol)
    assert set(back.prob.constraints) == set(opt.prob.constraints)
