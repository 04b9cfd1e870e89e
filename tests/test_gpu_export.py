"""Device export of the coefficient twin, selected-entry gather, JSON / log
export and save/load, through the C ABI (bit-exact against the oracle)."""
import numpy as np
import pytest
import torch

from autoparallel_amd import graphgen
from helpers import bits_equal
from oracle import cost_oracle as O
from test_serialization import oracle_twin

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def engine_mod():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from autoparallel_amd import engine

    return engine


GRAPHS = {
    "gpt2_tiny": lambda: graphgen.gpt2_graph((4,), n_layers=1, dim=64, n_heads=2, ffn_dim=128, vocab=256, seq=32, batch=8),
    "llama_1layer_8x8": lambda: graphgen.config_llama3_8b(1),
    "stress_3d": lambda: graphgen.stress_graph(120, (2, 2, 4), seed=4, s_min=2, s_max=40),
}


@pytest.mark.parametrize("name", list(GRAPHS))
def test_export_twin_matches_oracle(engine_mod, name):
    g = GRAPHS[name]()
    print(f"  export: {name} E={g.num_entries}", flush=True)
    eng = engine_mod.CostEngine(g).build(clamp_inf=True)
    keys, vals = eng.export_decision_vars()
    keys, vals = keys.cpu().numpy(), vals.cpu().numpy()
    want_keys, want_vals, *_ = oracle_twin(g)
    assert np.array_equal(keys, want_keys)
    assert bits_equal(vals, want_vals)
    # the order is decision_vars' insertion order: node, out_idx, argi, inp_idx
    k = keys.astype(np.int64)
    code = ((k[:, 0] * 4096 + k[:, 2]) * 64 + k[:, 1]) * 4096 + k[:, 3]
    assert (np.diff(code) > 0).all()


def test_solution_terms_and_json(engine_mod):
    from autoparallel_amd.sharding_problem import PackedShardingOptimizer

    g = GRAPHS["gpt2_tiny"]()
    opt = PackedShardingOptimizer(g)
    sol = opt.get_solution()
    terms, slot = opt.solution_terms(sol)
    r = opt.engine.results()
    # every edge's selected entry, gathered on the host for comparison
    for e in range(g.num_edges):
        v, u = int(g.edge_node[e]), int(g.edge_src_node[e])
        idx = int(g.edge_off[e]) + int(sol[v]) * int(g.edge_ssrc[e]) + (int(sol[u]) if u >= 0 else 0)
        assert slot[e] == idx
        assert terms[e, 1] == r["comm"][idx] and terms[e, 3] == r["cost"][idx]
        assert terms[e, 2] == (r["flags"][idx] & 1)
        assert terms[e, 0] == r["per_arg"][int(g.node_comp_off[v]) + int(sol[v])]
    assert sorted(opt.var_start[np.arange(g.num_edges)] + (slot - g.edge_off[:-1])) == sorted(opt.selected)
    # out-of-range assignment is reported, not read
    bad = sol.copy()
    bad[0] = 10**4
    t2, s2 = opt.solution_terms(bad)
    assert s2[int(g.node_edge_off[0])] == -1 and np.isnan(t2[int(g.node_edge_off[0]), 0])
    data = opt.get_json(sol)
    assert len(data["nodes"]) == g.num_nodes and data["mesh"]["shape"] == [4]
    score = opt.compute_solution_cost(sol)
    s = data["summary"]
    assert np.isclose(s["compute"], score["compute"], rtol=1e-12) and np.isclose(s["comm"], score["comm"], rtol=1e-12)
    assert np.isclose(s["total"], s["compute"] + s["comm"] + s["transition"])
    # sum of the selected variables' cost is the ILP objective (no clusters here)
    assert np.isclose(terms[:, 3].sum(), opt.objective_value, rtol=1e-12)
    rec = next(n for n in data["nodes"] if n["inputs"])
    assert {"name", "src_placement", "dst_placement", "comm_cost", "transition_cost"} <= set(rec["inputs"][0])
    log = opt.get_log(sol)
    assert f"total_cost: {terms[:, 3].sum():.2f}" in log and "# placement=" in log


def test_save_from_device_and_reload(engine_mod, tmp_path):
    from autoparallel_amd.sharding_problem import PackedShardingOptimizer

    g = GRAPHS["gpt2_tiny"]()
    opt = PackedShardingOptimizer(g)
    opt.add_node_constraint(g.roles.param_grad[0][0], (0x40,))
    sol = opt.get_solution()
    path = str(tmp_path / "opt.npz")
    opt.save(path)
    loaded = PackedShardingOptimizer.load(path)
    assert loaded.engine is None  # nothing touched the device yet
    assert bits_equal(loaded.coef.cost, opt.coef.cost) and bits_equal(loaded.coef.comm, opt.coef.comm)
    assert np.array_equal(loaded.coef.flags, opt.coef.flags)
    assert np.array_equal(loaded._extract(), sol)
    assert np.array_equal(loaded.resolve(), sol)
    # device entry points on the loaded optimizer use the uploaded saved arrays
    a, b = loaded.get_json(sol), opt.get_json(sol)
    assert a["summary"] == b["summary"] and a["nodes"] == b["nodes"]
    assert loaded.compute_solution_cost(sol) == opt.compute_solution_cost(sol)
    k1, v1 = loaded.decision_var_arrays()
    k2, v2 = opt.decision_var_arrays()
    assert np.array_equal(k1, k2) and bits_equal(v1, v2)


def test_full_size_export_properties(engine_mod):
    """Llama-3-8B, (8,8): the twin is a permutation of the entry arrays."""
    g = graphgen.config_llama3_8b()
    eng = engine_mod.CostEngine(g).build(clamp_inf=True)
    keys, vals = eng.export_decision_vars()
    torch.cuda.synchronize()
    E = g.num_entries
    assert keys.shape == (E, 4) and vals.shape == (E, 3)
    slots = torch.from_numpy(g.entry_slots()).cuda()
    comm = eng.comm[slots]
    fin = torch.isfinite(comm)
    assert torch.isclose(vals[:, 1][torch.isfinite(vals[:, 1])].sum(), comm[fin].sum(), rtol=1e-9)
    assert int(torch.isinf(vals[:, 1]).sum()) == int((~fin).sum())
    assert int(vals[:, 2].sum()) == int((eng.flags[slots] & 1).sum())
    k = keys.to(torch.int64)
    code = ((k[:, 0] * 4096 + k[:, 2]) * 64 + k[:, 1]) * 4096 + k[:, 3]
    assert bool((code[1:] > code[:-1]).all())


@pytest.mark.parametrize("name", list(GRAPHS))
def test_compacted_entries_are_the_real_slots(engine_mod, name):
    """apc_compact_entries: the three entry arrays per decision variable equal a
    host gather of the padded arrays at entry_slots(), bit for bit; with repeated
    nodes aliased to their roots too."""
    g = GRAPHS[name]()
    if name == "llama_1layer_8x8":
        # alias the edges of every second node with the same strategies on both sides as an earlier one
        from autoparallel_amd.packed import EDGE_HAS_PRODUCER

        seen, alias = {}, np.arange(g.num_edges, dtype=np.int64)
        for e in range(g.num_edges):
            key = (int(g.edge_dst_list[e]), int(g.edge_src_list[e]), int(g.edge_sdst[e]), int(g.edge_ssrc[e]),
                   int(g.edge_flags[e]) & EDGE_HAS_PRODUCER, int(g.edge_default_off[e]) < 0)
            if key[5] and key in seen:
                alias[e] = seen[key]
            else:
                seen.setdefault(key, e)
        assert (alias != np.arange(g.num_edges)).sum() > 10
        g = g.with_edge_alias(alias)
    print(f"  compact: {name} E={g.num_entries} slots={g.num_slots}", flush=True)
    assert g.num_slots > g.num_entries
    eng = engine_mod.CostEngine(g).build(clamp_inf=True)
    padded, packed = eng.results(), eng.results(compact=True)
    slots = g.entry_slots()
    for k in ("comm", "cost"):
        assert packed[k].shape == (g.num_entries,) and bits_equal(packed[k], padded[k][slots]), k
    assert np.array_equal(packed["flags"], padded["flags"][slots])
    for k in ("compute", "per_arg"):
        assert bits_equal(packed[k], padded[k])
