"""ILP assembly and solver hand-off on packed graphs.  Coefficients come from
the oracle here (CPU); tests/test_gpu_parity.py checks that the HIP engine's
coefficients, and therefore the solved plan, are identical."""
import os

import numpy as np
import pytest

from autoparallel_amd import graphgen, ilp
from autoparallel_amd.sharding_problem import Coefficients, PackedShardingOptimizer
from oracle import cost_oracle as O


def oracle_coefficients(g):
    r = O.GraphOracle(g).build()
    cost, bad = O.clamp_inf(r["cost"])
    flags = (r["transition"] | (bad << 1)).astype(np.uint8)
    per_arg = np.zeros(g.num_compute)
    for v in range(g.num_nodes):
        o0 = int(g.node_comp_off[v])
        per_arg[o0:o0 + int(g.node_nstrat[v])] = r["compute"][o0:o0 + int(g.node_nstrat[v])] / int(g.node_nargs[v])
    return Coefficients(g, r["comm"], cost, flags, r["compute"], per_arg), r


@pytest.fixture(scope="module")
def tiny():
    g = graphgen.gpt2_graph((4,), n_layers=1, dim=64, n_heads=2, ffn_dim=128, vocab=256, seq=32, batch=8)
    coef, raw = oracle_coefficients(g)
    return g, coef, raw


def test_row_counts(tiny):
    g, coef, _ = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    names = list(opt.prob.constraints)
    count = lambda p: sum(1 for n in names if n.rsplit("_", 1)[0] == p)
    assert count("unique_decision") == g.num_edges
    multi = [v for v in range(g.num_nodes) if opt._num_input_nodes(v) > 1]
    want = sum((int(g.node_edge_off[v + 1]) - int(g.node_edge_off[v]) - 1) * int(g.node_nstrat[v]) for v in multi)
    assert count("same_across_args") == want
    pairs = {(int(u), int(v)) for u, v in zip(g.edge_src_node, g.edge_node) if u >= 0}
    assert count("output_input_consistent") == sum(int(g.node_nstrat[u]) for u, _ in pairs)
    assert count("inf_cases") == int(((coef.flags >> 1) & 1).sum())
    assert count("grad_param_constraint") + count("grad_param_constraint_disable") > 0
    assert count("fwd_param_dtype") > 0  # fp32 master weights cast to bf16
    assert names[0] == "unique_decision_000"


def test_solution_is_feasible_and_consistent(tiny):
    g, coef, raw = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    sol = opt.get_solution()
    assert (sol >= 0).all() and (sol < g.node_nstrat).all()
    assert opt.prob.violated() == []
    # exactly one variable per (node, arg)
    assert len(opt.selected) == g.num_edges
    # flow: the selected inp_idx of every edge is the producer's out_idx
    keys = g.entry_keys()[opt.selected]
    for v, a, o, j in keys:
        u = int(g.edge_src_node[opt.edge_of(v, a)])
        if u >= 0:
            assert sol[u] == j
        assert sol[v] == o
    # objective == sum of selected costs; no forbidden variable selected
    assert np.isclose(opt.objective_value, coef.cost[opt.selected].sum())
    assert ((coef.flags[opt.selected] >> 1) & 1).sum() == 0
    # the ILP objective of this plan equals the oracle's evaluation of it
    cost, bad = O.clamp_inf(raw["cost"])
    obj, viol = O.ilp_objective(g, cost, bad, sol)
    assert viol == 0 and np.isclose(obj, opt.objective_value, rtol=1e-12)
    # forward/backward pairs agree on placement
    plc = opt.solution_placements(sol)
    for p, gr in g.roles.param_grad:
        if gr >= 0:
            assert plc[p] == plc[gr]


def test_optimum_not_worse_than_samples(tiny):
    g, coef, raw = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    sol = opt.get_solution()
    cost, bad = O.clamp_inf(raw["cost"])
    all_rep = np.zeros(g.num_nodes, np.int64)  # strategy 0 == replicate everywhere: feasible
    obj_rep, viol = O.ilp_objective(g, cost, bad, all_rep)
    assert viol == 0 and opt.objective_value <= obj_rep + 1e-9


def test_node_constraint_and_resolve(tiny):
    g, coef, _ = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    base = opt.get_solution()
    base_obj = opt.objective_value
    tok = g.node_names.index("tokens")
    names = opt.add_node_constraint(tok, (0x40,))  # Shard(0) on the batch
    sol = opt.resolve()
    assert opt.solution_placements(sol)[tok] == ("S(0)",)
    assert opt.objective_value >= base_obj - 1e-9
    opt.remove_constraints(names)
    again = opt.resolve()
    assert np.isclose(opt.objective_value, base_obj)
    with pytest.raises(RuntimeError):
        opt.add_node_constraint(tok, (0x47,))  # Shard(7) does not exist


def test_infeasible_raises(tiny):
    g, coef, _ = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    tok = g.node_names.index("tokens")
    opt.add_node_constraint(tok, (0x40,))
    opt.add_node_constraint(tok, (0x00,))
    with pytest.raises(RuntimeError):
        opt.get_solution()


def test_lp_file(tiny, tmp_path):
    g, coef, _ = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    opt._set_objective()
    path = os.path.join(tmp_path, "model.lp")
    opt.prob.write_lp(path, opt.var_names())
    text = open(path).read()
    assert text.startswith("\\* AutoParallel *\\") and "unique_decision_000:" in text and "Binaries" in text
    assert "n_tokens_s_" in text  # reference variable naming, sanitised for the LP format


def test_sparse_ilp_basics():
    p = ilp.SparseILP(3)
    p.objective = np.asarray([1.0, 2.0, 3.0])
    p.add_row("pick", [0, 1, 2], 1.0, ilp.EQ, 1.0)
    p.add_row("ban", [0], 1.0, ilp.EQ, 0.0)
    assert p.solve() == ilp.STATUS_OPTIMAL and list(p.x) == [0, 1, 0]
    p.add_row("ban", [1], 1.0, ilp.EQ, 0.0)
    p.add_row("ban", [2], 1.0, ilp.EQ, 0.0)
    assert p.solve() == ilp.STATUS_INFEASIBLE
    assert list(p.constraints) == ["pick_000", "ban_000", "ban_001", "ban_002"]


# ---------------------------------------------------------------------------
# repeated-subgraph clustering (host logic; hashes from the oracle here)
# ---------------------------------------------------------------------------
def test_clustered_ilp_matches_reference_semantics():
    from autoparallel_amd import clustering
    from oracle import cluster_oracle as CO

    g = graphgen.llama_graph((2, 4), 3, 64, 4, 2, 128, 256, 32, 8)
    hashes = CO.node_hashes(g, g.node_phase)
    # the hash groups nodes exactly as the exact content key does
    keys = [CO.node_key(g, v, g.node_phase) for v in range(g.num_nodes)]
    by_key, by_hash = {}, {}
    for v in range(g.num_nodes):
        by_key.setdefault(keys[v], []).append(v)
        by_hash.setdefault(hashes[v], []).append(v)
    assert sorted(by_key.values()) == sorted(by_hash.values())
    groups = clustering.identical_regions(g, hashes)
    assert groups, "three identical decoder layers must cluster"
    for grp in groups:
        assert len({len(r) for r in grp}) == 1 and len(grp) >= 2 and len(grp[0]) > 1
        for reg in grp:
            assert reg == sorted(reg)
            assert len({int(g.node_phase[v]) for v in reg}) == 1  # regions do not cross fwd/bwd
        for pos in range(len(grp[0])):
            assert len({hashes[r[pos]] for r in grp}) == 1  # identical position by position
    flat = [v for grp in groups for r in grp for v in r]
    assert len(flat) == len(set(flat))  # no node in two regions
    root = clustering.cluster_roots(g, groups)
    mult = clustering.multipliers(root)
    assert mult.sum() == g.num_nodes and (mult[root != np.arange(g.num_nodes)] == 0).all()
    # layers 1 and 2 link to layer 0: a good part of the graph is linked
    assert (root != np.arange(g.num_nodes)).sum() > g.num_nodes // 4

    coef, raw = oracle_coefficients(g)
    plain = PackedShardingOptimizer(g, coefficients=coef)
    sol_plain = plain.get_solution()
    g2 = graphgen.llama_graph((2, 4), 3, 64, 4, 2, 128, 256, 32, 8)
    coef2, _ = oracle_coefficients(g2)
    opt = PackedShardingOptimizer(g2, coefficients=coef2, cluster_root=root)
    names = list(opt.prob.constraints)
    count = lambda p, o: sum(1 for n in list(o.prob.constraints) if n.rsplit("_", 1)[0] == p)
    n_linked_edges = int(opt.linked[g2.edge_node].sum())
    assert count("unique_decision", opt) == g2.num_edges - n_linked_edges
    assert count("output_input_consistent", opt) < count("output_input_consistent", plain)
    sol = opt.get_solution()
    assert (sol >= 0).all()
    assert (sol[opt.linked] == sol[opt.root[opt.linked]]).all()  # repeated nodes follow their root
    assert opt.prob.violated() == []
    # the ILP objective (root cost x multiplicity) is the plain objective of the expanded plan
    cost, bad = O.clamp_inf(raw["cost"])
    obj, viol = O.ilp_objective(g, cost, bad, sol)
    assert viol == 0 and np.isclose(obj, opt.objective_value, rtol=1e-9)
    # tying the layers together cannot beat the free optimum, and on identical layers it matches it
    assert opt.objective_value >= plain.objective_value - 1e-6
    assert np.isclose(opt.objective_value, plain.objective_value, rtol=1e-6)
    assert opt.cluster_links and all(opt.root[r] == r for r in opt.cluster_links.values())
    with pytest.raises(RuntimeError, match="shares the variables"):
        opt.add_node_constraint(int(np.nonzero(opt.linked)[0][0]))


def test_violated_constraints_log(tiny):
    """The reference's layout (optimize_sharding.py:1115-1124): a list of the
    violated row names, then each row's terms with coefficient and value."""
    g, coef, _ = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    opt.get_solution()
    assert opt.get_violated_constraints_log() == "Violated constraints: []"
    # deselect the variable chosen for the first (node, arg): its uniqueness row now sums to 0
    first = int(opt.selected[0])
    opt.prob.x[first] = 0.0
    log = opt.get_violated_constraints_log()
    head, *rest = log.split("\n")
    assert head.startswith("Violated constraints: ['unique_decision_000'")
    assert rest[0] == "========= unique_decision_000 ============="
    names = opt.var_names()
    assert f"{names[first]}, coeff=1.0, value=0.0" in rest
    opt.prob.x[first] = 1.0
