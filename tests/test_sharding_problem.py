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


def test_lp_file_text_of_a_three_variable_model(tmp_path):
    """The LP text, character for character: objective with a unit, a fractional
    and a negative coefficient, one row of each sense, a negative right-hand
    side, a variable fixed out of the model (not declared binary), names
    sanitised for the format."""
    p = ilp.SparseILP(3)
    p.objective = np.asarray([1.0, 2.5, -3.0])
    p.add_row("pick", [0, 1, 2], 1.0, ilp.EQ, 1.0)
    p.add_row("cap", [0, 2], [2.0, -1.0], ilp.LE, 1.5)
    p.add_row("floor", [1], [1.0], ilp.GE, -2.0)
    p.upper[2] = 0.0
    path = os.path.join(tmp_path, "m.lp")
    p.write_lp(path, ["n=a,s=0,arg=0,output_p=0,input_p=0", "n=a,s=0,arg=0,output_p=0,input_p=1", "z z"])
    x0, x1 = "n_a_s_0_arg_0_output_p_0_input_p_0", "n_a_s_0_arg_0_output_p_0_input_p_1"
    assert open(path).read() == (
        "\\* AutoParallel *\\\n"
        "Minimize\n"
        f"OBJ: + {x0} + 2.5 {x1} - 3.0 z_z\n"
        "Subject To\n"
        f"pick_000: + {x0} + {x1} + z_z = 1.0\n"
        f"cap_000: + 2.0 {x0} - z_z <= 1.5\n"
        f"floor_000: + {x1} >= -2.0\n"
        "Binaries\n"
        f"{x0}\n{x1}\n"
        "End\n")
    # and without names
    p.write_lp(path)
    assert "OBJ: + x0 + 2.5 x1 - 3.0 x2\n" in open(path).read()


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
def test_a_row_that_names_a_variable_twice_is_merged_not_refused():
    """With repeated subgraphs sharing variables the two sides of a difference row can stand for
    the same variables.  The solver takes a matrix with duplicate entries for a model error, which
    is not the same as an infeasible problem: the entries are merged, and a row that cancels
    itself out says nothing."""
    p = ilp.SparseILP(3)
    p.objective[:] = [1.0, 2.0, 3.0]
    p.add_row("twice", [0, 0, 1], [1.0, -1.0, 1.0], ilp.EQ, 1.0)  # x0 - x0 + x1 == 1
    p.add_row("cancels", [2, 2], [1.0, -1.0], ilp.EQ, 0.0)        # x2 - x2 == 0
    p.add_row("doubles", [0, 0, 2], [1.0, 1.0, 1.0], ilp.GE, 1.0)  # 2 x0 + x2 >= 1
    A, lo, hi, ub = p.to_matrix()
    assert A.has_canonical_format and A.shape == (3, 3)
    assert A[0].toarray().tolist() == [[0.0, 1.0, 0.0]] and A[1].nnz == 0 and A[2].toarray().tolist() == [[2.0, 0.0, 1.0]]
    assert p.solve() == ilp.STATUS_OPTIMAL and p.x.tolist() == [1.0, 1.0, 0.0] and p.objective_value == 3.0
    # a problem without a solution is still reported as that
    q = ilp.SparseILP(2)
    q.add_row("too_much", [0, 1], [1.0, 1.0], ilp.EQ, 3.0)
    assert q.solve() == ilp.STATUS_INFEASIBLE and q.x is None


def test_a_failure_inside_the_solver_is_reported_as_that(monkeypatch):
    """The solver's own code can give up part-way on a very large problem (an exception out of its
    C++ side, not a status): the caller gets one error that says so and names the way out."""
    import scipy.optimize

    def broken(*a, **k):
        raise ValueError("vector::_M_default_append")

    monkeypatch.setattr(scipy.optimize, "milp", broken)
    p = ilp.SparseILP(2)
    p.add_row("one", [0, 1], [1.0, 1.0], ilp.EQ, 1.0)
    with pytest.raises(RuntimeError, match="failed inside on 2 variables x 1 rows.*write_lp"):
        p.solve(backend="highs")


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
    # a constraint on a repeated node lands on its root's variables
    # (autoparallel/optimize_sharding.py:1401-1417: the variable lookup resolves links)
    v = next(int(x) for x in np.nonzero(opt.linked)[0] if opt._first_out_placements(int(x))[int(sol[x])] is not None)
    r = int(opt.root[v])
    other = next(o for o, t in enumerate(opt._first_out_placements(v))
                 if t is not None and t != opt._first_out_placements(v)[int(sol[v])])
    want = tuple(int(x) for x in g2.tuple_plc[opt._first_out_placements(v)[other], : g2.ndim])
    n_log = len(opt._constraint_log)
    names = opt.add_node_constraint(v, want, "pin_linked")
    assert len(names) == int(g2.node_edge_off[v + 1] - g2.node_edge_off[v]) and len(opt._constraint_log) == n_log + 1
    for name, e in zip(names, range(int(g2.node_edge_off[r]), int(g2.node_edge_off[r + 1]))):
        row = opt.prob.constraints[name]
        assert int(opt.var_start[e]) <= row.idx.min() and row.idx.max() < int(opt.var_start[e + 1])
    sol2 = opt.get_solution()
    chosen = tuple(int(x) for x in g2.tuple_plc[opt._first_out_placements(v)[int(sol2[v])], : g2.ndim])
    assert chosen == want and sol2[v] == sol2[r]
    # a constraint that cannot be met is refused and leaves no trace in the log
    with pytest.raises(RuntimeError, match="Couldn't find"):
        opt.add_node_constraint(v, (0x47,) * g2.ndim)
    assert len(opt._constraint_log) == n_log + 1


def test_node_constraint_matches_the_first_output_that_has_a_spec():
    """For a tuple-valued node the placement is matched against the first output
    with a spec in each strategy (autoparallel/optimize_sharding.py:1696-1706)."""
    from autoparallel_amd.packed import DT_F32, GraphBuilder, NodeDesc

    b = GraphBuilder((2,), 8)
    m = b.meta((8, 8), (8, 1), 4, DT_F32)
    r_, s0 = b.spec(m, (0x00,)), b.spec(m, (0x40,))
    b.add_node(NodeDesc("x", [[r_], [s0]], [[r_], [s0]], inputs=[], default_rows=[[[0.0]], [[0.0]]]))
    # two outputs; strategy 1 has no spec for output 0, its first output with a spec is Shard(0)
    b.add_node(NodeDesc("pair", [[r_], [s0]], [[r_, r_], [-1, s0]], inputs=[0], tuple_output=True))
    g = b.pack()
    assert g.node_out_runs.shape == (2, 2) and g.node_out_runs[0, 1] == -1
    coef, _ = oracle_coefficients(g)
    opt = PackedShardingOptimizer(g, coefficients=coef)
    assert opt._out_placements(1)[1] is None and opt._first_out_placements(1)[1] is not None
    opt.add_node_constraint(1, (0x40,))
    assert opt.get_solution()[1] == 1


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


def _rows_one_at_a_time(opt):
    """The default rows written as the reference's loops write them
    (autoparallel/optimize_sharding.py:665-801), one row per iteration: what the
    block builders must reproduce, names and order included."""
    g = opt.g
    rows = []
    count = {}

    def add(prefix, idx, coef, rhs):
        k = count.get(prefix, 0)
        count[prefix] = k + 1
        rows.append((f"{prefix}_{k:03}", [int(i) for i in idx], [float(c) for c in coef], ilp.EQ, float(rhs)))

    def row_vars(e, o):
        e = int(opt.edge_alias[e])
        s = int(g.edge_ssrc[e])
        b = int(opt.var_start[e]) + o * s
        return list(range(b, b + s))

    def col_vars(e, j):
        e = int(opt.edge_alias[e])
        s = int(g.edge_ssrc[e])
        return [int(opt.var_start[e]) + o * s + j for o in range(int(g.edge_sdst[e]))]

    for e in range(g.num_edges):
        if not opt.linked[g.edge_node[e]]:
            idx = range(int(opt.var_start[e]), int(opt.var_start[e + 1]))
            add("unique_decision", idx, [1.0] * len(idx), 1.0)
    for v in range(g.num_nodes):
        e0, e1 = int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])
        if opt.linked[v] or int((g.edge_src_node[e0:e1] >= 0).sum()) <= 1:
            continue
        for e in range(e0 + 1, e1):
            for o in range(int(g.node_nstrat[v])):
                a0, ak = row_vars(e0, o), row_vars(e, o)
                add("same_across_args", a0 + ak, [1.0] * len(a0) + [-1.0] * len(ak), 0.0)
    seen, users = set(), {}
    for e in range(g.num_edges):
        u, v = int(g.edge_src_node[e]), int(g.edge_node[e])
        # an edge between two linked nodes has no rows of its own when the edge between their roots
        # stands for it (autoparallel/optimize_sharding.py:743-746); where the producer's root is not
        # what the consumer's root reads there, it keeps them
        covered = u >= 0 and opt.linked[u] and opt.linked[v] and int(g.edge_src_node[int(opt.edge_alias[e])]) == int(opt.root[u])
        if u < 0 or covered or (u, v) in seen:
            continue
        seen.add((u, v))
        users.setdefault(u, []).append(e)
    for u in sorted(users):
        eu = int(g.node_edge_off[u])
        for e in users[u]:
            for k in range(int(g.node_nstrat[u])):
                pu, cv = row_vars(eu, k), col_vars(e, k)
                add("output_input_consistent", pu + cv, [1.0] * len(pu) + [-1.0] * len(cv), 0.0)
    for i in np.nonzero((opt.coef.flags & 2) != 0)[0]:
        if opt.prob.upper[i] > 0:
            add("inf_cases", [i], [1.0], 0.0)
    return rows


@pytest.mark.parametrize("clustered", [False, True])
def test_block_rows_equal_the_loops(tiny, clustered):
    g, coef, _ = tiny
    root = None
    if clustered:  # link every other node to an earlier node with the same strategies on every edge
        root, first = np.arange(g.num_nodes), {}
        for v in range(g.num_nodes):
            e0, e1 = int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])
            key = (int(g.node_nstrat[v]), tuple(g.edge_ssrc[e0:e1].tolist()),
                   tuple(g.edge_dst_list[e0:e1].tolist()), tuple(g.edge_src_list[e0:e1].tolist()),
                   tuple(g.edge_default_off[e0:e1].tolist() if (g.edge_default_off[e0:e1] < 0).all() else [v]))
            if key in first and v % 2 == 0:
                root[v] = first[key]
            first.setdefault(key, v)
        assert (root != np.arange(g.num_nodes)).sum() > 5
    opt = PackedShardingOptimizer(g, coefficients=coef, cluster_root=root)
    want = _rows_one_at_a_time(opt)
    got = [(n, r.idx.tolist(), r.coef.tolist(), r.sense, r.rhs) for n, r in opt.prob.constraints.items()]
    assert got[: len(want)] == want
    assert all(n.rsplit("_", 1)[0] not in ("unique_decision", "same_across_args", "output_input_consistent",
                                            "inf_cases") for n, *_ in got[len(want):])


def test_row_container():
    """Rows live in blocks; the mapping view finds, removes and replaces them by name."""
    p = ilp.SparseILP(6)
    names = p.add_rows("pair", [0, 2, 4, 6], [0, 1, 2, 3, 4, 5], 1.0, ilp.LE, [1.0, 2.0, 3.0])
    assert names == ["pair_000", "pair_001", "pair_002"] and p.add_row("pair", [0], 1.0, ilp.GE, 0.0) == "pair_003"
    p.add_row("cap", [0, 5], [2.0, 3.0], ilp.LE, 4.0, exact_name=True)
    p.add_rows("pin", [0, 1, 2], [1, 4], 1.0, ilp.EQ, 0.0)
    assert list(p.constraints) == ["pair_000", "pair_001", "pair_002", "pair_003", "cap", "pin_000", "pin_001"]
    assert len(p.constraints) == 7 and "pair_001" in p.constraints and "pair_004" not in p.constraints
    assert "pair_1" not in p.constraints and "nothing" not in p.constraints
    r = p.constraints["pair_001"]
    assert (r.name, r.idx.tolist(), r.coef.tolist(), r.sense, r.rhs) == ("pair_001", [2, 3], [1.0, 1.0], ilp.LE, 2.0)
    p.remove("pair_001")
    assert "pair_001" not in p.constraints and len(p.constraints) == 6
    with pytest.raises(KeyError):
        p.remove("pair_001")
    assert p.constraints.pop("pair_001", None) is None and p.constraints.pop("cap").rhs == 4.0
    p.add_row("cap", [1], 1.0, ilp.LE, 1.0, exact_name=True)
    p.add_row("cap", [2], 1.0, ilp.LE, 1.0, exact_name=True)  # replaces
    assert [n for n in p.constraints].count("cap") == 1 and p.constraints["cap"].idx.tolist() == [2]
    A, lo, hi, ub = p.to_matrix()
    # pins become bounds; the rest in insertion order
    assert ub.tolist() == [1, 0, 1, 1, 0, 1] and A.shape == (4, 6)
    assert A.toarray().tolist() == [[1, 1, 0, 0, 0, 0], [0, 0, 0, 0, 1, 1], [1, 0, 0, 0, 0, 0], [0, 0, 1, 0, 0, 0]]
    assert lo.tolist() == [-np.inf, -np.inf, 0.0, -np.inf] and hi.tolist() == [1.0, 3.0, np.inf, 1.0]
    assert p.next_name("pair") == "pair_004"


# -- symbolic sizes made concrete (known answers of the reference's
#    tests/test_dynamic_shapes.py:296-480, restated) ---------------------------------
def _symbolic(shape, dynamic):
    import torch
    from torch._subclasses import FakeTensorMode
    from torch.fx.experimental.symbolic_shapes import DimDynamic, ShapeEnv, StatelessSymbolicContext

    mode = FakeTensorMode(shape_env=ShapeEnv(), static_shapes=False)
    ctx = StatelessSymbolicContext(dynamic_sizes=[DimDynamic.DYNAMIC if d else DimDynamic.STATIC for d in dynamic])
    return mode, mode.from_tensor(torch.empty(*shape, device="meta"), symbolic_context=ctx)


def test_concretize_args():
    import torch

    from autoparallel_amd.optimize_sharding import _produces_tensor, concretize_args, concretize_symint

    _, x = _symbolic((16, 128), (True, True))
    assert all(isinstance(d, torch.SymInt) for d in x.shape)
    out = concretize_args((x, x.shape[0], [x.shape[1], 32]))
    assert isinstance(out[0], torch.Tensor) and all(type(d) is int for d in out[0].shape) and out[0].shape == (16, 128)
    assert type(out[1]) is int and out[1] == 16
    assert type(out[2][0]) is int and out[2] == [128, 32]
    assert out[0].stride() == (128, 1) and out[0].dtype == x.dtype
    plain = concretize_args((torch.randn(4, 4), 42, [1, 2, 3]))
    assert plain[1] == 42 and plain[2] == [1, 2, 3]
    assert concretize_symint(7) == 7 and concretize_symint("s") == "s"
    assert _produces_tensor(torch.randn(4)) and _produces_tensor((torch.randn(4), None))
    assert not _produces_tensor(42) and not _produces_tensor(None) and not _produces_tensor((1, None))


def test_concretize_gm():
    import torch
    from torch.fx import Graph, GraphModule

    from autoparallel_amd.optimize_sharding import concretize_gm

    mode, t = _symbolic((16, 128), (True, False))
    graph = Graph()
    x = graph.placeholder("x")
    x.meta.update(val=t, desc="descriptor", custom_key=42)
    y = graph.call_function(torch.relu, (x,))
    with mode:
        y.meta["val"] = torch.relu(t)
    graph.output(y)
    gm = GraphModule({}, graph)
    concrete, to_c, to_o = concretize_gm(gm)
    orig, conc = list(gm.graph.nodes), list(concrete.graph.nodes)
    assert [(n.op, n.target) for n in orig] == [(n.op, n.target) for n in conc]
    assert all(to_c[a] is b and to_o[b] is a for a, b in zip(orig, conc)) and len(to_c) == len(to_o) == 3
    assert conc[1].args == (conc[0],)  # edges follow the copy
    for n in conc[:2]:
        assert all(type(d) is int for d in n.meta["val"].shape) and n.meta["val"].shape == (16, 128)
    assert isinstance(orig[0].meta["val"].shape[0], torch.SymInt)  # the caller's graph is untouched
    assert conc[0].meta["desc"] == "descriptor" and conc[0].meta["custom_key"] == 42
