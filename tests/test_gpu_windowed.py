"""A graph scored in windows of nodes gives, bit for bit, the sums of one pass
over the whole graph."""
import numpy as np
import pytest
import torch

from autoparallel_amd import graphgen, windowed
from oracle import cost_oracle as O

pytestmark = pytest.mark.gpu

N_TOTAL, S_MAX, SEED, N_ASSIGN = 240, 24, 5, 40000


def test_windows_equal_one_pass():
    from autoparallel_amd.engine import CostEngine

    g, gid, n_standin = graphgen.stress_dag_window(N_TOTAL, 0, N_TOTAL, (4, 8, 8), SEED, 4, S_MAX)
    assert n_standin == 0 and (gid == np.arange(N_TOTAL)).all()
    eng = CostEngine(g).build(clamp_inf=True)
    whole = eng.score_random(seed=1, first=0, count=N_ASSIGN).cpu().numpy()
    again = eng.score_random_window(1, 0, N_ASSIGN, gid, 0).cpu().numpy()
    assert (whole.view(np.uint64) == again.view(np.uint64)).all()
    for window in (60, 97):
        print(f"  windows of {window}", flush=True)
        got, st = windowed.score_in_windows(N_TOTAL, window, N_ASSIGN, seed=SEED, assign_seed=1, s_max=S_MAX,
                                            workers=1)
        assert st["nodes"] == N_TOTAL and st["edges"] == g.num_edges and st["entries"] == g.num_entries
        assert st["standin_nodes"] > 0
        assert (got.view(np.uint64) == whole.view(np.uint64)).all()
    # and the whole-graph sums are the oracle's for a few of the drawn assignments
    ref = O.GraphOracle(g).build()
    cost, bad = O.clamp_inf(ref["cost"])
    for a in (0, 1, 39999):
        asg = eng.random_assignment(1, a)
        want = O.score_assignment(g, ref["comm"], ref["transition"], ref["compute"], asg)
        obj, viol = O.ilp_objective(g, cost, bad, asg)
        assert tuple(whole[a, :4]) == tuple(float(x) for x in want)
        assert whole[a, 4] == obj and whole[a, 5] == viol


def test_window_arguments_are_checked():
    from autoparallel_amd.engine import CostEngine

    g, gid, ns = graphgen.stress_dag_window(60, 30, 60, (4, 8, 8), SEED, 4, 12)
    eng = CostEngine(g).build(clamp_inf=True)
    with pytest.raises(AssertionError):
        eng.score_random_window(1, 0, 16, gid[:-1], ns)
    with pytest.raises(AssertionError):
        eng.score_random_window(1, 0, 16, gid, ns, init=torch.zeros(8, 6, dtype=torch.float64, device="cuda"))


def test_a_window_of_the_full_dag_against_the_compiled_oracle():
    """One window deep inside the 200 000-node DAG (stand-in producers from all
    over the graph): every entry against the compiled C restatement."""
    from autoparallel_amd.engine import CostEngine
    from oracle import c_oracle

    g, gid, n_standin = graphgen.stress_dag_window(200000, 150000, 151000)
    assert n_standin > 1000 and int(gid[:n_standin].min()) < 50000
    print(f"  window: {g.num_nodes} nodes, E={g.num_entries}", flush=True)
    want = c_oracle.COracle(g).build(threads=16)
    eng = CostEngine(g).build(clamp_inf=False)
    got = eng.results()
    for k in ("comm", "cost", "compute"):
        assert (got[k].view(np.uint64) == want[k].view(np.uint64)).all(), k
    assert ((got["flags"] & 1) == want["transition"]).all()


def test_feasible_draws_in_windows_equal_one_pass():
    """Assignments drawn without forbidden entries where the graph allows it: the
    windows carry the choices of earlier nodes along, and give the sample and the
    sums of one pass over the whole graph, bit for bit; without the plan, where nodes
    fall back, and with it, where none does."""
    from autoparallel_amd import feasible_plan
    from autoparallel_amd.engine import CostEngine

    n = 4096
    g, gid, _ = graphgen.stress_dag_window(N_TOTAL, 0, N_TOTAL, (4, 8, 8), SEED, 4, S_MAX)
    eng = CostEngine(g).build(clamp_inf=True)
    plain = eng.score_random(1, 0, n).cpu().numpy()
    # with at most 24 strategies per node the plan cannot serve every node of this graph
    filters, stuck = feasible_plan.plan_filters(feasible_plan.window_masks(g))
    fallbacks = {}
    for plan in (False, True):
        assign, fb = eng.sample_feasible(1, 0, n, row_filter=filters if plan else None)
        whole = eng.score(assign).cpu().numpy()
        assert (whole[:, 5] == 0).sum() >= (plain[:, 5] == 0).sum() and whole[:, 5].mean() < plain[:, 5].mean()
        fallbacks[plan] = int(fb.sum().item())
        if plan and not stuck:
            assert fallbacks[plan] == 0 and (whole[:, 5] == 0).all()
        for window in (60, 97):
            got, st = windowed.score_in_windows(N_TOTAL, window, n, seed=SEED, assign_seed=1, s_max=S_MAX, workers=1,
                                                feasible=True, plan=plan)
            assert (got.view(np.uint64) == whole.view(np.uint64)).all(), (plan, window)
            assert st["assignments_without_fallback"] == int((fb == 0).sum().item())
            assert abs(st["fallback_nodes_per_assignment_mean"] - float(fb.double().mean().item())) < 1e-9
            assert ("plan_confined_nodes" in st) == plan
            if plan:
                assert st["plan_confined_nodes"] == len(filters) and st["plan_stuck_nodes"] == len(stuck)
    assert fallbacks[True] < fallbacks[False] / 2
    # a sample too large for the device is taken in batches, each a pass over the kept windows
    got, st = windowed.score_in_windows(N_TOTAL, 60, n, seed=SEED, assign_seed=1, s_max=S_MAX, workers=1,
                                        feasible=True, max_batch=1000)
    assert st["assignment_batches"] == 8 and (got.view(np.uint64) == whole.view(np.uint64)).all()
    assert st["nodes"] == N_TOTAL and st["entries"] == g.num_entries
    # a sample taken in several runs: assignments 100 .. 163 by themselves are those of the run from 0
    part, _ = windowed.score_in_windows(N_TOTAL, 60, 64, seed=SEED, assign_seed=1, s_max=S_MAX, workers=1,
                                        feasible=True, first=100)
    assert (part.view(np.uint64) == whole[100:164].view(np.uint64)).all()
    part, _ = windowed.score_in_windows(N_TOTAL, 60, 64, seed=SEED, assign_seed=1, s_max=S_MAX, workers=1, first=100)
    assert (part.view(np.uint64) == plain[100:164].view(np.uint64)).all()


def test_config5_at_full_size_in_windows():
    """The planner stress DAG at its full 200 000 nodes (2.4e10 cost entries, more
    than one GPU holds at once), built and scored window by window: sizes as the
    generator defines them, every window with the compressed block table, finite
    sums, and the same sums, bit for bit, from windows of another size."""
    n = 2048
    first, st = windowed.score_in_windows(200000, 3000, n, workers=14)
    assert st["nodes"] == 200000 and st["edges"] == 360006 and st["entries"] == 23981186946, st
    assert st["windows"] == 67 and st["modes"] == {"compressed": 67}
    assert np.isfinite(first).all() and (first[:, 4] > 0).all()
    print(f"  200k nodes in windows of 3000: wall {st['wall_s']:.1f} s, device build {st['build_device_s']:.2f} s, "
          f"scoring {st['score_device_s']:.2f} s", flush=True)
    second, st2 = windowed.score_in_windows(200000, 4500, n, workers=14)
    assert st2["entries"] == st["entries"] and st2["windows"] == 45
    assert (first.view(np.uint64) == second.view(np.uint64)).all()
    # and drawn node by node with the plan that confines the producers of the nodes that
    # would run out of strategies.  One node of this DAG (194 348: four strategies, each asking
    # a producer for Partials that none of the producer's strategies offers) selects a forbidden
    # entry whatever anyone chooses, so no assignment of the DAG is free of them; every other
    # node is served in every assignment.
    planned, st3 = windowed.score_in_windows(200000, 3000, n, workers=14, feasible=True)
    print(f"  planned draws: {st3['plan_confined_nodes']} confined nodes, plan {st3['plan_s']:.1f} s, "
          f"sampling {st3['sample_device_s']:.2f} s, {st3['fallback_nodes_per_assignment_mean']} fallbacks", flush=True)
    assert st3["plan_stuck_nodes"] == 1 and st3["unservable_nodes"] == [194348]
    assert st3["fallback_nodes_per_assignment_mean"] == 1.0 and st3["fallback_nodes_per_assignment_min"] == 1
    assert (planned[:, 5] >= 1).all() and (planned[:, 5] <= 4).all() and (first[:, 5] > 100).all()
    assert np.isfinite(planned).all()


def test_planned_draws_on_a_dag_of_the_same_size_that_has_feasible_assignments():
    """The same generator with seed 1: 200 000 nodes, every one of which can be served.
    With the plan no node of any assignment falls back and no forbidden entry is selected."""
    n = 1024
    scores, st = windowed.score_in_windows(200000, 3000, n, workers=14, feasible=True, seed=1)
    print(f"  seed 1: {st['entries']} entries, {st['plan_confined_nodes']} confined nodes, "
          f"sampling {st['sample_device_s']:.2f} s", flush=True)
    assert st["nodes"] == 200000 and st["windows"] == 67 and st["entries"] > 2e10
    assert st["plan_stuck_nodes"] == 0 and st["unservable_nodes"] == []
    assert st["assignments_without_fallback"] == n and st["fallback_nodes_per_assignment_mean"] == 0.0
    assert (scores[:, 5] == 0).all() and np.isfinite(scores).all()
    assert len({float(x) for x in scores[:, 4]}) == n  # and they are different assignments


def test_the_node_of_config5_that_no_assignment_can_serve():
    """Node 194 348 of the 200 000-node DAG, with its producers as stand-ins, from the
    flags the device writes: each of its strategies has an argument whose entries are
    forbidden against every strategy of the producer.  (So every assignment of the DAG
    selects a forbidden entry, and the ILP over it has no solution.)"""
    from autoparallel_amd.engine import CostEngine

    g, gid, n_standin = graphgen.stress_dag_window(200000, 194348, 194349)
    v = g.num_nodes - 1
    assert int(gid[v]) == 194348 and n_standin == v
    flags = CostEngine(g).build(clamp_inf=True).results()["flags"]
    S = int(g.node_nstrat[v])
    edges = range(int(g.node_edge_off[v]), int(g.node_edge_off[v + 1]))
    assert S == 4 and len(edges) >= 1
    for o in range(S):
        dead = []
        for e in edges:
            ssrc, off = int(g.edge_ssrc[e]), int(g.edge_off[e])
            dead.append(bool(((flags[off + o * ssrc: off + (o + 1) * ssrc] & 2) != 0).all()))
        assert any(dead), (o, dead)


def test_small_batches_of_explicit_assignments_in_a_window():
    """apc_score_assignments_window (entry arrays, a lane per assignment) gives the
    sums of the batch scorers for the same window, stand-ins and carried sums
    included."""
    from autoparallel_amd import engine as E
    from autoparallel_amd.engine import CostEngine

    g, gid, n_standin = graphgen.stress_dag_window(N_TOTAL, 100, 200, (4, 8, 8), SEED, 4, S_MAX)
    assert n_standin > 0
    eng = CostEngine(g).build(clamp_inf=True)
    n = 500
    rng = np.random.default_rng(0)
    assign = torch.from_numpy(np.stack([rng.integers(0, s, n) for s in g.node_nstrat]).astype(np.int16)).cuda()
    init = torch.rand(n, 6, dtype=torch.float64, device="cuda")
    got = eng.score_window(assign, n_standin, init=init)
    assert eng.last_score_backend == "entry_arrays"
    saved = E._SCORE_LANES_FROM
    try:
        E._SCORE_LANES_FROM = 0
        want = eng.score_window(assign, n_standin, init=init)
        assert eng.last_score_backend != "entry_arrays"
    finally:
        E._SCORE_LANES_FROM = saved
    assert torch.equal(got.view(torch.int64), want.view(torch.int64))
