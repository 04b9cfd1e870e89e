"""apc_schedule_metrics through the C ABI against the reference's vectors, the
oracle on permuted orders, and the reference's own FX-level tests."""
import json
import os

import numpy as np
import pytest
import torch
from torch.fx.experimental.proxy_tensor import make_fx

from autoparallel_amd import schedule_metrics as SM
from oracle import schedule_oracle as SO

import schedule_graphs as SG
from test_oracle_schedule import GOLDEN, HAND

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def golden():
    with open(GOLDEN) as f:
        return json.load(f)


def test_reference_vectors_on_device(golden):
    for case in golden["cases"]:
        print(f"  schedule seed {case['seed']}", flush=True)
        gm, est = SG.build_graph(case["desc"])
        m = SM.estimate_graph_metrics(gm, est)
        want = case["metrics"]
        got = [m.total_time, m.compute_time, m.communication_time, m.exposed_comm_time]
        assert got == want[:4], (case["seed"], got, want)  # bit-exact
        assert m.peak_memory == want[4]


@pytest.mark.parametrize("k", range(len(HAND)))
def test_hand_derived_timelines_on_device(k):
    ps, want = HAND[k]
    times, peak = SM.ScheduleEstimator(ps).evaluate()
    assert tuple(times[0]) == want and peak[0] == 0


def test_batch_of_orders_matches_oracle(golden):
    """Many valid orders of one graph in one launch, each against the oracle."""
    for case in golden["cases"][5::9]:
        gm, est = SG.build_graph(case["desc"])
        ps = SM.pack_schedule(gm, est)
        orders = ps.random_orders(150, seed=case["seed"] + 100)
        print(f"  seed {case['seed']}: {ps.n_node} nodes, {ps.n_storage} storages, {orders.shape[0]} orders", flush=True)
        times, peak = SM.ScheduleEstimator(ps).evaluate(orders)
        for b, order in enumerate(orders):
            want = SO.schedule_metrics(ps, order)
            assert tuple(times[b]) == want[:4], (case["seed"], b, times[b], want)
            assert int(peak[b]) == want[4]
        # order 0 is the graph's own: the reference's numbers
        assert list(times[0]) == case["metrics"][:4] and int(peak[0]) == case["metrics"][4]
        # different orders do give different answers (the batch is not degenerate)
        assert len({float(t) for t in times[:, 0]}) > 1


def test_large_batch_properties(golden):
    """20 000 orders of the largest graph: invariants that hold for any order."""
    case = golden["cases"][-1]
    gm, est = SG.build_graph(case["desc"])
    ps = SM.pack_schedule(gm, est)
    base = ps.random_orders(200, seed=7)
    orders = np.tile(base, (100, 1))
    times, peak = SM.ScheduleEstimator(ps).evaluate(orders)
    assert times.shape == (20000, 4)
    # replicas of an order agree bit for bit wherever they sit in the batch
    assert (times.reshape(100, 200, 4) == times[:200][None]).all()
    assert (peak.reshape(100, 200) == peak[:200][None]).all()
    launch = ps.n_node  # every node adds 1 us to its own stream
    comp = times[:, 1]
    assert np.allclose(comp, comp[0], rtol=1e-12)  # same terms, another order of summation
    assert (times[:, 0] >= comp + 0.0).all() and (times[:, 3] >= 0).all()
    assert (times[:, 0] <= times[:, 1] + times[:, 2] + 2 * launch + 1e-6).all()
    assert (peak >= ps.initial_bytes).all() and (peak <= ps.initial_bytes + ps.st_bytes.sum()).all()


def _constant_estimator(dur):
    return lambda node: dur if node.op == "call_function" else 0


def test_reference_fx_level_cases():
    """The reference's tests/test_estimate_graph_metrics.py cases that need no
    process group: compute-only graph, accumulation, determinism."""
    def f(a, b):
        return torch.mm(a, b)

    gm = make_fx(f, tracing_mode="fake")(torch.randn(4, 8), torch.randn(8, 16))
    m = SM.estimate_graph_metrics(gm, _constant_estimator(100))
    assert m.compute_time == 100.0 and m.communication_time == 0 and m.exposed_comm_time == 0
    assert m.total_time > m.compute_time and m.peak_memory >= 0
    assert m == SM.estimate_graph_metrics(gm, _constant_estimator(100))

    def g(a, b, c):
        return torch.mm(torch.relu(torch.mm(a, b)), c)

    gm = make_fx(g, tracing_mode="fake")(torch.randn(4, 8), torch.randn(8, 16), torch.randn(16, 32))
    assert sum(1 for n in gm.graph.nodes if n.op == "call_function") == 3
    assert SM.estimate_graph_metrics(gm, _constant_estimator(50)).compute_time == 150


def test_bad_arguments_are_refused():
    import ctypes as C

    from autoparallel_amd import _lib

    ps, _ = HAND[1]
    est = SM.ScheduleEstimator(ps)
    with pytest.raises(AssertionError):
        est.evaluate(np.asarray([[0, 0, 1]], np.int32))  # not a permutation
    s = est.sched
    out = torch.zeros(8, dtype=torch.float64, device="cuda")
    pk = torch.zeros(2, dtype=torch.int64, device="cuda")
    # the graph's own order is one schedule: two without an order array is an error
    rc = est.lib.apc_schedule_metrics(C.byref(s), None, 2, C.c_void_p(out.data_ptr()), None,
                                      C.c_void_p(out.data_ptr()), C.c_void_p(pk.data_ptr()), None)
    assert rc == -1 and b"one schedule" in est.lib.apc_last_error()
