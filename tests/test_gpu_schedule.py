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


@pytest.mark.parametrize("copies", [100, 350])
def test_large_batch_properties(golden, copies):
    """20 000 and 70 000 orders of the largest graph (a workgroup's 64 orders on two
    wavefronts and on one: the launch has several workgroups for every CU): the oracle's
    numbers for the distinct orders, and invariants that hold for any order."""
    case = golden["cases"][-1]
    gm, est = SG.build_graph(case["desc"])
    ps = SM.pack_schedule(gm, est)
    base = ps.random_orders(200, seed=7)
    orders = np.tile(base, (copies, 1))
    times, peak = SM.ScheduleEstimator(ps).evaluate(orders)
    assert times.shape == (200 * copies, 4)
    for b in range(0, 200, 7):
        want = SO.schedule_metrics(ps, base[b])
        assert tuple(times[b]) == want[:4] and int(peak[b]) == want[4], (b, times[b], want)
    # replicas of an order agree bit for bit wherever they sit in the batch
    assert (times.reshape(copies, 200, 4) == times[:200][None]).all()
    assert (peak.reshape(copies, 200) == peak[:200][None]).all()
    launch = ps.n_node  # every node adds 1 us to its own stream
    comp = times[:, 1]
    assert np.allclose(comp, comp[0], rtol=1e-12)  # same terms, another order of summation
    assert (times[:, 0] >= comp + 0.0).all() and (times[:, 3] >= 0).all()
    assert (times[:, 0] <= times[:, 1] + times[:, 2] + 2 * launch + 1e-6).all()
    assert (peak >= ps.initial_bytes).all() and (peak <= ps.initial_bytes + ps.st_bytes.sum()).all()


def test_an_empty_graph_takes_no_time():
    from test_oracle_schedule import _manual

    ps = _manual([], [], [], n_stream=1)
    times, peak = SM.ScheduleEstimator(ps).evaluate()
    assert times.tolist() == [[0.0, 0.0, 0.0, 0.0]] and peak.tolist() == [0]
    assert SO.schedule_metrics(ps)[:4] == (0.0, 0.0, 0.0, 0.0)


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


def test_runtime_estimator_of_a_lowered_graph():
    """make_custom_runtime_estimation (reference: graph_passes/debug_helpers.py:170-224):
    collectives priced on the mesh dim of their group with the oracle's
    alpha-beta forms (all-gather on the gathered volume), waits free, compute
    nodes at the unsharded roofline estimate; and the whole graph through
    estimate_graph_metrics with it."""
    import torch.distributed as dist
    import torch.fx as fx
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.device_mesh import init_device_mesh
    from torch.testing._internal.distributed.fake_pg import FakeStore

    from autoparallel_amd.cost_models import collective_runtime_estimation as cre
    from autoparallel_amd.schedule_metrics import estimate_graph_metrics, make_custom_runtime_estimation
    from oracle import cost_oracle as O

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    had = dist.is_initialized()
    if had:
        dist.destroy_process_group()
    dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=16)
    try:
        mesh = init_device_mesh("cpu", (2, 8), mesh_dim_names=("dp", "tp"))
        cre.configure(8, "AMD Instinct MI355X")
        names = [g.group_name for g in mesh.get_all_groups()]
        ops = torch.ops
        g = fx.Graph()
        with FakeTensorMode():
            x = g.placeholder("x")
            x.meta["val"] = torch.empty(512, 1024, dtype=torch.bfloat16, device="cuda")
            w = g.placeholder("w")
            w.meta["val"] = torch.empty(1024, 2048, dtype=torch.bfloat16, device="cuda")
            ag = g.call_function(ops._c10d_functional.all_gather_into_tensor.default, (x, 8, names[1]))
            ag.meta["val"] = torch.empty(4096, 1024, dtype=torch.bfloat16, device="cuda")
            wt = g.call_function(ops._c10d_functional.wait_tensor.default, (ag,))
            wt.meta["val"] = ag.meta["val"]
            mm = g.call_function(ops.aten.mm.default, (wt, w))
            mm.meta["val"] = torch.empty(4096, 2048, dtype=torch.bfloat16, device="cuda")
            ar = g.call_function(ops._c10d_functional.all_reduce.default, (mm, "sum", names[0]))
            ar.meta["val"] = mm.meta["val"]
            wt2 = g.call_function(ops._c10d_functional.wait_tensor.default, (ar,))
            wt2.meta["val"] = mm.meta["val"]
            other = g.call_function(ops._c10d_functional.all_reduce.default, (wt2, "sum", "not a group of this mesh"))
            other.meta["val"] = mm.meta["val"]
            v = g.call_function(ops.aten.view.default, (other, [2048, 4096]))
            v.meta["val"] = torch.empty(2048, 4096, dtype=torch.bfloat16, device="cuda")
            g.output((v,))
        gm = fx.GraphModule(torch.nn.Module(), g)
        est = make_custom_runtime_estimation(mesh)
        from torch.distributed.tensor._collective_utils import MeshTopoInfo

        def topo_of(m):  # bandwidth and latency as torch derives them for this mesh on this host, as the reference passes them
            t, mt = O.Topo(tuple(m.shape), 8), MeshTopoInfo.build_from_mesh(m)
            t.bw, t.lat = list(mt.mesh_dim_bandwidth), list(mt.mesh_dim_latency)
            return t

        topo = topo_of(mesh)
        dev = O.DeviceLimit()
        want_ag = O.collective_comm_cost("allgather", 512 * 1024 * 2 * 8, topo, 1)
        want_ar = O.collective_comm_cost("allreduce", 4096 * 2048 * 2, topo, 0)
        flat = O.collective_comm_cost("allreduce", 4096 * 2048 * 2, topo_of(mesh._flatten()), 0)  # the flattened mesh
        flops = 2 * 4096 * 1024 * 2048
        nbytes = 2 * (4096 * 1024 + 1024 * 2048 + 4096 * 2048)
        want_mm = O.roofline_cost(flops, nbytes, 3, dev)
        assert want_mm == max(flops / (2516.6e12) * 1e6 / 0.70, O.compute_read_write_time(nbytes, dev))
        assert est(ag) == want_ag and est(ar) == want_ar and est(other) == flat
        assert est(wt) == 0 and est(v) == 0 and est(x) == 0
        assert est(mm) == want_mm
        assert est(ag, override_size=0.5) == O.collective_comm_cost("allgather", 2**29 * 8, topo, 1)
        m = estimate_graph_metrics(gm, est)
        assert m.compute_time == want_mm and m.communication_time == want_ag + want_ar + flat
        assert abs(m.exposed_comm_time - (want_ag + want_ar)) < 1e-9 * m.exposed_comm_time  # both waited for right away; the last one never
        # the chain end to end (the last collective runs out on its own stream), plus 1 us of launch per node passed
        chain = want_ag + want_mm + want_ar + flat
        assert chain < m.total_time <= chain + len(list(gm.graph.nodes))
    finally:
        dist.destroy_process_group()
        if had:
            dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=8)


@pytest.mark.parametrize("n_layers", [32, 45, 80])
def test_synthetic_schedule_from_lds_and_from_scratch_memory(n_layers):
    """A graph whose records and reader counts fit a CU's LDS is walked from there (with
    the end times of its collectives when those fit too), a larger one from the caller's
    scratch arrays: each against the oracle, with a last wavefront that is only partly
    filled."""
    ps = SM.synthetic_schedule(n_layers, seed=3)
    state = 48 * ps.n_node + 264 * (ps.n_storage + 1)
    ends = 512 * (int((ps.stream != 0).sum()) + 2)
    assert (state <= 160 * 1024) == (n_layers < 80) and (state + ends <= 160 * 1024) == (n_layers == 32)
    orders = ps.random_orders(130, seed=5)
    print(f"  {ps.n_node} nodes, {ps.n_storage} storages, {state} + {ends} bytes", flush=True)
    times, peak = SM.ScheduleEstimator(ps).evaluate(orders)
    for b, order in enumerate(orders):
        want = SO.schedule_metrics(ps, order)
        assert tuple(times[b]) == want[:4] and int(peak[b]) == want[4], (b, times[b], peak[b], want)
    assert len({int(x) for x in peak}) > 1


def test_a_node_that_reads_more_storages_than_its_record_names():
    """Seven producers and one node that reads all of them (a record in LDS names four
    of a node's storages; the rest come from the use list)."""
    n_prod = 7
    N = n_prod + 3
    deps = [[] for _ in range(n_prod)] + [list(range(n_prod)), [n_prod], [n_prod + 1]]
    use_off = np.concatenate([[0], np.cumsum([len(d) for d in deps])]).astype(np.int32)
    use_st = np.asarray([u for d in deps for u in d], np.int32)
    flags = np.zeros(N, np.uint8)
    flags[-1] = SM.SCHED_NO_MEM
    alloc_st = np.arange(N - 1, dtype=np.int32)
    ps = SM.PackedSchedule(
        dur=np.arange(1.0, N + 1.0), stream=np.zeros(N, np.int32), flags=flags, wait_src=np.full(N, -1, np.int32),
        n_stream=1, st_bytes=(np.arange(N, dtype=np.int64) + 1) * 1000, st_freeable=np.ones(N, np.uint8),
        st_users=np.bincount(use_st, minlength=N).astype(np.int32),
        alloc_off=np.minimum(np.arange(N + 1), N - 1).astype(np.int32), alloc_st=alloc_st,
        use_off=use_off, use_st=use_st, initial_bytes=500, dep_off=use_off.copy(), dep_node=use_st.copy())
    ps.validate()
    orders = ps.random_orders(70, seed=1)
    times, peak = SM.ScheduleEstimator(ps).evaluate(orders)
    for b, order in enumerate(orders):
        want = SO.schedule_metrics(ps, order)
        assert tuple(times[b]) == want[:4] and int(peak[b]) == want[4], (b, order, peak[b], want)
    # all seven producers live when the reader allocates, then only its own output and its reader's
    assert int(peak[0]) == 500 + sum(1000 * (k + 1) for k in range(n_prod + 1))
