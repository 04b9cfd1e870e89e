"""The reference-shaped Python surface (ShardingOptimizer on an AOT joint
graph, the cost_models functions on DTensorSpecs) over the HIP engine."""
import contextlib

import numpy as np
import pytest
import torch
import torch.nn as nn

from helpers import bits_equal
from oracle import cost_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mesh():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import torch.distributed as dist
    from torch.distributed.device_mesh import init_device_mesh
    from torch.testing._internal.distributed.fake_pg import FakeStore

    if not dist.is_initialized():
        dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=8)
    yield init_device_mesh("cpu", (2, 4))
    dist.destroy_process_group()


class MLP(nn.Module):
    def __init__(self):
        super().__init__()
        self.a = nn.Linear(64, 128, bias=False)
        self.b = nn.Linear(128, 64, bias=False)

    def forward(self, x):
        return self.b(torch.relu(self.a(x)))


def _joint_graph():
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        m, x = MLP(), torch.randn(16, 32, 64)
        with contextlib.ExitStack() as stack:
            jd = aot_export_joint_with_descriptors(stack, m, (x,))
    return jd.graph_module


def test_sharding_optimizer_on_joint_graph(mesh):
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    gm = _joint_graph()
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    g = opt._packed
    assert len(opt.decision_vars) == g.num_entries > 1000
    # every coefficient equals the oracle's on the same packed problem
    ref = O.GraphOracle(g).build()
    slots = g.entry_slots()
    cost_ref, bad = O.clamp_inf(ref["cost"])
    assert bits_equal(opt._core.coef.comm, ref["comm"][slots])
    assert bits_equal(opt._core.coef.cost, cost_ref[slots])
    # mapping view: reference key order, attribute access, strategy objects
    keys = list(opt.decision_vars)
    assert keys == sorted(keys, key=lambda k: (k[0], k[2], k[1], k[3]))
    k = keys[len(keys) // 2]
    dv = opt.decision_vars[k]
    assert dv.cost == dv.comm_cost + dv.compute_cost + dv.sharding_transition_cost or dv.cost == 10000.0
    assert dv.strategy is opt.strats[opt.nodes[k[0]]].strategies[k[2]]
    assert opt.decision_vars.get((10**6, 0, 0, 0)) is None
    # redistribute_cost rows were written back (same object the strategies carry)
    node = opt.nodes[k[0]]
    assert opt.strats[node].strategies[k[2]].redistribute_cost[k[1]][k[3]] == dv.comm_cost
    # solve: one strategy per node, consistent with the flow constraints
    sol = opt.get_solution()
    assert set(sol) == {n for n in opt.nodes if n.op != "output"}
    base = opt._core.objective_value
    # the reference's accessors: variables by key with their solved values, strategies by node
    chosen = set(opt.selected_keys)
    assert all(opt.pulp_variables[key].varValue == 1.0 for key in list(chosen)[:50])
    others = [key for key in keys[:400] if key not in chosen]
    assert others and all(opt.pulp_variables[key].varValue == 0.0 for key in others)
    assert opt.pulp_variables[k].name == f"n={opt.nodes[k[0]]},s={k[0]},arg={k[1]},output_p={k[2]},input_p={k[3]}"
    assert opt.get_strategy(node) is opt.strats[node] and opt._concrete_to_orig[node] is node
    assert opt._resolve_decision_var(k).cost == dv.cost
    total = opt._compute_solution_cost(sol)["total"]
    assert np.isclose(total, base, rtol=1e-9)  # no clusters, no inf entries selected
    # parameters and their gradients get the same placement
    from torch._functorch._aot_autograd import fx_utils

    for p, gr in fx_utils.get_param_and_grad_nodes(gm.graph).values():
        assert sol[p].output_specs.placements == sol[gr].output_specs.placements
    # export: JSON (one record per graph node, output included), annotated log, save, placements
    data = opt.get_json()
    assert [n["name"] for n in data["nodes"]] == [n.name for n in gm.graph.nodes]
    assert data["nodes"][-1]["op"] == "output" and data["mesh"]["shape"] == [2, 4]
    assert np.isclose(data["summary"]["total"], total, rtol=1e-9)
    kinds = {n.get("placeholder_kind") for n in data["nodes"]}
    assert {"param", "input", "tangent"} <= kinds
    assert any(n.get("op", "").startswith("aten.") for n in data["nodes"])
    log = opt.get_log()
    assert "# placement=" in log and f"total_cost: {base:.2f}" in log
    import tempfile

    from autoparallel_amd.sharding_problem import PackedShardingOptimizer

    with tempfile.TemporaryDirectory() as tmp:
        opt.save(tmp + "/opt.npz")
        loaded = PackedShardingOptimizer.load(tmp + "/opt.npz")
        assert loaded.n_vars == len(opt.decision_vars) and loaded.g.num_nodes == opt._packed.num_nodes == len(opt.nodes) - 1
        assert np.isclose(loaded.objective_value, base)
        assert loaded.get_json()["summary"] == opt._core.get_json()["summary"]
        opt.save_placements(tmp + "/plc.json")
        back = opt.load_placements(tmp + "/plc.json")
        assert all(str(back[n].output_specs) == str(sol[n].output_specs) for n in sol)
    # counterfactual report: the all-Replicate plan is available everywhere and never cheaper in total
    from torch.distributed.tensor.placement_types import Replicate as _R

    text = opt.explain_placement((_R(), _R()))
    assert text.startswith("explain_placement: target=") and "Tgt.Comm" in text
    assert "UNAVAILABLE" not in text and ("CHOSEN CHEAPER" in text or "TIE" in text or "CHOSEN" in text)
    assert len(opt.explain_placement((_R(), _R()), max_nodes=3).strip().split("\n")) == 2 + 2 + 3
    # a user constraint moves the plan and can be removed again
    x = next(n for n in gm.graph.nodes if n.name == "primals_3")
    from torch.distributed.tensor.placement_types import Replicate, Shard

    names = opt.add_node_constraint(x, (Shard(0), Replicate()))
    sol2 = opt.resolve()
    assert sol2[x].output_specs.placements == (Shard(0), Replicate())
    assert opt._core.objective_value >= base - 1e-9
    opt.diff_solutions(sol, sol2)
    opt.remove_constraints(names)
    opt.resolve()
    assert np.isclose(opt._core.objective_value, base)


def test_cost_models_scalar_api(mesh, golden):
    from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

    from autoparallel_amd import cost_models as cm

    cm.configure(devices_per_host=8, device_name="AMD Instinct MI355X")
    shape = (6, 10)
    tm = TensorMeta(torch.Size(shape), (10, 1), torch.float32)
    topo, dev = O.Topo((2, 4), 8), O.DeviceLimit()
    code = {Replicate(): 0, Shard(0): 0x40, Shard(1): 0x41, Partial(): 0x80}
    opts = list(code)
    for a in [(Shard(0), Shard(1)), (Partial(), Partial()), (Replicate(), Shard(1)), (Shard(1), Partial())]:
        for b in [(Replicate(), Replicate()), (Shard(1), Shard(0)), (Shard(0), Shard(0)), (Partial(), Replicate())]:
            s, t = DTensorSpec(mesh, a, tensor_meta=tm), DTensorSpec(mesh, b, tensor_meta=tm)
            got = cm.estimate_strategy_comms_cost(s, t)
            sa, tb = tuple(code[p] for p in a), tuple(code[p] for p in b)
            want = O.estimate_strategy_comms_cost(sa, shape, (10, 1), 4, tb, topo, dev)
            assert got == want or (np.isinf(got) and np.isinf(want)), (a, b, got, want)
            fwd = cm.redistribute_cost(s, t, [0, 1])
            want_fwd = O.redistribute_cost(sa, shape, (10, 1), 4, tb, topo, dev, [0, 1])
            assert fwd == want_fwd or (np.isinf(fwd) and np.isinf(want_fwd))
    assert cm.compute_read_write_time(2**40) == float(O.compute_read_write_time(2**40, dev))
    got = cm.collective_comm_cost("allreduce", 2**30, (2, 4), 1, devices_per_host=8)
    assert got == O.collective_comm_cost("allreduce", 2**30, topo, 1)
    from autoparallel_amd.cost_models.compute_estimation import _get_sharded_shape_stride

    spec = DTensorSpec(mesh, (Shard(0), Shard(1)), tensor_meta=TensorMeta(torch.Size((64, 36)), (36, 1), torch.float32))
    assert _get_sharded_shape_stride(spec) == ([32, 9], [36, 1])


def test_nccl_model_through_reference_api(mesh):
    """set_nccl_topo_config switches every entry point to the NCCL model; the
    reference's own tests call these functions the same way
    (tests/test_nccl_cost_model.py there)."""
    from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

    from autoparallel_amd import cost_models as cm
    from autoparallel_amd.cost_models import nccl_cost_model as ncm
    from oracle import nccl_oracle as N

    cm.configure(devices_per_host=8, device_name="AMD Instinct MI355X")
    cfg = cm.h100_topo_config(num_nodes=2)
    ocfg = N.h100_config(num_nodes=2)
    t = cm.derive_mesh_dim_topo(cfg, (2, 8), 0)
    ot = N.derive_dim_topo(ocfg, (2, 8), 0)
    assert (t.n_ranks, t.n_nodes, t.ppn, t.n_channels, t.bw_intra, t.bw_inter) == (
        ot.n_ranks, ot.n_nodes, ot.ppn, ot.n_channels, ot.bw_intra, ot.bw_inter)
    t16 = cm.derive_mesh_dim_topo(cfg, (16,), 0)
    o16 = N.derive_dim_topo(ocfg, (16,), 0)
    for nb in (1 << 12, (1 << 21) + 5, 1 << 30):
        assert np.isclose(ncm.nccl_allreduce_cost(nb, t16, cfg), N.collective_time(N.AR, nb, o16, ocfg), rtol=1e-12)
        assert np.isclose(ncm.nccl_allgather_cost(nb, t16, cfg), N.collective_time(N.AG, nb, o16, ocfg), rtol=1e-12)
        assert np.isclose(ncm.nccl_reduce_scatter_cost(nb, t16, cfg), N.collective_time(N.RS, nb, o16, ocfg), rtol=1e-12)
        assert np.isclose(ncm.nccl_all_to_all_cost(nb, t16, cfg), N.all_to_all_time(nb, o16, ocfg), rtol=1e-12)
    # a hand-made topology with no tuning-table row falls back to the algorithm loop
    odd = ncm.MeshDimTopo(24, 3, 8, 20.0, 50.0 / 16, 16)
    want = N.collective_time(N.AR, 1 << 30, N.DimTopo(24, 3, 8, 20.0, 50.0 / 16, 16), ocfg)
    assert np.isclose(ncm.nccl_allreduce_cost(1 << 30, odd, cfg), want, rtol=1e-12)
    # the module-level switch
    shape = (256, 512)
    tm = TensorMeta(torch.Size(shape), (512, 1), torch.bfloat16)
    topo, dev = O.Topo((2, 4), 8, nccl=N.h100_config(num_nodes=1)), O.DeviceLimit()
    code = {Replicate(): 0, Shard(0): 0x40, Shard(1): 0x41, Partial(): 0x80}
    try:
        cm.set_nccl_topo_config(cm.h100_topo_config(num_nodes=1))
        assert cm.get_nccl_topo_config() is not None
        for a in [(Shard(0), Shard(1)), (Partial(), Partial()), (Shard(1), Partial())]:
            for b in [(Replicate(), Replicate()), (Shard(1), Shard(0)), (Shard(0), Shard(0))]:
                s, tt = DTensorSpec(mesh, a, tensor_meta=tm), DTensorSpec(mesh, b, tensor_meta=tm)
                got = cm.estimate_strategy_comms_cost(s, tt)
                want = O.estimate_strategy_comms_cost(tuple(code[p] for p in a), shape, (512, 1), 2,
                                                      tuple(code[p] for p in b), topo, dev)
                assert (np.isinf(got) and np.isinf(want)) or np.isclose(got, want, rtol=1e-12), (a, b, got, want)
        got = cm.collective_comm_cost("allreduce", 1 << 26, (2, 4), 1)
        assert got == N.comm_cost("allreduce", 1 << 26, (2, 4), 1, N.h100_config(num_nodes=1))
    finally:
        cm.set_nccl_topo_config(None)
    alpha = cm.collective_comm_cost("allreduce", 1 << 26, (2, 4), 1, devices_per_host=8)
    assert alpha == O.collective_comm_cost("allreduce", 1 << 26, O.Topo((2, 4), 8), 1)
    # presets and detection
    assert cm.a100_topo_config().bw_intra == 87.7 and cm.gb200_topo_config().gpus_per_node == 72

    class _M:
        def size(self):
            return 16

    assert cm.detect_nccl_topo_config(_M(), device_name="AMD Instinct MI355X") is None
    h = cm.detect_nccl_topo_config(_M(), device_name="NVIDIA H100 80GB HBM3")
    assert (h.arch, h.num_nodes, h.gpus_per_node, h.has_nvswitch) == (cm.GpuArch.HOPPER, 2, 8, True)
    assert cm.detect_nccl_topo_config(_M(), device_name="NVIDIA GB200") is None  # 16 % 72 != 0


def test_runtime_cost_api_routes(mesh):
    """estimate_strategy_runtime_cost on fx nodes: a closed-form operator through
    its program, one without (cumsum) through the explicit route, a view for
    nothing, each against the oracle's roofline.  (The reference's own vectors
    are reproduced through this function in test_gpu_fx_dispatch.py.)"""
    from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
    from torch.distributed.tensor._op_schema import OpSpec
    from torch.distributed.tensor.placement_types import Replicate, Shard

    from autoparallel_amd import cost_models as cm, fx_programs

    cm.configure(devices_per_host=8, device_name="AMD Instinct MI355X")
    aten = torch.ops.aten
    graph = torch.fx.Graph()

    def ph(name, shape, dtype):
        n = graph.placeholder(name)
        n.meta["val"] = torch.empty(shape, dtype=dtype, device="meta")
        return n

    a, b = ph("a", (512, 256), torch.float32), ph("b", (256, 1024), torch.float32)
    mm = graph.call_function(aten.mm.default, (a, b))
    mm.meta["val"] = torch.empty((512, 1024), dtype=torch.float32, device="meta")

    def spec(n, plc):
        v = n.meta["val"]
        return DTensorSpec(mesh, plc, tensor_meta=TensorMeta(v.shape, v.stride(), v.dtype))

    dev = O.DeviceLimit()
    for pa, pb, (m_, k_, n_) in [((Replicate(), Replicate()), (Replicate(), Replicate()), (512, 256, 1024)),
                                 ((Shard(0), Replicate()), (Replicate(), Shard(1)), (256, 256, 256))]:
        st = OpSpec(spec(mm, pa), input_specs=[spec(a, pa), spec(b, pb)])
        cm.reset_compute_cost_cache()
        got = cm.estimate_strategy_runtime_cost(mm, st)
        want = O.roofline_cost(2 * m_ * k_ * n_, 4 * (m_ * k_ + k_ * n_ + m_ * n_), 1, dev)
        assert got == float(want)
    # explicit route
    x = ph("x", (4096, 4096), torch.bfloat16)
    cs = graph.call_function(aten.cumsum.default, (x, 1))
    cs.meta["val"] = torch.empty((4096, 4096), dtype=torch.bfloat16, device="meta")
    st = OpSpec(spec(cs, (Shard(0), Replicate())), input_specs=[spec(x, (Shard(0), Replicate()))])
    before = sum(fx_programs.fallback_ops.values())
    got = cm.estimate_strategy_runtime_cost(cs, st)
    assert sum(fx_programs.fallback_ops.values()) == before + 1
    assert got == float(O.roofline_cost(0, 2 * (2048 * 4096 * 2), 3, dev))
    # views cost nothing
    v = graph.call_function(aten.view.default, (x, [16, 256, 4096]))
    v.meta["val"] = torch.empty((16, 256, 4096), dtype=torch.bfloat16, device="meta")
    assert cm.estimate_strategy_runtime_cost(v, st) == 0


class _Stack(nn.Module):
    def __init__(self, n=3):
        super().__init__()
        self.layers = nn.ModuleList([nn.Linear(64, 64, bias=False) for _ in range(n)])

    def forward(self, x):
        for layer in self.layers:
            x = torch.relu(layer(x))
        return x


def test_repeated_subgraphs_on_joint_graph(mesh):
    """The reference's clustered mode (optimize_sharding.py:261-266): repeated
    layers share decision variables; the plan and its cost match the
    unclustered optimizer on identical layers."""
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    def graph():
        with FakeTensorMode():
            m, x = _Stack(), torch.randn(16, 32, 64)
            with contextlib.ExitStack() as stack:
                return aot_export_joint_with_descriptors(stack, m, (x,)).graph_module

    plain = ShardingOptimizer(graph(), mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    plain.get_solution()
    opt = ShardingOptimizer(graph(), mesh, devices_per_host=8, device_name="AMD Instinct MI355X",
                            repeated_subgraphs=True)
    assert opt.cluster_links, "three identical layers must produce links"
    for linked, root in opt.cluster_links.items():
        assert linked[1:] == root[1:] and linked[0] != root[0]
        assert str(opt.nodes[linked[0]].target) == str(opt.nodes[root[0]].target)
    # as in the reference, decision_vars holds the root keys only; a linked key is resolved through the links
    linked, root = next(iter(opt.cluster_links.items()))
    assert root in opt.decision_vars and linked not in opt.decision_vars
    with pytest.raises(KeyError):
        opt.decision_vars[linked]
    assert opt._resolve_decision_var(linked).key == root
    assert opt.pulp_variables[linked].index == opt.pulp_variables[root].index
    assert all(k[0] not in opt._cluster_linked_node_idxs for k in opt.decision_vars)
    sol = opt.get_solution()
    for v in opt._cluster_linked_node_idxs:
        r = opt._core.root[v]
        assert str(sol[opt.nodes[v]].output_specs) == str(sol[opt.nodes[int(r)]].output_specs)
    assert np.isclose(opt._core.objective_value, plain._core.objective_value, rtol=1e-6)
    assert len(opt.selected_keys) == opt._packed.num_edges  # root keys plus the expanded linked keys
    assert "total_cost:" in opt.get_log()
    # the export names the cluster of every repeated node (autoparallel/export_json.py:396-401):
    # a linked node carries its root's name, root and linked nodes share the cluster's number
    data = opt.get_json()
    by_name = {n["name"]: n for n in data["nodes"]}
    linked = [n for n in data["nodes"] if "cluster_root" in n]
    assert len(linked) == len(opt._cluster_linked_node_idxs) > 0
    for n in linked:
        root = by_name[n["cluster_root"]]
        assert "cluster_root" not in root and root["cluster_id"] == n["cluster_id"] and root["op"] == n["op"]
        assert root["placement"] == n["placement"]
    assert all({"name", "op"} <= set(n) for n in data["nodes"]) and {"total", "comm", "compute"} <= set(data["summary"])
    assert any(n.get("module_path") for n in data["nodes"]) and {n.get("phase") for n in data["nodes"]} >= {"forward", "backward"}


def test_prefetch_discount_on_joint_graph(mesh):
    """apply_prefetch_discount(0) (reference tests/test_prefetch_derived_sets.py:262-296):
    discounted variables have comm 0 and cost == compute + transition."""
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    opt = ShardingOptimizer(_joint_graph(), mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    before = {k: dv.comm_cost for k, dv in opt.decision_vars.items() if 0 < dv.comm_cost < float("inf")}
    assert before
    n = opt.apply_prefetch_discount(scale=0.0)
    assert n > 0
    zeroed = 0
    for k, dv in opt.decision_vars.items():
        if k in before and dv.comm_cost == 0.0:
            assert dv.cost == dv.compute_cost + dv.sharding_transition_cost
            zeroed += 1
    assert zeroed == n
    # the strategies' redistribute_cost rows follow the discount
    k = next(k for k in before if opt.decision_vars[k].comm_cost == 0.0)
    assert opt.strats[opt.nodes[k[0]]].strategies[k[2]].redistribute_cost[k[1]][k[3]] == 0.0


def test_an_optimizer_is_freed_with_its_last_reference(mesh):
    """The mappings the optimizer holds (decision_vars, cluster_links) refer back
    to it weakly: no reference cycle keeps its strategies and coefficient arrays
    alive until the cyclic collector next runs."""
    import gc
    import weakref

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    gm = _joint_graph()
    was = gc.isenabled()
    gc.disable()
    try:
        opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X",
                                repeated_subgraphs=True)
        dvs, ref = opt.decision_vars, weakref.ref(opt)
        key = next(iter(dvs))
        dv = dvs[key]  # a view handed out keeps the optimizer alive
        del opt
        assert ref() is not None and dv.cost == dvs[key].cost
        del dv
        assert ref() is None
        with pytest.raises(ReferenceError):
            len(dvs)
    finally:
        if was:
            gc.enable()


def test_rebuild_after_mutating_strategies(mesh):
    """_build_decision_vars is re-entrant (reference tests/test_paired_output_constraint.py:30-158):
    after removing one placement from a gradient node's strategies, the rebuilt
    ILP disables the parameter strategies without a partner and the solution
    never picks them."""
    from torch._functorch._aot_autograd import fx_utils

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    gm = _joint_graph()
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    param, grad = next((p, g) for p, g in fx_utils.get_param_and_grad_nodes(gm.graph).values() if g is not None)
    removed = str(opt.strats[grad].strategies[-1].output_specs.placements)
    n_before = len(opt.decision_vars)
    opt.strats[grad].strategies = [s for s in opt.strats[grad].strategies
                                   if str(s.output_specs.placements) != removed]
    opt.decision_vars = opt._build_decision_vars()
    assert len(opt.decision_vars) < n_before
    assert any("grad_param_constraint_disable" in name for name in opt.prob.constraints)
    sol = opt.get_solution()
    grad_plc = {str(s.output_specs.placements) for s in opt.strats[grad].strategies}
    chosen = str(sol[param].output_specs.placements)
    assert chosen in grad_plc and chosen != removed
    # every variable of the unmatched parameter strategy is zero
    pidx = opt.node_map[param]
    bad = [i for i, s in enumerate(opt.strats[param].strategies) if str(s.output_specs.placements) == removed]
    assert len(bad) == 1
    assert all(k[2] != bad[0] for k in opt.selected_keys if k[0] == pidx)
    # the reference's own sequence, statement by statement (tests/test_paired_output_constraint.py:58-62):
    # counters cleared, variables rebuilt, a new problem assigned, the default rows added to it
    rows = sorted(opt.prob.constraints)
    objective = opt.prob.objective_value
    opt.add_node_constraint(param, constraint_name="gone_with_the_old_problem")
    opt._name_counters.clear()
    opt.decision_vars = opt._build_decision_vars()
    opt.prob = object()  # pulp.LpProblem("AutoParallel", pulp.LpMinimize) there
    assert len(opt.prob.constraints) == 0 and opt._name_counters == {}
    opt.add_default_constraints()
    assert sorted(opt.prob.constraints) == rows  # the same rows under the same names, none twice
    sol2 = opt.get_solution()
    assert opt.prob.objective_value == objective
    assert {n.name: str(s.output_specs) for n, s in sol2.items()} == {n.name: str(s.output_specs) for n, s in sol.items()}
    # one group at a time, and counters that can be assigned (serialization.py:266)
    opt.prob = None
    opt._name_counters = {}
    for add in (opt.add_unique_decision_constraint, opt.add_same_output_across_args_constraint,
                opt.add_output_input_consistent_constraint, opt.add_inf_cost_constraint,
                opt.add_forward_backward_consistency_constraints, opt.add_grad_reduce_dtype_constraints):
        add()
    assert sorted(opt.prob.constraints) == rows


def test_joint_graph_with_symbolic_batch_is_planned_on_its_concrete_twin(mesh):
    """A joint graph traced with symbolic input sizes (the reference's dynamic=True,
    autoparallel/api.py:129-154) is planned on a twin with the sizes' hints
    (optimize_sharding.py:160-218): the same coefficients and the same plan as
    the graph traced with plain sizes, and a solution keyed by the nodes of the
    graph that was handed in."""
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.fx.experimental.symbolic_shapes import DimDynamic, ShapeEnv, StatelessSymbolicContext

    from autoparallel_amd.optimize_sharding import ShardingOptimizer, _has_symbolic_sizes

    mode = FakeTensorMode(shape_env=ShapeEnv(), static_shapes=False)
    with mode:
        m = MLP()
    meta = torch.empty(16, 32, 64, device="meta")
    x = mode.from_tensor(meta, symbolic_context=StatelessSymbolicContext(dynamic_sizes=[DimDynamic.DYNAMIC] * 3))
    with mode:
        x = x.to("cpu")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (x,)).graph_module
    assert _has_symbolic_sizes(gm)
    dyn = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    static = ShardingOptimizer(_joint_graph(), mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    # planned on the twin: its graph is not the one handed in, and the maps between the two are total
    assert dyn.graph is not gm.graph and set(dyn._concrete_to_orig.values()) == set(gm.graph.nodes)
    assert all(not isinstance(d, torch.SymInt) for n in dyn.graph.nodes if isinstance(n.meta.get("val"), torch.Tensor)
               for d in n.meta["val"].shape)
    sol_d, sol_s = dyn.get_solution(), static.get_solution()
    assert set(sol_d) <= set(gm.graph.nodes)  # keyed by the caller's nodes
    assert dyn._core.objective_value == static._core.objective_value
    from autoparallel_amd.optimize_sharding import _produces_tensor

    # the symbolic trace only adds size arithmetic (sym_size, products of sizes): nodes without a tensor, not planned
    ops = lambda opt: [str(n.target) for n in opt.graph.nodes if n.op == "call_function" and _produces_tensor(n.meta.get("val"))]
    assert ops(dyn) == ops(static) and len(list(dyn.graph.nodes)) > len(list(static.graph.nodes))
    assert len(dyn.decision_vars) == len(static.decision_vars)
    assert bits_equal(dyn._core.coef.cost, static._core.coef.cost) and bits_equal(dyn._core.coef.comm, static._core.coef.comm)
    by_name = lambda sol: [(str(n.target), str(s.output_specs)) for n, s in sol.items() if n.op == "call_function"]
    assert by_name(sol_d) == by_name(sol_s)


class _Block(nn.Module):
    """Embedding, layer norms, attention through scaled_dot_product_attention,
    a GELU MLP with biases: the op mix of a decoder block."""

    def __init__(self, d=64, h=4):
        super().__init__()
        self.h = h
        self.ln1, self.ln2 = nn.LayerNorm(d), nn.LayerNorm(d)
        self.qkv, self.o = nn.Linear(d, 3 * d, bias=False), nn.Linear(d, d, bias=False)
        self.up, self.down = nn.Linear(d, 4 * d), nn.Linear(4 * d, d)
        self.emb = nn.Embedding(128, d)

    def forward(self, tok):
        import torch.nn.functional as F

        x = self.emb(tok)
        b, s, d = x.shape
        q, k, v = self.qkv(self.ln1(x)).view(b, s, 3, self.h, d // self.h).permute(2, 0, 3, 1, 4)
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        x = x + self.o(a.transpose(1, 2).reshape(b, s, d))
        x = x + self.down(F.gelu(self.up(self.ln2(x))))
        return x.float().pow(2).mean()


def test_transformer_block_joint_graph(mesh):
    """A decoder block traced fwd+bwd: every coefficient the facade builds equals
    the oracle's on the same packed problem, and the plan solves."""
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    from autoparallel_amd.shardings import placement_options as PO

    # traced on fake tensors of the GPU, so that attention is the fused kernel
    # DTensor has a strategy for (the CPU kernel has none)
    with FakeTensorMode():
        with torch.device("cuda"):
            m = _Block()
        tok = torch.randint(0, 128, (8, 32), device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (tok,)).graph_module
    ops = {str(n.target) for n in gm.graph.nodes if n.op == "call_function"}
    assert any("scaled_dot_product" in o for o in ops) and any("layer_norm" in o for o in ops)
    assert any("embedding" in o for o in ops)
    PO.fallback_nodes.clear()
    PO.fallback_reasons.clear()
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    # no operator was left with the all-Replicate stand-in, and the norms offer
    # more than one strategy although their arguments have different numbers of candidates
    assert PO.fallback_nodes == [], PO.fallback_reasons
    ln = next(n for n in gm.graph.nodes if "native_layer_norm.default" in str(n.target))
    assert len(opt.strats[ln].strategies) > 1
    assert all(isinstance(s.output_specs, tuple) and len(s.output_specs) == 3 for s in opt.strats[ln].strategies)
    g = opt._packed
    ref = O.GraphOracle(g).build()
    slots = g.entry_slots()
    cost_ref, _ = O.clamp_inf(ref["cost"])
    assert g.num_entries > 10000
    assert bits_equal(opt._core.coef.comm, ref["comm"][slots])
    assert bits_equal(opt._core.coef.cost, cost_ref[slots])
    assert bits_equal(opt._core.coef.compute, ref["compute"])
    assert (ref["compute"] > 0).any()
    sol = opt.get_solution()
    assert set(sol) == {n for n in opt.nodes if n.op != "output"}
    assert np.isclose(opt._compute_solution_cost(sol)["total"], opt._core.objective_value, rtol=1e-9)


class _WithFactories(nn.Module):
    """Operators without tensor inputs next to ordinary ones."""

    def __init__(self):
        super().__init__()
        self.w = nn.Linear(64, 64, bias=False)

    def forward(self, x):
        pos = torch.arange(x.shape[1], device=x.device)
        bias = torch.full((32, 64), 0.5, device=x.device)
        mask = torch.zeros(16, 32, 64, device=x.device)
        y = self.w(x) + bias + mask
        return (y * pos[None, :, None].to(y.dtype)).sum()


def test_operators_without_tensor_inputs(mesh):
    """Factories get the Shard/Replicate product with a stand-in input spec and a
    zero row as long as the unfiltered product; generators are Replicate only
    (autoparallel/shardings/propagation_rules.py:412-554).  The coefficients of
    the whole graph equal the oracle's and the plan solves."""
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.tensor.placement_types import Replicate

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    with FakeTensorMode():
        m, x = _WithFactories(), torch.randn(16, 32, 64)
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (x,)).graph_module
    by_op = {}
    for n in gm.graph.nodes:
        if n.op == "call_function":
            by_op.setdefault(str(n.target), n)
    assert "aten.full.default" in by_op and "aten.zeros.default" in by_op and "aten.arange.default" in by_op
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    full = opt.strats[by_op["aten.full.default"]].strategies
    # rank 2 on a 2-dim mesh: (2 + 1)^2 combinations, all valid for (32, 64) on (2, 4)
    assert len(full) == 9 and all(len(s.redistribute_cost[0]) == 9 for s in full)
    assert all(s.input_specs[0] is s.output_specs for s in full)
    assert full[-1].output_specs.placements == (Replicate(), Replicate())
    zeros = opt.strats[by_op["aten.zeros.default"]].strategies
    assert len(zeros) == 16 and all(len(s.redistribute_cost[0]) == 16 for s in zeros)
    ar = opt.strats[by_op["aten.arange.default"]].strategies
    assert len(ar) == 1 and ar[0].output_specs.placements == (Replicate(), Replicate())
    assert ar[0].redistribute_cost == [[0.0]]
    g = opt._packed
    v = opt.node_map[by_op["aten.full.default"]]
    e = int(g.node_edge_off[v])
    assert g.node_nargs[v] == 1 and g.edge_src_node[e] < 0 and g.edge_ssrc[e] == 9
    ref = O.GraphOracle(g).build()
    slots = g.entry_slots()
    cost_ref, _ = O.clamp_inf(ref["cost"])
    assert bits_equal(opt._core.coef.comm, ref["comm"][slots])
    assert bits_equal(opt._core.coef.cost, cost_ref[slots])
    assert bits_equal(opt._core.coef.compute, ref["compute"])
    sol = opt.get_solution()
    assert set(sol) == {n for n in opt.nodes if n.op != "output"}
    assert np.isclose(opt._compute_solution_cost(sol)["total"], opt._core.objective_value, rtol=1e-9)


def test_hf_gpt2_small_joint_graph():
    """GPT-2 small as transformers defines it (12 layers, d 768, vocab 50257,
    random weights), batch 8 x 1024 tokens, forward and backward, on a mesh of 8:
    every operator gets DTensor strategies, every coefficient equals the
    oracle's, and the solved plan shards the large matrices."""
    transformers = pytest.importorskip("transformers")
    import torch.distributed as dist
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.device_mesh import init_device_mesh
    from torch.testing._internal.distributed.fake_pg import FakeStore

    from autoparallel_amd.optimize_sharding import ShardingOptimizer
    from autoparallel_amd.shardings import placement_options as PO

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")

    class Wrap(nn.Module):
        def __init__(self, lm):
            super().__init__()
            self.lm = lm

        def forward(self, ids):
            t = self.lm.transformer
            x = t.wte(ids) + t.wpe(torch.arange(ids.shape[1], device=ids.device))[None]
            for blk in t.h:
                out = blk(x)
                x = out[0] if isinstance(out, tuple) else out
            logits = self.lm.lm_head(t.ln_f(x))
            return torch.nn.functional.cross_entropy(
                logits[:, :-1].reshape(-1, logits.shape[-1]).float(), ids[:, 1:].reshape(-1))

    cfg = transformers.GPT2Config(attn_pdrop=0.0, embd_pdrop=0.0, resid_pdrop=0.0, use_cache=False,
                                  attn_implementation="sdpa")
    assert (cfg.n_layer, cfg.n_embd, cfg.n_head, cfg.vocab_size) == (12, 768, 12, 50257)
    with FakeTensorMode():
        torch.manual_seed(0)
        with torch.device("cuda"):
            m = Wrap(transformers.GPT2LMHeadModel(cfg))
        ids = torch.randint(0, cfg.vocab_size, (8, 1024), device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (ids,)).graph_module
    own_pg = not dist.is_initialized()
    if own_pg:
        dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=8)
    try:
        mesh8 = init_device_mesh("cpu", (8,))
        PO.fallback_nodes.clear()
        PO.fallback_reasons.clear()
        opt = ShardingOptimizer(gm, mesh8, devices_per_host=8, device_name="AMD Instinct MI355X")
        assert PO.fallback_nodes == [], PO.fallback_reasons
        g = opt._packed
        assert g.num_nodes > 1500 and g.num_entries > 15000
        ref = O.GraphOracle(g).build()
        slots = g.entry_slots()
        cost_ref, _ = O.clamp_inf(ref["cost"])
        assert bits_equal(opt._core.coef.comm, ref["comm"][slots])
        assert bits_equal(opt._core.coef.cost, cost_ref[slots])
        assert bits_equal(opt._core.coef.compute, ref["compute"])
        assert (ref["compute"] > 0).sum() > 300
        sol = opt.get_solution()
        # the objective counts a transition on an edge out of a tuple-valued producer
        # (autoparallel/optimize_sharding.py:470-477, through getitem), the reference's
        # scorer does not (:1099-1104, pred_spec is a tuple there)
        import operator

        uncounted = sum(
            1 for n, st in sol.items()
            if n.op == "call_function" and n.target is operator.getitem
            and sol[n.args[0]].output_specs[n.args[1]].placements != st.input_specs[0].placements)
        assert np.isclose(opt._compute_solution_cost(sol)["total"] + uncounted, opt._core.objective_value, rtol=1e-9)
        big = [n for n in sol if n.op == "placeholder" and n.meta["val"].ndim == 2
               and n.meta["val"].numel() in (768 * 3072, 768 * 2304)]
        assert len(big) == 12 * 3
        assert all(any(p.is_shard() for p in sol[n].output_specs.placements) for n in big)
    finally:
        if own_pg:
            dist.destroy_process_group()


def test_encoder_layer_with_dropout_joint_graph(mesh):
    """torch's TransformerEncoderLayer in training mode (dropout, whose DTensor
    rule refuses Partial arguments): no operator on the all-Replicate stand-in,
    coefficients equal to the oracle's, and the plan solves."""
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.optimize_sharding import ShardingOptimizer
    from autoparallel_amd.shardings import placement_options as PO

    class Enc(nn.Module):
        def __init__(self):
            super().__init__()
            self.layer = nn.TransformerEncoderLayer(64, 4, 128, dropout=0.1, batch_first=True)
            self.head = nn.Linear(64, 1)

        def forward(self, x):
            return self.head(self.layer(x)).mean()

    with FakeTensorMode():
        with torch.device("cuda"):
            m = Enc()
        x = torch.randn(8, 16, 64, device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (x,)).graph_module
    assert any("native_dropout" in str(n.target) for n in gm.graph.nodes)
    PO.fallback_nodes.clear()
    PO.fallback_reasons.clear()
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    assert PO.fallback_nodes == [], PO.fallback_reasons
    g = opt._packed
    ref = O.GraphOracle(g).build()
    slots = g.entry_slots()
    cost_ref, _ = O.clamp_inf(ref["cost"])
    assert bits_equal(opt._core.coef.comm, ref["comm"][slots])
    assert bits_equal(opt._core.coef.cost, cost_ref[slots])
    assert bits_equal(opt._core.coef.compute, ref["compute"])
    sol = opt.get_solution()
    assert set(sol) == {n for n in opt.nodes if n.op != "output"}


def test_collectives_stay_on_the_narrow_side_of_a_cast(mesh):
    """fp32 parameters cast to bf16 for compute, gradients cast back to fp32
    (what the reference's mixed-precision parametrization produces, with
    aten._to_copy standing in for its cast operator): no redistribution on the
    nodes before the forward cast, nor, when reduction is asked for in the wider
    dtype, on the backward cast and the single-input nodes that precede it
    (autoparallel/optimize_sharding.py:1487-1606)."""
    from torch._functorch._aot_autograd import fx_utils
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    class Mixed(nn.Module):
        def __init__(self):
            super().__init__()
            self.w1 = nn.Parameter(torch.randn(256, 128))
            self.w2 = nn.Parameter(torch.randn(128, 256))

        def forward(self, x):
            h = torch.relu(x @ self.w1.to(torch.bfloat16).t())
            return (h @ self.w2.to(torch.bfloat16).t()).float().pow(2).mean()

    with FakeTensorMode():
        with torch.device("cuda"):
            m = Mixed()
        x = torch.randn(64, 128, device="cuda", dtype=torch.bfloat16)
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (x,)).graph_module
    cast = torch.ops.aten._to_copy.default
    pairs = list(fx_utils.get_param_and_grad_nodes(gm.graph).values())
    assert len(pairs) == 2 and all(g is not None and g.target is cast for _, g in pairs)
    old = ShardingOptimizer.dtype_cast_targets
    ShardingOptimizer.dtype_cast_targets = {cast}
    try:
        plain = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
        wide = ShardingOptimizer(gm, mesh, True, devices_per_host=8, device_name="AMD Instinct MI355X")
    finally:
        ShardingOptimizer.dtype_cast_targets = old
    for opt in (plain, wide):
        roles = opt._packed.roles
        fwd = {opt.nodes[i] for i in roles.fwd_pre_cast}
        assert fwd == {next(iter(p.users)) for p, _ in pairs} and all(n.target is cast for n in fwd)
        bwd = {opt.nodes[i] for i in roles.bwd_pre_cast}
        # the cast and the transposes between it and the weight-gradient matmul, which stays out
        assert {g for _, g in pairs} <= bwd and {n.target for n in bwd} == {cast, torch.ops.aten.t.default}
        heads = [n for n in bwd if n.all_input_nodes[0] not in bwd]
        assert len(heads) == 2 and all(n.all_input_nodes[0].target is torch.ops.aten.mm.default for n in heads)
        names = list(opt.prob.constraints)
        n_fwd = sum(1 for n in names if n.startswith("fwd_param_dtype_"))
        n_bwd = sum(1 for n in names if n.startswith("grad_reduce_dtype_"))
        comm = opt._core.coef.comm
        keys = opt._packed.entry_keys()
        on = lambda idx: int(((comm > 0) & np.isin(keys[:, 0], list(idx))).sum())
        assert n_fwd == on(roles.fwd_pre_cast) > 0
        assert n_bwd == (on(roles.bwd_pre_cast) if opt is wide else 0)
        sol = opt.get_solution()
        for p, g in pairs:
            c = next(iter(p.users))
            assert sol[c].input_specs[0].placements == sol[p].output_specs.placements  # gathered after the cast
        if opt is wide:
            for n in bwd:  # reduced after the cast: nothing moves on the way to it
                assert sol[n].input_specs[0].placements == sol[n.all_input_nodes[0]].output_specs.placements


@pytest.mark.parametrize("clusters", [True, "extended"])
def test_reduction_after_the_cast_holds_for_repeated_layers_too(mesh, clusters):
    """With gradients reduced in the higher precision and repeated layers sharing their
    variables, no selected variable on the way from a weight-gradient matmul to its cast
    moves data, the expanded variables of linked layers included (the reference's
    tests/test_grad_reduce_dtype.py:147-171 with its check :53-125)."""
    from torch._functorch._aot_autograd import fx_utils
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    class Stacked(nn.Module):
        def __init__(self, n=4, d=128):
            super().__init__()
            self.ws = nn.ParameterList([nn.Parameter(torch.randn(d, d)) for _ in range(n)])

        def forward(self, x):
            for w in self.ws:
                x = torch.relu(x @ w.to(torch.bfloat16).t())
            return x.float().pow(2).mean()

    with FakeTensorMode():
        with torch.device("cuda"):
            m = Stacked()
        x = torch.randn(64, 128, device="cuda", dtype=torch.bfloat16)
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (x,)).graph_module
    cast = torch.ops.aten._to_copy.default
    old = ShardingOptimizer.dtype_cast_targets
    ShardingOptimizer.dtype_cast_targets = {cast}
    try:
        opt = ShardingOptimizer(gm, mesh, True, repeated_subgraphs=clusters, devices_per_host=8,
                                device_name="AMD Instinct MI355X")
    finally:
        ShardingOptimizer.dtype_cast_targets = old
    assert opt.cluster_links
    sol = opt.get_solution()
    checked = checked_linked = 0
    for param, grad in fx_utils.get_param_and_grad_nodes(gm.graph).values():
        assert grad is not None and grad.target is cast
        chain, n = [grad], grad  # the unary chain that ends in the gradient
        while len(n.all_input_nodes) == 1 and len(n.all_input_nodes[0].all_input_nodes) == 1:
            n = n.all_input_nodes[0]
            chain.append(n)
        at = next(i for i, c in enumerate(chain) if c.target is cast)
        before = {opt.node_map[c] for c in chain[at:] if c in opt.node_map}
        for key in opt.selected_keys:
            if key[0] in before:
                dv = opt._resolve_decision_var(key)
                checked += 1
                checked_linked += key in opt.cluster_links
                assert dv.comm_cost == 0, (opt.nodes[key[0]].name, dv.comm_cost)
        assert any(p.is_partial() for p in sol[chain[at]].output_specs.placements) or \
            all(p.is_replicate() for p in sol[param].output_specs.placements)
    assert checked > 0 and checked_linked > 0


def test_hf_gpt2_layers_under_the_default_memory_budget(mesh):
    """Two GPT-2 layers prepared as the reference prepares its graph (alias nodes)
    with the batch-sharded input and the default parameter budget of 1 / mesh size
    (autoparallel/api.py:371-382): every parameter ends fully sharded, the
    layer-norm weights too, whose gradients leave layer_norm_backward Partial and
    reach their Shard on the alias edge."""
    transformers = pytest.importorskip("transformers")
    from torch._functorch._aot_autograd.fx_utils import get_param_and_grad_nodes
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.tensor.placement_types import Replicate, Shard

    from autoparallel_amd.graph_utils import add_alias_nodes
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    class Wrap(nn.Module):
        def __init__(self, lm):
            super().__init__()
            self.lm = lm

        def forward(self, ids):
            t = self.lm.transformer
            x = t.wte(ids) + t.wpe(torch.arange(ids.shape[1], device=ids.device))[None]
            for blk in t.h:
                out = blk(x)
                x = out[0] if isinstance(out, tuple) else out
            logits = self.lm.lm_head(t.ln_f(x))
            return torch.nn.functional.cross_entropy(
                logits[:, :-1].reshape(-1, logits.shape[-1]).float(), ids[:, 1:].reshape(-1))

    cfg = transformers.GPT2Config(n_layer=2, attn_pdrop=0.0, embd_pdrop=0.0, resid_pdrop=0.0, use_cache=False,
                                  attn_implementation="sdpa")
    with FakeTensorMode():
        with torch.device("cuda"):
            m = Wrap(transformers.GPT2LMHeadModel(cfg))
        ids = torch.randint(0, cfg.vocab_size, (8, 1024), device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (ids,)).graph_module
    add_alias_nodes(gm)
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    opt.add_sharded_input_constraint([(Shard(0), Replicate())])
    opt.add_parameter_memory_constraint(0.0, 1.0 / mesh.size())
    sol = opt.get_solution()
    pairs = list(get_param_and_grad_nodes(gm.graph).values())
    assert len(pairs) >= 28
    for p, g in pairs:
        plc = sol[p].output_specs.placements
        assert all(x.is_shard() for x in plc), (p.name, plc)
        assert g.target is torch.ops.aten.alias.default and sol[g].output_specs.placements == plc
    norm_w = [p for p, g in pairs if p.meta["val"].shape == (768,)]
    assert len(norm_w) >= 10


def test_unsharded_runtime_estimate(mesh):
    """estimate_strategy_runtime_cost(node, None) prices the operator on its
    traced arguments (autoparallel/cost_models/compute_estimation.py:334-339,
    438-493): the same figure as the all-Replicate strategy, whose local shapes
    are the traced ones."""
    from autoparallel_amd.cost_models.compute_estimation import estimate_strategy_runtime_cost
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    gm = _joint_graph()
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    checked = 0
    for node in gm.graph.nodes:
        if node.op != "call_function" or node not in opt.strats:
            continue
        rep = [st for st in opt.strats[node].strategies
               if all(s is None or all(p.is_replicate() for p in s.placements) for s in st.input_specs)]
        if not rep:
            continue
        a, b = estimate_strategy_runtime_cost(node, None), estimate_strategy_runtime_cost(node, rep[0])
        assert a == b, (node, a, b)
        checked += a > 0
    assert checked >= 4


def test_graph_with_symbolic_sizes_is_planned_on_a_concrete_copy(mesh):
    """A graph whose batch size is symbolic: the planner works on a copy at the
    hinted sizes (autoparallel/optimize_sharding.py:162-189, 228-237) and gives
    the same coefficients and plan as the static graph; the plan comes back on
    the caller's nodes, and nodes of either graph are accepted."""
    import torch.fx as fx
    from torch._subclasses import FakeTensorMode
    from torch.distributed.tensor.placement_types import Replicate, Shard
    from torch.fx.experimental.symbolic_shapes import DimDynamic, ShapeEnv, StatelessSymbolicContext

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    aten = torch.ops.aten

    def build(symbolic):
        if symbolic:
            mode = FakeTensorMode(shape_env=ShapeEnv(), static_shapes=False)
            ctx = StatelessSymbolicContext(dynamic_sizes=[DimDynamic.DYNAMIC, DimDynamic.STATIC])
            xv = mode.from_tensor(torch.empty(64, 128, device="meta"), symbolic_context=ctx)
        else:
            mode = FakeTensorMode()
            xv = mode.from_tensor(torch.empty(64, 128, device="meta"))
        wv = mode.from_tensor(torch.empty(128, 256, device="meta"))
        g = fx.Graph()
        x, w = g.placeholder("x"), g.placeholder("w")
        x.meta["val"], w.meta["val"] = xv, wv
        with mode:
            h = g.call_function(aten.mm.default, (x, w))
            h.meta["val"] = aten.mm.default(xv, wv)
            r = g.call_function(aten.relu.default, (h,))
            r.meta["val"] = aten.relu.default(h.meta["val"])
            t = g.call_function(aten.sum.dim_IntList, (r, [1]))
            t.meta["val"] = aten.sum.dim_IntList(r.meta["val"], [1])
        g.output((t,))
        return fx.GraphModule(torch.nn.Module(), g)

    sym, static = build(True), build(False)
    assert isinstance(next(iter(sym.graph.nodes)).meta["val"].shape[0], torch.SymInt)
    a = ShardingOptimizer(sym, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    b = ShardingOptimizer(static, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    assert a.gm is not sym and a.orig_gm is sym and b.gm is static
    assert all(type(d) is int for n in a.graph.nodes for v in [n.meta.get("val")] if isinstance(v, torch.Tensor)
               for d in v.shape)
    assert a._packed.num_entries == b._packed.num_entries > 0
    assert bits_equal(a._core.coef.cost, b._core.coef.cost) and bits_equal(a._core.coef.comm, b._core.coef.comm)
    x_sym = next(iter(sym.graph.nodes))
    names = a.add_node_constraint(x_sym, (Shard(0), Replicate()))  # a node of the caller's graph
    b.add_node_constraint(next(iter(static.graph.nodes)), (Shard(0), Replicate()))
    sa, sb = a.get_solution(), b.get_solution()
    assert set(sa) == {n for n in sym.graph.nodes if n.op != "output"}  # keyed by the caller's nodes
    assert [str(sa[n].output_specs) for n in sym.graph.nodes if n.op != "output"] == \
        [str(sb[n].output_specs) for n in static.graph.nodes if n.op != "output"]
    assert sa[x_sym].output_specs.placements == (Shard(0), Replicate())
    assert a.get_strategy(x_sym) is a.strats[a._orig_to_concrete[x_sym]]
    assert np.isclose(a._compute_solution_cost(sa)["total"], b._compute_solution_cost(sb)["total"], rtol=1e-12)
    a.remove_constraints(names)
    assert set(a.resolve()) == set(sa)


def test_redistribute_cost_in_any_mesh_dim_order(mesh):
    """redistribute_cost(current, target, order) for every permutation of a 3-D
    mesh's dims and for orders that leave dims out, against the oracle's fold
    in that order (autoparallel/cost_models/collective_runtime_estimation.py:115-229):
    ascending and descending run on the device as they are, the others on the
    relabelled mesh."""
    import itertools

    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

    from autoparallel_amd.cost_models import collective_runtime_estimation as cre
    from autoparallel_amd.dtensor_bridge import placement_codes

    m3 = init_device_mesh("cpu", (2, 2, 2))
    cre.configure(4, "AMD Instinct MI355X")  # 4 per host: the outer dim crosses hosts, the inner two do not
    try:
        topo, dev = O.Topo((2, 2, 2), 4), O.DeviceLimit()
        metas = [((1024, 512, 64), (512 * 64, 64, 1)), ((1024, 512, 64), (64, 65536, 1))]  # contiguous, permuted
        R, P, S = Replicate(), Partial(), Shard
        pairs = [((S(0), S(1), P), (R, S(0), S(2))), ((P, P, S(1)), (S(0), R, R)), ((S(2), S(0), S(1)), (S(0), S(1), R)),
                 ((P, S(0), R), (R, R, S(0))), ((S(0), R, P), (S(0), P, R))]
        orders = [list(p) for p in itertools.permutations(range(3))] + [[1], [2, 0], [0, 2], []]
        checked = 0
        for shape, stride in metas:
            tm = TensorMeta(torch.Size(shape), stride, torch.bfloat16)
            for src, tgt in pairs:
                a, b = DTensorSpec(m3, src, tensor_meta=tm), DTensorSpec(m3, tgt, tensor_meta=tm)
                for order in orders:
                    got = cre.redistribute_cost(a, b, order)
                    want = O.redistribute_cost(placement_codes(src), shape, stride, 2, placement_codes(tgt), topo, dev, order)
                    assert got == want or (np.isinf(got) and np.isinf(want)), (src, tgt, order, got, want)
                    checked += np.isfinite(want) and want > 0
        assert checked > 60
        # the order changes the price: gathering before or after the reduce-scatter moves different volumes
        a, b = DTensorSpec(m3, pairs[0][0], tensor_meta=tm), DTensorSpec(m3, pairs[0][1], tensor_meta=tm)
        assert len({cre.redistribute_cost(a, b, o) for o in orders[:6]}) > 1
    finally:
        cre.configure(8, "AMD Instinct MI355X")


def test_measured_runtime_of_a_strategy(mesh):
    """benchmark_strategy_runtime_cost (autoparallel/cost_models/compute_estimation.py:496-529)
    runs the operator at the strategy's local sizes on the device: a matmul takes
    time, sharded or whole; a view takes none."""
    from autoparallel_amd.cost_models.compute_estimation import (
        benchmark_strategy_runtime_cost,
        estimate_strategy_runtime_cost,
    )
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    gm = _joint_graph()
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    mm = next(n for n in gm.graph.nodes if n.op == "call_function" and n.target is torch.ops.aten.mm.default)
    view = next(n for n in gm.graph.nodes if n.op == "call_function" and n.target is torch.ops.aten.view.default)
    sts = opt.strats[mm].strategies
    whole = next(s for s in sts if all(p.is_replicate() for sp in s.input_specs for p in sp.placements))
    t_whole = benchmark_strategy_runtime_cost(mm, whole)
    assert t_whole > 0 and benchmark_strategy_runtime_cost(mm, None) > 0
    assert benchmark_strategy_runtime_cost(view, opt.strats[view].strategies[0]) == 0
    assert estimate_strategy_runtime_cost(mm, whole) > 0
    from autoparallel_amd.cost_models.compute_estimation import compare_estimated_with_benchmarked_throughput

    sol = opt.get_solution()
    table = compare_estimated_with_benchmarked_throughput(gm.graph, sol)
    mms = [n for n in gm.graph.nodes if n.op == "call_function" and n.target is torch.ops.aten.mm.default]
    assert set(table) == set(mms)
    for real_us, est_us, tflops, peak, eff in table.values():
        assert real_us > 0 and est_us > 0 and peak == 157.3 and np.isclose(eff, tflops / peak)  # fp32 model


def test_hf_llama3_8b_layers_joint_graph():
    """Llama-3-8B as transformers defines it (d 4096, 32 query / 8 key-value heads,
    SwiGLU 14336, RMSNorm, rotary embedding, vocab 128256, bf16), four of its
    layers, batch 64 x 8192 tokens, forward and backward, on an (8, 8) mesh:
    every operator gets DTensor strategies (the layers after the first from the
    query cache), and every coefficient equals the oracle's."""
    transformers = pytest.importorskip("transformers")
    import torch.distributed as dist
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.device_mesh import init_device_mesh
    from torch.testing._internal.distributed.fake_pg import FakeStore

    from autoparallel_amd.optimize_sharding import ShardingOptimizer
    from autoparallel_amd.shardings import placement_options as PO

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")

    class Wrap(nn.Module):
        def __init__(self, lm):
            super().__init__()
            self.lm = lm

        def forward(self, ids):
            m = self.lm.model
            x = m.embed_tokens(ids)
            pos = torch.arange(ids.shape[1], device=ids.device)[None]
            pe = m.rotary_emb(x, pos)
            for layer in m.layers:
                out = layer(x, attention_mask=None, position_ids=pos, position_embeddings=pe)
                x = out[0] if isinstance(out, tuple) else out
            logits = self.lm.lm_head(m.norm(x))
            return torch.nn.functional.cross_entropy(
                logits[:, :-1].reshape(-1, logits.shape[-1]).float(), ids[:, 1:].reshape(-1))

    cfg = transformers.LlamaConfig(
        vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_hidden_layers=4, num_attention_heads=32,
        num_key_value_heads=8, max_position_embeddings=8192, rope_theta=500000.0, attention_dropout=0.0,
        use_cache=False, attn_implementation="sdpa")
    with FakeTensorMode():
        torch.manual_seed(0)
        torch.set_default_dtype(torch.bfloat16)
        try:
            with torch.device("cuda"):
                m = Wrap(transformers.LlamaForCausalLM(cfg))
        finally:
            torch.set_default_dtype(torch.float32)
        ids = torch.randint(0, cfg.vocab_size, (64, 8192), device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (ids,)).graph_module
    ops = {str(n.target) for n in gm.graph.nodes if n.op == "call_function"}
    assert any("scaled_dot_product" in o for o in ops) and "aten.silu.default" in ops and "aten.rsqrt.default" in ops
    had_pg = dist.is_initialized()
    if had_pg:  # the module's 8-rank fake group: this mesh needs 64
        dist.destroy_process_group()
    dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=64)
    try:
        mesh88 = init_device_mesh("cpu", (8, 8))
        PO.fallback_nodes.clear()
        PO.fallback_reasons.clear()
        PO.reset_placement_options_cache()
        opt = ShardingOptimizer(gm, mesh88, devices_per_host=8, device_name="AMD Instinct MI355X")
        assert PO.fallback_nodes == [], PO.fallback_reasons
        assert PO.strategy_cache_stats["hits"] > 2 * PO.strategy_cache_stats["misses"]
        g = opt._packed
        assert g.num_nodes > 900 and g.num_entries > 200000
        ref = O.GraphOracle(g).build()
        slots = g.entry_slots()
        cost_ref, _ = O.clamp_inf(ref["cost"])
        assert bits_equal(opt._core.coef.comm, ref["comm"][slots])
        assert bits_equal(opt._core.coef.cost, cost_ref[slots])
        assert bits_equal(opt._core.coef.compute, ref["compute"])
        # the first and the last layer's nodes got the same strategy sets
        mms = [n for n in gm.graph.nodes if n.op == "call_function" and n.target is torch.ops.aten.mm.default]
        per_layer = {}
        for n in mms:
            per_layer.setdefault(tuple(n.meta["val"].shape), []).append(len(opt.strats[n].strategies))
        assert all(len(set(v)) == 1 for v in per_layer.values())
        # With repeated_subgraphs only the first copy of every layer node is priced
        # (autoparallel/optimize_sharding.py:501-507): far fewer entries, the same
        # coefficients where both have them, and the same plan.
        PO.reset_placement_options_cache()
        clustered = ShardingOptimizer(gm, mesh88, devices_per_host=8, device_name="AMD Instinct MI355X",
                                      repeated_subgraphs=True)
        gc = clustered._packed
        assert gc.edge_alias is not None and gc.num_entries < 0.45 * g.num_entries
        assert len(clustered.decision_vars) == gc.num_entries == clustered._core.n_vars
        # what the reference asks of its clustering on such a model (tests/test_graph_clustering.py:231-297):
        # no region mixes forward and backward nodes, no node sits in two regions, the regions of a
        # group are as long as each other, and most of the graph is covered
        groups = clustered._core.region_groups
        assert groups
        seen = set()
        for group in groups:
            assert len(group) >= 2 and len({len(region) for region in group}) == 1
            for region in group:
                tags = {clustered.nodes[v].meta.get("partitioner_tag") for v in region} - {None}
                assert len(tags) <= 1, tags
                assert not (seen & set(region))
                seen |= set(region)
        n_ops = sum(1 for n in clustered.nodes if n.op == "call_function")
        assert len(seen) >= 0.5 * n_ops, (len(seen), n_ops)
        own = np.repeat(gc.priced, g.block_sizes())
        assert bits_equal(clustered._core.coef.comm, opt._core.coef.comm[own])
        assert bits_equal(clustered._core.coef.cost, opt._core.coef.cost[own])
        # a repeated node's strategies carry its root's redistribution rows (:554-571)
        v = int(np.nonzero(clustered._core.linked)[0][-1])
        r = int(clustered._core.root[v])
        for s_l, s_r, s_p in zip(clustered.strats[clustered.nodes[v]].strategies,
                                 clustered.strats[clustered.nodes[r]].strategies,
                                 opt.strats[opt.nodes[v]].strategies):
            assert s_l.redistribute_cost == s_r.redistribute_cost == s_p.redistribute_cost
        sol_c = clustered.get_solution()
        opt.get_solution()
        # Tying the layers together is a restriction of the free problem (here the first and the
        # last layer would rather differ from the middle ones): its optimum cannot be lower, and
        # its plan, expanded to every node, costs on the optimizer that priced every node exactly
        # what the clustered objective says (root cost x multiplicity).
        assert clustered._core.objective_value >= opt._core.objective_value * (1 - 1e-9)
        idx = torch.from_numpy(clustered._out_indices(sol_c).astype(np.int16).reshape(-1, 1)).cuda()
        r = opt._core.engine.score(idx).cpu().numpy()[0]
        assert r[5] == 0 and np.isclose(r[4], clustered._core.objective_value, rtol=1e-9)
        rc = clustered._core.engine.score(idx).cpu().numpy()[0]
        assert (rc[:4] == r[:4]).all() and np.isclose(rc[4], r[4], rtol=1e-12)
    finally:
        dist.destroy_process_group()
        if had_pg:
            dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=8)


def test_local_map_region_in_a_graph(mesh):
    """A graph with a local_map region (one declared strategy, zero compute, a
    non-tensor argument, an output without a spec): coefficients equal the
    oracle's, the region's inputs are redistributed to the declared placements,
    and the plan solves."""
    from torch.distributed.tensor.placement_types import Replicate, Shard

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    def call_local_map(*args):  # stands in for the higher-order operator; never run
        raise AssertionError

    aten = torch.ops.aten
    g = torch.fx.Graph()
    x, w = g.placeholder("x"), g.placeholder("w")
    x.meta["val"] = torch.empty(256, 64, device="meta")
    w.meta["val"] = torch.empty(64, 64, device="meta")
    h = g.call_function(aten.mm.default, (x, w))
    h.meta["val"] = torch.empty(256, 64, device="meta")
    region = g.call_function(call_local_map, (h, w, 3))
    region.meta["val"] = (torch.empty(256, 64, device="meta"), torch.empty(4, device="meta"))
    region.meta["local_map_kwargs"] = {"in_placements": ((Shard(0), Replicate()), (Replicate(), Replicate()), None),
                                       "out_placements": ((Shard(0), Replicate()),)}
    y = g.call_function(__import__("operator").getitem, (region, 0))
    y.meta["val"] = region.meta["val"][0]
    r = g.call_function(aten.relu.default, (y,))
    r.meta["val"] = torch.empty(256, 64, device="meta")
    g.output((r,))
    gm = torch.fx.GraphModule(torch.nn.Module(), g)
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    reg = region
    assert len(opt.strats[reg].strategies) == 1
    pk = opt._packed
    ref = O.GraphOracle(pk).build()
    slots = pk.entry_slots()
    cost_ref, _ = O.clamp_inf(ref["cost"])
    assert bits_equal(opt._core.coef.comm, ref["comm"][slots])
    assert bits_equal(opt._core.coef.cost, cost_ref[slots])
    v = opt.node_map[reg]
    o0 = int(pk.node_comp_off[v])
    assert opt._core.coef.compute[o0] == 0.0  # a region is not priced (not an OpOverload)
    # the edge from the matmul into the region: free only from producer strategies that are (S(0), R) up to a local slice
    e = int(pk.node_edge_off[v])
    block = opt._core.coef.comm[opt._core.var_start[e]:opt._core.var_start[e + 1]]
    src = [s.output_specs.placements for s in opt.strats[h].strategies]
    tgt = (Shard(0), Replicate())
    free = [all(a == b or (a.is_replicate() and b.is_shard()) for a, b in zip(p, tgt)) for p in src]  # R -> S is a local slice
    assert [c == 0.0 for c in block] == free and not all(free) and sum(free) >= 2
    sol = opt.get_solution()
    assert sol[h].output_specs.placements == (Shard(0), Replicate())
    assert sol[r].output_specs.placements == (Shard(0), Replicate())


def test_hf_llama_linears_as_einsums():
    """Two layers of the traced Llama-3-8B with its linear layers rewritten as
    einsums, the way the reference prepares a joint graph before planning
    (autoparallel/api.py:208): no matmul is left, the einsums are offered
    strategies that shard batch and sequence on different mesh dims, nothing
    falls back, and every coefficient equals the oracle's."""
    transformers = pytest.importorskip("transformers")
    import torch.distributed as dist
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.tensor.placement_types import Shard
    from torch.testing._internal.distributed.fake_pg import FakeStore

    from autoparallel_amd.graph_utils import replace_view_mm_view_with_einsum
    from autoparallel_amd.optimize_sharding import ShardingOptimizer
    from autoparallel_amd.shardings import placement_options as PO

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")

    class Wrap(nn.Module):
        def __init__(self, lm):
            super().__init__()
            self.lm = lm

        def forward(self, ids):
            m = self.lm.model
            x = m.embed_tokens(ids)
            pos = torch.arange(ids.shape[1], device=ids.device)[None]
            pe = m.rotary_emb(x, pos)
            for layer in m.layers:
                out = layer(x, attention_mask=None, position_ids=pos, position_embeddings=pe)
                x = out[0] if isinstance(out, tuple) else out
            logits = self.lm.lm_head(m.norm(x))
            return torch.nn.functional.cross_entropy(
                logits[:, :-1].reshape(-1, logits.shape[-1]).float(), ids[:, 1:].reshape(-1))

    n_layers = 2
    cfg = transformers.LlamaConfig(
        vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_hidden_layers=n_layers,
        num_attention_heads=32, num_key_value_heads=8, max_position_embeddings=8192, rope_theta=500000.0,
        attention_dropout=0.0, use_cache=False, attn_implementation="sdpa")
    with FakeTensorMode():
        torch.set_default_dtype(torch.bfloat16)
        try:
            with torch.device("cuda"):
                m = Wrap(transformers.LlamaForCausalLM(cfg))
        finally:
            torch.set_default_dtype(torch.float32)
        ids = torch.randint(0, cfg.vocab_size, (64, 8192), device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (ids,)).graph_module
    n_mm = len(gm.graph.find_nodes(op="call_function", target=torch.ops.aten.mm.default))
    # seven linear layers per block and the head; each with its input and its weight gradient
    assert n_mm == 3 * (7 * n_layers + 1)
    assert replace_view_mm_view_with_einsum(gm) == n_mm
    assert not gm.graph.find_nodes(op="call_function", target=torch.ops.aten.mm.default)
    eins = gm.graph.find_nodes(op="call_function", target=torch.ops.aten.einsum.default)
    assert sorted({n.args[0] for n in eins}) == ["abk,kn->abn", "abn,abk->kn"]
    had_pg = dist.is_initialized()
    if had_pg:
        dist.destroy_process_group()
    dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=64)
    try:
        mesh88 = init_device_mesh("cpu", (8, 8))
        PO.fallback_nodes.clear()
        PO.fallback_reasons.clear()
        PO.reset_placement_options_cache()
        opt = ShardingOptimizer(gm, mesh88, devices_per_host=8, device_name="AMD Instinct MI355X")
        assert PO.fallback_nodes == [], PO.fallback_reasons
        for n in eins:
            activations = {s.input_specs[0].placements for s in opt.strats[n].strategies}
            assert (Shard(0), Shard(1)) in activations and (Shard(1), Shard(0)) in activations, n
        g = opt._packed
        ref = O.GraphOracle(g).build()
        slots = g.entry_slots()
        cost_ref, _ = O.clamp_inf(ref["cost"])
        assert bits_equal(opt._core.coef.comm, ref["comm"][slots])
        assert bits_equal(opt._core.coef.cost, cost_ref[slots])
        assert bits_equal(opt._core.coef.compute, ref["compute"])
        sol = opt.get_solution()
        assert all(n in sol for n in eins)
    finally:
        dist.destroy_process_group()
        if had_pg:
            dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=8)
