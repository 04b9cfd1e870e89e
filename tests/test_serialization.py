"""Save / load on the packed layout and the log formatter (host logic, CPU).
Coefficients come from the oracle; tests/test_gpu_export.py checks the device
export of the same arrays."""
import json

import numpy as np
import pytest
import torch

from autoparallel_amd import graphgen, serialization
from autoparallel_amd.log_formatting import format_sharding_log
from autoparallel_amd.sharding_problem import Coefficients, PackedShardingOptimizer
from oracle import cost_oracle as O


def oracle_twin(g):
    """(keys, vals, compute, per_arg) as the reference's save_optimizer lays
    them out (serialization.py:145-161): decision_vars order, vals = (per-arg
    compute, comm, transition)."""
    r = O.GraphOracle(g).build()
    per_arg = np.zeros(g.num_compute)
    for v in range(g.num_nodes):
        o0, S = int(g.node_comp_off[v]), int(g.node_nstrat[v])
        per_arg[o0:o0 + S] = r["compute"][o0:o0 + S] / int(g.node_nargs[v])
    order = g.decision_var_order()
    keys = g.entry_keys()[order]
    slots = g.entry_slots()[order]
    comp_base = g.node_comp_off[keys[:, 0]] + keys[:, 2]
    vals = np.stack([per_arg[comp_base], r["comm"][slots], r["transition"][slots].astype(np.float64)], axis=1)
    return keys, vals, r["compute"], per_arg, r


@pytest.fixture(scope="module")
def tiny():
    g = graphgen.gpt2_graph((4,), n_layers=1, dim=64, n_heads=2, ffn_dim=128, vocab=256, seq=32, batch=8)
    keys, vals, compute, per_arg, raw = oracle_twin(g)
    coef = Coefficients.from_decision_var_arrays(g, keys, vals, compute, per_arg)
    return g, coef, raw


def test_twin_rebuilds_the_coefficients(tiny):
    g, coef, raw = tiny
    slots = g.entry_slots()
    cost, bad = O.clamp_inf(raw["cost"])
    assert np.array_equal(coef.comm, raw["comm"][slots])
    assert np.array_equal(coef.cost, cost[slots])  # compute + comm + transition, then the inf rewrite
    assert np.array_equal(coef.flags, (raw["transition"] | (bad << 1)).astype(np.uint8)[slots])
    # any row order is accepted; a duplicate or foreign key is not
    keys, vals = coef.saved_arrays
    perm = np.random.default_rng(0).permutation(len(keys))
    again = Coefficients.from_decision_var_arrays(g, keys[perm], vals[perm], coef.compute, coef.per_arg)
    assert np.array_equal(again.cost, coef.cost)
    dup = keys.copy()
    dup[1] = dup[0]
    with pytest.raises(RuntimeError):
        Coefficients.from_decision_var_arrays(g, dup, vals, coef.compute, coef.per_arg)
    far = keys.copy()
    far[0, 3] = 10**6
    with pytest.raises(RuntimeError):
        Coefficients.from_decision_var_arrays(g, far, vals, coef.compute, coef.per_arg)


def test_save_load_roundtrip(tiny, tmp_path):
    g, coef, _ = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    param = g.roles.param_grad[0][0]
    opt.add_node_constraint(param, (0x40,))
    opt.add_parameter_memory_constraint(0.0, 1.0)
    opt._memory_constraint = None  # needs device local shapes; the log entry is what is under test
    sol = opt.get_solution()
    path = str(tmp_path / "opt.npz")
    opt.save(path)
    with np.load(path, allow_pickle=False) as d:  # plain arrays only
        assert d["dv_costs_keys"].dtype == np.int32 and d["dv_costs_keys"].shape == (g.num_entries, 4)
        assert d["dv_costs_vals"].dtype == np.float64 and d["dv_costs_vals"].shape == (g.num_entries, 3)
        assert all(v.dtype != object for v in d.values())
    loaded = PackedShardingOptimizer.load(path)
    # same structure (the reference's test_save_load_roundtrip: node and variable counts survive)
    assert loaded.g.num_nodes == g.num_nodes and loaded.n_vars == opt.n_vars
    assert loaded.g.node_names == g.node_names
    assert np.array_equal(loaded.coef.cost, opt.coef.cost) and np.array_equal(loaded.coef.comm, opt.coef.comm)
    for f in ("lists", "tuple_plc", "edge_off", "prog", "default_vals", "node_comp_off"):
        assert np.array_equal(getattr(loaded.g, f), getattr(g, f))
    assert loaded.g.roles == g.roles
    # constraint log replayed verbatim, not expanded
    assert [m for m, _ in loaded._constraint_log] == ["add_node_constraint", "add_parameter_memory_constraint"]
    assert set(loaded.prob.constraints) == set(opt.prob.constraints)
    # solution preserved (test_save_load_preserves_solution), and re-solving gives the same plan
    assert np.array_equal(np.sort(loaded.selected), np.sort(opt.selected))
    assert np.array_equal(loaded._extract(), sol)
    assert np.isclose(loaded.objective_value, opt.objective_value, rtol=1e-12)
    loaded._memory_constraint = None
    assert np.array_equal(loaded.resolve(), sol)
    # what code written for the reference reads on the object it loaded (its tests/test_serialization.py:136-168,
    # 183-190): node and variable counts, a mesh stand-in with the shape, the selected keys, variables by key
    assert len(loaded.nodes) == len(opt.nodes) == g.num_nodes and loaded.nodes == list(g.node_names)
    assert len(loaded.decision_vars) == len(opt.decision_vars) == g.num_entries
    assert loaded.mesh.shape == tuple(int(x) for x in g.mesh_shape) and loaded.mesh.ndim == len(g.mesh_shape)
    assert loaded.mesh.size() == int(np.prod(g.mesh_shape)) and loaded.mesh.mesh_dim_names is None
    keys = loaded.selected_keys
    assert len(keys) == g.num_edges and {k[0] for k in keys} == set(range(g.num_nodes))
    assert all(loaded.decision_vars[k].value == 1.0 and k in loaded.decision_vars for k in keys)
    total = sum(loaded.decision_vars[k].cost for k in keys)
    assert np.isclose(total, loaded.objective_value, rtol=1e-12)
    order = list(loaded.decision_vars)
    assert order == sorted(order, key=lambda k: (k[0], k[2], k[1], k[3])) and len(order) == g.num_entries
    k0 = order[len(order) // 2]
    dv = loaded.decision_vars[k0]
    assert dv.cost == dv.comm_cost + dv.compute_cost + dv.sharding_transition_cost or dv.cost == 10000.0
    for bad in ((g.num_nodes, 0, 0, 0), (0, 99, 0, 0), (k0[0], k0[1], 10**6, 0), "x"):
        assert bad not in loaded.decision_vars
        with pytest.raises(KeyError):
            loaded.decision_vars[bad]


def test_memory_ratios_travel_with_the_file(tiny, tmp_path):
    """A problem under a parameter-memory budget is saved with the local/global size of every
    parameter strategy and solved again from the file alone.  Here the ratios are the oracle's
    (sharded_shape_stride); tests/test_gpu_parity.py checks the device's against the same."""
    g, coef, _ = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    params = [p for p, _ in g.roles.param_grad]
    mesh = [int(x) for x in g.mesh_shape]
    for p in params:
        run, r = int(g.node_out_list[p]), []
        for o in range(int(g.node_nstrat[p])):
            w = int(g.lists[run + o])
            rk = int(g.meta_rank[w >> 12])
            shape = [int(x) for x in g.meta_shape[w >> 12, :rk]]
            local, _ = O.sharded_shape_stride(shape, [1] * rk, [int(x) for x in g.tuple_plc[w & 0xFFF, : g.ndim]], mesh)
            r.append(np.prod(local) / np.prod(shape))
        opt._memory_ratio_cache[p] = np.asarray(r)
    opt.add_parameter_memory_constraint(0.0, 0.0)  # every parameter at its smallest ratio
    sol = opt.get_solution()
    assert all(opt._memory_ratio_cache[p][sol[p]] == opt._memory_ratio_cache[p].min() for p in params)
    path = str(tmp_path / "budget.npz")
    opt.save(path)
    back = PackedShardingOptimizer.load(path)
    assert set(back._memory_ratio_cache) == set(params)
    assert all(np.array_equal(back._memory_ratio_cache[p], opt._memory_ratio_cache[p]) for p in params)
    assert np.array_equal(back.resolve(), sol) and "memory_constraint_high" in back.prob.constraints
    # without the ratios the budget rows need the device: no silent stand-in
    back._memory_ratio_cache = {}
    if not torch.cuda.is_available():
        with pytest.raises(Exception):
            back.resolve()


def test_load_takes_the_reference_argument_order_too(tiny, tmp_path):
    from autoparallel_amd import serialization

    g, coef, _ = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    path = str(tmp_path / "o.npz")
    serialization.save_optimizer(opt, path)
    a = serialization.load_optimizer(path)
    b = serialization.load_optimizer(PackedShardingOptimizer, path)  # load_optimizer(cls, path) there
    c = serialization.load_optimizer(path, object)  # a class that is not the packed one: the packed one is made
    assert type(a) is type(b) is type(c) is PackedShardingOptimizer and a.n_vars == b.n_vars == c.n_vars == opt.n_vars


def test_mesh_placeholder_known_answers():
    from autoparallel_amd.sharding_problem import MeshPlaceholder

    m = MeshPlaceholder((32, 8), ("dp", "tp"))
    assert m.shape == (32, 8) and m.mesh_dim_names == ("dp", "tp") and m.ndim == 2 and m.size() == 256
    m = MeshPlaceholder((64,), None)
    assert m.mesh_dim_names is None and m.ndim == 1 and m.size() == 64


def test_unsolved_save_and_version_check(tiny, tmp_path):
    g, coef, _ = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    path = str(tmp_path / "unsolved.npz")
    opt.save(path)
    loaded = PackedShardingOptimizer.load(path)
    assert loaded.selected is None
    assert len(loaded.get_solution()) == g.num_nodes
    with np.load(path) as d:
        arrays = dict(d)
    arrays["version"] = np.asarray(99)
    bad = str(tmp_path / "bad.npz")
    np.savez(bad, **arrays)
    with pytest.raises(RuntimeError, match="Unsupported save file version"):
        PackedShardingOptimizer.load(bad)


def test_placements_roundtrip(tiny, tmp_path):
    g, coef, _ = tiny
    opt = PackedShardingOptimizer(g, coefficients=coef)
    sol = opt.get_solution()
    path = str(tmp_path / "plc.json")
    serialization.save_placements(opt, sol, path, ["dp"])
    d = json.load(open(path))
    assert d["version"] == 1 and d["mesh_shape"] == [4] and len(d["placements"]) == g.num_nodes
    back = serialization.load_placements(opt, path, ["dp"])
    # the first strategy with the same placement strings: same placements as the solution
    for v in range(g.num_nodes):
        assert opt.output_placement_str(v, int(back[v])) == opt.output_placement_str(v, int(sol[v]))
        assert opt.input_placement_strs(v, int(back[v])) == opt.input_placement_strs(v, int(sol[v]))
    with pytest.raises(RuntimeError, match="Mesh dim names mismatch"):
        serialization.load_placements(opt, path, ["tp"])
    d["placements"]["no_such_node"] = {"output": "R", "inputs": []}
    json.dump(d, open(path, "w"))
    with pytest.raises(RuntimeError, match="not found in current graph"):
        serialization.load_placements(opt, path, ["dp"])
    d["placements"].pop("no_such_node")
    first = next(iter(d["placements"]))
    d["placements"][first]["output"] = "S(63)"
    json.dump(d, open(path, "w"))
    with pytest.raises(RuntimeError, match="not found in available strategies"):
        serialization.load_placements(opt, path, ["dp"])
    d["mesh_shape"] = [8]
    json.dump(d, open(path, "w"))
    with pytest.raises(RuntimeError, match="Mesh shape mismatch"):
        serialization.load_placements(opt, path, ["dp"])


# --- log formatter: the reference's own known answers (tests/test_log_formatting.py:47-148) ---
class _Strat:
    def __init__(self, name):
        self.name = name

    def __str__(self):
        return self.name


class _Entry:
    def __init__(self, name, comm=0.0, compute=0.0, transition=0.0):
        self.strategy = _Strat(name)
        self.comm_cost, self.compute_cost, self.sharding_transition_cost = comm, compute, transition
        self.cost = comm + compute + transition


def test_log_simple_graph_known_answers():
    class M(torch.nn.Module):
        def forward(self, x):
            return x + 1

    graph = torch.fx.symbolic_trace(M()).graph
    x, add, _ = list(graph.nodes)
    text = format_sharding_log(graph, {x: [_Entry("Replicate()")], add: [_Entry("Shard(0)", comm=1.0, compute=2.0)]})
    assert "# placement=Replicate()" in text and "# placement=Shard(0)" in text
    assert "cost=[(1.0, 2.0, 0.0)]" in text
    assert "total_cost: 3.00" in text and "comm_cost: 1.00" in text
    assert "compute_cost: 2.00" in text and "transition_cost: 0.00" in text
    # the annotation sits on the line that assigns the node
    line = next(ln for ln in text.split("\n") if ln.lstrip().startswith("add ="))
    assert "# placement=Shard(0)" in line


def test_log_multiple_ops_and_accumulation():
    class M(torch.nn.Module):
        def forward(self, x, y):
            a = x + y
            return a * 2

    graph = torch.fx.symbolic_trace(M()).graph
    x, y, add, mul, _ = list(graph.nodes)
    text = format_sharding_log(graph, {x: [_Entry("Replicate()")], y: [_Entry("Shard(0)")],
                                       add: [_Entry("Shard(0)", compute=1.0)], mul: [_Entry("Shard(0)", compute=0.5)]})
    assert text.count("# placement=Shard(0)") == 3 and "# placement=Replicate()" in text
    assert "total_cost: 1.50" in text and "compute_cost: 1.50" in text

    class S(torch.nn.Module):
        def forward(self, x):
            return x + 1

    graph = torch.fx.symbolic_trace(S()).graph
    x, add, _ = list(graph.nodes)
    text = format_sharding_log(graph, {x: [_Entry("R", 1.0, 2.0, 0.5)], add: [_Entry("S", 3.0, 4.0, 1.5)]},
                               violated_constraints_log="violated: foo")
    assert "total_cost: 12.00" in text and "comm_cost: 4.00" in text
    assert "compute_cost: 6.00" in text and "transition_cost: 2.00" in text
    assert text.endswith("violated: foo")
    # several variables per node (one per argument) are all listed
    text = format_sharding_log(graph, {add: [_Entry("S", 1.0, 0.5), _Entry("S", 2.0, 0.5)]})
    assert "cost=[(1.0, 0.5, 0.0), (2.0, 0.5, 0.0)]" in text and "total_cost: 4.00" in text
