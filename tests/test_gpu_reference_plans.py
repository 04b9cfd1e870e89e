"""The solved plans the reference's own tests expect
(tests/test_optimize_placement.py:67-299 there), reproduced through
ShardingOptimizer on this stack: same models, sizes, meshes (256 ranks, 8 per
host, planning device H100 with its NCCL model, as that suite's patches and the
default cost model set it up), same constraints, and the joint graph prepared
with alias nodes as the reference prepares it.  The expected placements below
are that file's expectations, not this repository's output."""
import contextlib

import pytest
import torch
import torch.nn as nn
from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

pytestmark = pytest.mark.gpu


class FFN(nn.Module):
    def __init__(self, dim1, dim2):
        super().__init__()
        self.linear1 = nn.Linear(dim1, dim2, bias=False)
        self.linear2 = nn.Linear(dim2, dim1, bias=False)

    def forward(self, x, y):
        return y + 2, self.linear2(self.linear1(x)), y + 2


class TransformerBlock(nn.Module):
    def __init__(self, nheads, dim1, dim2):
        super().__init__()
        self.nheads = nheads
        self.wq, self.wk, self.wv, self.wo = (nn.Linear(dim1, dim1, bias=False) for _ in range(4))
        self.w1, self.w2 = nn.Linear(dim1, dim2, bias=False), nn.Linear(dim2, dim1, bias=False)

    def forward(self, x):
        heads = lambda t: t.unflatten(-1, (self.nheads, -1)).permute(0, 2, 1, 3)
        o = nn.functional.scaled_dot_product_attention(heads(self.wq(x)), heads(self.wk(x)), heads(self.wv(x)))
        o0 = self.wo(o.permute(0, 2, 1, 3).flatten(-2)) + x
        return o0 + self.w2(torch.relu(self.w1(o0)))


@pytest.fixture(scope="module")
def meshes():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import torch.distributed as dist
    from torch.distributed.device_mesh import init_device_mesh
    from torch.testing._internal.distributed.fake_pg import FakeStore

    from autoparallel_amd.cost_models import get_nccl_topo_config, set_nccl_topo_config

    if dist.is_initialized():
        dist.destroy_process_group()
    dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=256)
    before = get_nccl_topo_config()
    yield (init_device_mesh("cpu", (256,), mesh_dim_names=("dp",)),
           init_device_mesh("cpu", (32, 8), mesh_dim_names=("dp", "tp")))
    set_nccl_topo_config(before)
    dist.destroy_process_group()


def _optimizer(mesh, model_type, high_mem):
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.cost_models import detect_nccl_topo_config, set_nccl_topo_config
    from autoparallel_amd.graph_utils import add_alias_nodes
    from autoparallel_amd.optimize_sharding import ShardingOptimizer
    from autoparallel_amd.shardings import placement_options as PO

    lead = mesh.shape[0]
    with FakeTensorMode():
        with torch.device("cuda"):
            m = FFN(1024, 4096) if model_type == "ffn" else TransformerBlock(48, 6144, 6144 * 4)
        if model_type == "ffn":
            xs = (torch.randn(2048 * lead, 1024, device="cuda"), torch.randn(2048 * lead, 1, device="cuda"))
        else:
            xs = (torch.randn(8 * lead, 256, 6144, device="cuda", requires_grad=True),)
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, xs).graph_module
    add_alias_nodes(gm)
    set_nccl_topo_config(detect_nccl_topo_config(mesh, "H100"))
    PO.fallback_nodes.clear()
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="H100")
    assert PO.fallback_nodes == [], PO.fallback_reasons
    batch = (Shard(0),) + (Replicate(),) * (mesh.ndim - 1)
    n_in, n_out = (2, 3) if model_type == "ffn" else (1, 1)
    opt.add_sharded_input_constraint([batch] * n_in)
    opt.add_sharded_output_constraint([batch] * n_out)
    opt.add_parameter_memory_constraint(0, 1.0 / mesh.size() if high_mem is None else high_mem)  # api.py:371-382
    return gm, opt


def _mm_nodes(gm):
    return [n for n in gm.graph.nodes if n.op == "call_function" and n.target is torch.ops.aten.mm.default]


@pytest.mark.parametrize("model_type", ["ffn", "transformer_block"])
@pytest.mark.parametrize("high_mem", [None, 1.0])
def test_fsdp_and_ddp_on_one_mesh_dim(meshes, model_type, high_mem):
    """tests/test_optimize_placement.py:100-183: parameters sharded (budget 1/256)
    or replicated (budget 1), forward matmuls batch-sharded with the whole weight,
    weight gradients Partial, input gradients batch-sharded."""
    from torch._functorch._aot_autograd.fx_utils import get_param_nodes

    gm, opt = _optimizer(meshes[0], model_type, high_mem)
    sol = opt.get_solution()
    want = (Shard(0),) if high_mem is None else (Replicate(),)
    for node in get_param_nodes(gm.graph):
        assert sol[node].output_specs.placements == want
    mms = _mm_nodes(gm)
    n_fwd = 2 if model_type == "ffn" else 6
    assert len(mms) == (5 if model_type == "ffn" else 18)
    for node in mms[:n_fwd]:
        p = sol[node]
        assert (p.input_specs[0].placements, p.input_specs[1].placements, p.output_specs.placements) == \
            ((Shard(0),), (Replicate(),), (Shard(0),))
    for node in mms[n_fwd::2]:  # weight gradients
        p = sol[node]
        assert (p.input_specs[0].placements, p.input_specs[1].placements, p.output_specs.placements) == \
            ((Shard(1),), (Shard(0),), (Partial("sum"),))
    for node in mms[n_fwd + 1::2]:  # input gradients
        p = sol[node]
        assert (p.input_specs[0].placements, p.input_specs[1].placements, p.output_specs.placements) == \
            ((Shard(0),), (Replicate(),), (Shard(0),))


_S, _R, _P = Shard, Replicate(), Partial("sum")
# matmul placements (input 0, input 1, output) of tests/test_optimize_placement.py:189-192
_MM1 = ((_S(0), _R), (_R, _S(1)), (_S(0), _S(1)))
_MM2 = ((_S(0), _S(1)), (_R, _S(0)), (_S(0), _P))
_MM3 = ((_S(1), _R), (_S(0), _S(1)), (_P, _S(1)))
_MM4 = ((_S(1), _S(0)), (_S(0), _R), (_P, _S(0)))
_EXPECTED_2D = {  # :186-233
    "ffn": ([(_S(0), _S(0)), (_S(0), _S(1))], [_MM1, _MM2, _MM3, _MM1, _MM4]),
    "transformer_block": (
        [(_S(0), _S(0))] * 3 + [(_S(0), _S(1)), (_S(0), _S(0)), (_S(0), _S(1))],
        [_MM1, _MM1, _MM1, _MM2, _MM1, _MM2, _MM3, _MM1, _MM4, _MM2, _MM3, _MM1, _MM4, _MM2, _MM4, _MM2, _MM4, _MM2]),
}


@pytest.mark.parametrize("model_type", ["ffn", "transformer_block"])
def test_fsdp_with_tensor_parallel_on_two_mesh_dims(meshes, model_type):
    """tests/test_optimize_placement.py:236-299: every parameter's placement,
    every matmul's input and output placements, and attention sharded on batch
    and heads."""
    from torch._functorch._aot_autograd.fx_utils import get_param_nodes

    gm, opt = _optimizer(meshes[1], model_type, None)
    sol = opt.get_solution()
    params, mms = _EXPECTED_2D[model_type]
    got = [sol[n].output_specs.placements for n in get_param_nodes(gm.graph)]
    assert got == params
    got = [(sol[n].input_specs[0].placements, sol[n].input_specs[1].placements, sol[n].output_specs.placements)
           for n in _mm_nodes(gm)]
    assert got == mms
    sdpa = [n for n in gm.graph.nodes if n.op == "call_function"
            and n.target is torch.ops.aten._scaled_dot_product_efficient_attention.default]
    assert len(sdpa) == (0 if model_type == "ffn" else 1)
    for node in sdpa:
        p = sol[node]
        assert [s.placements for s in p.input_specs[:3]] == [(_S(0), _S(1))] * 3
        assert p.output_specs[0].placements == (_S(0), _S(1))


class _TwoLinear(nn.Module):
    def __init__(self, dim1, dim2, bias):
        super().__init__()
        self.linear1, self.linear2 = nn.Linear(dim1, dim2, bias=bias), nn.Linear(dim2, dim1, bias=bias)

    def forward(self, x):
        return self.linear2(torch.relu(self.linear1(x)))


def _two_linear(mesh, dim1=1024, dim2=4096, bias=False, rows=None, memory=True):
    """Model, constraints and defaults of tests/test_optimize_placement.py:518-556, 598-655."""
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.cost_models import detect_nccl_topo_config, set_nccl_topo_config
    from autoparallel_amd.graph_utils import add_alias_nodes
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    with FakeTensorMode():
        with torch.device("cuda"):
            m = _TwoLinear(dim1, dim2, bias)
        x = torch.rand((2048 if rows is None else rows) * mesh.shape[0], dim1, device="cuda", requires_grad=True)
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (x,)).graph_module
    add_alias_nodes(gm)
    set_nccl_topo_config(detect_nccl_topo_config(mesh, "H100"))
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="H100")
    batch = (Shard(0),) + (Replicate(),) * (mesh.ndim - 1)
    opt.add_sharded_input_constraint([batch])
    opt.add_sharded_output_constraint([batch])
    if memory:
        opt.add_parameter_memory_constraint(0.0, 1.0 / mesh.size())
    return gm, opt


def test_memory_budget_with_a_parameter_that_does_not_divide(meshes):
    """:518-556: a bias of 280 elements on 256 ranks cannot be sharded all the
    way; the budget takes each parameter's best achievable ratio, so the problem
    stays feasible."""
    from torch._functorch._aot_autograd.fx_utils import get_param_nodes

    gm, opt = _two_linear(meshes[1], 1024, 280, bias=True, rows=8)
    sol = opt.get_solution()
    params = get_param_nodes(gm.graph)
    assert len(params) == 4 and all(p in sol for p in params)


def test_parameter_smaller_than_the_mesh_stays_replicated(meshes):
    """:559-595: a parameter of 128 elements on 256 ranks."""
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._functorch._aot_autograd.fx_utils import get_param_nodes
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.graph_utils import add_alias_nodes
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    class Model(nn.Module):
        def __init__(self, dim):
            super().__init__()
            self.param = nn.Parameter(torch.rand(dim))

        def forward(self, x):
            return x + self.param

    mesh = meshes[0]
    with FakeTensorMode():
        with torch.device("cuda"):
            m = Model(128)
        x = torch.rand(512, 128, device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (x,)).graph_module
    add_alias_nodes(gm)
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="H100")
    opt.add_sharded_input_constraint([(Shard(0),)])
    opt.add_sharded_output_constraint([(Shard(0),)])
    opt.add_parameter_memory_constraint(0.0, 1.0 / mesh.size())
    sol = opt.get_solution()
    for node in get_param_nodes(gm.graph):
        assert sol[node].output_specs.placements == (Replicate(),)


@pytest.mark.parametrize("memory_first", [True, False])
def test_node_constraint_is_left_out_of_the_memory_budget(meshes, memory_first):
    """:598-696: a parameter forced to Replicate does not make the sharding budget
    infeasible, whichever constraint was added first, on the first solve and on a
    re-solve."""
    from torch._functorch._aot_autograd.fx_utils import get_param_nodes

    gm, opt = _two_linear(meshes[0], memory=False)
    node = get_param_nodes(gm.graph)[0]
    if memory_first:
        opt.add_parameter_memory_constraint(0.0, 1.0 / 256)
        opt.add_node_constraint(node, placement=(Replicate(),))
    else:
        opt.add_node_constraint(node, placement=(Replicate(),))
        opt.add_parameter_memory_constraint(0.0, 1.0 / 256)
    assert opt.get_solution()[node].output_specs.placements == (Replicate(),)
    assert opt.resolve()[node].output_specs.placements == (Replicate(),)


def test_constraints_added_and_removed_between_solves(meshes):
    """:699-843: a node constraint added after a solve is honoured by resolve();
    removing it puts the parameter back under the budget (sharded again);
    removing the memory rows by name keeps them from being rebuilt."""
    from torch._functorch._aot_autograd.fx_utils import get_param_nodes

    gm, opt = _two_linear(meshes[0])
    params = get_param_nodes(gm.graph)
    sol = opt.get_solution()
    assert all(sol[p].output_specs.placements == (Shard(0),) for p in params)
    names = opt.add_node_constraint(params[0], placement=(Replicate(),))
    assert opt.resolve()[params[0]].output_specs.placements == (Replicate(),)
    opt.remove_constraints(names)
    assert opt.resolve()[params[0]].output_specs.placements == (Shard(0),)
    opt.remove_constraints(["memory_constraint_high", "memory_constraint_low"])
    opt.resolve()
    assert "memory_constraint_high" not in opt.prob.constraints
    assert "memory_constraint_low" not in opt.prob.constraints


def test_tensor_created_in_the_graph_and_a_buffer(meshes):
    """The model of tests/test_optimize_placement.py:302-335 (a tensor made by
    torch.full inside forward, a registered buffer): the factory gets its
    Shard/Replicate product, the buffer is planned like an input, and the plan
    solves with the batch-sharded input."""
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.graph_utils import add_alias_nodes
    from autoparallel_amd.optimize_sharding import ShardingOptimizer
    from autoparallel_amd.shardings import placement_options as PO

    dim = 128

    class Model(nn.Module):
        def __init__(self):
            super().__init__()
            self.linear = nn.Linear(dim, dim)
            self.register_buffer("buf", torch.empty(dim))

        def forward(self, x):
            x = x + torch.full([256, 256, 6144], 0, dtype=torch.bfloat16, device=x.device).sum()
            return self.linear(x) + self.buf

    mesh = meshes[0]
    with FakeTensorMode():
        with torch.device("cuda"):
            m = Model()
        x = torch.rand(512, dim, device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (x,)).graph_module
    add_alias_nodes(gm)
    PO.fallback_nodes.clear()
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="H100")
    assert PO.fallback_nodes == [], PO.fallback_reasons
    full = next(n for n in gm.graph.nodes if n.op == "call_function" and n.target is torch.ops.aten.full.default)
    sts = opt.strats[full].strategies
    # rank 3 on one mesh dim: Shard(0), Shard(1), Shard(2), Replicate; 256 ranks split 256, 256 and 6144
    assert [s.output_specs.placements for s in sts] == [(Shard(0),), (Shard(1),), (Shard(2),), (Replicate(),)]
    assert all(s.output_specs.tensor_meta.dtype == torch.bfloat16 and len(s.redistribute_cost[0]) == 4 for s in sts)
    opt.add_sharded_input_constraint([(Shard(0),)])
    opt.add_sharded_output_constraint([(Shard(0),)])
    sol = opt.get_solution()
    assert sol[full].output_specs.placements != (Replicate(),)  # 200 MB of zeros are cheaper to make in shards
    inputs = [n for n in gm.graph.nodes if n.op == "placeholder"]
    assert len(inputs) >= 4 and all(n in sol for n in inputs)


def test_constant_tensor_attribute_of_the_graph(meshes):
    """tests/test_optimize_placement.py:470-516: a constant made by new_tensor is
    an attribute of the traced graph; it gets placements like any input and, being
    eight elements broadcast over the batch, ends up Replicate."""
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.graph_utils import add_alias_nodes
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    class Model(nn.Module):
        def __init__(self):
            super().__init__()
            self.linear = nn.Linear(256, 1024)

        def forward(self, x):
            y = x.new_tensor([0, 1, 2, 3, 4, 5, 6, 7])[None, :, None]
            return self.linear(x) + y

    mesh = meshes[0]
    with FakeTensorMode(allow_non_fake_inputs=True):
        with torch.device("cuda"):
            m = Model()
        x = torch.rand(8 * 256, 8, 256, device="cuda", requires_grad=True)
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (x,)).graph_module
    add_alias_nodes(gm)
    consts = [n for n in gm.graph.nodes if n.op == "get_attr"]
    assert consts, [n.op for n in gm.graph.nodes]
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="H100")
    opt.add_parameter_memory_constraint(0.0, 1.0 / mesh.size())
    opt.add_sharded_input_constraint([(Shard(0),)])
    opt.add_sharded_output_constraint([(Shard(0),)])
    sol = opt.get_solution()
    for node in consts:
        assert node in sol and sol[node].output_specs.placements == (Replicate(),)
