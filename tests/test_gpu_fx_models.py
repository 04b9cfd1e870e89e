"""Small models of the reference's own end-to-end tests, traced the way the
reference traces (its decomposition choices, autoparallel/tracing.py:14-36) and
planned through ShardingOptimizer: the permute / LayerNorm / permute block with
its non-contiguous strides, torch.arange (prims.iota), advanced indexing
(index / index_put with a None among the indices), an MLP with biases (addmm
taken apart so that the matmul can be sharded) (tests/test_propagation_rules.py:15-193)."""
import contextlib
import copy

import numpy as np
import pytest
import torch
import torch.nn as nn

from helpers import bits_equal
from oracle import cost_oracle as O

pytestmark = pytest.mark.gpu


def reference_style_decompositions():
    from torch._inductor.decomposition import select_decomp_table

    aten = torch.ops.aten
    table = copy.copy(select_decomp_table())
    for op in (aten.full_like.default, aten.empty_like.default, aten.threshold_backward.default,
               aten.native_layer_norm.default, aten.embedding_dense_backward.default,
               aten.native_layer_norm_backward.default, aten._softmax_backward_data.default, aten._softmax.default,
               aten.stack.default, aten.addmm.default):
        table.pop(op, None)
    table[aten.addmm.default] = lambda self, mat1, mat2, beta=1, alpha=1: self + mat1 @ mat2
    return table


class PermuteLayerNorm(nn.Module):
    def __init__(self):
        super().__init__()
        self.norm = nn.LayerNorm(96, eps=1e-6)

    def forward(self, x):  # (N, C, H, W) -> (N, H, W, C) -> norm over C -> back
        return self.norm(x.permute(0, 2, 3, 1)).permute(0, 3, 1, 2)


class ArangeEmbedding(nn.Module):
    def __init__(self):
        super().__init__()
        self.embed = nn.Embedding(256, 64)

    def forward(self, x):
        return x + self.embed(torch.arange(x.shape[1], device=x.device))


class IndexPut(nn.Module):
    def __init__(self):
        super().__init__()
        self.weight = nn.Parameter(torch.randn(32, 64))

    def forward(self, x):
        out = torch.zeros_like(x)
        idx = torch.arange(x.shape[1], device=x.device)
        out[:, idx] = x[:, idx]
        return out @ self.weight


class BiasedMLP(nn.Module):
    def __init__(self):
        super().__init__()
        self.a, self.b = nn.Linear(64, 128), nn.Linear(128, 64)

    def forward(self, x):
        return self.b(torch.nn.functional.gelu(self.a(x)))


class ConvBatchNorm(nn.Module):
    def __init__(self):
        super().__init__()
        self.c1, self.bn, self.c2 = nn.Conv2d(3, 32, 3, padding=1), nn.BatchNorm2d(32), nn.Conv2d(32, 64, 3, stride=2, padding=1)
        self.fc = nn.Linear(64, 10)

    def forward(self, x):
        x = torch.relu(self.c2(torch.relu(self.bn(self.c1(x)))))
        return self.fc(x.mean((2, 3)))


CASES = {
    # model, input shape, operators the trace must hold, nodes that get the all-Replicate stand-in
    "permute_layer_norm": (PermuteLayerNorm, (256, 96, 56, 56), ("aten.permute.default", "aten.native_layer_norm.default"), set()),
    "arange_embedding": (ArangeEmbedding, (256, 256, 64), ("prims.iota.default", "aten.embedding.default"), set()),
    # torch 2.10's index_put rule takes no None index (index.Tensor is planned from its run-time rule)
    "index_put": (IndexPut, (256, 32), ("aten.index_put.default", "aten.index.Tensor"), {"index_put"}),
    "biased_mlp": (BiasedMLP, (64, 128, 64), ("aten.mm.default", "aten.add.Tensor"), set()),
    # convolution (batch-parallel rule), batch norm taken apart into var_mean / squeeze.dims / pointwise
    "conv_batch_norm": (ConvBatchNorm, (64, 3, 32, 32), ("aten.convolution.default", "aten.convolution_backward.default",
                                                          "aten.var_mean.correction", "aten.squeeze.dims"), set()),
}


@pytest.fixture(scope="module")
def meshes():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import torch.distributed as dist
    from torch.distributed.device_mesh import init_device_mesh
    from torch.testing._internal.distributed.fake_pg import FakeStore

    own = not dist.is_initialized()
    if own:
        dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=8)
    yield {"1d": init_device_mesh("cpu", (8,)), "2d": init_device_mesh("cpu", (2, 4))}
    if own:
        dist.destroy_process_group()


@pytest.mark.parametrize("mesh_name", ["1d", "2d"])
@pytest.mark.parametrize("case", list(CASES))
def test_reference_style_trace_is_planned(meshes, case, mesh_name):
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.optimize_sharding import ShardingOptimizer
    from autoparallel_amd.shardings import placement_options as PO

    cls, shape, must_have, stand_ins = CASES[case]
    with FakeTensorMode():
        model, x = cls(), torch.rand(*shape)
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, model, (x,), decompositions=reference_style_decompositions()).graph_module
    targets = {str(n.target) for n in gm.graph.nodes if n.op == "call_function"}
    assert set(must_have) <= targets, targets
    assert "aten.addmm.default" not in targets
    PO.fallback_nodes.clear()
    PO.fallback_reasons.clear()
    opt = ShardingOptimizer(gm, meshes[mesh_name], devices_per_host=8, device_name="AMD Instinct MI355X")
    assert set(PO.fallback_reasons) == stand_ins, PO.fallback_reasons
    # every coefficient against the oracle on the same packed problem
    g = opt._packed
    ref = O.GraphOracle(g).build()
    slots = g.entry_slots()
    cost_ref, _ = O.clamp_inf(ref["cost"])
    assert bits_equal(opt._core.coef.comm, ref["comm"][slots]) and bits_equal(opt._core.coef.cost, cost_ref[slots])
    sol = opt.get_solution()
    assert set(sol) == {n for n in opt.nodes if n.op != "output"}
    assert np.isfinite(opt._core.objective_value) and not opt._core.prob.violated()
    # a node with the stand-in is Replicate on every mesh dim, inputs and output
    for n, spec in sol.items():
        if n.name in stand_ins:
            assert all(p.is_replicate() for p in spec.output_specs.placements)


def test_uneven_shards_are_offered_and_can_be_forced(meshes):
    """A weight dim that the mesh dim does not divide is still offered sharded on it
    while every shard is non-empty (the reference's tests/test_dynamic_shapes.py:1537-1640,
    remove_invalid_configs: the local size is a ceiling division), and the plan can be
    pinned to such a placement."""
    from torch._functorch._aot_autograd.fx_utils import get_param_nodes
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.tensor.placement_types import Replicate, Shard

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    class FFN(nn.Module):
        def __init__(self, d1, d2):
            super().__init__()
            self.w1, self.w2 = nn.Linear(d1, d2, bias=False), nn.Linear(d2, d1, bias=False)

        def forward(self, x):
            return self.w2(torch.relu(self.w1(x)))

    mesh = meshes["2d"]  # (2, 4)
    d1, d2 = 102, 400    # 102 = 4 * 25 + 2: uneven on the second mesh dim, every shard non-empty
    with FakeTensorMode():
        model, x = FFN(d1, d2), torch.randn(16, d1)
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, model, (x,), decompositions=reference_style_decompositions()).graph_module
    opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    w1 = get_param_nodes(gm.graph)[0]
    assert tuple(w1.meta["val"].shape) == (d2, d1)
    on_tp = {s.output_specs.placements[1].dim for s in opt.strats[w1].strategies if s.output_specs.placements[1].is_shard()}
    assert on_tp == {0, 1}
    # a dim smaller than the mesh dim is not offered: 3 rows cannot fill 4 shards
    with FakeTensorMode():
        tiny, xt = FFN(3, 400), torch.randn(16, 3)
        with contextlib.ExitStack() as stack:
            gt = aot_export_joint_with_descriptors(stack, tiny, (xt,), decompositions=reference_style_decompositions()).graph_module
    ot = ShardingOptimizer(gt, mesh, devices_per_host=8, device_name="AMD Instinct MI355X")
    wt = get_param_nodes(gt.graph)[0]
    assert {s.output_specs.placements[1].dim for s in ot.strats[wt].strategies if s.output_specs.placements[1].is_shard()} == {0}
    # pinned to the uneven placement, the plan is found and the weight's bytes are those of the ceiling shard
    opt.add_node_constraint(w1, (Replicate(), Shard(1)))
    sol = opt.get_solution()
    assert sol[w1].output_specs.placements == (Replicate(), Shard(1))
    g = opt._packed
    ref = O.GraphOracle(g).build()
    assert bits_equal(opt._core.coef.comm, ref["comm"][g.entry_slots()])


# ---------------------------------------------------------------------------
# Architectures of the transformers library at toy sizes: encoder, encoder-decoder,
# vision, grouped-query decoder, mixture of experts.
# ---------------------------------------------------------------------------
def _hf_cases():
    import transformers as T

    small = dict(hidden_size=128, num_hidden_layers=2, num_attention_heads=4, intermediate_size=256, vocab_size=512,
                 max_position_embeddings=128)
    return {
        "bert": (T.BertConfig, T.BertForMaskedLM, dict(hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0, **small), torch.float32),
        "t5": (T.T5Config, T.T5ForConditionalGeneration,
               dict(d_model=128, d_kv=32, d_ff=256, num_layers=2, num_heads=4, vocab_size=512, dropout_rate=0.0), torch.float32),
        "vit": (T.ViTConfig, T.ViTForImageClassification,
                dict(hidden_size=128, num_hidden_layers=2, num_attention_heads=4, intermediate_size=256, image_size=32,
                     patch_size=8, hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0), torch.float32),
        "mistral": (T.MistralConfig, T.MistralForCausalLM, dict(num_key_value_heads=2, sliding_window=None, **small), torch.float32),
        "mixtral": (T.MixtralConfig, T.MixtralForCausalLM,
                    dict(num_key_value_heads=2, num_local_experts=4, num_experts_per_tok=2, **small), torch.bfloat16),
    }


class _HFLoss(nn.Module):
    def __init__(self, model, kind):
        super().__init__()
        self.m, self.kind = model, kind

    def forward(self, x):
        if self.kind in ("mistral", "mixtral"):  # the decoder layers themselves: no mask is built from data
            m = self.m.model
            h = m.embed_tokens(x)
            pos = torch.arange(x.shape[1], device=x.device)[None]
            pe = m.rotary_emb(h, pos)
            for layer in m.layers:
                o = layer(h, attention_mask=None, position_ids=pos, position_embeddings=pe)
                h = o[0] if isinstance(o, tuple) else o
            logits = self.m.lm_head(m.norm(h))
        elif self.kind == "vit":
            logits = self.m(pixel_values=x).logits
        elif self.kind == "t5":
            logits = self.m(input_ids=x, decoder_input_ids=x).logits
        else:
            logits = self.m(input_ids=x).logits
        return logits.float().pow(2).mean()


# operators for which torch 2.10 registers no strategy (they get the all-Replicate stand-in)
_NO_STRATEGY_IN_THIS_TORCH = {"aten.select_scatter.default"}


@pytest.mark.parametrize("kind", ["bert", "t5", "vit", "mistral", "mixtral"])
def test_transformers_architectures_are_planned(meshes, kind):
    pytest.importorskip("transformers")
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    from autoparallel_amd.optimize_sharding import ShardingOptimizer
    from autoparallel_amd.shardings import placement_options as PO

    cfg_cls, model_cls, kwargs, dtype = _hf_cases()[kind]
    cfg = cfg_cls(**kwargs)
    cfg.use_cache = False
    cfg._attn_implementation = "sdpa"
    with FakeTensorMode():
        torch.set_default_dtype(dtype)
        try:
            with torch.device("cuda"):
                model = _HFLoss(model_cls(cfg), kind)
        finally:
            torch.set_default_dtype(torch.float32)
        x = torch.rand(8, 3, 32, 32, device="cuda") if kind == "vit" else torch.randint(0, 512, (8, 64), device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, model, (x,)).graph_module
    PO.fallback_nodes.clear()
    PO.fallback_reasons.clear()
    opt = ShardingOptimizer(gm, meshes["2d"], devices_per_host=8, device_name="AMD Instinct MI355X")
    by_name = {n.name: n for n in opt.nodes}
    assert {str(by_name[k].target) for k in PO.fallback_reasons} <= _NO_STRATEGY_IN_THIS_TORCH, PO.fallback_reasons
    g = opt._packed
    assert g.num_nodes > 300 and g.num_entries > 40000
    ref = O.GraphOracle(g).build()
    slots = g.entry_slots()
    cost_ref, _ = O.clamp_inf(ref["cost"])
    assert bits_equal(opt._core.coef.comm, ref["comm"][slots]) and bits_equal(opt._core.coef.cost, cost_ref[slots])
    assert bits_equal(opt._core.coef.compute, ref["compute"])
    sol = opt.get_solution()
    assert set(sol) == {n for n in opt.nodes if n.op != "output"} and not opt._core.prob.violated()


@pytest.mark.parametrize("kind,clusters", [("bert", True), ("mistral", True), ("mixtral", True),
                                           ("mistral", "extended"), ("bert", "extended")])
def test_the_whole_planning_sequence_on_architectures(meshes, kind, clusters, tmp_path):
    """What a caller of the reference does around the planner, in its order: linear layers as
    einsums, alias nodes, repeated layers sharing variables, the batch-sharded input pinned, the
    default parameter budget, solve, the log and the export, save and reopen."""
    pytest.importorskip("transformers")
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.tensor.placement_types import Replicate, Shard

    from autoparallel_amd.graph_utils import add_alias_nodes, replace_view_mm_view_with_einsum
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    cfg_cls, model_cls, kwargs, dtype = _hf_cases()[kind]
    cfg = cfg_cls(**kwargs)
    cfg.use_cache = False
    cfg._attn_implementation = "sdpa"
    with FakeTensorMode():
        torch.set_default_dtype(dtype)
        try:
            with torch.device("cuda"):
                model = _HFLoss(model_cls(cfg), kind)
        finally:
            torch.set_default_dtype(torch.float32)
        x = torch.randint(0, 512, (8, 64), device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, model, (x,)).graph_module
    mesh = meshes["2d"]
    assert replace_view_mm_view_with_einsum(gm) > 10
    add_alias_nodes(gm)
    opt = ShardingOptimizer(gm, mesh, repeated_subgraphs=clusters, devices_per_host=8,
                            device_name="AMD Instinct MI355X")
    assert opt._cluster_linked_node_idxs
    opt.add_sharded_input_constraint([(Shard(0), Replicate())])
    opt.add_parameter_memory_constraint(0.0, 1.0 / mesh.size())
    plan = opt.get_solution()
    ids = next(n for n in opt.nodes if n.op == "placeholder" and type(n.meta.get("desc")).__name__ == "PlainAOTInput")
    assert plan[ids].output_specs.placements == (Shard(0), Replicate())
    assert "total_cost:" in opt.get_log() and "Violated constraints: []" in opt.get_log()
    data = opt.get_json()
    assert abs(data["summary"]["total"] - sum(data["summary"][k] for k in ("comm", "compute", "transition"))) < 1e-6
    assert sum("cluster_root" in n for n in data["nodes"]) == len(opt._cluster_linked_node_idxs)
    opt.save(str(tmp_path / "o.npz"))
    again = type(opt).load(str(tmp_path / "o.npz"))
    assert np.isclose(again.objective_value, opt._core.objective_value, rtol=1e-12)
    assert len(again.decision_vars) == len(opt.decision_vars) and len(again.selected_keys) == len(opt.selected_keys)
    opt.save_placements(str(tmp_path / "p.json"))
    back = opt.load_placements(str(tmp_path / "p.json"))
    assert all(str(back[n].output_specs) == str(plan[n].output_specs) for n in plan)


def test_regions_of_different_groups_that_meet(meshes):
    """The vision model's backward holds small repeated chains (a bias gradient: view, sum, view)
    whose producers belong to regions of another group, rooted elsewhere; and chains that hang off
    different outputs of one attention backward.  Two things went wrong there: a difference row
    named a variable twice, which the solver took for a broken model and the planner reported as
    infeasible; and an edge between two linked nodes was left to an edge between their roots that
    does not exist.  The clustered plan, expanded, must cost on the engine that priced every node
    exactly what the clustered objective says."""
    pytest.importorskip("transformers")
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.tensor.placement_types import Replicate, Shard

    from autoparallel_amd.graph_utils import add_alias_nodes, replace_view_mm_view_with_einsum
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    cfg_cls, model_cls, kwargs, dtype = _hf_cases()["vit"]
    cfg = cfg_cls(**kwargs)
    cfg._attn_implementation = "sdpa"
    with FakeTensorMode():
        with torch.device("cuda"):
            model = _HFLoss(model_cls(cfg), "vit")
        x = torch.rand(8, 3, 32, 32, device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, model, (x,)).graph_module
    replace_view_mm_view_with_einsum(gm)
    add_alias_nodes(gm)
    mesh = meshes["2d"]
    kw = dict(devices_per_host=8, device_name="AMD Instinct MI355X")
    full = ShardingOptimizer(gm, mesh, **kw)
    clustered = ShardingOptimizer(gm, mesh, repeated_subgraphs=True, **kw)
    core = clustered._core
    g = core.g
    u, v = g.edge_src_node.astype(np.int64), g.edge_node.astype(np.int64)
    has = np.nonzero(u >= 0)[0]
    both = core.linked[u[has]] & core.linked[v[has]]
    uncovered = both & (g.edge_src_node[core.edge_alias[has]] != core.root[u[has]])
    assert uncovered.sum() > 0  # the case is present in this graph
    for opt in (full, clustered):
        opt.add_sharded_input_constraint([(Shard(0), Replicate())])
        opt.add_parameter_memory_constraint(0.0, 1.0 / mesh.size())
    plan = clustered.get_solution()
    full.get_solution()
    assert clustered._core.objective_value >= full._core.objective_value * (1 - 1e-9)
    idx = torch.from_numpy(clustered._out_indices(plan).astype(np.int16).reshape(-1, 1)).cuda()
    r = full._core.engine.score(idx).cpu().numpy()[0]
    assert r[5] == 0 and np.isclose(r[4], clustered._core.objective_value, rtol=1e-9)


def test_extended_clustering_takes_what_the_first_pass_leaves(meshes):
    """With four decoder layers the reference's pass takes the first normalisation of every layer
    into the large backward region and then drops the whole list of its duplicates, so the second
    normalisation of every layer stays on its own.  repeated_subgraphs="extended" grows regions
    from the duplicates that are still free: more nodes share variables, fewer entries are priced,
    and the plan, expanded and scored on the engine that priced every node, costs what the
    clustered objective says and no less than the plan of the unclustered problem."""
    pytest.importorskip("transformers")
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.tensor.placement_types import Replicate, Shard

    from autoparallel_amd.graph_utils import add_alias_nodes, replace_view_mm_view_with_einsum
    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    cfg_cls, model_cls, kwargs, dtype = _hf_cases()["mistral"]
    cfg = cfg_cls(**{**kwargs, "num_hidden_layers": 4})
    cfg.use_cache = False
    cfg._attn_implementation = "sdpa"
    with FakeTensorMode():
        with torch.device("cuda"):
            model = _HFLoss(model_cls(cfg), "mistral")
        x = torch.randint(0, 512, (8, 64), device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, model, (x,)).graph_module
    replace_view_mm_view_with_einsum(gm)
    add_alias_nodes(gm)
    mesh = meshes["2d"]
    kw = dict(devices_per_host=8, device_name="AMD Instinct MI355X")
    full = ShardingOptimizer(gm, mesh, **kw)
    first = ShardingOptimizer(gm, mesh, repeated_subgraphs=True, **kw)
    ext = ShardingOptimizer(gm, mesh, repeated_subgraphs="extended", **kw)
    assert ext.repeated_subgraphs is True
    assert len(ext._cluster_linked_node_idxs) > len(first._cluster_linked_node_idxs) > 0
    assert ext._packed.num_entries < first._packed.num_entries < full._packed.num_entries
    # the regions of the first pass are all still there
    taken = {tuple(reg) for grp in ext._core.region_groups for reg in grp}
    assert all(tuple(reg) in taken for grp in first._core.region_groups for reg in grp)
    for opt in (full, first, ext):
        opt.add_sharded_input_constraint([(Shard(0), Replicate())])
        opt.add_parameter_memory_constraint(0.0, 1.0 / mesh.size())
    plan = ext.get_solution()
    first.get_solution()
    full.get_solution()
    assert "Violated constraints: []" in ext.get_log()
    assert ext._core.objective_value >= first._core.objective_value * (1 - 1e-9)
    assert first._core.objective_value >= full._core.objective_value * (1 - 1e-9)
    idx = torch.from_numpy(ext._out_indices(plan).astype(np.int16).reshape(-1, 1)).cuda()
    r = full._core.engine.score(idx).cpu().numpy()[0]
    assert r[5] == 0 and np.isclose(r[4], ext._core.objective_value, rtol=1e-9)
