"""Host post-processing of operator strategies: the known answers of the
reference's tests/test_placement_options_utils.py (:28-150), restated for
autoparallel_amd.shardings.placement_options on a fake (CPU) mesh."""
import pytest
import torch
from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
from torch.distributed.tensor._op_schema import OpSpec, OpStrategy
from torch.distributed.tensor.placement_types import Replicate, Shard

from autoparallel_amd.shardings.placement_options import (
    fill_redistribute_cost,
    keep_unique_configs,
    remove_invalid_configs,
)
from oracle import cost_oracle as O


@pytest.fixture(scope="module")
def meshes():
    import torch.distributed as dist
    from torch.distributed.device_mesh import init_device_mesh
    from torch.testing._internal.distributed.fake_pg import FakeStore

    if dist.is_initialized():
        dist.destroy_process_group()
    dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=256)
    yield init_device_mesh("cpu", (256,)), init_device_mesh("cpu", (32, 8))
    dist.destroy_process_group()


def _tm(shape, dtype=torch.float32):
    t = torch.empty(shape, dtype=dtype, device="meta")
    return TensorMeta(t.shape, t.stride(), t.dtype)


def _one(mesh, shape, plc):
    spec = DTensorSpec(mesh, plc, tensor_meta=_tm(shape))
    return OpSpec(spec, input_specs=[spec], redistribute_cost=[[0.0]])


@pytest.mark.parametrize("which,shape,plc,kept", [
    (0, (256, 64), (Shard(0),), 1),            # divisible
    (0, (100, 64), (Shard(0),), 0),            # 100 < 256: empty shards
    (0, (7, 3), (Replicate(),), 1),            # replicate always kept
    (1, (256, 10), (Shard(0), Shard(1)), 1),   # 10 >= 8: uneven but non-empty
    (1, (257, 64), (Shard(0), Replicate()), 1),
    (1, (31, 64), (Shard(0), Replicate()), 0),
    (1, (64, 64), (Shard(0), Shard(0)), 0),    # 64/32 = 2, then 2 < 8
    (1, (256, 64), (Shard(0), Shard(0)), 1),   # 256/32 = 8, then 8 >= 8
])
def test_remove_invalid_configs_known_answers(meshes, which, shape, plc, kept):
    mesh = meshes[which]
    out = remove_invalid_configs(OpStrategy([_one(mesh, shape, plc)]), mesh)
    assert len(out.strategies) == kept
    # the same rule as the oracle's per-spec test (and the device enumeration kernel's)
    code = tuple(0 if isinstance(p, Replicate) else 0x40 | p.dim for p in plc)
    assert O.is_valid_spec(shape, code, tuple(mesh.shape)) == bool(kept)


def test_remove_invalid_configs_none_output_and_mix(meshes):
    mesh = meshes[0]
    spec = DTensorSpec(mesh, (Replicate(),), tensor_meta=_tm((256,)))
    out = remove_invalid_configs(OpStrategy([OpSpec(None, input_specs=[spec], redistribute_cost=[[0.0]])]), mesh)
    assert len(out.strategies) == 1
    mix = OpStrategy([_one(mesh, (256, 64), (Shard(0),)), _one(mesh, (100, 64), (Shard(0),))])
    assert len(remove_invalid_configs(mix, mesh).strategies) == 1


def test_keep_unique_configs_known_answers(meshes):
    mesh = meshes[0]
    a = _one(mesh, (4, 8), (Replicate(),))
    assert len(keep_unique_configs(OpStrategy([a, a])).strategies) == 1
    b = _one(mesh, (256, 64), (Replicate(),))
    c = _one(mesh, (256, 64), (Shard(0),))
    assert len(keep_unique_configs(OpStrategy([b, c])).strategies) == 2
    # equal content in distinct objects is still a duplicate
    assert len(keep_unique_configs(OpStrategy([_one(mesh, (4, 8), (Replicate(),)), a])).strategies) == 1


def test_fill_redistribute_cost_shapes(meshes):
    mesh = meshes[0]
    prod = OpStrategy([_one(mesh, (256, 64), (Replicate(),)), _one(mesh, (256, 64), (Shard(0),))])
    spec = DTensorSpec(mesh, (Replicate(),), tensor_meta=_tm((256, 64)))
    st = OpStrategy([OpSpec(spec, input_specs=[spec, spec])])
    fill_redistribute_cost(st, [prod, prod])
    assert st.strategies[0].redistribute_cost == [[0.0, 0.0], [0.0, 0.0]]


def test_device_limit_interface():
    """The reference's device table values for the MI355X
    (compute_estimation.py:226-239) through the engine's table, and its errors."""
    import torch

    from autoparallel_amd.cost_models import compute_estimation as CE
    from autoparallel_amd.cost_models import collective_runtime_estimation as CRE

    CRE.configure(device_name="AMD Instinct MI355X")
    try:
        limit = CE._get_device_limit()
        assert limit.gmem_bandwidth == 8.0 * 1024**4
        assert limit.gemm_tflops == {torch.float64: 78.6, torch.float32: 157.3, torch.float16: 2516.6,
                                     torch.bfloat16: 2516.6, torch.int8: 5033.2}
        assert CE._get_device_tflops(torch.bfloat16) == 2516.6
        assert CE._get_device_gmem_bandwidth() == limit.gmem_bandwidth
        with pytest.raises(ValueError, match="not supported"):
            CE._get_device_tflops(torch.int64)
        CRE.configure(device_name="Some Unknown Accelerator")
        with pytest.raises(ValueError):
            CE._get_device_limit()
    finally:
        CRE.configure(device_name=None)


def test_einsum_flop_and_memory_cost_known_answers():
    import torch

    from autoparallel_amd.cost_models import compute_memory_cost, einsum_flop

    a, b = torch.empty(4, 8, 16, device="meta"), torch.empty(16, 32, device="meta")
    assert einsum_flop("bsk,kn->bsn", (a, b)) == 4 * 8 * 32 * 16 * 2
    g, x = torch.empty(4, 8, 32, device="meta"), torch.empty(4, 8, 16, device="meta")
    assert einsum_flop("bsn,bsk->kn", (g, x)) == 4 * 8 * 32 * 16 * 2
    with pytest.raises(NotImplementedError):
        einsum_flop("ij,jk->ik", (torch.empty(2, 3, device="meta"), torch.empty(3, 4, device="meta")))
    with pytest.raises(AssertionError):
        einsum_flop("bsk,kn->bsn", (a, torch.empty(15, 32, device="meta")))
    bf = torch.empty(8, 4, dtype=torch.bfloat16, device="meta")
    assert compute_memory_cost(None, (a, [bf, 3]), {"out": b}) == 4 * 8 * 16 * 4 + 8 * 4 * 2 + 16 * 32 * 4


def _fx_node(target, args, val, name=None):
    g = torch.fx.Graph()
    n = g.call_function(target, args)
    n.meta["val"] = val
    if name:
        n.name = name
    return n


def _candidates(mesh, shape, placements):
    return OpStrategy([_one(mesh, shape, p) for p in placements])


def test_operators_without_tensor_inputs_rules(meshes):
    """Size-taking factories: every {Shard(d), Replicate} combination, Replicate
    last per mesh dim, invalid ones dropped, a stand-in input spec that is the
    output spec, and a zero row as long as the unfiltered product
    (autoparallel/shardings/propagation_rules.py:486-554).  Generators and
    scalar_tensor: Replicate only with one zero (:412-421, :453-484)."""
    from autoparallel_amd.shardings.placement_options import get_placement_options_for_node

    aten = torch.ops.aten
    mesh = meshes[1]  # (32, 8)
    val = torch.empty(64, 16, device="meta")
    node = _fx_node(aten.zeros.default, ([64, 16],), val)
    out = get_placement_options_for_node(mesh, node, [], [], ([64, 16],))
    plcs = [s.output_specs.placements for s in out.strategies]
    # (S0|S1|R)^2 = 9; dim 1 (16) cannot take the mesh dim of 32; 64/32 = 2 cannot take 8 more
    assert plcs == [(Shard(0), Shard(1)), (Shard(0), Replicate()),
                    (Replicate(), Shard(0)), (Replicate(), Shard(1)), (Replicate(), Replicate())]
    assert all(s.input_specs[0] is s.output_specs and s.redistribute_cost == [[0.0] * 9] for s in out.strategies)
    assert out.strategies[0].output_specs.tensor_meta.shape == (64, 16)
    for target, args, v in ((aten.arange.default, (128,), torch.empty(128, dtype=torch.int64, device="meta")),
                            (aten.scalar_tensor.default, (1.0,), torch.empty((), device="meta"))):
        out = get_placement_options_for_node(mesh, _fx_node(target, args, v), [], [], args)
        assert len(out.strategies) == 1 and out.strategies[0].redistribute_cost == [[0.0]]
        assert out.strategies[0].output_specs.placements == (Replicate(), Replicate())
        assert out.strategies[0].output_specs.tensor_meta.dtype == v.dtype


def test_view_is_not_strict(meshes):
    """A view that splits a sharded dim keeps the strategy with the input demoted
    (autoparallel/shardings/propagation_rules.py:239-287) where DTensor's own
    rule refuses the whole operator."""
    from autoparallel_amd.shardings.placement_options import fallback_nodes, get_placement_options_for_node

    mesh = meshes[0]  # (256,)
    src = _candidates(mesh, (512, 1024, 768), [(Replicate(),), (Shard(0),), (Shard(2),)])
    val = torch.empty(512, 1024, 12, 64, device="meta")
    g = torch.fx.Graph()
    x = g.placeholder("x")
    x.meta["val"] = torch.empty(512, 1024, 768, device="meta")
    node = g.call_function(torch.ops.aten.view.default, (x, [512, 1024, 12, 64]))
    node.meta["val"] = val
    before = list(fallback_nodes)
    out = get_placement_options_for_node(mesh, node, [src], [x.meta["val"]], (src, [512, 1024, 12, 64]))
    assert fallback_nodes == before
    got = {(s.input_specs[0].placements, s.output_specs.placements) for s in out.strategies}
    # 768 -> (12, 64): 12 < 256, so Shard(2) cannot follow; the input is asked to be Replicate
    assert got == {((Replicate(),), (Replicate(),)), ((Shard(0),), (Shard(0),))}
    assert all(len(s.redistribute_cost[0]) == 3 for s in out.strategies)
    assert all(s.output_specs.tensor_meta.shape == (512, 1024, 12, 64) for s in out.strategies)


def test_norm_strategies_with_unequal_candidate_counts(meshes):
    """DTensor's layer-norm functions pair the arguments' strategies by index;
    with 3 candidates for the input and 2 for weight and bias they are asked one
    input strategy at a time: one strategy per input placement, weight and bias
    Replicate, three outputs that follow the input on the outer dims."""
    from autoparallel_amd.shardings.placement_options import fallback_nodes, get_placement_options_for_node

    mesh = meshes[1]  # (32, 8)
    x_val = torch.empty(256, 64, 128, device="meta")
    w_val = torch.empty(128, device="meta")
    xs = _candidates(mesh, (256, 64, 128), [(Replicate(), Replicate()), (Shard(0), Replicate()),
                                            (Shard(0), Shard(1)), (Replicate(), Shard(2))])
    ws = _candidates(mesh, (128,), [(Replicate(), Replicate()), (Replicate(), Shard(0))])
    g = torch.fx.Graph()
    x, w, b = g.placeholder("x"), g.placeholder("w"), g.placeholder("b")
    x.meta["val"], w.meta["val"], b.meta["val"] = x_val, w_val, w_val
    node = g.call_function(torch.ops.aten.native_layer_norm.default, (x, [128], w, b, 1e-5))
    node.meta["val"] = (x_val, torch.empty(256, 64, 1, device="meta"), torch.empty(256, 64, 1, device="meta"))
    before = list(fallback_nodes)
    out = get_placement_options_for_node(mesh, node, [xs, ws, ws], [x_val, w_val, w_val], (xs, [128], ws, ws, 1e-5))
    assert fallback_nodes == before
    got = [(tuple(s.placements for s in st.input_specs), tuple(s.placements for s in st.output_specs))
           for st in out.strategies]
    rr = (Replicate(), Replicate())
    assert got == [((p, rr, rr), (p, p, p)) for p in (rr, (Shard(0), Replicate()), (Shard(0), Shard(1)))]
    assert [len(r) for r in out.strategies[0].redistribute_cost] == [4, 2, 2]
    assert out.strategies[0].output_specs[1].tensor_meta.shape == (256, 64, 1)


def test_partial_candidates_do_not_cost_the_operator_its_strategies(meshes):
    """DTensor's dropout rule raises when an argument may arrive Partial; the
    query is repeated without those candidates instead of giving the operator up
    to the all-Replicate stand-in (rows keep one column per real candidate)."""
    from torch.distributed.tensor.placement_types import Partial

    from autoparallel_amd.shardings.placement_options import fallback_nodes, get_placement_options_for_node

    mesh = meshes[0]
    src = _candidates(mesh, (512, 64), [(Replicate(),), (Shard(0),), (Partial(),)])
    g = torch.fx.Graph()
    x = g.placeholder("x")
    x.meta["val"] = torch.empty(512, 64, device="meta")
    node = g.call_function(torch.ops.aten.native_dropout.default, (x, 0.1, True))
    node.meta["val"] = (torch.empty(512, 64, device="meta"), torch.empty(512, 64, dtype=torch.bool, device="meta"))
    before = list(fallback_nodes)
    out = get_placement_options_for_node(mesh, node, [src], [x.meta["val"]], (src, 0.1, True))
    assert fallback_nodes == before
    assert {st.input_specs[0].placements for st in out.strategies} == {(Replicate(),), (Shard(0),)}
    assert all(len(st.redistribute_cost[0]) == 3 and len(st.output_specs) == 2 for st in out.strategies)


def test_failures_raise_and_only_unregistered_operators_get_the_stand_in(meshes, caplog, monkeypatch):
    """As in the reference (dtensor_sharding_helpers.py:327-361 under
    with_implicit_strategies, placement_options.py:328-346): an operator without
    a registered strategy function is planned all-Replicate, with a warning; a
    rule that raises is an error, unless the caller opts into the stand-in."""
    import logging

    from autoparallel_amd.shardings import placement_options as PO

    mesh = meshes[0]
    PO.reset_placement_options_cache()
    src = _candidates(mesh, (512, 64), [(Replicate(),), (Shard(0),)])
    g = torch.fx.Graph()
    x = g.placeholder("x")
    x.meta["val"] = torch.empty(512, 64, device="meta")
    # 1. no strategy function: stand-in + warning
    prop = PO.DTensor._op_dispatcher.sharding_propagator
    op = torch.ops.aten.flip.default
    assert op not in prop.op_strategy_funcs
    node = g.call_function(op, (x, [0]))
    node.meta["val"] = torch.empty(512, 64, device="meta")
    PO.fallback_nodes.clear()
    with caplog.at_level(logging.WARNING, logger=PO.logger.name):
        out = PO.get_placement_options_for_node(mesh, node, [src], [x.meta["val"]], (src, [0]))
    assert PO.fallback_nodes == [node.name] and "no strategy registered" in PO.fallback_reasons[node.name]
    assert any("all-Replicate stand-in" in r.message for r in caplog.records)
    assert [st.output_specs.placements for st in out.strategies] == [(Replicate(),)]
    # 2. a rule that raises: the error reaches the caller
    def broken(mesh, node, producer):
        raise KeyError("boom")

    monkeypatch.setattr(PO, "_view_rule", broken)
    view = g.call_function(torch.ops.aten.view.default, (x, [64, 512]))
    view.meta["val"] = torch.empty(64, 512, device="meta")
    PO.fallback_nodes.clear()
    with pytest.raises(KeyError, match="boom"):
        PO.get_placement_options_for_node(mesh, view, [src], [x.meta["val"]], (src, [64, 512]))
    assert PO.fallback_nodes == []
    # 3. ... unless asked for the stand-in
    with PO.replicate_stand_in_on_error(), caplog.at_level(logging.WARNING, logger=PO.logger.name):
        out = PO.get_placement_options_for_node(mesh, view, [src], [x.meta["val"]], (src, [64, 512]))
    assert PO.fallback_nodes == [view.name] and "KeyError" in PO.fallback_reasons[view.name]
    assert [st.output_specs.placements for st in out.strategies] == [(Replicate(),)]
    PO.reset_placement_options_cache()
    PO.fallback_nodes.clear()


def test_local_map_region_has_its_declared_strategy(meshes):
    """A local_map region offers exactly the placements its author declared
    (autoparallel/shardings/placement_options.py:380-490): leading arguments
    beyond the declared ones are Replicate, an argument with placement None or a
    non-tensor has no spec, trailing outputs are Replicate, and the cost rows
    have one zero per candidate of each tensor argument."""
    from torch.distributed.tensor.placement_types import Partial

    from autoparallel_amd.shardings.placement_options import get_placement_options_for_node

    mesh = meshes[1]  # (32, 8)

    def call_local_map(*args):  # stands in for the higher-order operator
        raise AssertionError("never run")

    g = torch.fx.Graph()
    sub = g.get_attr("body")  # the region's graph module: not a tensor
    act, x, w, n = g.placeholder("act"), g.placeholder("x"), g.placeholder("w"), g.placeholder("n")
    act.meta["val"] = torch.empty(64, 32, device="meta")
    x.meta["val"] = torch.empty(256, 64, device="meta")
    w.meta["val"] = torch.empty(64, 64, device="meta")
    n.meta["val"] = 7
    node = g.call_function(call_local_map, (sub, act, x, w, n))
    node.meta["val"] = (torch.empty(256, 64, device="meta"), None, torch.empty(8, device="meta"))
    node.meta["local_map_kwargs"] = {
        "in_placements": ((Shard(0), Replicate()), None, None),
        "out_placements": ((Shard(0), Partial()), None),
    }
    cands = {
        act: _candidates(mesh, (64, 32), [(Replicate(), Replicate()), (Shard(0), Replicate())]),
        x: _candidates(mesh, (256, 64), [(Replicate(), Replicate()), (Shard(0), Replicate()), (Shard(0), Shard(1))]),
        w: _candidates(mesh, (64, 64), [(Replicate(), Replicate())]),
    }
    schema = (None, cands[act], cands[x], cands[w], 7)
    out = get_placement_options_for_node(mesh, node, [cands[act], cands[x], cands[w]],
                                         [act.meta["val"], x.meta["val"], w.meta["val"]], schema)
    assert len(out.strategies) == 1
    st = out.strategies[0]
    rr = (Replicate(), Replicate())
    assert [None if s is None else s.placements for s in st.input_specs] == [rr, (Shard(0), Replicate()), None]
    assert st.input_specs[1].tensor_meta.shape == (256, 64)
    assert [None if s is None else s.placements for s in st.output_specs] == [(Shard(0), Partial()), None, rr]
    assert st.redistribute_cost == [[0.0, 0.0], [0.0, 0.0, 0.0], [0.0]]


def test_select_does_not_write_into_its_producer(meshes):
    """DTensor's select hands back one spec object as input and output when the
    selected dim is not sharded; the tensor-meta fill must not reach the
    producer's or the input's meta through it."""
    from autoparallel_amd.shardings.placement_options import get_placement_options_for_node

    mesh = meshes[1]
    src = _candidates(mesh, (256, 16, 64), [(Replicate(), Replicate()), (Shard(0), Replicate()), (Shard(0), Shard(2))])
    g = torch.fx.Graph()
    x = g.placeholder("x")
    x.meta["val"] = torch.empty(256, 16, 64, device="meta")
    node = g.call_function(torch.ops.aten.select.int, (x, 1, 3))
    node.meta["val"] = torch.empty(256, 64, device="meta")
    out = get_placement_options_for_node(mesh, node, [src], [x.meta["val"]], (src, 1, 3))
    assert len(out.strategies) >= 3
    for st in src.strategies:
        assert st.output_specs.tensor_meta.shape == (256, 16, 64)
    for st in out.strategies:
        assert st.output_specs.tensor_meta.shape == (256, 64)
        assert st.input_specs[0].tensor_meta.shape == (256, 16, 64)
        assert st.input_specs[0] is not st.output_specs
    assert {st.output_specs.placements for st in out.strategies} >= {(Replicate(), Replicate()), (Shard(0), Shard(1))}


def _plcs(strategy):
    out = []
    for st in strategy.strategies:
        o = st.output_specs[0] if isinstance(st.output_specs, tuple) else st.output_specs
        out.append((tuple(s.placements for s in st.input_specs), o.placements))
    return out


def test_rules_the_reference_keeps_for_itself(meshes):
    """stack, uniform_, split_with_sizes, view(dtype) and alias as the reference's
    own rules define them (autoparallel/shardings/propagation_rules.py:289-315,
    358-409, 621-680), on a (32, 8) mesh."""
    from torch.distributed.tensor.placement_types import Partial

    from autoparallel_amd.shardings import placement_options as PO

    mesh = meshes[1]
    aten = torch.ops.aten
    R, S = Replicate(), Shard
    g = torch.fx.Graph()
    a, b = g.placeholder("a"), g.placeholder("b")
    a.meta["val"] = b.meta["val"] = torch.empty(256, 64, device="meta")
    two = _candidates(mesh, (256, 64), [(R, R), (S(0), R)])

    # stack at dim 1: inputs alike, the output's shard dim moves past the new dim
    node = g.call_function(aten.stack.default, ([a, b], 1))
    node.meta["val"] = torch.empty(256, 2, 64, device="meta")
    out = PO.get_placement_options_for_node(mesh, node, [two, two], [a.meta["val"]] * 2, ([two, two], 1))
    got = _plcs(out)
    # 3 x 3 combinations less (S(1), S(1)): 64 / 32 = 2 rows cannot be split 8 ways
    assert len(got) == 8 and all(i[0] == i[1] for i, _ in got)
    assert ((((S(0), S(1)),) * 2, (S(0), S(2))) in got) and ((((R, R),) * 2, (R, R)) in got)
    assert all(len(r) == 2 for st in out.strategies for r in st.redistribute_cost)

    # uniform_: output as input, every sharding of the tensor
    node = g.call_function(aten.uniform.default, (a, 0.0, 1.0))
    node.meta["val"] = a.meta["val"]
    got = _plcs(PO.get_placement_options_for_node(mesh, node, [two], [a.meta["val"]], (two, 0.0, 1.0)))
    assert len(got) == 8 and all(i == (o,) for i, o in got) and ((S(1), S(1)),) not in [i for i, _ in got]

    # split_with_sizes on dim 1: no candidate sharded there, none Partial
    many = _candidates(mesh, (256, 64), [(R, R), (S(0), R), (S(1), R), (R, Partial()), (S(0), S(0)), (S(0), R)])
    node = g.call_function(aten.split_with_sizes.default, (a, [32, 32], 1))
    node.meta["val"] = (torch.empty(256, 32, device="meta"), torch.empty(256, 32, device="meta"))
    out = PO.get_placement_options_for_node(mesh, node, [many], [a.meta["val"]], (many, [32, 32], 1))
    assert [st.input_specs[0].placements for st in out.strategies] == [(R, R), (S(0), R), (S(0), S(0))]
    assert all(len(st.output_specs) == 2 and st.output_specs[1].tensor_meta.shape == (256, 32) and
               st.output_specs[0].placements == st.input_specs[0].placements for st in out.strategies)
    assert all(len(st.redistribute_cost[0]) == 6 for st in out.strategies)

    # view(dtype): nothing sharded on the last dim
    node = g.call_function(aten.view.dtype, (a, torch.int32))
    node.meta["val"] = torch.empty(256, 64, dtype=torch.int32, device="meta")
    out = PO.get_placement_options_for_node(mesh, node, [many], [a.meta["val"]], (many, torch.int32))
    assert [st.output_specs.placements for st in out.strategies] == [(R, R), (S(0), R), (R, Partial()), (S(0), S(0))]
    assert all(st.output_specs.tensor_meta.dtype == torch.int32 and st.input_specs[0].tensor_meta.dtype == torch.float32
               for st in out.strategies)


def test_select_takes_negative_dim_and_index(meshes):
    from autoparallel_amd.shardings.placement_options import fallback_nodes, get_placement_options_for_node

    mesh = meshes[1]
    src = _candidates(mesh, (256, 16, 64), [(Replicate(), Replicate()), (Shard(0), Shard(2))])
    g = torch.fx.Graph()
    x = g.placeholder("x")
    x.meta["val"] = torch.empty(256, 16, 64, device="meta")
    outs = []
    for dim, index in ((1, 15), (-2, -1)):
        node = g.call_function(torch.ops.aten.select.int, (x, dim, index))
        node.meta["val"] = torch.empty(256, 64, device="meta")
        before = list(fallback_nodes)
        outs.append(_plcs(get_placement_options_for_node(mesh, node, [src], [x.meta["val"]], (src, dim, index))))
        assert fallback_nodes == before
    assert outs[0] == outs[1] and (((Shard(0), Shard(2)),), (Shard(0), Shard(1))) in outs[0]


def test_flex_attention_strategies(meshes):
    """flex_attention: {Replicate, Shard(batch), Shard(head)} per mesh dim; grouped
    key/value heads shard only where they divide; block-mask tensors and the
    buffers of the score function are Replicate
    (autoparallel/shardings/placement_options.py:493-650).  Mesh (32, 8), 64 query
    heads over 8 key/value heads, batch 64."""
    from torch._higher_order_ops.flex_attention import flex_attention

    from autoparallel_amd.shardings.placement_options import get_placement_options_for_node

    mesh = meshes[1]
    R, S = Replicate(), Shard
    g = torch.fx.Graph()
    mk = lambda name, *shape, dtype=torch.bfloat16: (lambda n: (n.meta.__setitem__("val", torch.empty(*shape, dtype=dtype, device="meta")), n)[1])(g.placeholder(name))
    q, k, v = mk("q", 64, 64, 128, 32), mk("k", 64, 8, 128, 32), mk("v", 64, 8, 128, 32)
    kv_num = mk("kv_num_blocks", 1, 1, 4, dtype=torch.int32)
    kv_idx = mk("kv_indices", 1, 1, 4, 4, dtype=torch.int32)
    bias = mk("bias", 64, 128)
    score_mod = g.get_attr("score_mod")
    mask_mod = g.get_attr("mask_mod")
    block_mask = (128, 128, kv_num, kv_idx, None, None, None, None, None, None, 32, 32, mask_mod)
    node = g.call_function(flex_attention, (q, k, v, score_mod, block_mask, 0.17, {}, (bias,), ()))
    node.meta["val"] = (torch.empty(64, 64, 128, 32, dtype=torch.bfloat16, device="meta"),
                        torch.empty(64, 64, 128, device="meta"), torch.empty(64, 64, 128, device="meta"))
    tens = [q, k, v, kv_num, kv_idx, bias]
    cands = [_candidates(mesh, tuple(t.meta["val"].shape), [(R, R), (S(0), R)]) for t in tens]
    out = get_placement_options_for_node(mesh, node, cands, [t.meta["val"] for t in tens], None)
    assert len(out.strategies) == 9
    by_q = {st.input_specs[0].placements: st for st in out.strategies}
    assert set(by_q) == set(__import__("itertools").product((R, S(0), S(1)), repeat=2))
    for plc, st in by_q.items():
        ins = [s.placements for s in st.input_specs]
        # 8 key/value heads: Shard(1) holds on the mesh dim of 8 only, not on the one of 32
        kv = tuple(R if (p.is_shard() and p.dim == 1 and n != 8) else p for p, n in zip(plc, mesh.shape))
        assert ins[1] == ins[2] == kv
        assert ins[3] == ins[4] == (R, R)  # block-mask tensors have extent 1 on batch and heads
        assert ins[5] == (R, R)            # a buffer of the score function
        assert [s.placements for s in st.output_specs] == [plc, plc, plc]
        assert [len(r) for r in st.redistribute_cost] == [2] * 6
    assert by_q[(S(0), S(1))].output_specs[1].tensor_meta.shape == (64, 64, 128)


def test_flat_args_and_map_nodes_equal_pytree():
    """The argument walks of the strategy enumeration against torch's pytree on
    the structures FX arguments have (nested tuples, lists, dicts, slices,
    repeated nodes, None)."""
    from torch.utils._pytree import tree_flatten, tree_map_only

    from autoparallel_amd.optimize_sharding import _flat_args, _map_nodes

    g = torch.fx.Graph()
    a, b = g.placeholder("a"), g.placeholder("b")
    cases = [
        (a, b), (a, a, 1.5), ([a, None, b], 2), ((a, [b, (a, 3)]), {"k": b, "j": [a]}), (slice(0, 4, None), a),
        (), (None,), ("ij,jk->ik", [a, b]),
    ]
    for args in cases:
        node = g.call_function(torch.ops.aten.add.Tensor, args)  # FX turns the lists into immutable ones
        assert _flat_args(node.args, []) == tree_flatten(node.args)[0]
        f = lambda n: ("strategy of", n.name)
        assert _map_nodes(node.args, f) == tree_map_only(torch.fx.Node, f, node.args)


def test_torch_cost_rows_are_restored(meshes):
    """While a query runs torch's strategy functions fill their rows with zeros;
    afterwards, and after an error inside the query, torch's own function is
    back in every module that imported it."""
    import torch.distributed.tensor._ops._matrix_ops as MO
    import torch.distributed.tensor._ops.utils as OU

    from autoparallel_amd.shardings import placement_options as PO

    real = OU.generate_redistribute_costs
    assert MO.generate_redistribute_costs is real
    with PO._without_torch_cost_rows():
        assert OU.generate_redistribute_costs is PO._zero_cost_rows and MO.generate_redistribute_costs is PO._zero_cost_rows
        with PO._without_torch_cost_rows():  # nested: the inner exit must not bring the real one back early
            pass
        assert MO.generate_redistribute_costs is PO._zero_cost_rows
    assert OU.generate_redistribute_costs is real and MO.generate_redistribute_costs is real
    with pytest.raises(KeyError):
        with PO._without_torch_cost_rows():
            raise KeyError("inside")
    assert OU.generate_redistribute_costs is real and MO.generate_redistribute_costs is real


def test_strategies_do_not_depend_on_torchs_cost_rows(meshes):
    """The strategy functions of the installed torch fill in cost rows but do not
    select or order by them: with the rows made of zeros (as during a query) and
    with torch's own rows, the operators a transformer graph uses answer with the
    same input and output specs, in the same order."""
    from torch.distributed.tensor import DTensor
    from torch.distributed.tensor._op_schema import OpSchema

    from torch.distributed.tensor.placement_types import Partial

    from autoparallel_amd.shardings import placement_options as PO

    mesh = meshes[1]  # (32, 8)
    R, S, P = Replicate(), Shard, Partial()
    x = _candidates(mesh, (64, 32), [(R, R), (S(0), R), (S(1), S(0)), (P, R)])
    y = _candidates(mesh, (64, 32), [(R, R), (S(0), R), (R, S(1))])
    w = _candidates(mesh, (32, 48), [(R, R), (R, S(1)), (S(0), R)])
    x3 = _candidates(mesh, (32, 64, 32), [(R, R), (S(0), S(1)), (S(2), R)])
    aten = torch.ops.aten
    queries = [
        (aten.add.Tensor, (x, y), {}), (aten.mul.Tensor, (x, y), {}), (aten.mm.default, (x, w), {}),
        (aten.silu.default, (x,), {}), (aten.sum.dim_IntList, (x, [1], True), {}), (aten.mean.dim, (x, [-1], True), {}),
        (aten._softmax.default, (x, -1, False), {}), (aten.t.default, (x,), {}), (aten.transpose.int, (x3, 1, 2), {}),
        (aten.clone.default, (x,), {}), (aten._to_copy.default, (x,), {"dtype": torch.bfloat16}),
        (aten.rsqrt.default, (x,), {}), (aten.neg.default, (x,), {}), (aten.pow.Tensor_Scalar, (x, 2), {}),
        (aten.bmm.default, (x3, _candidates(mesh, (32, 32, 16), [(R, R), (S(0), R)])), {}),
    ]
    funcs = DTensor._op_dispatcher.sharding_propagator.op_strategy_funcs
    asked = nonzero = 0
    for op, args, kwargs in queries:
        fn = funcs.get(op)
        if fn is None:
            continue
        plain = fn(OpSchema(op, args, kwargs))
        with PO._without_torch_cost_rows():
            zeroed = fn(OpSchema(op, args, kwargs))
        summary = lambda st: [(str(s.input_specs), str(s.output_specs)) for s in st.strategies]
        assert summary(plain) == summary(zeroed), op
        nonzero += any(c != 0 for s in plain.strategies for row in (s.redistribute_cost or []) for c in row)
        asked += 1
    assert asked >= 12 and nonzero >= 6  # torch's own rows really differ from the zeros


def test_strategy_summaries_keep_the_cache_hits(meshes):
    """A query key holds one token per argument strategy; strategies with the
    same output specs get the same token wherever they come from, and tokens
    are not reused after the cache is reset."""
    from autoparallel_amd.shardings import placement_options as PO

    mesh = meshes[0]
    R, S = Replicate(), Shard
    x = _candidates(mesh, (64, 32), [(R, R), (S(0), R)])
    y = _candidates(mesh, (64, 32), [(R, R), (S(0), R)])  # other objects, same content
    z = _candidates(mesh, (64, 32), [(R, R), (S(1), R)])
    assert PO._fingerprint(x) == PO._fingerprint(y) != PO._fingerprint(z)
    assert PO._fingerprint(PO._copy_strategy(x)) == PO._fingerprint(x)
    old = PO._fingerprint(x)
    PO.reset_placement_options_cache()
    w = _candidates(mesh, (64, 32), [(R, S(1))])
    assert PO._fingerprint(w) != old  # x still carries `old`; nothing else may get it


def test_collector_state_is_restored():
    import gc

    from autoparallel_amd.optimize_sharding import _gc_paused

    assert gc.isenabled()
    with _gc_paused():
        assert not gc.isenabled()
        with _gc_paused():
            pass
        assert not gc.isenabled()
    assert gc.isenabled()
    gc.disable()
    try:
        with _gc_paused():
            pass
        assert not gc.isenabled()  # it was off before: stays off
    finally:
        gc.enable()


def _reduce_node(target, shape, args, out_shape):
    g = torch.fx.Graph()
    x = g.placeholder("x")
    x.meta["val"] = torch.empty(shape, device="meta")
    node = g.call_function(target, (x,) + tuple(args))
    node.meta["val"] = torch.empty(out_shape, device="meta")
    return x, node


@pytest.mark.parametrize("cands, must_have", [
    # both sharded dims are reduced: pending sums on both mesh dims
    ([(Shard(0), Shard(1))], [("P(sum)", "P(sum)")]),
    # the shards are on the dim that stays: it is dim 0 of the result
    ([(Shard(2), Shard(2))], [("S(0)", "S(0)")]),
    # a candidate that is Partial(avg) must not cost the later ones their shards
    ([(Replicate(), Replicate()), (Replicate(), "avg"), (Shard(0), Shard(1)), (Shard(0), Shard(2))],
     [("P(sum)", "P(sum)"), ("P(sum)", "S(0)"), ("R", "R")]),
    ([(Replicate(), "avg"), (Shard(0), Shard(1))], [("R", "R"), ("P(sum)", "P(sum)")]),
])
def test_sum_treats_every_candidate_on_its_own(meshes, cands, must_have):
    """The known answers of the reference's tests/test_reduction_strategies.py:38-117 for
    sum over dims [0, 1] of a (32, 8192, 4096) tensor on a 2-D mesh, asked through the node
    query: each candidate of the input keeps its own answer, whatever precedes it in the
    list (torch 2.10's rule decides once per call; the query then asks candidate by candidate)."""
    from torch.distributed.tensor.placement_types import Partial

    from autoparallel_amd.shardings.placement_options import get_placement_options_for_node, reset_placement_options_cache

    mesh = meshes[1]
    shape = (32, 8192, 4096)
    as_plc = lambda c: tuple(Partial(p) if isinstance(p, str) else p for p in c)
    src = OpStrategy([_one(mesh, shape, as_plc(c)) for c in cands])
    x, node = _reduce_node(torch.ops.aten.sum.dim_IntList, shape, ([0, 1],), (4096,))
    reset_placement_options_cache()
    out = get_placement_options_for_node(mesh, node, [src], [x.meta["val"]], (src, [0, 1]))

    def short(p):
        return "R" if p.is_replicate() else (f"S({p.dim})" if p.is_shard() else f"P({p.reduce_op})")

    got = {tuple(short(p) for p in st.output_specs.placements) for st in out.strategies}
    assert set(must_have) <= got, got
    # one column per candidate of the input in every cost row
    assert all(len(st.redistribute_cost) == 1 and len(st.redistribute_cost[0]) == len(cands) for st in out.strategies)


def test_mean_of_sharded_and_replicated_candidates(meshes):
    """mean over [0, 1] (tests/test_reduction_strategies.py:119-140): the replicated candidate
    stays replicated, the one sharded on the reduced dims ends in a pending average."""
    from autoparallel_amd.shardings.placement_options import get_placement_options_for_node, reset_placement_options_cache

    mesh = meshes[1]
    shape = (32, 8192, 4096)
    src = OpStrategy([_one(mesh, shape, (Replicate(), Replicate())), _one(mesh, shape, (Shard(0), Shard(1)))])
    x, node = _reduce_node(torch.ops.aten.mean.dim, shape, ([0, 1],), (4096,))
    reset_placement_options_cache()
    out = get_placement_options_for_node(mesh, node, [src], [x.meta["val"]], (src, [0, 1]))
    got = {st.output_specs.placements for st in out.strategies}
    assert (Replicate(), Replicate()) in got
    assert any(all(p.is_partial() and p.reduce_op == "avg" for p in plc) for plc in got), got


def test_tensor_meta_of_the_result_is_written_over_filled_in_or_left_alone(meshes):
    """The three cases of the reference's tests/test_placement_options_utils.py:193-240:
    an existing tensor meta on the output spec is replaced by the result's, a missing one
    is filled in, a strategy without an output spec (a non-tensor getitem) is skipped."""
    from autoparallel_amd.shardings.placement_options import propagate_tensor_meta

    mesh = meshes[0]
    val = torch.empty(4, 8, device="meta")
    node = _fx_node(torch.ops.aten.neg.default, (), val)
    stale = _tm((2, 2))
    spec = DTensorSpec(mesh, (Replicate(),), tensor_meta=stale)
    strat = OpStrategy([OpSpec(spec, input_specs=[DTensorSpec(mesh, (Replicate(),))], redistribute_cost=[[0.0]])])
    propagate_tensor_meta(node, [val], strat, mesh)
    got = strat.strategies[0].output_specs.tensor_meta
    assert got is not stale and got.shape == torch.Size([4, 8]) and got.stride == (8, 1)
    assert strat.strategies[0].input_specs[0].tensor_meta.shape == torch.Size([4, 8])  # inputs are filled in too
    bare = OpStrategy([OpSpec(DTensorSpec(mesh, (Replicate(),)), input_specs=[spec], redistribute_cost=[[0.0]])])
    assert bare.strategies[0].output_specs.tensor_meta is None
    propagate_tensor_meta(node, [val], bare, mesh)
    assert bare.strategies[0].output_specs.tensor_meta.shape == torch.Size([4, 8])
    none = OpStrategy([OpSpec(None, input_specs=[spec], redistribute_cost=[[0.0]])])
    propagate_tensor_meta(node, [val], none, mesh)
    assert none.strategies[0].output_specs is None


@pytest.mark.parametrize("target, extra", [
    (torch.ops.aten.floor_divide.default, None), (torch.ops.aten.hardswish.default, ()), (torch.ops.aten.leaky_relu.default, (0.1,)),
    (torch.ops.aten.mish.default, ()), (torch.ops.aten.softplus.default, ()),
])
def test_elementwise_operators_without_a_registered_strategy_are_pointwise(meshes, target, extra):
    """torch 2.10 registers nothing for these; they are elementwise (some carry the pointwise
    tag, some not), so they take DTensor's pointwise rule: the result follows the input's
    shards instead of forcing everything to Replicate."""
    from autoparallel_amd.shardings.placement_options import (fallback_reasons, get_placement_options_for_node,
                                                              reset_placement_options_cache)

    mesh = meshes[1]
    shape = (256, 64)
    cands = [(Replicate(), Replicate()), (Shard(0), Replicate()), (Shard(0), Shard(1)), (Replicate(), Shard(1))]
    src = OpStrategy([_one(mesh, shape, c) for c in cands])
    g = torch.fx.Graph()
    x = g.placeholder("x")
    x.meta["val"] = torch.empty(shape, device="meta")
    if extra is None:  # binary: the same tensor on both sides
        node = g.call_function(target, (x, x))
        producers, vals, schema = [src, src], [x.meta["val"]] * 2, (src, src)
    else:
        node = g.call_function(target, (x,) + tuple(extra))
        producers, vals, schema = [src], [x.meta["val"]], (src,) + tuple(extra)
    node.meta["val"] = torch.empty(shape, device="meta")
    reset_placement_options_cache()
    fallback_reasons.clear()
    out = get_placement_options_for_node(mesh, node, producers, vals, schema)
    assert not fallback_reasons
    got = {st.output_specs.placements for st in out.strategies}
    assert set(cands) <= got
    for st in out.strategies:  # elementwise: every input is placed like the output
        assert all(s.placements == st.output_specs.placements for s in st.input_specs)


def test_a_candidate_the_rule_refuses_costs_only_that_candidate(meshes):
    """nll_loss with reduction mean: torch's rule raises for an input candidate whose shards are
    of unequal size (the mean over shards would be biased).  Asked candidate by candidate, the
    operator simply offers nothing that follows that candidate; the others keep their answers and
    every cost row still has a column per real candidate.  When every candidate is refused the
    error is the rule's own."""
    from autoparallel_amd.shardings.placement_options import get_placement_options_for_node, reset_placement_options_cache

    mesh = meshes[1]  # (32, 8)
    n, v = 16 * 2047, 512  # 32752 rows: 8 divides them, 32 does not
    cands = [(Replicate(), Replicate()), (Replicate(), Shard(0)), (Shard(0), Replicate()), (Shard(0), Shard(0))]
    logits = OpStrategy([_one(mesh, (n, v), c) for c in cands])
    target = OpStrategy([_one(mesh, (n,), (Replicate(), Replicate()))])
    g = torch.fx.Graph()
    x, t = g.placeholder("x"), g.placeholder("t")
    x.meta["val"] = torch.empty(n, v, device="meta")
    t.meta["val"] = torch.empty(n, dtype=torch.int64, device="meta")
    node = g.call_function(torch.ops.aten.nll_loss_forward.default, (x, t, None, 1, -100))
    node.meta["val"] = (torch.empty((), device="meta"), torch.empty((), device="meta"))
    reset_placement_options_cache()
    out = get_placement_options_for_node(mesh, node, [logits, target], [x.meta["val"], t.meta["val"]], (logits, target, None, 1, -100))
    followed = {st.input_specs[0].placements for st in out.strategies}
    assert (Replicate(), Replicate()) in followed and (Replicate(), Shard(0)) in followed
    assert (Shard(0), Replicate()) not in followed and (Shard(0), Shard(0)) not in followed
    assert all(len(st.redistribute_cost[0]) == len(cands) and len(st.redistribute_cost[1]) == 1 for st in out.strategies)
    only_uneven = OpStrategy([_one(mesh, (n, v), (Shard(0), Replicate()))])
    reset_placement_options_cache()
    with pytest.raises(ValueError, match="evenly sharded"):
        get_placement_options_for_node(mesh, node, [only_uneven, target], [x.meta["val"], t.meta["val"]],
                                       (only_uneven, target, None, 1, -100))


def test_convolution_is_offered_replicated_or_batch_sharded(meshes):
    """torch 2.10 registers no strategy for convolution: per mesh dim, all Replicate or the batch
    sharded with the weights Replicate; backward the same with the weight and bias gradients as
    pending sums, and no spec for an output the mask switches off."""
    from torch.distributed.tensor.placement_types import Partial

    from autoparallel_amd.shardings.placement_options import (fallback_reasons, get_placement_options_for_node,
                                                              reset_placement_options_cache)

    mesh = meshes[1]  # (32, 8)
    g = torch.fx.Graph()
    vals = {"x": (512, 3, 16, 16), "w": (8, 3, 3, 3), "b": (8,), "go": (512, 8, 16, 16)}
    ph = {}
    for k, shape in vals.items():
        ph[k] = g.placeholder(k)
        ph[k].meta["val"] = torch.empty(shape, device="meta")
    full = lambda shape: OpStrategy([_one(mesh, shape, p) for p in
                                    [(Replicate(), Replicate()), (Shard(0), Replicate()), (Shard(0), Shard(0)), (Shard(1), Replicate())]])
    sx, sw, sb, sgo = full(vals["x"]), full(vals["w"]), OpStrategy([_one(mesh, vals["b"], (Replicate(), Replicate()))]), full(vals["go"])
    conv = g.call_function(torch.ops.aten.convolution.default, (ph["x"], ph["w"], ph["b"], [1, 1], [1, 1], [1, 1], False, [0, 0], 1))
    conv.meta["val"] = torch.empty(vals["go"], device="meta")
    reset_placement_options_cache()
    fallback_reasons.clear()
    out = get_placement_options_for_node(mesh, conv, [sx, sw, sb], [ph[k].meta["val"] for k in "xwb"],
                                         (sx, sw, sb, [1, 1], [1, 1], [1, 1], False, [0, 0], 1))
    assert not fallback_reasons
    got = {(st.output_specs.placements, tuple(s.placements for s in st.input_specs)) for st in out.strategies}
    R, S0 = Replicate(), Shard(0)
    assert got == {((a, b), ((a, b), (R, R), (R, R))) for a in (R, S0) for b in (R, S0)}
    assert all([len(r) for r in st.redistribute_cost] == [4, 4, 1] for st in out.strategies)
    bwd = g.call_function(torch.ops.aten.convolution_backward.default,
                          (ph["go"], ph["x"], ph["w"], [8], [1, 1], [1, 1], [1, 1], False, [0, 0], 1, [False, True, True]))
    bwd.meta["val"] = (None, torch.empty(vals["w"], device="meta"), torch.empty(vals["b"], device="meta"))
    out = get_placement_options_for_node(mesh, bwd, [sgo, sx, sw], [ph[k].meta["val"] for k in ("go", "x", "w")],
                                         (sgo, sx, sw, [8], [1, 1], [1, 1], [1, 1], False, [0, 0], 1, [False, True, True]))
    assert not fallback_reasons and len(out.strategies) == 4
    for st in out.strategies:
        gi, gw, gb = st.output_specs
        a = st.input_specs[0].placements
        assert gi is None and st.input_specs[1].placements == a and st.input_specs[2].placements == (R, R)
        want = tuple(Partial() if p.is_shard() else R for p in a)
        assert gw.placements == gb.placements == want and gw.tensor_meta.shape == torch.Size(vals["w"])


def test_gather_strategies_come_from_the_run_time_rule(meshes):
    """``x[idx]`` (aten.index.Tensor): torch 2.10 has a propagation rule for it, no strategy
    function.  One answer per candidate of the indexed tensor: a shard on a dim that is not
    indexed survives (moved past the index's dims), a shard on the indexed dim is given up
    for Replicate, the index itself Replicate."""
    from autoparallel_amd.shardings.placement_options import (fallback_reasons, get_placement_options_for_node,
                                                              reset_placement_options_cache)

    mesh = meshes[1]
    R = Replicate()
    g = torch.fx.Graph()
    x, i = g.placeholder("x"), g.placeholder("i")
    x.meta["val"] = torch.empty(512, 256, device="meta")
    i.meta["val"] = torch.empty(1024, dtype=torch.int64, device="meta")
    sx = OpStrategy([_one(mesh, (512, 256), p) for p in [(R, R), (Shard(1), R), (Shard(0), R), (R, Shard(1)), (Shard(0), Shard(1))]])
    si = OpStrategy([_one(mesh, (1024,), p) for p in [(R, R), (Shard(0), R)]])
    node = g.call_function(torch.ops.aten.index.Tensor, (x, [i]))
    node.meta["val"] = torch.empty(1024, 256, device="meta")
    reset_placement_options_cache()
    fallback_reasons.clear()
    out = get_placement_options_for_node(mesh, node, [sx, si], [x.meta["val"], i.meta["val"]], (sx, [si]))
    assert not fallback_reasons
    got = {(st.input_specs[0].placements, st.input_specs[1].placements, st.output_specs.placements) for st in out.strategies}
    assert got == {((R, R), (R, R), (R, R)), ((Shard(1), R), (R, R), (Shard(1), R)), ((R, Shard(1)), (R, R), (R, Shard(1)))}
    assert all([len(r) for r in st.redistribute_cost] == [5, 2] for st in out.strategies)
    assert all(st.output_specs.tensor_meta.shape == torch.Size([1024, 256]) for st in out.strategies)


def test_squeeze_of_several_dims_and_var_mean_have_strategies(meshes):
    """Both come out of the decomposition of batch norm; torch 2.10 registers neither.  squeeze.dims
    is a reshape to the result's shape; var_mean takes var's strategies, one spec for both results."""
    from autoparallel_amd.shardings.placement_options import (fallback_reasons, get_placement_options_for_node,
                                                              reset_placement_options_cache)

    mesh = meshes[1]
    R = Replicate()
    g = torch.fx.Graph()
    x = g.placeholder("x")
    x.meta["val"] = torch.empty(1, 64, 1, 512, device="meta")
    sx = OpStrategy([_one(mesh, (1, 64, 1, 512), p) for p in [(R, R), (Shard(1), R), (Shard(3), Shard(1))]])
    sq = g.call_function(torch.ops.aten.squeeze.dims, (x, [0, 2]))
    sq.meta["val"] = torch.empty(64, 512, device="meta")
    reset_placement_options_cache()
    fallback_reasons.clear()
    out = get_placement_options_for_node(mesh, sq, [sx], [x.meta["val"]], (sx, [0, 2]))
    assert not fallback_reasons
    assert {(st.input_specs[0].placements, st.output_specs.placements) for st in out.strategies} == {
        ((R, R), (R, R)), ((Shard(1), R), (Shard(0), R)), ((Shard(3), Shard(1)), (Shard(1), Shard(0)))}
    y = g.placeholder("y")
    y.meta["val"] = torch.empty(256, 64, 8, 8, device="meta")
    sy = OpStrategy([_one(mesh, (256, 64, 8, 8), p) for p in [(R, R), (Shard(0), R), (Shard(1), R)]])
    vm = g.call_function(torch.ops.aten.var_mean.correction, (y, [0, 2, 3]), {"correction": 0, "keepdim": True})
    vm.meta["val"] = (torch.empty(1, 64, 1, 1, device="meta"), torch.empty(1, 64, 1, 1, device="meta"))
    out = get_placement_options_for_node(mesh, vm, [sy], [y.meta["val"]], (sy, [0, 2, 3]))
    assert not fallback_reasons
    for st in out.strategies:
        var, mean = st.output_specs
        assert var.placements == mean.placements and var.tensor_meta.shape == torch.Size([1, 64, 1, 1])
        # not linear: nothing stays sharded on a reduced dim, the channel shard survives
        assert all(not p.is_shard() or p.dim == 1 for p in st.input_specs[0].placements)
    assert ((Shard(1), R), (Shard(1), R)) in {(st.input_specs[0].placements, st.output_specs[0].placements) for st in out.strategies}
