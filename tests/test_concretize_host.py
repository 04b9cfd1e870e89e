"""The host helpers that turn a traced graph with symbolic sizes into the
concrete twin the planner prices (autoparallel/optimize_sharding.py:111-218),
on the scenarios the reference's tests/test_dynamic_shapes.py:293-478 states."""
import pytest
import torch
from torch._subclasses import FakeTensorMode
from torch.fx import Graph, GraphModule
from torch.fx.experimental.symbolic_shapes import DimDynamic, ShapeEnv, StatelessSymbolicContext

from autoparallel_amd.optimize_sharding import (_has_symbolic_sizes, _produces_tensor, concretize_args,
                                                concretize_gm, concretize_symint)

DYN, STATIC = DimDynamic.DYNAMIC, DimDynamic.STATIC


def _symbolic(shape, dynamic, device="cpu"):
    mode = FakeTensorMode(shape_env=ShapeEnv(), static_shapes=False)
    t = mode.from_tensor(torch.empty(*shape, device=device), symbolic_context=StatelessSymbolicContext(dynamic_sizes=list(dynamic)))
    return mode, t


def test_symints_and_symbolic_tensors_become_concrete():
    _, x = _symbolic((16, 128), (DYN, DYN))
    assert all(isinstance(s, torch.SymInt) for s in x.shape)
    tensor, n, nested = concretize_args((x, x.shape[0], [x.shape[1], 32]))
    assert isinstance(tensor, torch.Tensor) and all(type(s) is int for s in tensor.shape)
    assert tuple(tensor.shape) == (16, 128) and tuple(tensor.stride()) == (128, 1) and tensor.dtype == x.dtype
    assert type(n) is int and n == 16
    assert type(nested[0]) is int and nested == [128, 32]
    assert concretize_symint(x.shape[1]) == 128 and concretize_symint(7) == 7 and concretize_symint("s") == "s"


def test_concrete_values_pass_through():
    t = torch.randn(4, 4)
    out = concretize_args((t, 42, [1, 2, 3], None, {"k": 2.5}))
    assert out[0] is t and out[1] == 42 and out[2] == [1, 2, 3] and out[3] is None and out[4] == {"k": 2.5}


def _relu_graph(dynamic):
    mode, sym = _symbolic((16, 128), dynamic, device="meta")
    graph = Graph()
    x = graph.placeholder("x")
    x.meta["val"] = sym
    x.meta["desc"] = "descriptor of x"
    x.meta["custom_key"] = 42
    y = graph.call_function(torch.relu, (x,))
    with mode:
        y.meta["val"] = torch.relu(sym)
    graph.output(y)
    return GraphModule({}, graph)


def test_twin_graph_has_the_same_structure_and_a_total_mapping():
    gm = _relu_graph((DYN, STATIC))
    assert _has_symbolic_sizes(gm)
    twin, to_twin, to_orig = concretize_gm(gm)
    a, b = list(gm.graph.nodes), list(twin.graph.nodes)
    assert len(a) == len(b) == len(to_twin) == len(to_orig)
    for orig, conc in zip(a, b):
        assert (orig.op, orig.target, orig.name) == (conc.op, conc.target, conc.name)
        assert to_twin[orig] is conc and to_orig[conc] is orig
        assert [to_twin[u] for u in orig.all_input_nodes] == list(conc.all_input_nodes)  # edges follow the mapping
    assert not _has_symbolic_sizes(twin)


def test_twin_metadata_is_concrete_and_the_rest_is_kept():
    gm = _relu_graph((DYN, DYN))
    twin, _, _ = concretize_gm(gm)
    for n in twin.graph.nodes:
        if n.op == "output":
            continue
        val = n.meta["val"]
        assert all(type(s) is int for s in val.shape) and tuple(val.shape) == (16, 128)
    x = next(n for n in twin.graph.nodes if n.op == "placeholder")
    assert x.meta["desc"] == "descriptor of x" and x.meta["custom_key"] == 42
    # the original keeps its symbols
    ox = next(n for n in gm.graph.nodes if n.op == "placeholder")
    assert any(isinstance(s, torch.SymInt) for s in ox.meta["val"].shape)


def test_graph_without_symbols_is_recognised():
    mode = FakeTensorMode()
    graph = Graph()
    x = graph.placeholder("x")
    with mode:
        x.meta["val"] = torch.empty(4, 8)
    graph.output(x)
    assert not _has_symbolic_sizes(GraphModule({}, graph))


@pytest.mark.parametrize("val, want", [
    (torch.randn(4), True), ((torch.randn(4), torch.randn(4)), True), ((torch.randn(4), None), True),
    ([None, (torch.randn(2),)], True), (42, False), (None, False), ((None, 3), False), ((), False),
])
def test_produces_tensor(val, want):
    assert _produces_tensor(val) is want


def test_collector_pause_hands_long_lived_objects_over_without_a_walk():
    """_gc_paused: the collector is off inside, on again after (if it was on), and what was
    allocated inside does not sit in the youngest generation afterwards; a frozen generation
    of the caller's own is left as it is."""
    import gc

    from autoparallel_amd.optimize_sharding import _gc_paused

    class Box:
        def __init__(self):
            self.ref = [self]  # a container the collector tracks

    assert gc.isenabled()
    gc.collect()
    with _gc_paused():
        assert not gc.isenabled()
        keep = [Box() for _ in range(5000)]
    assert gc.isenabled() and gc.get_freeze_count() == 0
    assert gc.get_count()[0] < 5000  # the 10 000 new containers are not counted as young
    assert len(keep) == 5000
    # nested use and a collector that was off before: left off
    gc.disable()
    try:
        with _gc_paused():
            pass
        assert not gc.isenabled()
    finally:
        gc.enable()
    # the caller's frozen generation survives
    gc.freeze()
    try:
        frozen = gc.get_freeze_count()
        assert frozen > 0
        with _gc_paused():
            more = [Box() for _ in range(100)]
        assert gc.get_freeze_count() == frozen and gc.isenabled() and len(more) == 100
    finally:
        gc.unfreeze()
