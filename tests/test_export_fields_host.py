"""The fields of the plan export that come from the FX graph (module path,
phase, repeated-layer index, cluster roots): autoparallel_amd.export_json against
the scenarios of the reference's tests/test_export_json.py:44-128 and the rules
of its export_json.py:23-215."""
import contextlib
from types import SimpleNamespace

import torch
from torch import nn

from autoparallel_amd import export_json as X


class Repeated(nn.Module):
    def __init__(self, dim, n_layers):
        super().__init__()
        self.embed = nn.Linear(dim, dim, bias=False)
        self.layers = nn.ModuleList([nn.Linear(dim, dim, bias=False) for _ in range(n_layers)])
        self.head = nn.Linear(dim, dim, bias=False)

    def forward(self, x):
        x = self.embed(x)
        for layer in self.layers:
            x = layer(x)
        return self.head(x)


def _joint(n_layers):
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        m, x = Repeated(64, n_layers), torch.rand(16, 64)
        with contextlib.ExitStack() as stack:
            return aot_export_joint_with_descriptors(stack, m, (x,)).graph_module


def test_layer_index_from_the_module_stack():
    gm = torch.fx.symbolic_trace(Repeated(64, 3))  # a tracer that records the module stack
    layers, outside = set(), 0
    for n in gm.graph.nodes:
        i = X.layer_index(n)
        if i is not None:
            layers.add(i)
        elif n.op not in ("placeholder", "output"):
            outside += 1
    assert layers == {0, 1, 2} and outside == 2  # embed and head are in no numbered layer
    assert {X.module_path(n) for n in gm.graph.nodes if n.op == "call_module"} == {"embed", "layers.0", "layers.1", "layers.2", "head"}
    assert X.layer_index(SimpleNamespace(meta={})) is None
    assert X.layer_index(SimpleNamespace(meta={"nn_module_stack": {}})) is None
    assert X.layer_index(SimpleNamespace(meta={"fwd_nn_module_stack": {"a": ("model.layers.17.mlp", nn.Linear)}})) == 17


def test_phase_module_path_and_kinds_on_a_joint_graph():
    gm = _joint(2)
    nodes = list(gm.graph.nodes)
    info = X.fx_node_info(nodes)
    assert len(info) == len(nodes)
    by_name = {n.name: i for n, i in zip(nodes, info)}
    params = [n for n in nodes if n.op == "placeholder" and X.placeholder_kind(n) == "param"]
    assert len(params) == 4 and all(by_name[p.name]["phase"] == "forward" for p in params)
    assert {by_name[p.name]["module_path"] for p in params} == {"embed.weight", "layers.0.weight", "layers.1.weight", "head.weight"}
    tangents = [n for n in nodes if X.placeholder_kind(n) == "tangent"]
    assert tangents and all(by_name[t.name]["phase"] == "backward" and by_name[t.name]["placeholder_kind"] == "tangent" for t in tangents)
    assert {i["phase"] for i in info} == {"forward", "backward"}
    # this tracer records no module stack: a node next to a parameter is placed by it, the parameter counted by its module
    first_use = [next(iter(p.users)) for p in params]
    assert {by_name[n.name]["module_path"] for n in first_use} == {"embed", "layers.0", "layers.1", "head"}
    assert all(i["op"] for i in info) and all("placeholder_kind" not in i for n, i in zip(nodes, info) if n.op != "placeholder")


class _Node(SimpleNamespace):
    __hash__ = object.__hash__  # nodes are dictionary keys, by identity

    def __eq__(self, other):
        return self is other


def _fake(name, layer=None, op="call_function", inputs=(), users=(), **meta):
    if layer is not None:
        meta["nn_module_stack"] = {"m": (f"layers.{layer}.ffn", nn.Linear)}
    return _Node(name=name, op=op, target=name, meta=meta, all_input_nodes=list(inputs), users=list(users))


def test_module_path_of_a_node_that_lost_its_stack():
    a = _fake("a", nn_module_stack={"m": ("model.layers.3.attn.wq", nn.Linear)})
    b = _fake("b", op="placeholder", desc=SimpleNamespace(target="model.layers.3.attn.wq.weight"))
    c = _fake("c", nn_module_stack={"m": ("model.layers.3.mlp", nn.Linear)})
    assert X.module_path(a) == "model.layers.3.attn.wq" and X.module_path(b) == "model.layers.3.attn.wq.weight"
    assert X.module_path(_fake("lost", inputs=[a, b])) == "model.layers.3.attn.wq"  # the parameter counts by its module
    assert X.module_path(_fake("lost", inputs=[a], users=[c])) == "model.layers.3"
    assert X.module_path(_fake("lost", inputs=[a], users=[_fake("z", nn_module_stack={"m": ("other.block", nn.Linear)})])) is None
    assert X.module_path(_fake("lost", inputs=[_fake("r", nn_module_stack={"m": ("L['self']", nn.Module)})])) is None
    assert X.module_path(_fake("alone")) is None
    assert X.module_path(_fake("saved", module_path="kept.as.written")) == "kept.as.written"


def test_phase_rules_in_their_order():
    assert X.phase(_fake("n", phase="backward", partitioner_tag="is_forward")) == "backward"  # what a saved graph says wins
    assert X.phase(_fake("n", partitioner_tag="is_backward")) == "backward"
    assert X.phase(_fake("n", partitioner_tag="is_forward")) == "forward"
    assert X.phase(_fake("tangents_1", op="placeholder")) == "backward" and X.phase(_fake("primals_1", op="placeholder")) == "forward"
    assert X.phase(_fake("n", layer=0)) == "forward"
    assert X.phase(_fake("n", fwd_nn_module_stack={"m": ("layers.0", nn.Linear)})) == "backward"
    # nothing to go by: position relative to the first tangent input
    graph = SimpleNamespace()
    seq = [_fake("primals_1", op="placeholder"), _fake("x"), _fake("tangents_1", op="placeholder"), _fake("y")]
    graph.nodes = seq
    for n in seq:
        n.graph = graph
    assert X.phase(seq[1]) == "forward" and X.phase(seq[3]) == "backward"


def test_clusters_are_rerooted_at_the_lowest_layer():
    X.normalize_cluster_layer({})
    # forward cluster rooted in layer 0, backward cluster rooted in layer 3 (topological order)
    f = [_fake(f"f{i}", layer=i) for i in range(4)]
    b = [_fake(f"b{i}", layer=i) for i in range(4)]
    roots = {f[1]: f[0], f[2]: f[0], f[3]: f[0], b[0]: b[3], b[1]: b[3], b[2]: b[3]}
    X.normalize_cluster_layer(roots)
    assert roots == {f[1]: f[0], f[2]: f[0], f[3]: f[0], b[1]: b[0], b[2]: b[0], b[3]: b[0]}
    # a cluster without a copy in the lowest layer moves to its nearest one; nodes outside numbered layers stay
    c = [_fake(f"c{i}", layer=i) for i in (1, 2, 3)]
    u = [_fake("u0"), _fake("u1")]
    roots = {f[1]: f[0], c[0]: c[2], c[1]: c[2], u[1]: u[0]}
    X.normalize_cluster_layer(roots)
    assert roots == {f[1]: f[0], c[1]: c[0], c[2]: c[0], u[1]: u[0]}
    # the export numbers clusters by root and names the root on the linked nodes only
    info = X.fx_node_info(f + b, {f[1]: f[0], b[0]: b[3], b[1]: b[3]})
    by = {n.name: i for n, i in zip(f + b, info)}
    assert by["f0"]["cluster_id"] == by["f1"]["cluster_id"] and by["f1"]["cluster_root"] == "f0" and "cluster_root" not in by["f0"]
    assert by["b0"]["cluster_id"] == by["b1"]["cluster_id"] == by["b3"]["cluster_id"] != by["f0"]["cluster_id"]
    assert by["b1"]["cluster_root"] == by["b3"]["cluster_root"] == "b0" and "cluster_id" not in by["f2"]


def test_cluster_keys_follow_the_reference_hash_key():
    """What the packed arrays do not hold of the reference's clustering key
    (graph_clustering.py:35-52, 68-73): operator name, tag, source position and arguments
    (tensors by metadata, integers by value).  Same on all of them: same id."""
    from torch.fx.experimental.proxy_tensor import make_fx

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    def f(x):
        for _ in range(2):
            x = torch.relu(x)  # one source line, same argument metadata: duplicates
        s0, s1 = x.sum(0), x.sum(1)
        return torch.sigmoid(x), s0, s1

    gm = make_fx(f)(torch.randn(4, 4))
    nodes = [n for n in gm.graph.nodes if n.op != "output"]
    ids = dict(zip((n.name for n in nodes), ShardingOptimizer._cluster_keys(nodes)))
    relus = [n.name for n in nodes if "relu" in n.name]
    sums = [n.name for n in nodes if "sum" in n.name]
    assert len(relus) == 2 and ids[relus[0]] == ids[relus[1]]
    assert len(sums) == 2 and ids[sums[0]] != ids[sums[1]]  # the dimension is part of the key
    assert len({ids[relus[0]], ids[sums[0]], ids[sums[1]], ids[next(n.name for n in nodes if "sigmoid" in n.name)]}) == 4
    nodes[1].meta["partitioner_tag"] = "is_backward"
    again = ShardingOptimizer._cluster_keys(nodes)
    assert again[1] != again[2]  # a different tag separates them


def test_cluster_keys_partition_like_the_pickled_key_of_the_reference():
    """The reference hashes a pickle, made by torch's InputPickler, of (operator name, tag, source
    position, argument values with tensors by their fake-tensor metadata, strategies)
    (graph_clustering.py:35-52, 68-81).  On a traced joint graph the ids of _cluster_keys group the
    nodes exactly as the non-strategy part of that pickle does (the strategies are the packed
    arrays' part of the key)."""
    from torch._dynamo.graph_region_tracker import InputPickler
    from torch.utils._pytree import tree_flatten

    from autoparallel_amd.optimize_sharding import ShardingOptimizer

    gm = _joint(4)
    nodes = [n for n in gm.graph.nodes if n.op != "output"]
    assert {n.meta.get("partitioner_tag") for n in nodes} >= {"is_forward", "is_backward"}
    # this tracer records no source positions; give the matmuls of the layers two different ones
    mms = [n for n in nodes if n.target is torch.ops.aten.mm.default]
    for i, n in enumerate(mms):
        n.meta["stack_trace"] = f'File "model.py", line {20 + i % 2}, in forward'
    pickler = InputPickler()

    def extract(a):
        if isinstance(a, torch.fx.Node):
            return a.meta.get("val")
        return a if isinstance(a, (torch.Tensor, int)) else None

    def pickled(n):
        flat, _ = tree_flatten(n.args)
        kw = sorted(n.kwargs.items(), key=lambda kv: kv[0])
        flat_kw, _ = tree_flatten(kw)
        key = (str(n.target), n.meta.get("partitioner_tag"), n.meta.get("stack_trace"),
               (tuple(sorted(n.kwargs)), tuple(extract(a) for a in flat + flat_kw)))
        return pickler.dumps(key)

    theirs = {}
    for i, n in enumerate(nodes):
        theirs.setdefault(pickled(n), []).append(i)
    mine = {}
    for i, k in enumerate(ShardingOptimizer._cluster_keys(nodes)):
        mine.setdefault(int(k), []).append(i)
    assert sorted(theirs.values()) == sorted(mine.values())
    assert max(len(v) for v in mine.values()) >= 4  # the repeated layers do fall together
    by_node = dict(zip(nodes, ShardingOptimizer._cluster_keys(nodes)))
    assert all(by_node[a] != by_node[b] for a, b in zip(mms, mms[1:]))  # neighbours differ in source position
