"""Parameter-derived and terminal-derived node sets on hand-built joint graphs:
the known answers of the reference's tests/test_prefetch_derived_sets.py
(:53-245)."""
import torch
import torch.fx
from torch._functorch._aot_autograd.descriptors import GradAOTOutput, ParamAOTInput, PlainAOTInput, PlainAOTOutput

from autoparallel_amd.graph_utils import build_param_derived_set, build_terminal_derived_set

_op = torch.ops.aten.abs.default


def _ph(graph, name, desc):
    n = graph.placeholder(name)
    n.meta["desc"] = desc
    return n


def _call(graph, *args):
    return graph.call_function(_op, args=args)


def _out(graph, outs, descs):
    o = graph.output(tuple(outs))
    o.meta["desc"] = descs
    return o


def test_param_derived_chain_fan_in_and_stop():
    g = torch.fx.Graph()
    w, x = _ph(g, "w", ParamAOTInput("w")), _ph(g, "x", PlainAOTInput(0))
    cast = _call(g, w)
    alias = _call(g, cast)
    mm = _call(g, x, alias)
    post = _call(g, mm)
    _out(g, [post], [PlainAOTOutput(0)])
    d = build_param_derived_set(g)
    assert {w, cast, alias} <= d and x not in d and mm not in d and post not in d

    g = torch.fx.Graph()
    p1, p2, inp = _ph(g, "p1", ParamAOTInput("a")), _ph(g, "p2", ParamAOTInput("b")), _ph(g, "i", PlainAOTInput(0))
    both, mixed = _call(g, p1, p2), _call(g, p1, inp)
    _out(g, [both, mixed], [PlainAOTOutput(0), PlainAOTOutput(1)])
    d = build_param_derived_set(g)
    assert both in d and mixed not in d

    g = torch.fx.Graph()
    x = _ph(g, "x", PlainAOTInput(0))
    _out(g, [_call(g, x)], [PlainAOTOutput(0)])
    assert len(build_param_derived_set(g)) == 0

    g = torch.fx.Graph()
    node = p = _ph(g, "p", ParamAOTInput("w"))
    chain = [p]
    for _ in range(10):
        node = _call(g, node)
        chain.append(node)
    _out(g, [node], [PlainAOTOutput(0)])
    assert set(chain) <= build_param_derived_set(g)


def test_terminal_derived_known_answers():
    g = torch.fx.Graph()
    pd = ParamAOTInput("w")
    param, inp = _ph(g, "param", pd), _ph(g, "inp", PlainAOTInput(0))
    fwd = _call(g, inp, param)
    bwd = _call(g, fwd)
    view = _call(g, bwd)
    alias = _call(g, view)
    _out(g, [fwd, alias], [PlainAOTOutput(0), GradAOTOutput(grad_of=pd)])
    t = build_terminal_derived_set(g)
    assert {alias, view, bwd} <= t and fwd not in t

    g = torch.fx.Graph()
    param, inp = _ph(g, "param", pd), _ph(g, "inp", PlainAOTInput(0))
    fwd = _call(g, inp, param)
    bwd = _call(g, fwd)
    grad, compute = _call(g, bwd), _call(g, bwd)
    _out(g, [fwd, grad, compute], [PlainAOTOutput(0), GradAOTOutput(grad_of=pd), PlainAOTOutput(1)])
    t = build_terminal_derived_set(g)
    assert grad in t and bwd not in t

    g = torch.fx.Graph()
    inp = _ph(g, "inp", PlainAOTInput(0))
    _out(g, [_call(g, inp)], [PlainAOTOutput(0)])
    assert len(build_terminal_derived_set(g)) == 0

    g = torch.fx.Graph()
    da, db = ParamAOTInput("a"), ParamAOTInput("b")
    pa, pb, inp = _ph(g, "pa", da), _ph(g, "pb", db), _ph(g, "inp", PlainAOTInput(0))
    fwd = _call(g, inp, pa, pb)
    ca = _call(g, fwd)
    ga = _call(g, ca)
    cb = _call(g, fwd)
    gb = _call(g, cb)
    _out(g, [fwd, ga, gb], [PlainAOTOutput(0), GradAOTOutput(grad_of=da), GradAOTOutput(grad_of=db)])
    t = build_terminal_derived_set(g)
    assert {ga, ca, gb, cb} <= t and fwd not in t


def test_add_alias_nodes():
    """An alias after every tensor node with two or more users (the users read
    the alias) and after every returned node
    (autoparallel/graph_passes/graph_utils.py:99-183, "v2")."""
    import torch

    from autoparallel_amd.graph_utils import add_alias_nodes

    aten = torch.ops.aten
    g = torch.fx.Graph()
    x = g.placeholder("x")
    x.meta["val"] = torch.empty(4, 4, device="meta")
    a = g.call_function(aten.relu.default, (x,))
    a.meta["val"] = torch.empty(4, 4, device="meta")
    b = g.call_function(aten.add.Tensor, (a, x))
    b.meta["val"] = torch.empty(4, 4, device="meta")
    c = g.call_function(aten.mul.Tensor, (a, b))
    c.meta["val"] = torch.empty(4, 4, device="meta")
    g.output((c, b))
    gm = add_alias_nodes(torch.fx.GraphModule(torch.nn.Module(), g))
    gm.graph.lint()
    nodes = list(gm.graph.nodes)
    alias = [n for n in nodes if n.op == "call_function" and n.target is aten.alias.default]
    # x (relu, add), relu (add, mul) and add (mul, output) fan out; mul and add's alias are returned
    assert len(alias) == 5
    of = lambda n: [al for al in alias if al.args[0] is n]
    assert len(of(x)) == 1 and set(of(x)[0].users) == {a, b} and list(x.users) == of(x)
    assert len(of(a)) == 1 and set(of(a)[0].users) == {b, c}
    fan = of(b)[0]
    out = nodes[-1]
    returned = list(out.all_input_nodes)
    assert all(r.target is aten.alias.default for r in returned)
    # the returned add already fans out: its second alias takes over every user of the first, as in the reference
    assert returned[0].args[0] is c and returned[1].args[0] is fan and c.args[1] is returned[1]
    assert list(fan.users) == [returned[1]]
    assert all(al.meta["val"].shape == (4, 4) for al in alias)
    # the alias of a fanned-out node sits before its first user
    assert nodes.index(of(x)[0]) < nodes.index(a)
