"""format_sharding_log on records built the way callers of the reference build
them (``DecisionVar(var=..., cost=..., ...)``, autoparallel/optimize_sharding.py:
191-203): the scenarios of the reference's tests/test_log_formatting.py:47-470."""
import pytest
import torch
import torch.fx

from autoparallel_amd.log_formatting import format_sharding_log
from autoparallel_amd.optimize_sharding import DecisionVar


class _Named:
    def __init__(self, name):
        self.name = name

    def __str__(self):
        return self.name


def entry(name, comm=0.0, compute=0.0, transition=0.0):
    return DecisionVar(var=None, cost=comm + compute + transition, compute_cost=compute, comm_cost=comm,
                       sharding_transition_cost=transition, strategy=_Named(name), output_spec=None, input_spec=None)


def graph_of(fn):
    return torch.fx.symbolic_trace(fn).graph


def test_record_holds_its_fields_and_refuses_others():
    e = entry("Shard(0)", comm=1.0, compute=2.0, transition=1.0)
    assert (e.cost, e.comm_cost, e.compute_cost, e.sharding_transition_cost) == (4.0, 1.0, 2.0, 1.0)
    assert str(e.strategy) == "Shard(0)" and e.var is None and e.output_spec is None and e.input_spec is None
    e.cost, e.comm_cost = 10.0, 7.0
    assert (e.cost, e.comm_cost) == (10.0, 7.0) and e.value() is None and "comm_cost=7.0" in repr(e)
    with pytest.raises(TypeError, match="missing"):
        DecisionVar(var=None, cost=1.0)
    with pytest.raises(TypeError, match="unexpected"):
        DecisionVar(var=None, cost=1.0, compute_cost=0.0, comm_cost=0.0, sharding_transition_cost=0, strategy=None,
                    output_spec=None, input_spec=None, weight=3)


def test_every_assignment_line_gets_its_own_annotation():
    graph = graph_of(lambda x: ((x + 1) * 2) - 3)
    x, add, mul, sub, out = list(graph.nodes)
    text = format_sharding_log(graph, {add: [entry("Strategy_A")], mul: [entry("Strategy_B")], sub: [entry("Strategy_C")]})
    for name, node in (("Strategy_A", "add"), ("Strategy_B", "mul"), ("Strategy_C", "sub")):
        lines = [ln for ln in text.split("\n") if name in ln]
        assert len(lines) == 1 and node in lines[0].lower()


def test_placeholders_are_annotated_and_the_output_is_not():
    graph = graph_of(lambda x, y: x + y)
    x, y, add, out = list(graph.nodes)
    text = format_sharding_log(graph, {x: [entry("Replicate()")], y: [entry("Shard(0)")], out: [entry("ShouldNotAppear")]})
    assert "Replicate()" in text and "Shard(0)" in text and "ShouldNotAppear" not in text
    # a node without an entry gets no annotation
    text = format_sharding_log(graph, {add: [entry("OnlyThis")]})
    assert text.count("# placement=") == 1 and "OnlyThis" in text


def test_empty_dict_colour_verbose_and_shard_order():
    graph = graph_of(lambda x: x + 1)
    x, add, out = list(graph.nodes)
    text = format_sharding_log(graph, {})
    assert "def forward" in text and "total_cost: 0.00" in text
    opt = {add: [entry("Shard(0)")]}
    assert "\x1b[" in format_sharding_log(graph, opt, colored=True) and "\x1b[" not in format_sharding_log(graph, opt)
    assert len(format_sharding_log(graph, opt, verbose=True)) > len(format_sharding_log(graph, opt, verbose=False))
    add.meta["shard_order"] = (1, 0)
    assert "shard_order=(1, 0)" in format_sharding_log(graph, opt)


def test_strategy_strings_and_cost_extremes():
    graph = graph_of(lambda x: x + 1)
    x, add, out = list(graph.nodes)
    long_name = "(Shard(dim=0), Replicate()) -> (Shard(dim=1), Partial(sum))"
    assert long_name in format_sharding_log(graph, {add: [entry(long_name)]})
    text = format_sharding_log(graph, {add: [entry("S")]})
    assert "total_cost: 0.00" in text and "[(0.0, 0.0, 0.0)]" in text
    text = format_sharding_log(graph, {add: [entry("S", comm=1e10, compute=2e10, transition=3e10)]})
    assert "total_cost: 60000000000.00" in text
    text = format_sharding_log(graph, {add: [entry("S")]},
                               violated_constraints_log="WARNING: Constraint X was violated\nWARNING: Constraint Y was violated")
    assert "WARNING: Constraint X was violated" in text and "WARNING: Constraint Y was violated" in text
