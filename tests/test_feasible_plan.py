"""Host side of the feasible draws on the planner stress DAG: the Partial masks read off
the spec words, the rule they stand for against the oracle's forbidden entries, and the
plan that confines the producers of the nodes that would run out of strategies."""
import numpy as np
import pytest

from autoparallel_amd import feasible_plan as FP
from autoparallel_amd import graphgen as G
from oracle import cost_oracle as O

MESH = (4, 8, 8)


@pytest.fixture(scope="module")
def small_dag():
    # few strategies per node: many nodes without a strategy that asks for no Partial
    g, gid, _ = G.stress_dag_window(600, 0, 600, MESH, 0, 4, 48)
    ref = O.GraphOracle(g).build()
    _, forbidden = O.clamp_inf(ref["cost"])
    return g, forbidden


def test_mask_rule_is_the_forbidden_entries(small_dag):
    """An entry is forbidden exactly where the consumer's input spec has a Partial on a
    mesh dim where the producer's output spec has none (every entry of the graph)."""
    g, forbidden = small_dag
    nodes = FP.window_masks(g)
    checked = 0
    for v, nm in nodes.items():
        k = 0
        for e in range(int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])):
            u = int(g.edge_src_node[e])
            if u < 0:
                continue
            sdst, ssrc, off = int(g.edge_sdst[e]), int(g.edge_ssrc[e]), int(g.edge_off[e])
            block = forbidden[off: off + sdst * ssrc].reshape(sdst, ssrc) != 0
            rule = (nm.wants[k][:, None] & ~nodes[u].out[None, :]) != 0
            assert (rule == block).all(), (v, e)
            assert nm.producers[k] == u
            checked += block.size
            k += 1
    assert checked == g.num_entries - sum(int(g.node_nstrat[v]) for v in nodes if not nodes[v].producers)
    assert 0.2 < forbidden.mean() < 0.6


def test_plan_leaves_no_node_without_a_strategy(small_dag):
    g, forbidden = small_dag
    nodes = FP.window_masks(g)
    filters, stuck = FP.plan_filters(nodes)
    assert not stuck and filters
    fragile = [v for v, nm in nodes.items() if nm.wants and not nm.has_safe]
    assert len(fragile) > 5
    for v, keep in filters.items():
        assert keep.shape == nodes[v].out.shape and keep.any() and not keep.all()
    # every node keeps a strategy that is allowed whatever its producers take from their filters
    for v, nm in nodes.items():
        rows = filters.get(v, np.ones(nm.out.shape[0], bool))
        served = rows.copy()
        for u, w in zip(nm.producers, nm.wants):
            least = np.bitwise_and.reduce(nodes[u].out[filters.get(u, np.ones(nodes[u].out.shape[0], bool))])
            served &= (w & ~least) == 0  # what every strategy left to u offers covers what the row asks for
        assert served.any(), v
    # and the walk: fallbacks without the plan, none with it, and no forbidden entry selected
    without = with_plan = 0
    for a in range(12):
        without += O.sample_feasible(g, forbidden, 3, a)[1]
        assign, fb = O.sample_feasible(g, forbidden, 3, a, row_filter=filters)
        with_plan += fb
        for v in filters:
            assert filters[v][assign[v]]
        for e in range(g.num_edges):
            u = int(g.edge_src_node[e])
            if u >= 0:
                o, j = assign[int(g.edge_node[e])], assign[u]
                assert not forbidden[int(g.edge_off[e]) + o * int(g.edge_ssrc[e]) + j]
    assert without > 12 and with_plan == 0


def test_masks_without_the_window_equal_the_window_s():
    g, gid, n_standin = G.stress_dag_window(20000, 9000, 9250, MESH, 0, 4, 512)
    a = FP.window_masks(g, gid, n_standin)
    b = G.stress_dag_partial_masks(20000, 9000, 9250, MESH, 0, 4, 512)
    assert sorted(a) == sorted(b) == list(range(9000, 9250))
    for v in a:
        assert (a[v].out == b[v].out).all() and a[v].producers == b[v].producers and a[v].has_safe == b[v].has_safe
        assert len(a[v].wants) == len(b[v].wants) and all((x == y).all() for x, y in zip(a[v].wants, b[v].wants))


def test_a_node_nobody_can_serve_is_reported():
    """A consumer whose only strategy asks for a Partial that no strategy of its producer offers."""
    nodes = {
        0: FP.NodeMasks(out=np.asarray([0, 2], np.uint8)).finish(),
        1: FP.NodeMasks(out=np.asarray([0], np.uint8), producers=[0], wants=[np.asarray([1], np.uint8)]).finish(),
        2: FP.NodeMasks(out=np.asarray([0], np.uint8), producers=[0], wants=[np.asarray([2], np.uint8)]).finish(),
    }
    filters, stuck = FP.plan_filters(nodes)
    assert stuck == [1] and list(filters) == [0] and filters[0].tolist() == [False, True]
