"""Pins for the oracle that do not come from the reference's output: closed
forms derived by hand, exact rational arithmetic, the installed torch functions
the reference calls, and invariants a plausible mistake would break."""
import itertools
import math
from fractions import Fraction

import numpy as np
import pytest

from oracle import cost_oracle as O

R, P, PA = 0x00, 0x80, 0x81


def S(d):
    return 0x40 | d


def test_topology_matches_torch_rule():
    # innermost dims are intra-host until the running product exceeds 8
    t = O.Topo((8, 8), 8)
    assert t.bw == [87.7 * 0.22, 87.7] and t.lat == [2.7, 0.6]
    t = O.Topo((4, 8, 8), 8)
    assert t.lat == [2.7, 2.7, 0.6]
    t = O.Topo((2, 4), 8)
    assert t.lat == [0.6, 0.6]
    t = O.Topo((8, 8), 1)  # no device visible: everything is inter-host
    assert t.lat == [2.7, 2.7]
    t = O.Topo((8,), 8)
    assert t.bw == [87.7]


def test_collectives_against_torch_functions():
    # the reference calls these torch functions directly
    # (collective_runtime_estimation.py:12-18); MeshTopoInfo is a plain
    # dataclass, so it can be built without a process group
    from torch.distributed.tensor._collective_utils import (
        MeshTopoInfo, allgather_cost, allreduce_cost, reduce_scatter_cost)

    topo = O.Topo((4, 8), 8)
    tt = MeshTopoInfo(None, [4, 8], list(topo.bw), list(topo.lat))
    rng = np.random.default_rng(0)
    for g in list(rng.random(50) * 8.0) + [0.0, 1e-9, 123.456]:
        for d in (0, 1):
            assert O.allgather_cost(g, topo, d) == allgather_cost(g, tt, d)
            assert O.allreduce_cost(g, topo, d) == allreduce_cost(g, tt, d)
            assert O.reduce_scatter_cost(g, topo, d) == reduce_scatter_cost(g, tt, d)


def test_collective_closed_form_rational():
    # latency + bytes*hops/n/bw in exact arithmetic agrees to double rounding
    topo = O.Topo((8,), 8)
    g = 0.75
    exact = Fraction(66, 10) + 7 * Fraction(6, 10) + Fraction(3, 4) * 7 / 8 / Fraction(877, 10) * 10**6
    assert math.isclose(O.allgather_cost(g, topo, 0), float(exact), rel_tol=1e-14)
    exact_ar = Fraction(66, 10) + 14 * Fraction(6, 10) + Fraction(3, 4) * 14 / 8 / Fraction(877, 10) * 10**6
    assert math.isclose(O.allreduce_cost(g, topo, 0), float(exact_ar), rel_tol=1e-14)
    assert O.all_to_all_cost(g, topo, 0) == O.allgather_cost(g, topo, 0) * 5


def test_hand_derived_single_dim_cases():
    """1-D mesh of 8 intra-host devices, 1 GiB contiguous fp32 tensor."""
    topo, dev = O.Topo((8,), 8), O.DeviceLimit()
    shape, stride, isz = (16384, 16384), (16384, 1), 4  # 2**30 bytes
    cost = lambda s, t: O.estimate_strategy_comms_cost(s, shape, stride, isz, t, topo, dev)
    lat = 6.6 + 7 * 0.6
    # S(0)->R: shard is 1/8 GiB, gathered to 1 GiB; no reshuffle for dim 0
    assert cost((S(0),), (R,)) == lat + (1.0 * 7 / 8) / 87.7 * 1e6
    # S(1)->R adds a read+write of the gathered tensor: 2 GiB at 8 TiB/s / 0.7
    rw = max((2 * 2**30) / (8.0 * 1024**4) * 1e6 / 0.70, 7)
    assert cost((S(1),), (R,)) == (lat + (1.0 * 7 / 8) / 87.7 * 1e6) + rw
    # P->R: all-reduce of the whole 1 GiB, 14 hops
    assert cost((P,), (R,)) == (6.6 + 14 * 0.6) + (1.0 * 14 / 8) / 87.7 * 1e6
    # P->S(0): reduce-scatter of 1 GiB
    assert cost((P,), (S(0),)) == lat + (1.0 * 7 / 8) / 87.7 * 1e6
    # S(0)->S(1): all-to-all of the 1/8 GiB shard (x5) plus one reshuffle of 2/8 GiB
    rw8 = max((2 * 2**27) / (8.0 * 1024**4) * 1e6 / 0.70, 7)
    assert cost((S(0),), (S(1),)) == (lat + (0.125 * 7 / 8) / 87.7 * 1e6) * 5 + 1 * rw8
    # forbidden
    assert cost((S(0),), (P,)) == math.inf
    assert cost((R,), (P,)) == math.inf
    # free
    assert cost((R,), (S(0),)) == 0.0
    assert cost((R,), (R,)) == 0.0
    assert cost((P,), (PA,)) == 0.0  # Partial(sum)->Partial(avg): no branch


def test_invariants_brute_force_small_meshes():
    dev = O.DeviceLimit()
    for mesh in [(2,), (4,), (2, 2), (2, 4), (3, 2)]:
        topo = O.Topo(mesh, 8)
        for shape in [(8, 12), (64, 6, 10)]:
            stride = tuple(int(np.prod(shape[i + 1:])) for i in range(len(shape)))
            opts = [R] + [S(i) for i in range(len(shape))] + [P]
            for s in itertools.product(opts, repeat=len(mesh)):
                for t in itertools.product(opts, repeat=len(mesh)):
                    c = O.estimate_strategy_comms_cost(s, shape, stride, 4, t, topo, dev)
                    assert c >= 0.0
                    if s == t:
                        assert c == 0.0
                    # R->P or S->P on any dim that is reached is forbidden
                    if all(x == R for x in s):
                        assert c == (math.inf if any(x == P for x in t) else 0.0)
                    # doubling the tensor never lowers a finite cost
                    c2 = O.estimate_strategy_comms_cost(s, (shape[0] * 2,) + shape[1:],
                                                        (stride[0],) + stride[1:], 4, t, topo, dev)
                    if math.isfinite(c):
                        assert c2 >= c


def test_noncontiguous_source_pays_one_extra_copy():
    topo, dev = O.Topo((8,), 8), O.DeviceLimit()
    shape = (4096, 8192)
    contig = O.estimate_strategy_comms_cost((S(0),), shape, (8192, 1), 2, (R,), topo, dev)
    transposed = O.estimate_strategy_comms_cost((S(0),), shape, (1, 4096), 2, (R,), topo, dev)
    gb = 2 * 4096 * 8192 / 8 / 1024 / 1024 / 1024
    # cost = (0.0 + rw(unsharded-by-this-dim bytes * 2)) + allgather
    assert transposed == O.compute_read_write_time(gb * 2 * 1024**3, dev) + contig
    assert transposed > contig


def test_contiguity_rule():
    assert O.check_contiguous((4, 5), (5, 1))
    assert not O.check_contiguous((4, 5), (1, 4))
    assert O.check_contiguous((1, 5), (999, 1))  # size-1 dims are skipped
    assert O.check_contiguous((4, 1, 5), (5, 7, 1))
    assert O.check_contiguous((), ())
    import torch
    from torch._prims_common import check_contiguous_sizes_strides
    for shape, perm in [((2, 3, 4), (0, 1, 2)), ((2, 3, 4), (2, 0, 1)), ((1, 3, 1), (2, 1, 0)),
                        ((5,), (0,)), ((2, 1, 4), (1, 0, 2))]:
        t = torch.empty(shape, device="meta").permute(perm)
        assert O.check_contiguous(tuple(t.shape), tuple(t.stride())) == \
            check_contiguous_sizes_strides(t.shape, t.stride())


def test_rw_time_floor_and_slope():
    dev = O.DeviceLimit()
    assert O.compute_read_write_time(0, dev) == 7
    # 7 us * 0.7 * 8 TiB/s = 43.1 MB is where the floor ends
    edge = 7e-6 * 0.70 * 8.0 * 1024**4
    assert O.compute_read_write_time(int(edge) - 1000, dev) == 7
    assert O.compute_read_write_time(int(edge) + 1000, dev) > 7
    assert O.compute_read_write_time(2**40, dev) == (2**40 / (8.0 * 1024**4) * 1e6) / 0.70


def test_sequential_ceil_division():
    # same convention the reference pins for its sibling _localize_shape_arg
    # (tests/test_dynamic_shapes.py:708-738 there): 1024 over (4, 64) -> 4; 10 over 3 -> 4
    assert O.sharded_shape_stride((1024,), (1,), (S(0), S(0)), (4, 64))[0] == [4]
    assert O.sharded_shape_stride((10,), (1,), (S(0),), (3,))[0] == [4]
    # stride quirk: only dims with d-1 > 0 adjust the previous stride
    shape, stride = (8, 6, 4), (24, 4, 1)
    assert O.sharded_shape_stride(shape, stride, (S(1),), (2,)) == ([8, 3, 4], [24, 4, 1])
    assert O.sharded_shape_stride(shape, stride, (S(2),), (2,)) == ([8, 6, 2], [24, 2, 1])


def test_validity_rule_cases_of_reference_tests():
    # expectations of the reference's tests/test_placement_options_utils.py:28-124
    assert O.is_valid_spec((256, 64), (S(0),), (256,))
    assert not O.is_valid_spec((100, 64), (S(0),), (256,))
    assert O.is_valid_spec((7, 3), (R,), (256,))
    assert O.is_valid_spec((256, 10), (S(0), S(1)), (32, 8))  # uneven but non-empty
    assert O.is_valid_spec((257, 64), (S(0), R), (32, 8))
    # same dim sharded twice: second division sees the already divided size
    assert O.is_valid_spec((64,), (S(0), S(0)), (8, 8))

def test_create_all_options_counts_and_order():
    opts = O.create_all_options((64, 8192, 4096), (8, 8))
    assert len(opts) == 16 and opts[0] == (R, R) and opts[1] == (R, S(0)) and opts[4] == (S(0), R)
    # a dim of 4 cannot be sharded over 8
    opts = O.create_all_options((4, 4096), (8, 8))
    assert all(S(0) not in o for o in opts) and len(opts) == 4
    assert O.create_all_options((), (8, 8)) == [(R, R)]


def test_validity_63():
    # 63 over (8, 8) on the same dim: 63 >= 8 -> 8, then 8 >= 8 -> 1: valid
    assert O.is_valid_spec((63,), (S(0), S(0)), (8, 8))


def test_roofline_closed_form():
    dev = O.DeviceLimit()
    # compute bound: 2*8192*4096*14336 flops at 2516.6 TFLOPS / 0.7
    fl = 2 * 8192 * 4096 * 14336
    assert O.roofline_cost(fl, 1000, 3, dev) == (fl / (2516.6 * 10**12) * 1e6) / 0.70
    # memory bound
    assert O.roofline_cost(1, 2**36, 3, dev) == (2**36 / (8.0 * 1024**4) * 1e6) / 0.70
    assert O.roofline_cost(0, 10, 3, dev) == 7
    with pytest.raises(ValueError):
        O.roofline_cost(10, 10, 5, dev)


# ---------------------------------------------------------------------------
# the sampler of assignments without a forbidden variable (no reference counterpart)
# ---------------------------------------------------------------------------
def _sampler_graph():
    from autoparallel_amd import graphgen

    g = graphgen.llama_graph((2, 4), 1, 64, 4, 2, 128, 256, 32, 16)
    ref = O.GraphOracle(g).build()
    _, forbidden = O.clamp_inf(ref["cost"])
    return g, ref, forbidden


def test_sampled_assignments_select_no_forbidden_variable():
    g, ref, forbidden = _sampler_graph()
    assert forbidden.any()
    clamped, _ = O.clamp_inf(ref["cost"])
    plain_hits = clean = 0
    for a in range(40):
        assign, fallbacks = O.sample_feasible(g, forbidden, 11, a)
        _, viol = O.ilp_objective(g, clamped, forbidden, assign)
        if fallbacks == 0:  # every node found an allowed strategy: nothing forbidden is selected
            assert viol == 0
            clean += 1
        plain = [O.plain_draw(11, a, v, int(g.node_nstrat[v])) for v in range(g.num_nodes)]
        plain_hits += O.ilp_objective(g, clamped, forbidden, plain)[1] > 0
    assert clean > 0
    assert plain_hits == 40  # the plain draws all select something forbidden on this graph


def test_sampler_is_uniform_over_the_allowed_strategies_of_a_node():
    """Frequencies of a node's choice over many assignments with its producer's
    choice given: every allowed strategy is reached, no other one is, and none is
    favoured (chi-square against the flat distribution).  The forbidden mask is
    made by hand, so the allowed set is known without the sampler."""
    from helpers import graph_from_pairs

    n_src, n_tgt = 3, 12
    g = graph_from_pairs((2, 4), 8, (64, 64), (64, 1), 4, [(0, 0), (0x40, 0), (0, 0x41)],
                         [(0, 0)] * n_tgt)
    assert g.num_nodes == 2 and int(g.node_nstrat[1]) == n_tgt
    e = int(g.node_edge_off[1])
    forbidden = np.zeros(g.num_slots, np.uint8)
    allowed = {0: [1, 2, 3, 5, 8, 11], 1: [4], 2: []}
    for j in range(n_src):
        for o in range(n_tgt):
            if o not in allowed[j]:
                forbidden[int(g.edge_off[e]) + o * n_src + j] = 1
    n = 6000
    for j in range(n_src):
        hist, fallback_total = {}, 0
        for a in range(n):
            assign, fallbacks = O.sample_feasible(g, forbidden, 5, a, first_node=1, given=[j])
            hist[assign[1]] = hist.get(assign[1], 0) + 1
            fallback_total += fallbacks
        if not allowed[j]:  # nothing allowed: the plain draw over all strategies, counted
            assert fallback_total == n and len(hist) == n_tgt
            assert all(O.plain_draw(5, a, 1, n_tgt) == O.sample_feasible(g, forbidden, 5, a, first_node=1, given=[j])[0][1]
                       for a in range(50))
            continue
        assert fallback_total == 0 and sorted(hist) == allowed[j], (j, sorted(hist))
        k = len(allowed[j])
        chi2 = sum((hist[o] - n / k) ** 2 / (n / k) for o in allowed[j])
        assert chi2 < 20.5, (j, chi2)  # 99.9th percentile of chi-square with 5 degrees of freedom
