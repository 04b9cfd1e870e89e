"""apc_build_all_noalloc (block table in the library's static device array)
against apc_build_all (block table in a buffer of the caller's), through the C
ABI: two builds in a row, the second on a smaller problem, bit for bit; and the
refusal of a table beyond the static array."""
import ctypes as C

import numpy as np
import pytest

from autoparallel_amd import graphgen

pytestmark = pytest.mark.gpu


def _both(CE, g, **kw):
    import torch

    from autoparallel_amd import _lib

    eng = CE(g, **kw)
    assert eng.use_table and 0 < eng.problem.table_size <= (1 << 20)
    eng.build(clamp_inf=True)
    want = {k: v.copy() for k, v in eng.results().items()}
    for t in (eng.comm, eng.cost, eng.flags, eng.compute, eng.per_arg, eng.status):
        t.zero_()
    eng.table.fill_(float("nan"))  # the caller's table is not touched by the other entry point
    torch.cuda.synchronize()
    rc = eng.lib.apc_build_all_noalloc(
        C.byref(eng.problem), eng._ptr(eng.compute), eng._ptr(eng.per_arg), eng._ptr(eng.status),
        eng._ptr(eng.comm), eng._ptr(eng.cost), eng._ptr(eng.flags), 1, eng._stream())
    _lib.check(rc, "apc_build_all_noalloc")
    got = eng.results()
    assert bool(torch.isnan(eng.table).all())
    for k in ("comm", "cost", "compute", "per_arg"):
        a, b = got[k].view(np.uint64), want[k].view(np.uint64)
        assert (a == b).all(), f"{k}: {(a != b).sum()} of {a.size} differ"
    assert (got["flags"] == want["flags"]).all()
    return eng


def test_noalloc_build_matches_build_all_twice_second_smaller():
    from autoparallel_amd.engine import CostEngine

    big = graphgen.llama_graph((8, 8), 2, 1024, 8, 4, 2048, 8192, 512, 16)
    small = graphgen.llama_graph((2, 4), 1, 64, 4, 2, 128, 256, 32, 16)
    assert small.num_entries < big.num_entries
    _both(CostEngine, big, table_mode="full")
    _both(CostEngine, small, table_mode="full")
    # and the compressed layout, after the two above left their tables in the array
    _both(CostEngine, graphgen.stress_graph(40, (4, 8, 8), seed=5, s_max=24), table_mode="compressed")


def test_noalloc_build_refuses_a_table_beyond_the_static_array():
    from autoparallel_amd.engine import CostEngine

    g = graphgen.stress_graph(120, (4, 8, 8), seed=1)
    eng = CostEngine(g, table_mode="full")
    assert eng.problem.table_size > (1 << 20)
    rc = eng.lib.apc_build_all_noalloc(
        C.byref(eng.problem), eng._ptr(eng.compute), eng._ptr(eng.per_arg), eng._ptr(eng.status),
        eng._ptr(eng.comm), eng._ptr(eng.cost), eng._ptr(eng.flags), 1, eng._stream())
    assert rc == -1
    assert b"static scratch" in eng.lib.apc_last_error()


def test_noalloc_build_of_a_problem_without_a_block_table():
    """table_size == 0: every entry is evaluated directly, as apc_build_all does
    with table == NULL; with and without the problem's tile list."""
    import torch

    from autoparallel_amd import _lib
    from autoparallel_amd.engine import CostEngine

    g = graphgen.stress_graph(60, (2, 4, 4), seed=3, s_max=48)
    for lut in (False, True):
        eng = CostEngine(g, table_mode="direct", lut=lut)
        assert eng.table is None
        # the problem as a caller without a block table describes it
        eng.problem.table_size, eng.problem.n_table_unit, eng.problem.n_block = 0, 0, 0
        assert (eng.problem.n_lut_entry_tile > 0) == lut
        rc = eng.lib.apc_build_all(
            C.byref(eng.problem), None, eng._ptr(eng.compute), eng._ptr(eng.per_arg), eng._ptr(eng.status),
            eng._ptr(eng.comm), eng._ptr(eng.cost), eng._ptr(eng.flags), 1, eng._stream())
        _lib.check(rc, "apc_build_all")
        eng.built = True
        want = {k: v.copy() for k, v in eng.results().items()}
        for t in (eng.comm, eng.cost, eng.flags, eng.compute, eng.per_arg, eng.status):
            t.zero_()
        torch.cuda.synchronize()
        rc = eng.lib.apc_build_all_noalloc(
            C.byref(eng.problem), eng._ptr(eng.compute), eng._ptr(eng.per_arg), eng._ptr(eng.status),
            eng._ptr(eng.comm), eng._ptr(eng.cost), eng._ptr(eng.flags), 1, eng._stream())
        _lib.check(rc, "apc_build_all_noalloc")
        got = eng.results()
        for k in ("comm", "cost", "compute", "per_arg"):
            assert (got[k].view(np.uint64) == want[k].view(np.uint64)).all(), (lut, k)
        assert (got["flags"] == want["flags"]).all()
