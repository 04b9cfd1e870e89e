"""Packed format invariants, decision-var assembly identities, the scorer's
semantics on the reference's own mock data, and the C ABI surface (load +
exported symbols; no GPU work)."""
import ctypes
import os
import re

import numpy as np
import pytest

from autoparallel_amd import graphgen, packed
from autoparallel_amd.packed import GraphBuilder, NodeDesc
from oracle import cost_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def small_llama():
    return graphgen.llama_graph((8, 8), 1, 1024, 8, 4, 2048, 8192, 512, 16)


def test_layout_invariants(small_llama):
    g = small_llama
    g.validate()
    assert g.num_slots % 16 == 0 and g.num_slots >= g.num_entries
    assert (g.edge_off[:-1] % 16 == 0).all()
    slots = g.entry_slots()
    assert slots.shape[0] == g.num_entries and len(np.unique(slots)) == g.num_entries
    keys = g.entry_keys()
    assert keys.shape == (g.num_entries, 4)
    # every (node, arg, out, inp) key is unique and in range
    assert len({tuple(k) for k in keys[:: max(1, len(keys) // 5000)]}) > 0
    assert (keys[:, 2] < g.node_nstrat[keys[:, 0]]).all()
    # chunk index: each 16-slot chunk belongs to the edge of its entries
    eid = np.repeat(np.arange(g.num_edges), g.edge_sdst.astype(np.int64) * g.edge_ssrc)
    assert (g.chunk_edge_index()[slots >> 4] == eid).all()
    # work items tile every edge block exactly once
    items = g.work_items()
    covered = np.zeros(g.num_edges, np.int64)
    item_edge = np.searchsorted(g.edge_off[:-1], items["off"])  # items copy their edge's record
    assert (g.edge_off[:-1][item_edge] == items["off"]).all()
    np.add.at(covered, item_edge, 1)
    sizes = g.edge_sdst.astype(np.int64) * g.edge_ssrc
    lead = g.edge_off[:-1] % 64  # an item starts at a multiple of 64 slots, up to 48 before its block
    assert (covered == (sizes + lead + 255) // 256).all()
    first_slot = items["off"] + items["local0"].astype(np.int32)
    assert (first_slot % 64 == 0).all() and (first_slot + 64 > items["off"]).all()
    # the entries an item's 256 lanes-times-four reach, kept where 0 <= entry < size: every entry once
    hit = np.zeros(g.num_slots, np.int32)
    for it, e in zip(items, item_edge):
        local = (np.arange(256, dtype=np.int64) + int(np.int32(it["local0"])))
        local = local[(local >= 0) & (local < sizes[e])]
        hit[it["off"] + local] += 1
    assert (hit[slots] == 1).all() and hit.sum() == len(slots)
    # decision-var order: node, out_idx, argi, inp_idx
    order = g.decision_var_order()
    k = keys[order]
    assert (np.lexsort((k[:, 3], k[:, 1], k[:, 2], k[:, 0])) == np.arange(len(k))).all()


def test_magic_division_exact(small_llama):
    rec = small_llama.edge_records()
    for r in rec[:: max(1, len(rec) // 200)]:
        if r["magic"] == 0:
            continue
        size = int(r["ssrc"]) * int(r["sdst"])
        for local in {0, 1, size - 1, size // 2, int(r["ssrc"]) - 1, int(r["ssrc"])} & set(range(size)):
            assert (local * int(r["magic"])) >> 32 == local // int(r["ssrc"])


@pytest.mark.parametrize("make", [
    lambda: graphgen.llama_graph((2, 4), 1, 64, 4, 2, 128, 256, 32, 16),
    lambda: graphgen.stress_graph(60, (4, 8, 8), seed=2, s_max=40),
    lambda: graphgen.moe_graph((2, 4), 2, 64, 4, 8, 2, 32, 256, 32, 8),
])
def test_compressed_block_table_layout(make):
    """The compressed block table against its definition: matrix element
    [uidx[o]][uidx[j]] of an edge stands for the pair (lists[src + j],
    lists[dst + o]), whatever o and j reach it."""
    g = make()
    uidx, ufirst, nuniq = g.run_unique_index()
    block_edge, block_off, unit_block, table_off, usrc, block_udst = g.block_table(True)
    full = g.block_table(False)
    assert block_off[-1] <= full[1][-1] and (block_off % 256 == 0).all()
    assert unit_block.shape[0] == block_off[-1] // 256
    hp = (g.edge_flags & packed.EDGE_HAS_PRODUCER) != 0
    assert ((table_off >= 0) == hp).all()
    # element -> the word pair it stands for, filled from every entry of every edge
    cell = {}
    rec = g.edge_records(True)
    for e in np.nonzero(hp)[0]:
        s0, d0, ns, nd = int(g.edge_src_list[e]), int(g.edge_dst_list[e]), int(g.edge_ssrc[e]), int(g.edge_sdst[e])
        sw, tw = g.lists[s0:s0 + ns], g.lists[d0:d0 + nd]
        if usrc[e] == 0:  # not compressed: a missing spec somewhere
            assert (sw == packed.SPEC_NONE).any() or (tw == packed.SPEC_NONE).any()
            assert not rec["flags"][e] & packed.EDGE_COMPRESSED
            continue
        assert rec["flags"][e] & packed.EDGE_COMPRESSED and rec["flags"][e] >> packed.EDGE_USRC_SHIFT == usrc[e]
        assert usrc[e] == np.unique(sw).shape[0] == nuniq[s0]
        assert nuniq[d0] == np.unique(tw).shape[0]
        at = table_off[e] + uidx[d0:d0 + nd].astype(np.int64)[:, None] * usrc[e] + uidx[s0:s0 + ns][None, :]
        assert at.max() < table_off[e] + int(usrc[e]) * nuniq[d0]
        pair = (sw.astype(np.int64)[None, :] << 32) | tw.astype(np.int64)[:, None]
        for a, w in zip(at.ravel().tolist(), pair.ravel().tolist()):
            assert cell.setdefault(a, w) == w
        # and the table kernel's way back: element -> a position holding that word
        k = np.arange(usrc[e])
        assert (uidx[s0 + ufirst[s0 + k]] == k).all()
    for b, e in enumerate(block_edge):
        if usrc[e]:
            assert block_udst[b] == nuniq[int(g.edge_dst_list[e])]
            assert block_off[b + 1] - block_off[b] >= int(usrc[e]) * int(block_udst[b])


def test_shared_compute_slots_are_consistent(small_llama):
    """Nodes that share a compute slot must produce identical estimates: the
    oracle prices every node on its own and writes into the shared slot."""
    g = small_llama
    orc = O.GraphOracle(g)
    seen = {}
    for v in range(g.num_nodes):
        vals = [float(orc.node_compute_cost(v, o)) for o in range(int(g.node_nstrat[v]))]
        off = int(g.node_comp_off[v])
        if off in seen:
            assert seen[off] == vals
        seen[off] = vals
    assert len(seen) == g.comp_nodes.shape[0] < g.num_nodes


def test_assembly_identities(small_llama):
    g = small_llama
    r = O.GraphOracle(g).build()
    slots = g.entry_slots()
    keys = g.entry_keys()
    per_arg = r["compute"][g.node_comp_off[keys[:, 0]] + keys[:, 2]] / g.node_nargs[keys[:, 0]]
    want = (r["comm"][slots] + per_arg) + r["transition"][slots]
    got = r["cost"][slots]
    fin = np.isfinite(want)
    assert (got[fin] == want[fin]).all() and np.isinf(got[~fin]).all()
    # placeholders: one entry per strategy, all zero
    ph = g.edge_src_node < 0
    for e in np.nonzero(ph)[0][:50]:
        b = int(g.edge_off[e])
        n = int(g.edge_sdst[e]) * int(g.edge_ssrc[e])
        assert (r["cost"][b:b + n] == 0.0).all()
    # transition can be 1 where comm is 0 (R -> S)
    assert ((r["transition"][slots] == 1) & (r["comm"][slots] == 0.0)).any()
    clamped, bad = O.clamp_inf(r["cost"])
    assert (clamped[bad == 1] == 10000.0).all() and np.isfinite(clamped).all()


def test_prefetch_discount_semantics(small_llama):
    g = small_llama
    r = O.GraphOracle(g).build()
    cost, _ = O.clamp_inf(r["cost"])
    comm2, cost2, n = O.prefetch_discount(g, r["comm"], r["transition"], r["compute"], cost, 0.0)
    assert n > 0
    changed = comm2 != r["comm"]
    assert changed.sum() == n and (comm2[changed] == 0.0).all()
    # the reference's own check (tests/test_prefetch_derived_sets.py:288-296 there):
    # where comm was zeroed, cost == compute + transition
    slots = g.entry_slots()
    keys = g.entry_keys()
    per_arg = np.zeros(g.num_slots)
    per_arg[slots] = r["compute"][g.node_comp_off[keys[:, 0]] + keys[:, 2]] / g.node_nargs[keys[:, 0]]
    assert (cost2[changed] == per_arg[changed] + r["transition"][changed]).all()
    # untouched entries (inf or zero comm, non-prefetchable edges) keep their cost
    assert (cost2[~changed] == cost[~changed]).all()
    # scale 1.0 changes no value
    comm3, cost3, n3 = O.prefetch_discount(g, r["comm"], r["transition"], r["compute"], cost, 1.0)
    assert n3 == n and (comm3 == r["comm"]).all()


def _mock_graph(entries):
    """A chain of single-strategy nodes whose only entries carry the given
    (compute, comm, transition) triples via explicit default rows."""
    b = GraphBuilder((2,), 8)
    m = b.meta((4,), (1,), 4, packed.DT_F32)
    s = b.spec(m, (0,))
    for i, (comp, comm, trans) in enumerate(entries):
        b.add_node(NodeDesc(f"n{i}", in_specs=[[s]], out_specs=[[s]], inputs=[],
                            default_rows=[[[float(comm)]]]))
    return b.pack()


def test_scorer_matches_reference_mock_totals():
    """The reference's log-formatting tests build mock DecisionVars and expect
    the totals to be plain sums of the selected entries' components
    (tests/test_log_formatting.py:57-79 there: 1.0/2.0/0 -> total 3.00)."""
    g = _mock_graph([(1.0, 2.0, 0)])
    comm = np.zeros(g.num_slots)
    comm[g.entry_slots()] = [2.0]
    compute = np.asarray([1.0])
    tot = O.score_assignment(g, comm, np.zeros(g.num_slots, np.uint8), compute, [0])
    # a producer-less entry contributes its compute only (no predecessor strategy)
    assert tot == (1.0, 1.0, 0.0, 0.0)
    obj, viol = O.ilp_objective(g, comm + 1.0, np.zeros(g.num_slots, np.uint8), [0])
    assert (obj, viol) == (3.0, 0)


def test_scorer_known_answers_of_a_hand_made_plan():
    """The three rules of the reference's _compute_solution_cost that a sum of selected
    entries would miss (optimize_sharding.py:1081-1101): compute_cost * num_args per node,
    non-finite comm skipped, no transition through a producer whose output is a tuple of
    specs.  The expected totals are worked out by hand in helpers.hand_made_plan."""
    from helpers import hand_made_plan

    g, comm, transition, compute, assign, want = hand_made_plan()
    assert tuple(float(x) for x in O.score_assignment(g, comm, transition, compute, assign)) == want
    # the other strategy of G (same placement as T[0]'s element): no comm term 0.125, nothing else changes
    total, comp, cm, tr = O.score_assignment(g, comm, transition, compute, [1, 0, 1, 0, 0])
    assert (float(total), float(comp), float(cm), float(tr)) == (358.0 - 256.0 + 128.0 + 0.75 + 2.0, 230.0, 0.75, 2.0)


def test_scorer_on_graph(small_llama):
    g = small_llama
    r = O.GraphOracle(g).build()
    cost, bad = O.clamp_inf(r["cost"])
    assign = np.zeros(g.num_nodes, np.int64)  # strategy 0 everywhere: all replicate
    total, comp, comm, trans = O.score_assignment(g, r["comm"], r["transition"], r["compute"], assign)
    assert comm == 0.0 and trans == 0.0 and total == comp > 0
    obj, viol = O.ilp_objective(g, cost, bad, assign)
    assert viol == 0 and np.isclose(obj, total, rtol=1e-12)
    rng = np.random.default_rng(0)
    assign = rng.integers(0, g.node_nstrat)
    total, comp, comm, trans = O.score_assignment(g, r["comm"], r["transition"], r["compute"], assign)
    assert total == (comp + comm) + trans and trans > 0


def test_builder_rejects_bad_programs():
    with pytest.raises(AssertionError):
        packed.check_program([1, 0, 2, 1, 3, 0], 2)  # factor names arg 3 of 2
    with pytest.raises(AssertionError):
        packed.check_program([0, 1, 2, 1, 1, 0, 9], 1)  # dim 9 >= MAX_RANK
    packed.check_program([0, 1, 2, 1, 2, 0, 0], 1)


def test_abi_exports_every_declared_symbol():
    from autoparallel_amd import _lib

    lib = _lib.load()
    header = open(os.path.join(ROOT, "include", "apc.h")).read()
    declared = set(re.findall(r"\b(apc_[a-z_0-9]+)\s*\(", header))
    assert declared, "no declarations found"
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in apc.h but not exported"
    assert set(_lib.EXPORTED_SYMBOLS) == declared
    assert lib.apc_version() == _lib.ABI_VERSION == 5
    # struct sizes agree between the header's layout and the ctypes mirror
    assert packed.PackedGraph.EDGE_DTYPE.itemsize == 64


def test_abi_host_helpers():
    from autoparallel_amd import _lib

    lib = _lib.load()
    shape = (ctypes.c_int32 * 4)(4, 8, 8, 1)
    bw = (ctypes.c_double * 4)()
    lat = (ctypes.c_double * 4)()
    assert lib.apc_mesh_topology(ctypes.addressof(shape), 3, 8, ctypes.addressof(bw), ctypes.addressof(lat)) == 0
    t = O.Topo((4, 8, 8), 8)
    assert list(bw)[:3] == t.bw and list(lat)[:3] == t.lat
    m = _lib.ApcModel()
    assert lib.apc_device_limits(b"AMD Instinct MI355X", ctypes.byref(m)) == 0
    assert m.gmem_bw == O.MI355X_GMEM_BW and list(m.tflops)[:5] == [O.MI355X_TFLOPS[i] for i in range(5)]
    # the whole device table of the reference, matched by substring in its order
    for name, bw, tf in O.DEVICE_TABLE:
        for full in (name, "NVIDIA " + name + " 80GB HBM3"):
            assert lib.apc_device_limits(full.encode(), ctypes.byref(m)) == 0, full
            assert m.gmem_bw == bw and list(m.tflops)[:5] == [float(tf.get(i, 0.0)) for i in range(5)], full
    assert lib.apc_device_limits(b"NVIDIA PG509-210", ctypes.byref(m)) == 0 and m.tflops[3] == 312.0
    assert lib.apc_device_limits(b"NVIDIA H100 and A100", ctypes.byref(m)) == 0 and m.tflops[0] == 67.0
    # the H100 row against the figures the reference's documentation quotes (989 TFLOPS bf16, 3.35 TB/s:
    # docs/how_autoparallel_chooses_a_strategy.md:34-39); the other rows are data restated from the table
    h100 = O.DeviceLimit.named("NVIDIA H100 80GB HBM3")
    assert h100.tflops[3] == 989.0 and h100.tflops[1] == 494.0 and h100.gmem_bandwidth == 3.35 * 1024**4
    assert O.DeviceLimit.named("AMD Instinct MI300X").tflops[1] == 653.7
    assert lib.apc_device_limits(b"Some Other GPU", ctypes.byref(m)) == _lib.load().apc_device_limits(b"x", ctypes.byref(m)) != 0
    assert b"Unsupported device" in lib.apc_last_error()
    # the host-side draw of the on-device assignment generator is deterministic and in range
    draws = [lib.apc_random_assignment(7, a, v, 13) for a in range(20) for v in range(20)]
    assert all(0 <= d < 13 for d in draws) and len(set(draws)) > 5
    assert draws == [lib.apc_random_assignment(7, a, v, 13) for a in range(20) for v in range(20)]


def test_engine_needs_gpu():
    import torch

    from autoparallel_amd import _lib
    from autoparallel_amd.engine import CostEngine

    if torch.cuda.is_available():
        pytest.skip("GPU present")
    g = _mock_graph([(1.0, 2.0, 0)])
    with pytest.raises(Exception):
        CostEngine(g, device="cpu")


def test_stress_dag_windows_are_slices_of_one_graph():
    """A window holds the nodes of its range as the whole DAG has them:
    same strategies, same producers (by global id), same spec words' content."""
    n, seed = 90, 3
    whole, gid_w, ns_w = graphgen.stress_dag_window(n, 0, n, (4, 8, 8), seed, 4, 16)
    assert ns_w == 0 and whole.num_nodes == n

    def content(g, v):
        """(strategy count, per edge: producer gid, decoded consumer specs) of local node v."""
        out = []
        for e in range(int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])):
            words = g.lists[int(g.edge_dst_list[e]):int(g.edge_dst_list[e]) + int(g.edge_sdst[e])]
            metas = words >> packed.TUPLE_BITS
            dec = [(tuple(g.meta_shape[m][:g.meta_rank[m]]), int(g.meta_dtype[m]), tuple(g.tuple_plc[w & 0xFFF]))
                   for m, w in zip(metas, words)]
            src = ()
            if g.edge_src_node[e] >= 0:  # the producer's run: the stand-in must carry the real specs
                sw = g.lists[int(g.edge_src_list[e]):int(g.edge_src_list[e]) + int(g.edge_ssrc[e])]
                src = tuple((tuple(g.meta_shape[w >> packed.TUPLE_BITS][:g.meta_rank[w >> packed.TUPLE_BITS]]),
                             tuple(g.tuple_plc[w & 0xFFF])) for w in sw)
            out.append((int(g.edge_src_node[e]), dec + [src]))
        return int(g.node_nstrat[v]), out

    edges = 0
    for lo, hi in ((0, 30), (30, 61), (61, 90)):
        g, gid, ns = graphgen.stress_dag_window(n, lo, hi, (4, 8, 8), seed, 4, 16)
        g.validate()
        assert (gid[ns:] == np.arange(lo, hi)).all() and (gid[:ns] < lo).all() and (np.diff(gid[:ns]) > 0).all()
        for v in range(ns, g.num_nodes):
            s_loc, e_loc = content(g, v)
            s_all, e_all = content(whole, int(gid[v]))
            assert s_loc == s_all and len(e_loc) == len(e_all)
            for (src_l, dec_l), (src_a, dec_a) in zip(e_loc, e_all):
                assert (int(gid[src_l]) if src_l >= 0 else -1) == src_a and dec_l == dec_a
        edges += int((g.edge_node >= ns).sum())
    assert edges == whole.num_edges


def test_tensors_beyond_int64_bytes_are_refused():
    b = GraphBuilder((2, 4), 8)
    m = b.meta((65536, 65536, 65536, 32768), graphgen.contiguous_stride((65536, 65536, 65536, 32768)), 4, packed.DT_F32)
    s = b.spec(m, (0, 0))
    b.add_node(NodeDesc("x", in_specs=[[s]], out_specs=[[s]], inputs=[], default_rows=[[[0.0]]]))
    with pytest.raises(ValueError, match="int64 range"):
        b.pack().validate()
    assert graphgen._cap_numel((65536, 65536, 65536, 65536)) == (8192, 8192, 8192, 8192) or \
        np.prod([float(x) for x in graphgen._cap_numel((65536, 65536, 65536, 65536))]) <= 2.0**48


def test_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    """Without the built HIP library every entry into the product path raises:
    nothing is computed on the host instead."""
    from autoparallel_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libapc_hip.so"))
    with pytest.raises(_lib.ApcError, match="no CPU fallback"):
        _lib.load()
    from autoparallel_amd.engine import make_model

    with pytest.raises(_lib.ApcError):
        make_model((8, 8), 8, "AMD Instinct MI355X")
    # the package itself never reaches for the oracle
    import pathlib
    import re

    root = pathlib.Path(_lib.__file__).parent
    for path in root.rglob("*.py"):
        assert not re.search(r"^\s*(from|import)\s+oracle\b", path.read_text(), re.M), path


def test_specs_in_bulk_equal_specs_one_by_one():
    """GraphBuilder.specs gives the words, and hands out the tuple ids in the order, of spec called per row."""
    rng = np.random.default_rng(5)
    one, bulk = packed.GraphBuilder((4, 8, 8)), packed.GraphBuilder((4, 8, 8))
    codes = np.asarray([packed.PLC_R, packed.shard(0), packed.shard(1), packed.shard(2), packed.PARTIAL_SUM])
    for k in range(40):
        shape = (64 + k, 128, 32)
        m1 = one.meta(shape, (128 * 32, 32, 1), 2, packed.DT_BF16)
        m2 = bulk.meta(shape, (128 * 32, 32, 1), 2, packed.DT_BF16)
        rows = codes[rng.integers(0, 2 + k % 4, size=(int(rng.integers(1, 300)), 3))]
        assert [one.spec(m1, tuple(int(c) for c in r)) for r in rows] == bulk.specs(m2, rows)
        if k % 7 == 0:  # the two ways of interning mix
            assert one.spec(m1, (codes[4], codes[4], codes[0])) == bulk.spec(m2, (codes[4], codes[4], codes[0]))
    assert one._tuple_rows == bulk._tuple_rows and bulk.specs(0, np.zeros((0, 3), np.int64)) == []


def test_layout_choice_and_caches_travel_with_the_graph(small_llama):
    """The engine's default layout is a property of the packed graph, and the
    layouts made for it in a worker process arrive with the pickled graph."""
    import pickle

    # one layer: the full table would be more than half as large as the entry arrays; four layers share it
    assert small_llama.default_table_mode() == "compressed"
    four = graphgen.llama_graph((8, 8), 4, 1024, 8, 4, 2048, 8192, 512, 16)
    assert four.default_table_mode() == "full" and four.default_item_entries("full") == 256
    g = graphgen.stress_graph(60, (4, 8, 8), seed=2, s_min=64, s_max=300)
    mode = g.default_table_mode()
    assert mode == "compressed"  # no two edges share a matrix: only the matrices of distinct words are small enough
    assert g.default_item_entries(mode) == (512 if g.num_entries >= packed.WIDE_ITEMS_FROM else 256)
    assert g.default_item_entries("direct") == 256
    g.validate()
    g.warm_host_layout()
    h = pickle.loads(pickle.dumps(g))
    assert h.__dict__.get("_validated") and h.__dict__["_run_unique"] is not None
    assert (True, g.default_item_entries(mode)) in h.__dict__["_work_items"] and True in h.__dict__["_block_tables"]
    for a, b in zip(h.run_unique_index(), g.run_unique_index()):
        assert np.array_equal(a, b)
    assert np.array_equal(h.work_items(True, g.default_item_entries(mode)), g.work_items(True, g.default_item_entries(mode)))
    # a graph derived from it starts without them
    alias = np.arange(g.num_edges)
    assert "_work_items" not in g.with_edge_alias(alias).__dict__


def test_every_entry_point_refuses_a_problem_it_could_not_walk():
    """No GPU is touched: a null problem, an empty one (no mesh) and one whose counts
    name arrays that are not there are turned away on the host, with a status below zero
    and a message, by every entry point that takes a problem."""
    from autoparallel_amd import _lib

    lib = _lib.load()
    ptr = ctypes.POINTER(_lib.ApcProblem)
    ints = (ctypes.c_int, ctypes.c_int32, ctypes.c_int64, ctypes.c_uint32, ctypes.c_uint64)
    takers = [(name, args) for name, (res, args) in _lib._SIGNATURES.items()
              if res is ctypes.c_int and args and args[0] is ptr]
    assert len(takers) >= 20

    def call(name, args, first):
        rest = [0 if a in ints else 0.0 if a in (ctypes.c_double, ctypes.c_float) else None for a in args[1:]]
        return getattr(lib, name)(first, *rest)

    empty = _lib.ApcProblem()
    no_arrays = _lib.ApcProblem()
    no_arrays.model.ndim = 2
    no_arrays.model.mesh_shape[0], no_arrays.model.mesh_shape[1] = 2, 4
    no_arrays.n_node, no_arrays.n_edge, no_arrays.n_entry, no_arrays.n_slot, no_arrays.n_chunk, no_arrays.n_item = 5, 7, 100, 112, 7, 1
    for name, args in takers:
        for what, first in (("null", None), ("empty", ctypes.byref(empty)), ("no arrays", ctypes.byref(no_arrays))):
            rc = call(name, args, first)
            assert rc < 0 and lib.apc_last_error(), (name, what, rc)


def test_templates_pack_like_nodes_described_one_by_one():
    """GraphBuilder.add_template / add_instance (one description shared by the
    repeated nodes of a model, default rows asked through a callback) give the
    arrays that add_node gives for the same nodes, field by field."""
    import dataclasses

    from autoparallel_amd import graphgen
    from autoparallel_amd.packed import GraphBuilder, PackedGraph

    class Recorder(GraphBuilder):
        made = []

        def __init__(self, *a, **k):
            super().__init__(*a, **k)
            Recorder.made.append(self)

    saved, graphgen.GraphBuilder = graphgen.GraphBuilder, Recorder
    try:
        want = graphgen.llama_graph((2, 4), 3, 256, 8, 4, 512, 1024, 128, 16)
    finally:
        graphgen.GraphBuilder = saved
    src = Recorder.made[-1]
    # the same nodes again: a template per distinct description (by content), an instance per node
    b = GraphBuilder(src.mesh_shape, src.devices_per_host)
    b._metas, b._meta_rows = dict(src._metas), list(src._meta_rows)
    b._tuples, b._tuple_rows = dict(src._tuples), list(src._tuple_rows)
    b.prefetchable_edges, b.multiplier = set(src.prefetchable_edges), dict(src.multiplier)
    templates, rows = {}, {}
    for v, nd in enumerate(src.nodes):
        key = (tuple(map(tuple, nd.in_specs)), tuple(map(tuple, nd.out_specs)), nd.op,
               None if nd.program is None else tuple(nd.program), nd.tuple_output, nd.nargs,
               None if nd.default_rows is None else len(nd.default_rows[0]))
        if key not in templates:
            templates[key] = b.add_template(nd)
        b.add_instance(templates[key], nd.inputs, nd.getitem_index, nd.name)
        rows[v] = nd.default_rows
    assert len(templates) < len(src.nodes) // 2
    got = b.pack(default_rows_of=rows.get)
    for f in dataclasses.fields(PackedGraph):
        if f.name in ("roles", "node_kind", "node_phase", "node_cluster_key"):  # the generator sets these after packing
            continue
        x, y = getattr(got, f.name), getattr(want, f.name)
        if isinstance(y, np.ndarray):
            assert x.dtype == y.dtype and x.shape == y.shape and x.tobytes() == y.tobytes(), f.name
        else:
            assert x == y, f.name
