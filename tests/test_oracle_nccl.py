"""The NCCL-model oracle against (a) vectors written by the reference's own
module (tests/golden/make_nccl_vectors.py) and (b) the closed-form known
answers of the reference's tests/test_nccl_cost_model.py, restated here.

The vectors are bit-exact on this machine (same libm ``log2``/``pow`` as the
generator); the assertion allows 1e-12 relative so that the suite also holds
on a host whose libm rounds ``log2`` differently in the last place."""
import math

import numpy as np
import pytest

from oracle import cost_oracle as O
from oracle import nccl_oracle as N

REL = 1e-12


def cfg_of(row) -> N.NcclConfig:
    arch, nn, gpn, bwi, bwe, nch, sw, cn, nl = row
    return N.NcclConfig(int(arch), int(nn), int(gpn), float(bwi), float(bwe), None if nch < 0 else int(nch),
                        bool(sw), bool(cn), float(nl))


def close(a, b, rel=REL):
    if math.isinf(a) or math.isinf(b):
        return a == b
    return abs(a - b) <= rel * max(abs(a), abs(b))


def test_collective_vectors(nccl_golden):
    g = nccl_golden
    cfgs = [cfg_of(r) for r in g["cfg"]]
    meshes = [tuple(int(x) for x in r[1:1 + r[0]]) for r in g["mesh"]]
    names = ["allgather", "reduce_scatter", "allreduce", "all_to_all"]
    exact = 0
    case, cost, topo = g["case"], g["cost"], g["topo"]
    for i in range(case.shape[0]):
        ci, mi, d, coll, nb = (int(x) for x in case[i])
        t = N.derive_dim_topo(cfgs[ci], meshes[mi], d)
        assert (t.n_ranks, t.n_nodes, t.ppn, t.n_channels) == tuple(int(x) for x in topo[i])
        got = N.comm_cost(names[coll], nb, meshes[mi], d, cfgs[ci])
        assert close(got, float(cost[i])), (cfgs[ci], meshes[mi], d, names[coll], nb, got, cost[i])
        exact += got == cost[i]
    assert case.shape[0] > 100000
    assert exact >= 0.999 * case.shape[0]


def test_vectors_cover_every_path(nccl_golden):
    """The fixture must exercise each dispatch path, or it would not pin it."""
    g = nccl_golden
    cfgs = [cfg_of(r) for r in g["cfg"]]
    meshes = [tuple(int(x) for x in r[1:1 + r[0]]) for r in g["mesh"]]
    seen = set()
    for ci, mi, d, coll, nb in g["case"][::31].tolist():
        c, t = cfgs[ci], N.derive_dim_topo(cfgs[ci], meshes[mi], d)
        sw = c.arch in (N.HOPPER, N.BLACKWELL) and c.has_nvswitch
        if coll == 3:
            seen.add("a2a_ce" if sw and t.n_nodes == 1 else "a2a_nic" if t.n_nodes > 1 and c.has_nvswitch else "a2a_sm")
        elif sw and t.n_nodes == 1:
            seen.add("nvswitch")
        elif sw and N.table_collective_time(coll, nb, t, c) is not None:
            seen.add("table_ar" if coll == N.AR else "table_agrs")
        else:
            seen.add("loop")
            if c.has_collnet:
                seen.add("loop_collnet")
            if t.n_nodes > 4:
                seen.add("loop_depth")
    assert seen == {"a2a_ce", "a2a_nic", "a2a_sm", "nvswitch", "table_ar", "table_agrs", "loop", "loop_collnet",
                    "loop_depth"}
    assert np.isinf(g["cost"]).any()  # zero NIC bandwidth config


def test_depth_scaled_tables(nccl_golden):
    for n in (8, 16, 32, 64):
        want = nccl_golden[f"ring_depth_{n}"]
        got = np.asarray(N.depth_scaled_ring_table(n))
        assert np.allclose(got, want, rtol=1e-15, atol=0)
        # clamp: no entry more than twice its predecessor (reference test :1293-1300)
        assert all(got[i] <= 2.0 * got[i - 1] + 1e-15 for i in range(1, 24))


def test_redistribute_under_nccl_model(nccl_golden):
    g = nccl_golden
    dev = O.DeviceLimit()
    total = 0
    for k in range(int(g["n_pair"])):
        cfg = cfg_of(g["cfg"][int(g[f"pair_{k}_cfg"])])
        mesh = [int(x) for x in g[f"pair_{k}_mesh"]]
        topo = O.Topo(mesh, 8, nccl=cfg)
        shape = [int(x) for x in g[f"pair_{k}_shape"]]
        stride = [int(x) for x in g[f"pair_{k}_stride"]]
        itemsize = int(g[f"pair_{k}_itemsize"])
        src, tgt, want = g[f"pair_{k}_src"], g[f"pair_{k}_tgt"], g[f"pair_{k}_cost"]
        for i in range(src.shape[0]):
            s = tuple(int(x) for x in src[i])
            t = tuple(int(x) for x in tgt[i])
            got = O.estimate_strategy_comms_cost(s, shape, stride, itemsize, t, topo, dev)
            assert close(got, float(want[i])), (k, s, t, got, want[i])
            total += 1
    assert total > 15000


# --- known answers restated from the reference's tests -----------------------
def test_derive_topology_known_answers():
    # tests/test_nccl_cost_model.py:45-105
    t = N.derive_dim_topo(N.a100_config(), (8,), 0)
    assert (t.n_ranks, t.n_nodes, t.ppn, t.n_channels) == (8, 1, 8, 12)
    t = N.derive_dim_topo(N.a100_config(num_nodes=2), (2, 8), 1)
    assert (t.n_ranks, t.ppn, t.n_nodes) == (8, 8, 1)
    t = N.derive_dim_topo(N.a100_config(num_nodes=2), (2, 8), 0)
    assert (t.n_ranks, t.ppn, t.n_nodes) == (2, 1, 2)
    t = N.derive_dim_topo(N.h100_config(num_channels=16), (8,), 0)
    assert t.bw_intra == pytest.approx(20.0) and t.bw_inter == pytest.approx(50.0 / 16)
    assert N.derive_dim_topo(N.a100_config(num_channels=8), (8,), 0).n_channels == 8
    c = N.NcclConfig(N.HOPPER, 4, 8, 320.0, 50.0)
    assert [(N.derive_dim_topo(c, (2, 4, 4), d).ppn, N.derive_dim_topo(c, (2, 4, 4), d).n_nodes) for d in (2, 1, 0)] == [
        (4, 1), (2, 2), (1, 2)]


def test_bw_latency_known_answers():
    # :109-198
    c = N.a100_config()
    t = N.derive_dim_topo(c, (8,), 0)
    assert N.algo_bw(N.AR, N.RING, N.SIMPLE, t, c) == pytest.approx(12 * (87.7 / 12) * 8 / 14)
    assert N.algo_bw(N.AG, N.RING, N.SIMPLE, t, c) == pytest.approx(12 * (87.7 / 12) * 8 / 7)
    assert N.algo_bw(N.AR, N.TREE, N.SIMPLE, t, c) == pytest.approx(min(87.7 * 0.92, 12 * 24.0) * 0.5)
    assert N.algo_bw(N.AG, N.TREE, N.SIMPLE, t, c) == 0.0
    assert N.algo_latency(N.AR, N.RING, N.SIMPLE, t, c) == pytest.approx(8.4 + 14 * 3.4)
    assert N.algo_latency(N.AR, N.TREE, N.SIMPLE, t, c) == pytest.approx(8.4 + 2 * 7 * 4.0)
    h = N.h100_config()
    th = N.derive_dim_topo(h, (8,), 0)
    assert N.algo_bw(N.AR, N.NVLS, N.SIMPLE, th, h) > 0
    assert N.algo_bw(N.AR, N.NVLS, N.LL, th, h) == 0.0 and N.algo_bw(N.AR, N.NVLS, N.LL128, th, h) == 0.0
    a = N.a100_config(has_nvswitch=True)
    assert N.algo_bw(N.AR, N.NVLS, N.SIMPLE, N.derive_dim_topo(a, (8,), 0), a) == 0.0
    c2 = N.a100_config(num_nodes=2, gpus_per_node=1)
    t2 = N.derive_dim_topo(c2, (2,), 0)
    assert N.algo_latency(N.AR, N.RING, N.SIMPLE, t2, c2) == pytest.approx(8.4 + 2 * 14.0 + 4.7 * 2)


def test_eligibility():
    # :236-310
    assert N.NVLS not in N.eligible_algos(N.AR, N.h100_config(has_nvswitch=False), 1)
    assert N.NVLS in N.eligible_algos(N.AR, N.h100_config(), 1)
    assert N.NVLS_TREE not in N.eligible_algos(N.AR, N.h100_config(), 1)
    assert N.NVLS_TREE in N.eligible_algos(N.AR, N.h100_config(), 2)
    assert N.COLLNET_DIRECT not in N.eligible_algos(N.AR, N.a100_config(), 1)
    assert {N.COLLNET_DIRECT, N.COLLNET_CHAIN} <= set(N.eligible_algos(N.AR, N.a100_config(has_collnet=True), 1))
    assert N.NVLS not in N.eligible_algos(N.AR, N.a100_config(has_nvswitch=True), 1)
    ag = N.eligible_algos(N.AG, N.h100_config(has_collnet=True), 1)
    assert N.RING in ag and N.NVLS in ag and N.COLLNET_DIRECT in ag and N.TREE not in ag
    assert N.eligible_protos(N.RING) == [N.LL, N.LL128, N.SIMPLE] == N.eligible_protos(N.TREE)
    for a in (N.NVLS, N.NVLS_TREE, N.COLLNET_DIRECT, N.COLLNET_CHAIN):
        assert N.eligible_protos(a) == [N.SIMPLE]


def test_ring_plateau_known_answer():
    # :569-611
    c = N.a100_config(num_nodes=4, gpus_per_node=1)
    t = N.derive_dim_topo(c, (4,), 0)
    thr = 64 * t.n_channels * t.n_ranks
    bw = N.algo_bw(N.AR, N.RING, N.SIMPLE, t, c)
    lat = N.algo_latency(N.AR, N.RING, N.SIMPLE, t, c)

    def corrected(n):
        lg = N.log2i((n // t.n_ranks) >> 6)
        return bw * N.RING_CORR[lg]

    assert N.algo_time(N.AR, N.RING, N.SIMPLE, thr - 1, t, c) == pytest.approx(lat + (thr - 1) / (1000.0 * corrected(thr - 1)))
    assert N.algo_time(N.AR, N.RING, N.SIMPLE, thr, t, c) == pytest.approx(lat * 1.4 + thr / (1000.0 * corrected(thr)))
    n = 1 << 20
    bl, ll = N.algo_bw(N.AR, N.RING, N.LL, t, c), N.algo_latency(N.AR, N.RING, N.LL, t, c)
    assert N.algo_time(N.AR, N.RING, N.LL, n, t, c) == pytest.approx(ll + n / (1000.0 * bl * N.RING_CORR[N.log2i((n // 4) >> 6)]))


def test_all_to_all_known_answers():
    # :841-852, :873-885
    c = N.h100_config(num_nodes=2)
    t = N.derive_dim_topo(c, (16,), 0)
    n = 1 << 30
    want = 37.0 + n * ((16 - 8) / 16) / (1000.0 * (50.0 * (1.0 - 0.44 / 2)))
    assert N.all_to_all_time(n, t, c) == pytest.approx(want)
    n = 2 << 20
    assert N.all_to_all_time(n, t, c) > 37.0 + n * 0.5 / (1000.0 * 50.0 * 0.78)
    # CE path (:1248-1255 of the model)
    h = N.h100_config()
    assert N.all_to_all_time(1 << 24, N.derive_dim_topo(h, (8,), 0), h) == 50.0 + (1 << 24) / (1000.0 * 380.0)


def test_nvswitch_known_answers():
    # :1155-1169, :1016-1032
    h = N.h100_config()
    t = N.derive_dim_topo(h, (8,), 0)
    n = 1 << 30
    assert N.collective_time(N.AR, n, t, h) == pytest.approx(31.0 + n / (1000.0 * 267.0))
    c2, c3, c4 = (N.collective_time(N.AG, 1 << 24, N.derive_dim_topo(h, (k,), 0), h) for k in (2, 3, 4))
    assert c2 < c3 < c4
    assert N.collective_time(N.AG, n, t, h) == N.collective_time(N.RS, n, t, h)


def test_table_path_known_answers():
    # :1145-1153, :1216-1226, :1268-1286
    c = N.h100_config(num_nodes=2)
    t = N.derive_dim_topo(c, (16,), 0)
    n = 1 << 30
    tab = N.table_collective_time(N.AR, n, t, c)
    assert tab is not None
    assert N.collective_time(N.AR, n, t, c) == pytest.approx(tab)
    odd = N.DimTopo(24, 3, 8, 20.0, 50.0 / 16, 16)
    assert N.table_collective_time(N.AR, n, odd, c) is None
    assert N.table_collective_time(N.AG, n, odd, c) is None
    assert 0 < N.collective_time(N.AR, n, odd, c) < float("inf")


def test_interp_correction_known_answers():
    # :1332-1362
    tab = (0.10, 0.20, 0.40, 0.80, 1.00)
    for i, v in enumerate(tab):
        assert N.interp_correction(tab, (1 << i) << 6) == pytest.approx(v)
    f = math.log2(3) - 1
    assert N.interp_correction(tab, 3 << 6) == pytest.approx(tab[1] * (1 - f) + tab[2] * f, abs=1e-10)
    assert N.interp_correction(tab, 0) == tab[0] and N.interp_correction(tab, 1) == tab[0]
    assert N.interp_correction(tab, (1 << 20) << 6) == tab[-1]


@pytest.mark.parametrize("n_nodes", [8, 16, 32])
def test_no_jump_at_power_of_two(n_nodes):
    # :1364-1382
    c = N.h100_config(num_nodes=n_nodes, gpus_per_node=8)
    t = N.derive_dim_topo(c, (n_nodes * 8,), 0)
    for e in range(16, 26):
        lo = N.collective_time(N.AG, (1 << e) - 1, t, c)
        hi = N.collective_time(N.AG, (1 << e) + 1, t, c)
        assert 0.85 < hi / lo < 1.15


@pytest.mark.parametrize("func", [N.AG, N.RS, N.AR])
def test_monotone_in_size(func):
    # :639-666
    for c, mesh in ((N.a100_config(), (8,)), (N.h100_config(), (8,)), (N.a100_config(num_nodes=4), (4, 8))):
        t = N.derive_dim_topo(c, mesh, 0)
        prev = 0.0
        for k in range(10, 31):
            v = N.collective_time(func, 1 << k, t, c)
            assert v > 0 and v >= prev
            prev = v
