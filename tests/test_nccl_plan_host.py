"""Host half of the NCCL model (apc_nccl_plan_build, no GPU needed): the
candidates it resolves, evaluated here with the same per-entry rule the
kernels apply, must reproduce the reference's vectors; the derived topology
and every candidate's latency/bandwidth must equal the oracle's."""
import math

import numpy as np
import pytest

from autoparallel_amd import _lib
from autoparallel_amd.engine import build_nccl_plan
from oracle import nccl_oracle as N
from tests.test_oracle_nccl import cfg_of, close

NC_TREE, NC_TREE24, NC_RING, NC_NVLS, NC_FULL, NC_PLATEAU, NC_NIC = 1, 2, 4, 8, 16, 32, 64
ABI_KIND = {0: 0, 1: 3, 2: 2, 3: 1}  # fixture collective code -> C ABI kind


def eval_plan(plan, kind, nbytes, i):
    """Python transcription of the device-side candidate evaluation."""
    d = plan.dim[i]
    best = math.inf
    for c in range(d.n_cand[kind]):
        k = d.cand[kind][c]
        bw, lat, f = k.bw, k.lat, k.flags
        if f & NC_NIC:
            lg = N.log2i((nbytes // d.n_ranks) >> 6)
            corr = plan.a2a_nic_ramp[lg] if lg < 24 else 1.0
            if d.a2a_log_nodes > 1 and corr < 1.0:
                corr = 1.0 - (1.0 - corr) / d.a2a_log_nodes
            t = lat + nbytes * d.a2a_remote / (1000.0 * bw * corr)
        else:
            if f & (NC_TREE | NC_TREE24):
                ls = N.log2i(nbytes >> 6)
                if ls < (24 if f & NC_TREE24 else 23):
                    bw *= plan.tree_corr[k.proto][ls]
            per = nbytes // d.n_ranks
            if f & NC_RING:
                bw *= N.interp_correction(list(d.ring_corr), per)
            if f & NC_NVLS:
                bw *= N.interp_correction(list(plan.nvls_tree_ramp), per)
            if f & NC_FULL and N.log2i(per >> 6) < 24:
                bw *= N.interp_correction(list(plan.full_mesh_ramp), per)
            if f & NC_PLATEAU and nbytes / (d.n_channels * d.n_ranks) >= 64:
                lat *= 1.4
            t = lat + nbytes / (1000.0 * bw)
        best = min(best, t)
    return best


def test_symbol_and_struct_sizes():
    lib = _lib.load()
    assert hasattr(lib, "apc_nccl_plan_build")
    import ctypes as C

    assert C.sizeof(_lib.ApcNcclCand) == 24
    assert C.sizeof(_lib.ApcNcclDim) == 16 + 16 + 16 + 4 * 10 * 24 + 24 * 8 + 16
    assert C.sizeof(_lib.ApcNcclPlan) == 8 + 4 * C.sizeof(_lib.ApcNcclDim) + 6 * 24 * 8


def test_plan_reproduces_reference_vectors(nccl_golden):
    g = nccl_golden
    cfgs = [cfg_of(r) for r in g["cfg"]]
    meshes = [tuple(int(x) for x in r[1:1 + r[0]]) for r in g["mesh"]]
    plans = {}
    case, cost, topo = g["case"], g["cost"], g["topo"]
    exact = 0
    for i in range(case.shape[0]):
        ci, mi, d, coll, nb = (int(x) for x in case[i])
        key = (ci, mi)
        if key not in plans:
            plans[key] = build_nccl_plan(cfgs[ci], meshes[mi])
        plan = plans[key]
        pd = plan.dim[d]
        assert (pd.n_ranks, pd.n_nodes, pd.ppn, pd.n_channels) == tuple(int(x) for x in topo[i])
        got = eval_plan(plan, ABI_KIND[coll], nb, d)
        assert close(got, float(cost[i])), (cfgs[ci], meshes[mi], d, coll, nb, got, cost[i])
        exact += got == cost[i]
    assert exact >= 0.999 * case.shape[0]


def test_candidates_match_oracle_terms():
    """Algorithm-loop candidates: latency and bandwidth equal the oracle's
    _compute_algo_latency / _compute_algo_bw restatement bit for bit."""
    c = N.a100_config(num_nodes=4, has_collnet=True, net_latency=1.25)
    mesh = (4, 8)
    plan = build_nccl_plan(c, mesh)
    t = N.derive_dim_topo(c, mesh, 0)
    want = []
    for a in N.eligible_algos(N.AR, c, t.n_nodes):
        for p in N.eligible_protos(a):
            bw = N.algo_bw(N.AR, a, p, t, c)
            if bw > 0:
                want.append((N.algo_latency(N.AR, a, p, t, c), bw, p))
    d = plan.dim[0]
    got = [(d.cand[2][k].lat, d.cand[2][k].bw, d.cand[2][k].proto) for k in range(d.n_cand[2])]
    assert got == want and len(got) == 8
    assert list(d.ring_corr) == list(N.RING_CORR)
    c8 = N.h100_config(num_nodes=16, has_nvswitch=False)
    assert list(build_nccl_plan(c8, (16, 8)).dim[0].ring_corr) == list(N.depth_scaled_ring_table(16))


def test_one_device_dim_and_bad_arguments():
    lib = _lib.load()
    plan = build_nccl_plan(N.a100_config(), (1, 8))
    assert plan.dim[0].n_cand[0] == 0 and plan.dim[0].n_cand[2] == 0  # reference divides by zero steps there
    assert plan.dim[1].n_cand[0] == 3
    with pytest.raises(_lib.ApcError):
        build_nccl_plan(N.NcclConfig(5, 1, 8, 1.0, 1.0), (8,))
    with pytest.raises(_lib.ApcError):
        build_nccl_plan(N.NcclConfig(0, 1, 0, 1.0, 1.0), (8,))
