"""NCCL-tuning collective model on the device, through the C ABI, against the
vectors written by the reference's module and against the CPU oracle.

Tolerance: 1e-12 relative.  The model interpolates correction tables at
log2(bytes >> 6); the reference takes that logarithm from the host libm, the
kernel from the device math library, and the two may round the last bit
differently (everything else is the same binary64 operation sequence; entries
that use no interpolation are asserted bit-exact)."""
import ctypes as C

import numpy as np
import pytest
import torch

from helpers import bits_equal, graph_from_pairs
from oracle import cost_oracle as O
from oracle import nccl_oracle as N
from test_oracle_nccl import cfg_of

pytestmark = pytest.mark.gpu
REL = 1e-12
ABI_KIND = np.asarray([0, 3, 2, 1], np.int32)  # fixture collective code -> C ABI kind


def _close(got, want):
    inf = np.isinf(want)
    if not (np.isinf(got) == inf).all():
        return False
    g, w = got[~inf], want[~inf]
    return bool((np.abs(g - w) <= REL * np.maximum(np.abs(g), np.abs(w))).all())


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from autoparallel_amd import _lib, engine

    return _lib, engine


def test_collective_vectors_through_c_abi(gpu, nccl_golden):
    _lib, engine = gpu
    lib = _lib.load()
    g = nccl_golden
    cfgs = [cfg_of(r) for r in g["cfg"]]
    meshes = [tuple(int(x) for x in r[1:1 + r[0]]) for r in g["mesh"]]
    case, cost = g["case"], g["cost"]
    keys = case[:, 0] * 1000 + case[:, 1]
    total = exact = 0
    for key in np.unique(keys):
        sel = np.nonzero(keys == key)[0]
        ci, mi = int(key) // 1000, int(key) % 1000
        model = engine.make_model(meshes[mi], 8, "AMD Instinct MI355X")
        keep = engine.upload_nccl_plan(model, cfgs[ci], "cuda")
        kind = torch.from_numpy(ABI_KIND[case[sel, 3]]).cuda()
        nb = torch.from_numpy(np.ascontiguousarray(case[sel, 4])).cuda()
        dim = torch.from_numpy(case[sel, 2].astype(np.int32)).cuda()
        out = torch.empty(sel.shape[0], dtype=torch.float64, device="cuda")
        rc = lib.apc_collective_costs(C.byref(model), sel.shape[0], kind.data_ptr(), nb.data_ptr(), dim.data_ptr(),
                                      out.data_ptr(), None)
        assert rc == 0
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert _close(got, cost[sel]), (cfgs[ci], meshes[mi])
        exact += int((got == cost[sel]).sum())
        total += sel.shape[0]
        del keep
    assert total == case.shape[0] > 100000
    assert exact >= 0.98 * total
    print(f"  nccl collective vectors: {total} checked, {exact} bit-identical", flush=True)


def test_no_interpolation_is_bit_exact(gpu, nccl_golden):
    """Single-node configurations use no log2 interpolation: exact bits."""
    _lib, engine = gpu
    lib = _lib.load()
    for cfg, mesh in ((N.a100_config(), (8,)), (N.h100_config(), (2, 4)), (N.gb200_config(), (72,))):
        model = engine.make_model(mesh, 8, "AMD Instinct MI355X")
        keep = engine.upload_nccl_plan(model, cfg, "cuda")
        rng = np.random.default_rng(11)
        q = 4000
        kind = rng.integers(0, 4, q).astype(np.int32)
        nb = (2.0 ** rng.uniform(0, 38, q)).astype(np.int64)
        dim = rng.integers(0, len(mesh), q).astype(np.int32)
        tk, tb, td = (torch.from_numpy(a).cuda() for a in (kind, nb, dim))
        out = torch.empty(q, dtype=torch.float64, device="cuda")
        assert lib.apc_collective_costs(C.byref(model), q, tk.data_ptr(), tb.data_ptr(), td.data_ptr(),
                                        out.data_ptr(), None) == 0
        torch.cuda.synchronize()
        names = ["allgather", "all_to_all", "allreduce", "reduce_scatter"]
        want = np.asarray([N.comm_cost(names[k], int(b), mesh, int(d), cfg) for k, b, d in zip(kind, nb, dim)])
        assert bits_equal(out.cpu().numpy(), want)
        del keep


@pytest.mark.parametrize("use_table", [True, False])
def test_redistribution_vectors_under_nccl(gpu, nccl_golden, use_table):
    """estimate_strategy_comms_cost of the reference with an NCCL topology
    config set, through the entry kernel."""
    _lib, engine = gpu
    g = nccl_golden
    for k in range(int(g["n_pair"])):
        cfg = cfg_of(g["cfg"][int(g[f"pair_{k}_cfg"])])
        mesh = [int(x) for x in g[f"pair_{k}_mesh"]]
        shape = [int(x) for x in g[f"pair_{k}_shape"]]
        stride = [int(x) for x in g[f"pair_{k}_stride"]]
        src, tgt, want = g[f"pair_{k}_src"], g[f"pair_{k}_tgt"], g[f"pair_{k}_cost"]
        src_t = sorted({tuple(int(x) for x in r) for r in src})
        tgt_t = sorted({tuple(int(x) for x in r) for r in tgt})
        pg = graph_from_pairs(mesh, 8, shape, stride, int(g[f"pair_{k}_itemsize"]), src_t, tgt_t)
        print(f"  nccl pair case {k}: mesh={mesh} pairs={len(want)} table={use_table}", flush=True)
        eng = engine.CostEngine(pg, use_table=use_table, nccl_config=cfg).build(clamp_inf=False)
        comm = eng.results()["comm"]
        base, ssrc = int(pg.edge_off[1]), int(pg.edge_ssrc[1])
        si = {t: i for i, t in enumerate(src_t)}
        ti = {t: i for i, t in enumerate(tgt_t)}
        idx = np.asarray([base + ti[tuple(int(x) for x in t)] * ssrc + si[tuple(int(x) for x in s)]
                          for s, t in zip(src, tgt)])
        assert _close(comm[idx], want), k
        # and the whole build against the oracle with the same model
        ref = O.GraphOracle(pg, nccl=cfg).build()
        got = eng.results()
        assert _close(got["comm"], ref["comm"]) and _close(got["cost"], ref["cost"])
        assert ((got["flags"] & 1) == ref["transition"]).all()
