"""Writes tests/golden/nccl_vectors.npz from the reference's NCCL cost model.

Run in the build container only:   python tests/golden/make_nccl_vectors.py

``autoparallel/cost_models/nccl_cost_model.py`` imports only the standard
library, so it is loaded by file path on its own.  The second part loads
``collective_runtime_estimation`` the way make_cost_vectors.py does, selects the
NCCL model with ``set_nccl_topo_config`` and records
``estimate_strategy_comms_cost`` over placement pairs.

The output holds inputs and expected outputs only:
  cfg        float64[K, 9]  arch, num_nodes, gpus_per_node, bw_intra, bw_inter,
                            num_channels (-1 = default), has_nvswitch,
                            has_collnet, net_latency
  mesh       int64[M, 5]    ndim, shape[4] (0-padded)
  case       int64[N, 5]    cfg index, mesh index, mesh dim, collective
                            (0 allgather, 1 reduce_scatter, 2 allreduce,
                            3 all_to_all), n_bytes
  cost       float64[N]     _nccl_comm_cost-equivalent value
  topo       int64[N, 4]    derived n_ranks, n_nodes, ppn, n_channels
  ring_depth_<n>            _depth_scaled_ring_correction(n)
  pair_<k>_* redistribution cases under the NCCL model (same field layout as
             cost_vectors.npz plus pair_<k>_cfg = cfg index)
"""
import importlib.util
import itertools
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

REF = "/root/reference/autoparallel/cost_models/nccl_cost_model.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "nccl_vectors.npz")

# arch, num_nodes, gpus_per_node, bw_intra, bw_inter, num_channels, nvswitch, collnet, net_latency
CONFIGS = [
    (0, 1, 8, 87.7, 25.0, -1, 0, 0, 0.0),
    (0, 2, 8, 87.7, 25.0, -1, 0, 0, 0.0),
    (0, 4, 8, 87.7, 25.0, -1, 0, 0, 0.0),
    (0, 8, 1, 87.7, 25.0, -1, 0, 0, 0.0),
    (0, 2, 8, 87.7, 25.0, -1, 1, 0, 0.0),
    (0, 4, 8, 87.7, 12.5, -1, 0, 1, 0.0),
    (0, 4, 8, 87.7, 25.0, 8, 0, 0, 2.5),
    (1, 1, 8, 320.0, 50.0, -1, 1, 0, 0.0),
    (1, 8, 8, 320.0, 50.0, -1, 1, 0, 0.0),
    (1, 8, 8, 320.0, 25.0, -1, 1, 0, 1.5),
    (1, 8, 8, 320.0, 50.0, -1, 0, 0, 0.0),
    (1, 8, 8, 320.0, 50.0, -1, 1, 1, 0.0),
    (1, 4, 8, 320.0, 50.0, 1, 1, 0, 0.0),
    (1, 16, 4, 320.0, 50.0, -1, 1, 0, 0.0),
    (1, 4, 8, 320.0, 50.0, 24, 0, 1, 0.5),
    (2, 1, 72, 640.0, 50.0, -1, 1, 0, 0.0),
    (2, 8, 8, 640.0, 50.0, -1, 1, 0, 0.0),
    (2, 8, 8, 640.0, 100.0, -1, 0, 0, 0.0),
    (2, 8, 8, 640.0, 100.0, -1, 1, 1, 0.0),
    (1, 8, 8, 320.0, 0.0, -1, 1, 0, 0.0),
]
MESHES = [(8,), (2,), (4,), (6,), (16,), (64,), (2, 8), (4, 8), (8, 8), (16, 8), (32, 8), (64, 8), (3, 8),
          (8, 4), (4, 2), (2, 4, 4), (4, 8, 8), (2, 2, 2, 8), (32, 2), (16, 4), (72,), (2, 72), (5, 4)]
BYTES = [0, 1, 63, 64, 100, 4095, 4096, 65537, 1 << 17, (1 << 18) + 1, 3 * (1 << 18), 1 << 20, 3 * (1 << 20) + 17,
         (1 << 22) - 1, 1 << 24, (1 << 26) + 12345, 5 * (1 << 26), 1 << 28, 1 << 30, 7 * (1 << 30) + 1, 1 << 34,
         (1 << 37) + 99]


def load_nccl():
    spec = importlib.util.spec_from_file_location("ref_nccl_cost_model", REF)
    m = importlib.util.module_from_spec(spec)
    sys.modules[spec.name] = m
    spec.loader.exec_module(m)
    return m


def make_cfg(m, row):
    arch, nn, gpn, bwi, bwe, nch, sw, cn, nl = row
    return m.NCCLTopoConfig(arch=m.GpuArch(arch), num_nodes=nn, gpus_per_node=gpn, bw_intra=bwi, bw_inter=bwe,
                            num_channels=None if nch < 0 else nch, has_nvswitch=bool(sw), has_collnet=bool(cn),
                            net_latency=nl)


def main():
    m = load_nccl()
    rng = np.random.default_rng(7)
    extra = [int(2 ** x) for x in rng.uniform(6, 36, 10)]
    sizes = BYTES + extra
    cases, cost, topo = [], [], []
    fns = [m.nccl_allgather_cost, m.nccl_reduce_scatter_cost, m.nccl_allreduce_cost, m.nccl_all_to_all_cost]
    for ci, row in enumerate(CONFIGS):
        cfg = make_cfg(m, row)
        for mi, mesh in enumerate(MESHES):
            for d in range(len(mesh)):
                t = m.derive_mesh_dim_topo(cfg, mesh, d)
                if t.n_ranks < 2:
                    continue
                for coll in range(4):
                    for nb in sizes:
                        cases.append((ci, mi, d, coll, nb))
                        cost.append(fns[coll](nb, t, cfg))
                        topo.append((t.n_ranks, t.n_nodes, t.ppn, t.n_channels))
    out = {
        "cfg": np.asarray(CONFIGS, np.float64),
        "mesh": np.asarray([(len(s),) + tuple(s) + (0,) * (4 - len(s)) for s in MESHES], np.int64),
        "case": np.asarray(cases, np.int64),
        "cost": np.asarray(cost, np.float64),
        "topo": np.asarray(topo, np.int64),
    }
    for n in (8, 16, 32, 64):
        out[f"ring_depth_{n}"] = np.asarray(m._depth_scaled_ring_correction(n), np.float64)

    # redistribution under the NCCL model
    import make_cost_vectors as mcv

    mcv.patch_device()
    mods = mcv.load_reference_cost_models()
    cre = mods["collective_runtime_estimation"]
    nc = mods["nccl_cost_model"]
    import torch
    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard
    from torch.testing._internal.distributed.fake_pg import FakeStore

    pair_cases = [
        # cfg index, mesh, shape, stride, itemsize
        (8, (8, 8), (4096, 4096), (4096, 1), 2),
        (8, (8, 8), (64, 8192, 512), (512, 32768, 1), 4),
        (1, (2, 8), (8192, 1024), (1024, 1), 2),
        (13, (2, 4, 4), (128, 256, 64), (16384, 64, 1), 2),
        (7, (8,), (1024, 1024), (1, 1024), 4),
    ]
    k = 0
    for ci, mesh_shape, shape, stride, itemsize in pair_cases:
        world = int(np.prod(mesh_shape))
        if torch.distributed.is_initialized():
            torch.distributed.destroy_process_group()
        torch.distributed.init_process_group("fake", store=FakeStore(), rank=0, world_size=world)
        mesh = init_device_mesh("cpu", mesh_shape)
        cfg = make_cfg(nc, CONFIGS[ci])
        cre.set_nccl_topo_config(cfg)
        dtype = {2: torch.bfloat16, 4: torch.float32}[itemsize]
        tm = TensorMeta(torch.Size(shape), tuple(stride), dtype)
        opts = [Replicate(), Partial()] + [Shard(i) for i in range(len(shape))]
        src, tgt, vals = [], [], []
        for s in itertools.product(opts, repeat=len(mesh_shape)):
            for t in itertools.product(opts, repeat=len(mesh_shape)):
                a = DTensorSpec(mesh, s, tensor_meta=tm)
                b = DTensorSpec(mesh, t, tensor_meta=tm)
                vals.append(cre.estimate_strategy_comms_cost(a, b))
                src.append([mcv.code_of(p) for p in s])
                tgt.append([mcv.code_of(p) for p in t])
        cre.set_nccl_topo_config(None)
        out[f"pair_{k}_cfg"] = np.asarray(ci)
        out[f"pair_{k}_mesh"] = np.asarray(mesh_shape, np.int64)
        out[f"pair_{k}_shape"] = np.asarray(shape, np.int64)
        out[f"pair_{k}_stride"] = np.asarray(stride, np.int64)
        out[f"pair_{k}_itemsize"] = np.asarray(itemsize)
        out[f"pair_{k}_src"] = np.asarray(src, np.uint8)
        out[f"pair_{k}_tgt"] = np.asarray(tgt, np.uint8)
        out[f"pair_{k}_cost"] = np.asarray(vals, np.float64)
        k += 1
    out["n_pair"] = np.asarray(k)
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, "cases", len(cases), "pair cases", k, "pairs", sum(len(out[f'pair_{i}_cost']) for i in range(k)))


if __name__ == "__main__":
    main()
