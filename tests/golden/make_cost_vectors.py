"""Writes tests/golden/cost_vectors.npz from the reference's own cost functions.

Run in the build container only (the reference tree is not present anywhere
else):   python tests/golden/make_cost_vectors.py

No reference test pins a numeric value of ``redistribute_cost``,
``estimate_strategy_comms_cost``, ``compute_read_write_time``,
``_get_sharded_shape_stride`` or ``estimate_strategy_runtime_cost``; these
vectors do.  The three ``cost_models`` modules are loaded by file path under a
stub parent package (the package ``__init__`` needs ``pulp`` and nightly-only
torch APIs), with the device patched the way the reference's tests/conftest.py
does it, but to an MI355X: 8 devices per host, name "AMD Instinct MI355X".

The output holds inputs and expected outputs only (no reference code):
  comm_<k>_{mesh,dph,shape,stride,itemsize}   one case per k
  comm_<k>_src / _tgt   uint8[n, ndim] placement bytes (packed-format encoding)
  comm_<k>_cost         float64[n]  estimate_strategy_comms_cost(src, tgt)
  comm_<k>_cost_fwd     float64[n]  redistribute_cost(src, tgt, [0..ndim))
  rw_bytes / rw_time    compute_read_write_time
  shard_*               _get_sharded_shape_stride
  rt_*                  estimate_strategy_runtime_cost on hand-built fx nodes
"""
import importlib.util
import itertools
import os
import sys
import types

import numpy as np
import torch

REF = "/root/reference/autoparallel"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cost_vectors.npz")


def load_reference_cost_models():
    pkg = types.ModuleType("autoparallel")
    pkg.__path__ = [REF]
    sys.modules["autoparallel"] = pkg
    sub = types.ModuleType("autoparallel.cost_models")
    sub.__path__ = [REF + "/cost_models"]
    sys.modules["autoparallel.cost_models"] = sub
    mods = {}
    for name in ("nccl_cost_model", "compute_estimation", "collective_runtime_estimation"):
        spec = importlib.util.spec_from_file_location(
            "autoparallel.cost_models." + name, f"{REF}/cost_models/{name}.py"
        )
        m = importlib.util.module_from_spec(spec)
        sys.modules[spec.name] = m
        spec.loader.exec_module(m)
        mods[name] = m
    return mods


def patch_device():
    torch.cuda.device_count = lambda: 8
    torch.cuda.get_device_name = lambda device=None: "AMD Instinct MI355X"
    torch.cuda.is_available = lambda: True
    torch.cuda.set_device = lambda *a, **k: None
    torch.cuda.current_device = lambda: 0
    # no accelerator in the build container: route device-name queries to the
    # patched torch.cuda module
    torch.get_device_module = lambda device=None: torch.cuda


def code_of(p):
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

    if isinstance(p, Replicate):
        return 0
    if isinstance(p, Shard):
        return 0x40 | p.dim
    assert isinstance(p, Partial)
    return 0x80 | {"sum": 0, "avg": 1, "min": 2, "max": 3, "product": 4}[p.reduce_op]


def main():
    patch_device()
    mods = load_reference_cost_models()
    cre = mods["collective_runtime_estimation"]
    ce = mods["compute_estimation"]

    import torch.distributed as dist
    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
    from torch.distributed.tensor._op_schema import OpSpec
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard
    from torch.testing._internal.distributed.fake_pg import FakeStore

    dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=256)
    out = {}
    rng = np.random.default_rng(1234)

    # ---------------- communication cost ----------------
    cases = [
        # mesh, shape, stride, dtype
        ((8,), (64, 8192, 4096), None, torch.bfloat16),
        ((8,), (50257, 768), None, torch.float32),
        ((8, 8), (64, 8192, 4096), None, torch.bfloat16),
        ((8, 8), (4096, 14336), None, torch.bfloat16),
        ((8, 8), (4096, 14336), (1, 4096), torch.bfloat16),  # transposed view
        ((8, 8), (64, 32, 8192, 128), (33554432, 128, 4096, 1), torch.bfloat16),
        ((8, 8), (128256,), None, torch.float32),
        ((2, 4), (6, 10), None, torch.float32),
        ((3, 5), (30, 45, 7), None, torch.float64),  # non power-of-two mesh
        ((32, 8), (1000, 333), (333, 1), torch.float16),
        ((4, 8, 8), (256, 8192, 8192), None, torch.bfloat16),
        ((4, 8, 8), (8192, 28672), (1, 8192), torch.bfloat16),
        ((2, 3, 4), (24, 36, 48), None, torch.float32),
        ((8, 8), (1, 8192, 1), None, torch.float32),  # size-1 dims
        ((8, 8), (64, 8192, 4096), (33554432, 1, 8192), torch.bfloat16),
    ]
    for k, (mesh_shape, shape, stride, dtype) in enumerate(cases):
        mesh = init_device_mesh("cuda", mesh_shape)
        ndim = len(mesh_shape)
        t = torch.empty(shape, device="meta", dtype=dtype)
        if stride is None:
            stride = t.stride()
        tm = TensorMeta(torch.Size(shape), tuple(stride), dtype)
        opts = [Replicate()] + [Shard(i) for i in range(len(shape))] + [Partial(), Partial("avg")]
        tuples = list(itertools.product(opts, repeat=ndim))
        pairs = [(a, b) for a in tuples for b in tuples]
        if len(pairs) > 4000:
            idx = rng.choice(len(pairs), size=4000, replace=False)
            idx.sort()
            pairs = [pairs[i] for i in idx]
        src = np.zeros((len(pairs), ndim), np.uint8)
        tgt = np.zeros((len(pairs), ndim), np.uint8)
        cost = np.zeros(len(pairs), np.float64)
        cost_fwd = np.zeros(len(pairs), np.float64)
        for i, (a, b) in enumerate(pairs):
            s_spec = DTensorSpec(mesh, a, tensor_meta=tm)
            t_spec = DTensorSpec(mesh, b, tensor_meta=tm)
            cre.reset_comms_cost_cache()
            cost[i] = cre.estimate_strategy_comms_cost(s_spec, t_spec)
            cost_fwd[i] = cre.redistribute_cost(s_spec, t_spec, list(range(ndim)))
            src[i] = [code_of(p) for p in a]
            tgt[i] = [code_of(p) for p in b]
        out[f"comm_{k}_mesh"] = np.asarray(mesh_shape, np.int64)
        out[f"comm_{k}_dph"] = np.asarray([8], np.int64)
        out[f"comm_{k}_shape"] = np.asarray(shape, np.int64)
        out[f"comm_{k}_stride"] = np.asarray(stride, np.int64)
        out[f"comm_{k}_itemsize"] = np.asarray([dtype.itemsize], np.int64)
        out[f"comm_{k}_src"] = src
        out[f"comm_{k}_tgt"] = tgt
        out[f"comm_{k}_cost"] = cost
        out[f"comm_{k}_cost_fwd"] = cost_fwd
    out["comm_ncases"] = np.asarray([len(cases)], np.int64)

    # ---------------- read/write time ----------------
    b = np.concatenate(
        [
            np.asarray([0, 1, 7, 1000, 43110, 43111, 43112, 2**20, 2**30, 2**40 + 12345], np.int64),
            rng.integers(1, 2**44, size=200),
        ]
    )
    out["rw_bytes"] = b
    out["rw_time"] = np.asarray([float(ce.compute_read_write_time(int(x))) for x in b], np.float64)
    # float-valued byte counts, as redistribute_cost passes them
    bf = rng.random(200) * 2.0**36
    out["rw_fbytes"] = bf
    out["rw_ftime"] = np.asarray([float(ce.compute_read_write_time(float(x))) for x in bf], np.float64)

    # ---------------- sharded shape/stride ----------------
    mesh = init_device_mesh("cuda", (4, 8, 8))
    shapes = [(256, 8192, 8192), (10, 3, 1000), (7,), (64, 32, 8192, 128)]
    rows = []
    for shape in shapes:
        t = torch.empty(shape, device="meta")
        tm = TensorMeta(torch.Size(shape), t.stride(), torch.float32)
        opts = [Replicate()] + [Shard(i) for i in range(len(shape))] + [Partial()]
        for plc in itertools.product(opts, repeat=3):
            spec = DTensorSpec(mesh, plc, tensor_meta=tm)
            ns, nst = ce._get_sharded_shape_stride(spec)
            rows.append((shape, t.stride(), [code_of(p) for p in plc], ns, nst))
    n = len(rows)
    sh = np.zeros((n, 4), np.int64)
    st = np.zeros((n, 4), np.int64)
    rk = np.zeros(n, np.int64)
    pl = np.zeros((n, 3), np.uint8)
    osh = np.zeros((n, 4), np.int64)
    ost = np.zeros((n, 4), np.int64)
    for i, (shape, stride, plc, ns, nst) in enumerate(rows):
        r = len(shape)
        rk[i] = r
        sh[i, :r], st[i, :r], pl[i], osh[i, :r], ost[i, :r] = shape, stride, plc, ns, nst
    out.update(shard_rank=rk, shard_shape=sh, shard_stride=st, shard_plc=pl,
               shard_out_shape=osh, shard_out_stride=ost,
               shard_mesh=np.asarray([4, 8, 8], np.int64))

    # ---------------- runtime (compute) estimate ----------------
    # Hand-built fx nodes whose args carry meta-device tensors; strategies are
    # OpSpecs with the given input placements.  Stored: op name, the global
    # input shapes/dtypes, per-case input placements, expected cost.
    import contextlib

    mesh = init_device_mesh("cuda", (8, 8))
    fake_mode = contextlib.nullcontext()  # meta tensors stand in for FakeTensors
    aten = torch.ops.aten

    def mk(shape, dtype):
        return torch.empty(shape, dtype=dtype, device="meta")

    rt_ops = []  # (name, target, [(shape, dtype)], extra_args, [in placements per case])
    R, S, P = Replicate(), Shard, Partial()
    bf16, f32 = torch.bfloat16, torch.float32
    rt_ops.append(("mm", aten.mm.default, [((8192, 4096), bf16), ((4096, 14336), bf16)], (),
                   [((R, R), (R, R)), ((S(0), R), (R, R)), ((S(0), S(1)), (R, S(0))),
                    ((R, S(0)), (R, S(1))), ((S(1), S(0)), (S(0), S(1)))]))
    rt_ops.append(("mm_f32", aten.mm.default, [((512, 256), f32), ((256, 1024), f32)], (),
                   [((R, R), (R, R)), ((S(0), S(0)), (R, R)), ((S(1), R), (S(0), R))]))
    rt_ops.append(("bmm", aten.bmm.default, [((64, 1024, 128), bf16), ((64, 128, 1024), bf16)], (),
                   [((R, R), (R, R)), ((S(0), R), (S(0), R)), ((S(0), S(1)), (S(0), R))]))
    rt_ops.append(("addmm", aten.addmm.default,
                   [((3072,), bf16), ((8192, 768), bf16), ((768, 3072), bf16)], (),
                   [((R, R), (R, R), (R, R)), ((R, S(0)), (S(0), R), (R, S(1))),
                    ((R, R), (S(0), S(0)), (R, R))]))
    rt_ops.append(("add", aten.add.Tensor, [((64, 8192, 4096), bf16), ((64, 8192, 4096), bf16)], (),
                   [((R, R), (R, R)), ((S(0), S(1)), (S(0), S(1))), ((S(0), S(2)), (S(0), S(2))),
                    ((S(2), S(2)), (S(2), S(2)))]))
    rt_ops.append(("mul_bcast", aten.mul.Tensor, [((64, 8192, 4096), bf16), ((4096,), bf16)], (),
                   [((R, R), (R, R)), ((S(0), S(2)), (R, S(0))), ((S(1), R), (R, R))]))
    rt_ops.append(("small_add", aten.add.Tensor, [((16, 16), f32), ((16, 16), f32)], (),
                   [((R, R), (R, R)), ((S(0), R), (S(0), R))]))
    rt_ops.append(("silu", aten.silu.default, [((64, 8192, 14336), bf16)], (),
                   [((R, R),), ((S(0), S(2)),), ((S(1), S(1)),)]))
    rt_ops.append(("sum_dim", aten.sum.dim_IntList, [((64, 8192, 4096), f32)], ([2], True),
                   [((R, R),), ((S(0), S(1)),), ((S(0), S(2)),)]))
    rt_ops.append(("mean_dim", aten.mean.dim, [((64, 8192, 4096), f32)], ([-1], True),
                   [((R, R),), ((S(0), S(1)),)]))
    rt_ops.append(("einsum_fwd", aten.einsum.default,
                   [((64, 8192, 4096), bf16), ((4096, 14336), bf16)], "bsk,kn->bsn",
                   [((R, R), (R, R)), ((S(0), R), (R, S(1))), ((S(0), S(2)), (R, S(0))),
                    ((S(1), S(0)), (R, R))]))
    rt_ops.append(("einsum_bwd", aten.einsum.default,
                   [((64, 8192, 14336), bf16), ((64, 8192, 4096), bf16)], "bsn,bsk->kn",
                   [((R, R), (R, R)), ((S(0), S(1)), (S(0), S(1))), ((S(0), S(2)), (S(0), R))]))
    rt_ops.append(("softmax", aten._softmax.default, [((64, 32, 1024, 1024), f32)], (-1, False),
                   [((R, R),), ((S(0), S(1)),)]))
    rt_ops.append(("embedding", aten.embedding.default,
                   [((128256, 4096), bf16), ((64, 8192), torch.int64)], (),
                   [((R, R), (R, R)), ((R, R), (S(0), S(1))), ((R, S(1)), (S(0), R))]))
    rt_ops.append(("view", aten.view.default, [((64, 8192, 4096), bf16)], ([64, 8192, 32, 128],),
                   [((R, R),)]))
    rt_ops.append(("sdpa_flash", aten._scaled_dot_product_flash_attention.default,
                   [((64, 32, 8192, 128), bf16)] * 3, (0.0, True),
                   [((R, R),) * 3, ((S(0), S(1)),) * 3, ((S(0), R),) * 3]))

    names, shapes_all, dtypes_all, plcs_all, costs_all, flops_all, bytes_all = [], [], [], [], [], [], []
    for name, target, ins, extra, cases_ in rt_ops:
        graph = torch.fx.Graph()
        phs = []
        for i, (shape, dtype) in enumerate(ins):
            ph = graph.placeholder(f"x{i}")
            ph.meta["val"] = mk(shape, dtype)
            phs.append(ph)
        if isinstance(extra, str):
            node = graph.call_function(target, (extra, phs))
        else:
            node = graph.call_function(target, tuple(phs) + tuple(extra))
        for plcs in cases_:
            in_specs = []
            for (shape, dtype), plc, ph in zip(ins, plcs, phs):
                v = ph.meta["val"]
                in_specs.append(DTensorSpec(mesh, plc, tensor_meta=TensorMeta(v.shape, v.stride(), v.dtype)))
            strat = OpSpec(output_specs=in_specs[0], input_specs=in_specs)
            ce.reset_compute_cost_cache()
            with fake_mode:
                c = ce.estimate_strategy_runtime_cost(node, strat)
                args, kwargs = ce._shard_args_for_node(node, strat)
                fl, o = ce._compute_flops(node.target, *args, **kwargs)
                nb = ce.compute_memory_cost(node.target, args, o)
            names.append(name)
            shapes_all.append([list(s) for s, _ in ins])
            dtypes_all.append([str(d) for _, d in ins])
            plcs_all.append([[code_of(p) for p in plc] for plc in plcs])
            costs_all.append(float(c))
            flops_all.append(int(fl))
            bytes_all.append(int(nb))
    import json

    out["rt_json"] = np.frombuffer(
        json.dumps(
            {"names": names, "shapes": shapes_all, "dtypes": dtypes_all, "placements": plcs_all,
             "flops": flops_all, "bytes": bytes_all,
             "cost_hex": [float(c).hex() for c in costs_all], "mesh": [8, 8]}
        ).encode(),
        dtype=np.uint8,
    )
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes;", len(names), "runtime cases")


if __name__ == "__main__":
    main()
