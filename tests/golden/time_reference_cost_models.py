"""Calibration of the CPU baseline: microseconds per cost entry of the
reference's own ``estimate_strategy_comms_cost`` beside the Python port
(oracle/cost_oracle.py) on the same cases, the ones of cost_vectors.npz.

Run in the build container only (the reference tree is not present anywhere
else):   python tests/golden/time_reference_cost_models.py

The reference modules are loaded exactly as make_cost_vectors.py loads them.
The reference is timed twice: with its memo cache cleared before every call
(every entry is computed: what a graph without repeated spec pairs costs) and
with the cache kept (its normal mode; no pair repeats within a case, so this
shows the cost of the cache itself).  The port's function has no memo of its
own (GraphOracle keeps one, keyed like the reference's).  Prints one JSON line.
"""
import json
import os
import sys
import time

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import make_cost_vectors as M  # noqa: E402
from oracle import cost_oracle as O  # noqa: E402

CASES = [2, 3, 10]  # (8,8) activations, (8,8) weight, (4,8,8) activations
N_PER_CASE = 1500


def main():
    M.patch_device()
    cre = M.load_reference_cost_models()["collective_runtime_estimation"]
    import torch.distributed as dist
    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard
    from torch.testing._internal.distributed.fake_pg import FakeStore

    dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=256)
    golden = np.load(os.path.join(HERE, "cost_vectors.npz"))
    dev = O.DeviceLimit()

    def placement(code):
        code = int(code)
        if code == 0:
            return Replicate()
        if code & 0x40:
            return Shard(code & 0x3F)
        return Partial(["sum", "avg", "min", "max", "product"][code & 0x3F])

    res = {"reference": {}, "port": {}}
    n_total = 0
    t_ref = {"cleared": 0.0, "kept": 0.0}
    t_port = 0.0
    for k in CASES:
        mesh_shape = tuple(int(x) for x in golden[f"comm_{k}_mesh"])
        shape = [int(x) for x in golden[f"comm_{k}_shape"]]
        stride = [int(x) for x in golden[f"comm_{k}_stride"]]
        itemsize = int(golden[f"comm_{k}_itemsize"][0])
        dtype = {2: torch.bfloat16, 4: torch.float32, 8: torch.float64}[itemsize]
        src, tgt = golden[f"comm_{k}_src"][:N_PER_CASE], golden[f"comm_{k}_tgt"][:N_PER_CASE]
        want = golden[f"comm_{k}_cost"][:N_PER_CASE]
        mesh = init_device_mesh("cuda", mesh_shape)
        tm = TensorMeta(torch.Size(shape), tuple(stride), dtype)
        specs = [(DTensorSpec(mesh, tuple(placement(c) for c in s), tensor_meta=tm),
                  DTensorSpec(mesh, tuple(placement(c) for c in t), tensor_meta=tm)) for s, t in zip(src, tgt)]
        topo = O.Topo(list(mesh_shape), int(golden[f"comm_{k}_dph"][0]))
        keys = [(tuple(int(x) for x in s), tuple(int(x) for x in t)) for s, t in zip(src, tgt)]
        n_total += len(specs)
        for mode in ("cleared", "kept"):
            cre.reset_comms_cost_cache()
            t0 = time.perf_counter()
            for a, b in specs:
                if mode == "cleared":
                    cre.reset_comms_cost_cache()
                got = cre.estimate_strategy_comms_cost(a, b)
            t_ref[mode] += time.perf_counter() - t0
            assert got == want[len(keys) - 1] or (np.isinf(got) and np.isinf(want[len(keys) - 1]))
        t0 = time.perf_counter()
        for s, t in keys:
            got = O.estimate_strategy_comms_cost(s, shape, stride, itemsize, t, topo, dev)
        t_port += time.perf_counter() - t0
        assert got == want[len(keys) - 1] or (np.isinf(got) and np.isinf(want[len(keys) - 1]))
    for mode in ("cleared", "kept"):
        res["reference"][f"us_per_entry_cache_{mode}"] = t_ref[mode] / n_total * 1e6
    res["port"]["us_per_entry"] = t_port / n_total * 1e6
    res["entries"] = n_total
    res["cases"] = CASES
    res["what"] = "estimate_strategy_comms_cost, one call per (src, tgt) placement pair of cost_vectors.npz"
    print(json.dumps(res))


if __name__ == "__main__":
    main()
