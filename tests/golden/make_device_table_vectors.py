"""Writes tests/golden/device_table_vectors.json from the reference's device lookups.

Run in the build container only (the reference tree is not present anywhere
else):   python tests/golden/make_device_table_vectors.py

For a list of device-name strings as drivers report them, the file holds what
the reference's ``_get_device_gmem_bandwidth()`` and ``_get_device_tflops(dtype)``
(autoparallel/cost_models/compute_estimation.py:257-289) answer when
``get_device_name`` returns that string: the bandwidth and the five dtype
figures as hex floats, ``null`` where the lookup raises for the dtype, and
``{"error": ...}`` where it raises for the device.  Inputs and expected
outputs only (no reference code).  ``compute_estimation`` is loaded by file
path under a stub parent package, as make_cost_vectors.py does.
"""
import json
import os

import torch

from make_cost_vectors import load_reference_cost_models, patch_device

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "device_table_vectors.json")

# names as torch.cuda.get_device_name / the vendors' tools print them, one or more
# per row of the table, plus strings that match two rows, one only by its board
# name, and none
NAMES = [
    "NVIDIA H100 80GB HBM3", "NVIDIA H100 PCIe", "NVIDIA H100 NVL", "NVIDIA B200",
    "NVIDIA A100-SXM4-80GB", "NVIDIA A100-PCIE-40GB", "NVIDIA PG509-210", "NVIDIA A30",
    "NVIDIA A10G", "Tesla T4", "Tesla V100-SXM2-16GB", "Tesla V100-PCIE-32GB", "Tesla P100-PCIE-16GB",
    "AMD Instinct MI200X", "AMD Instinct MI300X", "AMD Instinct MI300X VF", "AMD Instinct MI325X",
    "AMD Instinct MI350X", "AMD Instinct MI355X", "Intel(R) Data Center GPU Max 1550",
    "H100", "A100", "A30", "A10G", "T4", "V100", "P100", "B200", "Max 1550",
    "NVIDIA H100 and A100", "NVIDIA A100 and H100", "A30 next to an A10G", "MI300X",
    "NVIDIA GeForce RTX 4090", "AMD Instinct MI250X", "AMD Instinct MI300A", "NVIDIA H200", "",
]
DTYPES = (("float64", torch.float64), ("float32", torch.float32), ("float16", torch.float16),
          ("bfloat16", torch.bfloat16), ("int8", torch.int8))


def main():
    patch_device()
    ce = load_reference_cost_models()["compute_estimation"]
    out = {}
    for name in NAMES:
        torch.cuda.get_device_name = lambda device=None, _n=name: _n
        try:
            bw = ce._get_device_gmem_bandwidth()
        except ValueError as e:
            out[name] = {"error": str(e).split(".")[0]}
            continue
        row = {"gmem_bandwidth": float(bw).hex(), "tflops": {}}
        for label, dt in DTYPES:
            try:
                row["tflops"][label] = float(ce._get_device_tflops(dt)).hex()
            except ValueError:
                row["tflops"][label] = None
        out[name] = row
    with open(OUT, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", OUT, os.path.getsize(OUT), "bytes;", len(out), "names,",
          sum("error" in v for v in out.values()), "unsupported")


if __name__ == "__main__":
    main()
