"""The reference's ``autoparallel.cost_models.nccl_cost_model`` interface
(autoparallel/cost_models/nccl_cost_model.py:40-92, 1001-1021, 1321-1465) on
top of the HIP engine.  The configuration types and presets are plain data;
topology derivation and candidate resolution run in the library's host helper,
and every cost is evaluated on the device (a single query is a batch of one).
"""
from __future__ import annotations

import ctypes as C
import logging
from dataclasses import dataclass
from enum import Enum
from typing import Optional, Tuple

import torch

from .. import _lib
from ..engine import build_nccl_plan, detect_device_name, nccl_config_struct

logger = logging.getLogger(__name__)


class GpuArch(Enum):
    AMPERE = 0
    HOPPER = 1
    BLACKWELL = 2


class NCCLFunc(Enum):
    ALLGATHER = 0
    REDUCESCATTER = 1
    ALLREDUCE = 2


@dataclass
class NCCLTopoConfig:
    arch: GpuArch
    num_nodes: int
    gpus_per_node: int
    bw_intra: float  # GB/s per GPU inside a node
    bw_inter: float  # GB/s per GPU between nodes
    num_channels: Optional[int] = None  # None: 12 on Ampere, 16 on Hopper/Blackwell
    has_nvswitch: bool = False
    has_collnet: bool = False
    net_latency: float = 0.0


@dataclass
class MeshDimTopo:
    n_ranks: int
    n_nodes: int
    ppn: int
    bw_intra: float  # per channel
    bw_inter: float  # per channel
    n_channels: int


def derive_mesh_dim_topo(config: NCCLTopoConfig, mesh_shape: Tuple[int, ...], dim_idx: int) -> MeshDimTopo:
    d = build_nccl_plan(config, tuple(mesh_shape)).dim[dim_idx]
    return MeshDimTopo(d.n_ranks, d.n_nodes, d.ppn, d.bw_intra, d.bw_inter, d.n_channels)


# C ABI collective codes
_KIND = {"allgather": 0, "all_to_all": 1, "allreduce": 2, "reduce_scatter": 3}


def _plan_cost(plan: _lib.ApcNcclPlan, kind: int, n_bytes: int, dim: int) -> float:
    import numpy as np

    lib = _lib.load()
    model = _lib.ApcModel()
    model.ndim = plan.ndim
    for i in range(plan.ndim):
        model.mesh_shape[i] = plan.dim[i].n_ranks
    dev_plan = torch.from_numpy(np.frombuffer(bytes(plan), dtype=np.uint8).copy()).cuda()
    model.nccl_plan = dev_plan.data_ptr()
    k = torch.tensor([kind], dtype=torch.int32, device="cuda")
    nb = torch.tensor([int(n_bytes)], dtype=torch.int64, device="cuda")
    dm = torch.tensor([dim], dtype=torch.int32, device="cuda")
    out = torch.empty(1, dtype=torch.float64, device="cuda")
    _lib.check(lib.apc_collective_costs(C.byref(model), 1, k.data_ptr(), nb.data_ptr(), dm.data_ptr(),
                                        out.data_ptr(), None), "apc_collective_costs")
    return float(out.item())


def _topo_cost(kind: str, n_bytes: int, topo: MeshDimTopo, config: NCCLTopoConfig) -> float:
    lib = _lib.load()
    plan = _lib.ApcNcclPlan()
    c = nccl_config_struct(config)
    _lib.check(lib.apc_nccl_plan_for_topo(C.byref(c), int(topo.n_ranks), int(topo.n_nodes), int(topo.ppn),
                                          int(topo.n_channels), float(topo.bw_intra), float(topo.bw_inter),
                                          C.byref(plan)), "apc_nccl_plan_for_topo")
    return _plan_cost(plan, _KIND[kind], n_bytes, 0)


def nccl_allgather_cost(n_bytes: int, topo: MeshDimTopo, config: NCCLTopoConfig) -> float:
    return _topo_cost("allgather", n_bytes, topo, config)


def nccl_allreduce_cost(n_bytes: int, topo: MeshDimTopo, config: NCCLTopoConfig) -> float:
    return _topo_cost("allreduce", n_bytes, topo, config)


def nccl_reduce_scatter_cost(n_bytes: int, topo: MeshDimTopo, config: NCCLTopoConfig) -> float:
    return _topo_cost("reduce_scatter", n_bytes, topo, config)


def nccl_all_to_all_cost(n_bytes: int, topo: MeshDimTopo, config: NCCLTopoConfig) -> float:
    return _topo_cost("all_to_all", n_bytes, topo, config)


def nccl_collective_time(func: NCCLFunc, n_bytes: int, topo: MeshDimTopo, config: NCCLTopoConfig) -> float:
    return _topo_cost({0: "allgather", 1: "reduce_scatter", 2: "allreduce"}[NCCLFunc(func).value], n_bytes, topo,
                      config)


def nccl_mesh_collective_cost(collective: str, n_bytes: int, mesh_shape: Tuple[int, ...], mesh_dim: int,
                              config: NCCLTopoConfig) -> float:
    """_nccl_comm_cost (autoparallel/cost_models/collective_runtime_estimation.py:44-62)."""
    if collective not in _KIND:
        return 0.0
    return _plan_cost(build_nccl_plan(config, tuple(mesh_shape)), _KIND[collective], n_bytes, mesh_dim)


# most specific first, so "B200" does not match inside "GB200"
_CANONICAL_GPUS_PER_NODE = (("GB200", 72), ("B200", 72), ("H200", 8), ("H100", 8), ("A100", 8))


def a100_topo_config(num_nodes: int = 1, gpus_per_node: int = 8, bw_inter: float = 25.0, **kw) -> NCCLTopoConfig:
    return NCCLTopoConfig(arch=GpuArch.AMPERE, num_nodes=num_nodes, gpus_per_node=gpus_per_node, bw_intra=87.7,
                          bw_inter=bw_inter, **kw)


def h100_topo_config(num_nodes: int = 1, gpus_per_node: int = 8, bw_inter: float = 50.0,
                     has_nvswitch: bool = True, **kw) -> NCCLTopoConfig:
    return NCCLTopoConfig(arch=GpuArch.HOPPER, num_nodes=num_nodes, gpus_per_node=gpus_per_node, bw_intra=320.0,
                          bw_inter=bw_inter, has_nvswitch=has_nvswitch, **kw)


def gb200_topo_config(num_nodes: int = 1, gpus_per_node: int = 72, bw_inter: float = 50.0,
                      has_nvswitch: bool = True, **kw) -> NCCLTopoConfig:
    return NCCLTopoConfig(arch=GpuArch.BLACKWELL, num_nodes=num_nodes, gpus_per_node=gpus_per_node, bw_intra=640.0,
                          bw_inter=bw_inter, has_nvswitch=has_nvswitch, **kw)


def detect_nccl_topo_config(mesh, device_name: Optional[str] = None) -> Optional[NCCLTopoConfig]:
    """Preset for the planning device, or None when the device is not one the
    NCCL model was fitted for (every AMD part: the caller then keeps the
    default alpha-beta model) or the mesh does not divide into whole nodes."""
    if device_name is None:
        try:
            device_name = detect_device_name()
        except (RuntimeError, AssertionError):
            logger.info("No device available for NCCL cost model detection; using the default cost model.")
            return None
    total = mesh.size()
    for name, gpn in _CANONICAL_GPUS_PER_NODE:
        if name in device_name:
            break
    else:
        logger.warning("Unrecognized GPU '%s' for NCCL cost model; using the default cost model.", device_name)
        return None
    if total % gpn != 0:
        logger.warning("Mesh size %d is not divisible by %d GPUs/node for %s; using the default cost model.", total,
                       gpn, device_name)
        return None
    nodes = total // gpn
    if name == "A100":
        return a100_topo_config(num_nodes=nodes, gpus_per_node=gpn)
    if name in ("H100", "H200"):
        return h100_topo_config(num_nodes=nodes, gpus_per_node=gpn)
    return gb200_topo_config(num_nodes=nodes, gpus_per_node=gpn)
