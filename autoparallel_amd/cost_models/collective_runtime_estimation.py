"""The reference's ``autoparallel.cost_models.collective_runtime_estimation``
interface on top of the HIP engine (same names, arguments and return values;
autoparallel/cost_models/collective_runtime_estimation.py:34-41, 65-110,
115-229, 235-262).  Every number is computed on the device through the C ABI:
a single query is a batch of one."""
from __future__ import annotations

import ctypes as C
import dataclasses
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import _lib
from ..dtensor_bridge import devices_per_host, placement_codes, tensor_meta_key
from ..engine import CostEngine, detect_device_name, make_model
from ..packed import GraphBuilder, NodeDesc

_nccl_topo_config = None
_mesh_topo_config = None
_comms_cost_cache: Dict[tuple, float] = {}
_settings = {"devices_per_host": None, "device_name": None}

_COLLECTIVES = {"allgather": 0, "all_to_all": 1, "allreduce": 2, "reduce_scatter": 3}


def configure(devices_per_host: Optional[int] = None, device_name: Optional[str] = None) -> None:
    """Pin the two host-dependent inputs of the model (the reference reads
    them from the planning host: device count per host and device name)."""
    _settings["devices_per_host"] = devices_per_host
    _settings["device_name"] = device_name
    _comms_cost_cache.clear()


def _dph(mesh) -> int:
    return _settings["devices_per_host"] if _settings["devices_per_host"] is not None else devices_per_host(mesh)


def _device_name() -> str:
    return _settings["device_name"] or detect_device_name()


def set_nccl_topo_config(config) -> None:
    """Select the NCCL-tuning collective model (an NCCLTopoConfig) or, with
    None, the default alpha-beta model.  Clears the comm-cost memo, as the
    reference does (:34-38)."""
    global _nccl_topo_config
    _nccl_topo_config = config
    _comms_cost_cache.clear()


def get_nccl_topo_config():
    return _nccl_topo_config


def reset_comms_cost_cache() -> None:
    _comms_cost_cache.clear()


# ---------------------------------------------------------------------------
# xGMI node topology for the default (alpha-beta) model.  Not in the reference:
# its presets cover NVLink/NVSwitch systems (nccl_cost_model.py:1413-1470) and its
# detector returns None on an MI355X (:1341-1410), which leaves the alpha-beta
# model with torch's NVLink-era constants (87.7 GB/s per dim, 0.22 of it between
# hosts).  Outside the parity claim: with no config set, every number is the
# reference's.
# ---------------------------------------------------------------------------
@dataclasses.dataclass(frozen=True)
class XGMITopoConfig:
    """A node of GPUs joined pairwise by xGMI links, nodes joined by one NIC per
    GPU.  A ring collective inside a node is bound by one link per direction;
    an all-to-all drives all the links of a GPU at once."""

    gpus_per_node: int = 8
    links_per_gpu: int = 7
    link_gbps: float = 153.6  # one link, both directions together
    nic_gbps: float = 50.0  # per GPU between nodes (a 400 Gb/s NIC each)
    lat_intra_us: float = 0.6
    lat_inter_us: float = 2.7


def mi355x_topo_config(nic_gbps: float = 50.0) -> XGMITopoConfig:
    """MI355X / MI350X platform: 8 GPUs, 7 Infinity Fabric links of 153.6 GB/s each."""
    return XGMITopoConfig(nic_gbps=float(nic_gbps))


def mi300x_topo_config(nic_gbps: float = 50.0) -> XGMITopoConfig:
    """MI300X / MI325X platform: 8 GPUs, 7 links of 128 GB/s each."""
    return XGMITopoConfig(link_gbps=128.0, nic_gbps=float(nic_gbps))


def detect_mesh_topo_config(device_name: Optional[str] = None) -> Optional[XGMITopoConfig]:
    """The preset for the planning host's GPU, or None where the reference's
    constants apply (the counterpart of detect_nccl_topo_config for the default
    model)."""
    name = device_name or _device_name()
    if "MI355X" in name or "MI350X" in name:
        return mi355x_topo_config()
    if "MI300X" in name or "MI325X" in name:
        return mi300x_topo_config()
    return None


def set_mesh_topo_config(config: Optional[XGMITopoConfig]) -> None:
    """Select the link constants of the alpha-beta model (None: the
    reference's).  Clears the comm-cost memo, as set_nccl_topo_config does."""
    global _mesh_topo_config
    _mesh_topo_config = config
    _comms_cost_cache.clear()


def get_mesh_topo_config() -> Optional[XGMITopoConfig]:
    return _mesh_topo_config


def mi355x_topo(mesh_shape: Sequence[int], devices_per_host: int = 8,
                config: Optional[XGMITopoConfig] = None) -> Tuple[List[float], List[float], List[float]]:
    """(GB/s, us per hop, all-to-all GB/s) per mesh dim on MI355X nodes of
    ``devices_per_host`` GPUs (apc_xgmi_topology)."""
    cfg = dataclasses.replace(config or mi355x_topo_config(), gpus_per_node=int(devices_per_host))
    m = make_model(tuple(mesh_shape), devices_per_host, "AMD Instinct MI355X", topo_config=cfg)
    nd = len(mesh_shape)
    return ([m.mesh_bw[i] for i in range(nd)], [m.mesh_lat[i] for i in range(nd)],
            [m.mesh_a2a_bw[i] for i in range(nd)])


def comms_cost_matrix(src_specs: Sequence, tgt_specs: Sequence, order_mode: int = 0,
                      bandwidth_latency=None) -> np.ndarray:
    """cost[t][s] of redistributing src_specs[s] into the placements of
    tgt_specs[t] (all on one mesh): one edge block on the device.
    ``bandwidth_latency``: (GB/s, us per hop, all-to-all GB/s or 0) per mesh dim
    in place of what the mesh shape and the devices per host give."""
    mesh = src_specs[0].mesh
    b = GraphBuilder(tuple(mesh.shape), _dph(mesh) if hasattr(mesh, "device_type") else (_settings["devices_per_host"] or 1))
    src_words = [b.spec(b.meta(*tensor_meta_key(s.tensor_meta)), placement_codes(s.placements)) for s in src_specs]
    tgt_words = [b.spec(b.meta(*tensor_meta_key(t.tensor_meta)), placement_codes(t.placements)) for t in tgt_specs]
    b.add_node(NodeDesc("src", in_specs=[[w] for w in src_words], out_specs=[[w] for w in src_words],
                        inputs=[], default_rows=[[[0.0]] for _ in src_words]))
    b.add_node(NodeDesc("tgt", in_specs=[[w] for w in tgt_words], out_specs=[[w] for w in tgt_words], inputs=[0]))
    g = b.pack()
    eng = CostEngine(g, device_name=_device_name(), use_table=False, order_mode=order_mode,
                     nccl_config=_nccl_topo_config, topo_config=_mesh_topo_config)
    if bandwidth_latency is not None:
        for i, (bw, lat, a2a) in enumerate(zip(*bandwidth_latency)):
            m = eng.problem.model
            m.mesh_bw[i], m.mesh_lat[i], m.mesh_a2a_bw[i] = float(bw), float(lat), float(a2a)
    eng.build(clamp_inf=False)
    comm = eng.results()["comm"]
    base = int(g.edge_off[1])
    return comm[base : base + len(tgt_words) * len(src_words)].reshape(len(tgt_words), len(src_words))


def redistribute_cost(current_spec, target_spec, order: List[int]) -> float:
    if current_spec.mesh != target_spec.mesh:
        return float("inf")
    ndim = current_spec.mesh.ndim
    order = [int(i) for i in order]
    if order == list(range(ndim)):
        return float(comms_cost_matrix([current_spec], [target_spec], order_mode=1)[0, 0])
    if order == list(reversed(range(ndim))):
        return float(comms_cost_matrix([current_spec], [target_spec], order_mode=2)[0, 0])
    return _redistribute_cost_in_order(current_spec, target_spec, order)


def _redistribute_cost_in_order(current_spec, target_spec, order: List[int]) -> float:
    """Any other visiting order of the mesh dims (a permutation, or a subset: the
    dims left out are never touched, :154-156).  The fold only sees, per step, the
    two placements, the size, bandwidth and latency of the dim it visits, and the
    running volume; so it is evaluated in ascending order on the mesh relabelled
    in visiting order, with the bandwidth and latency each dim has on the real
    mesh carried along."""
    from types import SimpleNamespace

    if _nccl_topo_config is not None:
        raise NotImplementedError("an explicit mesh-dim order with the NCCL model is not built")
    mesh = current_spec.mesh
    ndim = mesh.ndim
    assert len(set(order)) == len(order) and all(0 <= i < ndim for i in order), order
    rest = [i for i in range(ndim) if i not in order]
    perm = order + rest
    model = make_model(tuple(mesh.shape), _dph(mesh), _device_name(), topo_config=_mesh_topo_config)
    bw, lat = [model.mesh_bw[i] for i in perm], [model.mesh_lat[i] for i in perm]
    a2a = [model.mesh_a2a_bw[i] for i in perm]
    relabelled = SimpleNamespace(shape=tuple(mesh.shape[i] for i in perm), ndim=ndim)
    src_plc = tuple(current_spec.placements[i] for i in perm)
    tgt_plc = tuple(target_spec.placements[i] if i in order else current_spec.placements[i] for i in perm)
    src = SimpleNamespace(mesh=relabelled, placements=src_plc, tensor_meta=current_spec.tensor_meta)
    tgt = SimpleNamespace(mesh=relabelled, placements=tgt_plc, tensor_meta=target_spec.tensor_meta)
    return float(comms_cost_matrix([src], [tgt], order_mode=1, bandwidth_latency=(bw, lat, a2a))[0, 0])


def estimate_strategy_comms_cost(src_spec, tgt_spec) -> float:
    key = (src_spec.placements, src_spec.tensor_meta, tgt_spec.placements, tgt_spec.tensor_meta,
           tuple(src_spec.mesh.shape))
    try:
        hash(key)
    except TypeError:
        key = None
    if key is not None:
        cached = _comms_cost_cache.get(key)
        if cached is not None:
            return cached
    if src_spec.mesh != tgt_spec.mesh:
        cost = float("inf")
    else:
        cost = float(comms_cost_matrix([src_spec], [tgt_spec], order_mode=0)[0, 0])
    if key is not None:
        _comms_cost_cache[key] = cost
    return cost


def collective_comm_cost(collective: str, comm_bytes: int, mesh_shape: Tuple[int, ...], mesh_dim: int,
                         mesh_topo=None, devices_per_host: Optional[int] = None) -> float:
    """Cost in microseconds of one collective on one mesh dim.  ``mesh_topo``
    (a torch MeshTopoInfo) supplies per-dim bandwidth/latency when given;
    otherwise they are derived from ``devices_per_host``."""
    if _nccl_topo_config is not None:
        from .nccl_cost_model import nccl_mesh_collective_cost

        return nccl_mesh_collective_cost(collective, comm_bytes, tuple(mesh_shape), mesh_dim, _nccl_topo_config)
    lib = _lib.load()
    dph = devices_per_host if devices_per_host is not None else (_settings["devices_per_host"] or 1)
    model = make_model(tuple(mesh_shape), dph, _device_name(), topo_config=_mesh_topo_config)
    if mesh_topo is not None:
        for i in range(len(mesh_shape)):
            model.mesh_bw[i] = float(mesh_topo.mesh_dim_bandwidth[i])
            model.mesh_lat[i] = float(mesh_topo.mesh_dim_latency[i])
            model.mesh_a2a_bw[i] = 0.0
    kind = torch.tensor([_COLLECTIVES.get(collective, -1)], dtype=torch.int32, device="cuda")
    nb = torch.tensor([int(comm_bytes)], dtype=torch.int64, device="cuda")
    dim = torch.tensor([int(mesh_dim)], dtype=torch.int32, device="cuda")
    out = torch.empty(1, dtype=torch.float64, device="cuda")
    _lib.check(lib.apc_collective_costs(C.byref(model), 1, kind.data_ptr(), nb.data_ptr(), dim.data_ptr(),
                                        out.data_ptr(), None), "apc_collective_costs")
    return float(out.item())


def all_to_all_cost(bytes_gb: float, mesh_topo, mesh_dim: int) -> float:
    shape = tuple(mesh_topo.mesh_dim_devices)
    return collective_comm_cost("all_to_all", int(bytes_gb * 1024**3), shape, mesh_dim, mesh_topo)
