"""The reference's ``autoparallel.cost_models.compute_estimation`` interface
on top of the HIP engine (autoparallel/cost_models/compute_estimation.py:
258-331, 391-403, 426-493)."""
from __future__ import annotations

import ctypes as C
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from .. import _lib, fx_programs
from ..dtensor_bridge import placement_codes, tensor_meta_key
from ..engine import CostEngine, detect_device_name, make_model
from ..packed import OP_EXPLICIT, OP_PROGRAM, OP_ZERO, GraphBuilder, NodeDesc

_compute_cost_cache: Dict[tuple, float] = {}


def reset_compute_cost_cache() -> None:
    _compute_cost_cache.clear()


def _model(mesh_shape=(1,)):
    from .collective_runtime_estimation import _device_name

    return make_model(tuple(mesh_shape), 1, _device_name())


def compute_read_write_time(read_write_bytes) -> float:
    lib = _lib.load()
    b = torch.tensor([float(read_write_bytes)], dtype=torch.float64, device="cuda")
    out = torch.empty_like(b)
    m = _model()
    _lib.check(lib.apc_rw_times(C.byref(m), 1, b.data_ptr(), out.data_ptr(), None), "apc_rw_times")
    return float(out.item())


def _get_sharded_shape_stride(spec) -> Tuple[List[int], List[int]]:
    lib = _lib.load()
    shape, stride, _, _ = tensor_meta_key(spec.tensor_meta)
    r = len(shape)
    pad = lambda xs, fill: list(xs) + [fill] * (8 - r)
    t_rank = torch.tensor([r], dtype=torch.int32, device="cuda")
    t_shape = torch.tensor([pad(shape, 1)], dtype=torch.int64, device="cuda")
    t_stride = torch.tensor([pad(stride, 0)], dtype=torch.int64, device="cuda")
    codes = list(placement_codes(spec.placements))
    t_plc = torch.tensor([codes + [0] * (4 - len(codes))], dtype=torch.uint8, device="cuda")
    o_shape, o_stride = torch.empty_like(t_shape), torch.empty_like(t_stride)
    m = _model(tuple(spec.mesh.shape))
    _lib.check(lib.apc_local_shapes(C.byref(m), 1, t_rank.data_ptr(), t_shape.data_ptr(), t_stride.data_ptr(),
                                    t_plc.data_ptr(), o_shape.data_ptr(), o_stride.data_ptr(), None),
               "apc_local_shapes")
    return o_shape[0, :r].tolist(), o_stride[0, :r].tolist()


def _has_zero_cost(node) -> bool:
    if node.op != "call_function":
        return True
    if not isinstance(node.target, torch._ops.OpOverload):
        return True
    return bool(node.target.is_view) or node.target is torch.ops.aten._unsafe_view.default


def runtime_cost_vector(node, strategies) -> np.ndarray:
    """estimate_strategy_runtime_cost for every strategy of one node: one
    compute slot evaluated on the device."""
    if _has_zero_cost(node):
        return np.zeros(len(strategies))
    from .collective_runtime_estimation import _device_name, _dph

    mesh = next(s for st in strategies for s in st.input_specs if s is not None).mesh
    b = GraphBuilder(tuple(mesh.shape), _dph(mesh))
    desc = fx_programs.describe_node(node, strategies, b)
    prods = []
    n_args = len(desc.in_specs[0])
    for a in range(n_args):
        col = list(dict.fromkeys(row[a] for row in desc.in_specs if row[a] >= 0))
        if not col:
            prods.append(-1)
            continue
        prods.append(b.add_node(NodeDesc(f"arg{a}", in_specs=[[w] for w in col], out_specs=[[w] for w in col],
                                         inputs=[], default_rows=[[[0.0]] for _ in col])))
    desc.inputs = prods
    desc.default_rows = [[[0.0] * (len(b.nodes[p].in_specs) if p >= 0 else 1) for p in prods] for _ in strategies]
    v = b.add_node(desc)
    b.share_compute_slots = False
    g = b.pack()
    eng = CostEngine(g, device_name=_device_name())
    eng.prepare()
    res = eng.results()
    off = int(g.node_comp_off[v])
    return res["compute"][off : off + len(strategies)].copy()


def estimate_strategy_runtime_cost(node, strategy):
    if _has_zero_cost(node):
        return 0
    if strategy is None:
        raise NotImplementedError("unsharded runtime estimates (strategy=None) are not built")
    key = None
    try:
        key = (node.target, tuple((s.placements, s.tensor_meta) for s in strategy.input_specs),
               fx_programs.non_tensor_args_key(node))
        hash(key)
    except TypeError:
        key = None
    if key is not None and key in _compute_cost_cache:
        return _compute_cost_cache[key]
    cost = float(runtime_cost_vector(node, [strategy])[0])
    if key is not None:
        _compute_cost_cache[key] = cost
    return cost
