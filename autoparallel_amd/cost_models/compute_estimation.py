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


# dtype order of apc_model.tflops (packed.DT_*: float64, float32, float16, bfloat16, int8)
_TFLOPS_DTYPES = (torch.float64, torch.float32, torch.float16, torch.bfloat16, torch.int8)


class DeviceLimit:
    """Bandwidth and GEMM throughput of the current device, as the reference's
    DeviceLimit carries them (compute_estimation.py:47-66), read from the
    engine's device table (apc_device_limits)."""

    def __init__(self, name: str, gmem_bandwidth: float, gemm_tflops: Dict[torch.dtype, float]):
        self.name, self.gmem_bandwidth, self.gemm_tflops = name, gmem_bandwidth, gemm_tflops


def _get_device_limit() -> DeviceLimit:
    """Raises ValueError for a device the table does not know, as the reference
    does (compute_estimation.py:258-275)."""
    from .collective_runtime_estimation import _device_name

    name = _device_name()
    try:
        m = _model()
    except _lib.ApcError as exc:
        raise ValueError(str(exc)) from None
    tf = {dt: float(m.tflops[i]) for i, dt in enumerate(_TFLOPS_DTYPES) if m.tflops[i] > 0.0}
    return DeviceLimit(name, float(m.gmem_bw), tf)


def _get_device_tflops(dtype) -> float:
    limit = _get_device_limit()
    if dtype not in limit.gemm_tflops:
        raise ValueError(f"Dtype {dtype} not supported on {limit.name}. "
                         f"Supported dtypes: {list(limit.gemm_tflops.keys())}")
    return limit.gemm_tflops[dtype]


def _get_device_gmem_bandwidth() -> float:
    return _get_device_limit().gmem_bandwidth


def einsum_flop(equation, tensors, out=None, **kwargs) -> int:
    """Flops of the two einsum forms a linear layer lowers to (reference
    compute_estimation.py:17-44): "{batch}k,kn->{batch}n" and
    "{batch}n,{batch}k->kn", 2 * batch * n * k each.  The device evaluates the
    same products from opprog.einsum_fwd / einsum_bwd."""
    assert len(tensors) == 2
    a, b = (tuple(t.shape) for t in tensors)
    batch = 1
    for d in a[:-1]:
        batch *= d
    if len(b) == 2 and len(a) >= 3:
        assert a[-1] == b[0], f"Contracting dim mismatch: {a[-1]} vs {b[0]}"
        return batch * b[1] * a[-1] * 2
    if len(a) == len(b) and len(a) >= 3:
        assert a[:-1] == b[:-1], f"Batch dims mismatch: {a[:-1]} vs {b[:-1]}"
        return batch * a[-1] * b[-1] * 2
    raise NotImplementedError(f"Unsupported einsum shapes: {a} {b}")


def compute_memory_cost(op, args, outs) -> int:
    """Bytes read plus bytes written by an op (reference compute_estimation.py:321-331)."""
    from torch.utils._pytree import tree_flatten

    def nbytes(data):
        return sum(x.numel() * x.element_size() for x in tree_flatten(data)[0] if isinstance(x, torch.Tensor))

    return nbytes(args) + nbytes(outs)


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


def _unsharded_strategy(node):
    """Stand-in strategy for an operator evaluated on its traced arguments:
    Replicate on a mesh of one device (the local shape is the traced shape)."""
    from types import SimpleNamespace

    from torch.distributed.tensor._dtensor_spec import TensorMeta
    from torch.distributed.tensor.placement_types import Replicate
    from torch.utils._pytree import tree_flatten

    one = SimpleNamespace(shape=(1,), ndim=1)
    spec = lambda t: SimpleNamespace(mesh=one, placements=(Replicate(),),
                                     tensor_meta=TensorMeta(t.shape, t.stride(), t.dtype))
    ins = [spec(a.meta["val"]) for a in tree_flatten(node.args)[0]
           if isinstance(a, torch.fx.Node) and isinstance(a.meta.get("val"), torch.Tensor)]
    val = node.meta.get("val")
    if isinstance(val, torch.Tensor):
        outs = spec(val)
    else:
        outs = tuple(spec(v) if isinstance(v, torch.Tensor) else None for v in val)
    return SimpleNamespace(input_specs=ins, output_specs=outs)


def runtime_cost_vector(node, strategies) -> np.ndarray:
    """estimate_strategy_runtime_cost for every strategy of one node: one
    compute slot evaluated on the device."""
    if _has_zero_cost(node):
        return np.zeros(len(strategies))
    from .collective_runtime_estimation import _device_name, _dph

    mesh = next((s for st in strategies for s in st.input_specs if s is not None), None)
    if mesh is None:  # no tensor argument: a factory, priced on its output alone
        mesh = next(s for s in (lambda o: o if isinstance(o, (tuple, list)) else (o,))(strategies[0].output_specs)
                    if s is not None)
    mesh = mesh.mesh
    b = GraphBuilder(tuple(mesh.shape), _dph(mesh) if hasattr(mesh, "device_type") else 1)
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
        # the operator on its arguments as traced, no sharding
        # (compute_estimation.py:334-339): every tensor argument whole on one device
        return float(runtime_cost_vector(node, [_unsharded_strategy(node)])[0])
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


def benchmark_fn(fn, *args, **kwargs) -> float:
    """Mean time of ``fn(*args, **kwargs)`` on the current stream in
    microseconds: 3 untimed calls, then 10 between two events
    (compute_estimation.py:513-529)."""
    for _ in range(3):
        fn(*args, **kwargs)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(10):
        fn(*args, **kwargs)
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / 10 * 1e3


def _shard_args_for_node(node, strategy=None, rand_init: bool = False):
    """(args, kwargs) of the node with every tensor argument at the size and
    stride the strategy leaves on one device (the traced ones without a
    strategy); real random ones on the device with
    ``rand_init`` (compute_estimation.py:334-365).  Without it the tensors are on
    the meta device."""
    from torch.utils._pytree import tree_flatten, tree_map_only

    args = tree_map_only(torch.fx.Node, lambda x: x.meta["val"], node.args)
    kwargs = tree_map_only(torch.fx.Node, lambda x: x.meta["val"], node.kwargs)
    assert not any(isinstance(v, torch.Tensor) for v in kwargs.values()), f"{node}: tensors are expected in args"
    flat, spec = tree_flatten(args)
    specs = iter(strategy.input_specs if strategy is not None else ())
    out = []
    for x in flat:
        if isinstance(x, torch.Tensor):
            sizes, strides = (list(x.shape), list(x.stride())) if strategy is None else _get_sharded_shape_stride(next(specs))
            if rand_init:
                t = torch.empty_strided(sizes, strides, dtype=x.dtype, device="cuda")
                x = t.normal_() if t.dtype.is_floating_point else t.random_(0, 256)
            else:
                x = torch.empty_strided(sizes, strides, dtype=x.dtype, device="meta")  # sizes are all the counters need
        out.append(x)
    return spec.unflatten(out), kwargs


def _compute_flops(fn, *args, **kwargs):
    """(flops torch counts for fn on these arguments, its output) (:383-388)."""
    from torch.utils.flop_counter import FlopCounterMode

    with FlopCounterMode(display=False) as counter:
        out = fn(*args, **kwargs)
    return counter.get_total_flops(), out


def compare_estimated_with_benchmarked_throughput(graph, sharding_placement, tgt_ops="mm"):
    """For the chosen strategy of every node of the target operators: measured
    time, estimated time, achieved TFLOP/s, the device's figure and their ratio
    (:532-556)."""
    if tgt_ops == "mm":
        tgt_ops = [torch.ops.aten.mm.default, torch.ops.aten.bmm.default]
    data = {}
    for node in graph.nodes:
        if node.op != "call_function" or (tgt_ops is not None and node.target not in tgt_ops):
            continue
        strategy = sharding_placement[node]
        args, kwargs = _shard_args_for_node(node, strategy)
        flops = _compute_flops(node.target, *args, **kwargs)[0]
        real_us = benchmark_strategy_runtime_cost(node, strategy)
        throughput = flops / (real_us / 1e6) * 1e-12
        peak = _get_device_tflops(strategy.input_specs[0].tensor_meta.dtype)
        data[node] = (real_us, estimate_strategy_runtime_cost(node, strategy), throughput, peak, throughput / peak)
    return data


def benchmark_strategy_runtime_cost(node, strategy) -> float:
    """The measured counterpart of estimate_strategy_runtime_cost, for checking
    the model against the device: the operator is run on random tensors of the
    sizes the strategy leaves on one device (compute_estimation.py:496-510)."""
    if _has_zero_cost(node):
        return 0
    from torch._subclasses.fake_tensor import unset_fake_temporarily

    with unset_fake_temporarily():
        args, kwargs = _shard_args_for_node(node, strategy, rand_init=True)
        return benchmark_fn(node.target, *args, **kwargs)
