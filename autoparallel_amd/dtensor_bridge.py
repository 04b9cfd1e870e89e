"""Conversions between torch DTensor objects and the packed format."""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch
from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

from .packed import DT_BF16, DT_F16, DT_F32, DT_F64, DT_I8, DT_OTHER, PLC_OTHER, PLC_PARTIAL, PLC_R, PLC_SHARD

_DTYPE_CODES = {
    torch.float64: DT_F64,
    torch.float32: DT_F32,
    torch.float16: DT_F16,
    torch.bfloat16: DT_BF16,
    torch.int8: DT_I8,
}
_REDUCE_OPS = {"sum": 0, "avg": 1, "min": 2, "max": 3, "product": 4}

# placements that are not plain Replicate / Shard / Partial(reduce_op) are
# interned under Python equality, which is what the reference's
# ``current == target`` test uses (collective_runtime_estimation.py:157)
_interned: List[object] = []


def dtype_code(dtype: torch.dtype) -> int:
    return _DTYPE_CODES.get(dtype, DT_OTHER)


def _intern(p) -> int:
    for i, q in enumerate(_interned):
        if type(q) is type(p) and q == p:
            return i
    _interned.append(p)
    assert len(_interned) <= 48, "too many distinct exotic placements"
    return len(_interned) - 1


def placement_code(p) -> int:
    if type(p) is Replicate or (isinstance(p, Replicate) and p.is_replicate()):
        return PLC_R
    if type(p) is Shard:
        return PLC_SHARD | int(p.dim)
    if type(p) is Partial and p.reduce_op in _REDUCE_OPS:
        return PLC_PARTIAL | _REDUCE_OPS[p.reduce_op]
    if p.is_partial():  # MaskPartial, _NormPartial, exotic reduce ops
        return PLC_PARTIAL | (8 + _intern(p))
    if p.is_shard():  # Shard subclasses
        return PLC_SHARD | int(p.dim)
    return PLC_OTHER | _intern(p)  # e.g. _StridedShard: none of the three kinds


def placement_codes(placements: Sequence) -> Tuple[int, ...]:
    return tuple(placement_code(p) for p in placements)


def tensor_meta_key(tm) -> Tuple[Tuple[int, ...], Tuple[int, ...], int, int]:
    return (
        tuple(int(s) for s in tm.shape),
        tuple(int(s) for s in tm.stride),
        int(tm.dtype.itemsize),
        dtype_code(tm.dtype),
    )


def devices_per_host(mesh) -> int:
    """What MeshTopoInfo.build_from_mesh reads
    (torch/distributed/tensor/_collective_utils.py:254)."""
    from torch.distributed.device_mesh import _mesh_resources

    try:
        return int(_mesh_resources.num_devices_per_host(mesh.device_type))
    except Exception:
        return 1
