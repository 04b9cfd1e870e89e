"""CPU oracle for the NCCL-tuning collective cost model.  TEST INFRASTRUCTURE ONLY.

Nothing under ``autoparallel_amd/`` may import this module.

Per-call restatement, on Python ints and floats, of
``autoparallel/cost_models/nccl_cost_model.py``:

  derive_dim_topo             :1001-1021   (derive_mesh_dim_topo)
  algo_bw                     :323-465     (_compute_algo_bw)
  algo_latency                :473-551     (_compute_algo_latency)
  algo_time                   :559-613     (_nccl_algo_time)
  eligible_algos / protos     :616-649
  interp_correction           :294-315
  depth_scaled_ring_table     :700-719
  interp_clamped              :980-992
  table_algo_time             :1024-1075
  table_collective_time       :1081-1160
  collective_time             :1163-1212   (nccl_collective_time)
  all_to_all_time             :1215-1313   (nccl_all_to_all_cost)
  comm_cost                   collective_runtime_estimation.py:44-62 (_nccl_comm_cost)

Codes: func 0 allgather, 1 reduce_scatter, 2 allreduce; algo 0 tree, 1 ring,
2 collnet-direct, 3 collnet-chain, 4 nvls, 5 nvls-tree; proto 0 LL, 1 LL128,
2 Simple; arch 0 Ampere, 1 Hopper, 2 Blackwell.  The numeric tables are the
model's data (NCCL tuning constants and the reference's fitted corrections).

Pinning: golden vectors written by tests/golden/make_nccl_vectors.py from the
reference's module (stdlib-only, loaded by file path), and the closed-form
known answers of the reference's tests/test_nccl_cost_model.py restated in
tests/test_oracle_nccl.py.
"""
from __future__ import annotations

import functools
import math
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

INF = float("inf")

AG, RS, AR = 0, 1, 2
TREE, RING, COLLNET_DIRECT, COLLNET_CHAIN, NVLS, NVLS_TREE = range(6)
LL, LL128, SIMPLE = 0, 1, 2
AMPERE, HOPPER, BLACKWELL = 0, 1, 2

DEFAULT_CHANNELS = (12, 16, 16)

#                 tree              ring              cdirect          cchain           nvls             nvls-tree
BASE_LAT = ((6.8, 14.0, 8.4), (6.6, 14.0, 8.4), (0.0, 0.0, 0.0), (0.0, 0.0, 0.0), (0.0, 0.0, 0.0), (0.0, 0.0, 0.0))
HW_LAT_NVLINK = ((0.6, 1.25, 4.0), (0.6, 1.9, 3.4), (0.0, 0.0, 3.7), (0.0, 0.0, 2.8), (0.0, 0.0, 25.0), (0.0, 0.0, 25.0))
HW_LAT_NET = ((5.0, 8.5, 14.0), (2.7, 4.0, 14.0), (0.0, 0.0, 31.0), (0.0, 0.0, 30.0), (0.0, 0.0, 18.0), (0.0, 0.0, 20.9))

# [arch][node bucket]
MAX_TREE_BW = ((24.0, 23.6, 17.8), (38.7, 41.4, 36.0), (70.0, 42.8, 24.0))
MAX_NVLS_TREE_BW = ((24.0, 23.6, 17.8), (0.0, 57.7, 45.5), (0.0, 96.0, 43.8))
LL_MAX_BW = ((87.7, 39.0, 20.4), (141.0, 39.0, 20.4), (282.0, 39.0, 20.4))
MAX_RING_LL128_BW = ((20.0, 20.0, 20.0), (36.7, 36.7, 36.7), (40.0, 40.0, 40.0))
MAX_TREE_LL128_BW = ((20.0, 20.0, 20.0), (36.7, 36.7, 29.0), (55.6, 31.67, 20.0))
NVLS_EFF = (0.0, 0.85, 0.74)

TREE_CORR = (
    (1.0, 1.0, 1.0, 1.0, 0.9, 0.8, 0.7, 0.7, 0.7, 0.7, 0.6, 0.5, 0.4, 0.4, 0.5, 0.6, 0.7, 0.8, 0.9, 1.0, 1.0, 1.0, 1.0, 1.0),
    (1.0, 1.0, 1.0, 1.0, 1.0, 0.9, 0.8, 0.8, 0.8, 0.7, 0.6, 0.6, 0.6, 0.6, 0.6, 0.6, 0.8, 0.9, 0.9, 0.9, 0.9, 1.0, 1.0, 1.0),
    (0.9, 0.9, 0.9, 0.9, 0.9, 0.9, 0.9, 0.8, 0.7, 0.6, 0.6, 0.5, 0.5, 0.5, 0.5, 0.6, 0.7, 0.8, 0.7, 0.7, 0.8, 0.9, 0.9, 0.9),
)
RING_CORR = (1.0,) * 11 + (0.10, 0.18, 0.30, 0.43, 0.63, 0.55, 0.78, 0.93) + (1.0,) * 5
NVLS_TREE_RAMP = (1.0,) * 8 + (0.10, 0.10, 0.15, 0.28, 0.41, 0.55, 0.72, 0.88) + (1.0,) * 8
FULL_MESH_RING_RAMP = (0.01, 0.02, 0.03, 0.06, 0.10, 0.16, 0.25, 0.36) + (0.68,) * 10 + (0.79,) + (0.87,) * 5
A2A_NIC_RAMP = (1.0,) * 8 + (0.28, 0.28, 0.35, 0.43, 0.62, 0.71, 0.82, 0.89, 0.92, 0.95) + (1.0,) * 6
assert len(RING_CORR) == len(NVLS_TREE_RAMP) == len(FULL_MESH_RING_RAMP) == len(A2A_NIC_RAMP) == 24

NET_OVERHEAD = 1.0
RING_SYNC_PER_NODE = 4.7
BLACKWELL_BW_SCALE = 640.0 / 320.0
A2A_CE_BW = {HOPPER: 380.0, BLACKWELL: 675.0}
A2A_CE_LAT = 50.0
A2A_SM_BW_CORR = 0.7
A2A_NIC_OVERHEAD = 0.44
A2A_MULTI_NODE_LAT = ((2, 37.0), (4, 42.0), (8, 60.0), (16, 98.0), (32, 290.0))

# intra-node NVSwitch measurements, (ranks, value): [func]
NVSWITCH_BW = (((2, 537.0), (4, 434.0), (8, 394.0)),) * 2 + (((2, 324.0), (4, 236.0), (8, 267.0)),)
NVSWITCH_LAT = (((2, 8.0), (4, 17.0), (8, 30.0)),) * 2 + (((2, 10.0), (4, 15.0), (8, 31.0)),)

# multi-node H100 NVSwitch tuning tables: rows for nodes in (2,4,8,16,32) x ppn
# in (1,2,4,8), each ((lat, bw) LL, LL128, Simple)
_NODES = (2, 4, 8, 16, 32)
_PPN = (1, 2, 4, 8)
_AGRS_RING = (
    ((11.6, 48.0), (22.5, 88.3), (22.4, 96.0)), ((11.3, 52.0), (21.8, 117.8), (29.2, 128.0)),
    ((15.3, 44.6), (29.4, 201.9), (42.8, 219.4)), ((23.3, 41.6), (44.6, 313.2), (70.0, 409.6)),
    ((21.6, 27.2), (39.5, 58.9), (50.4, 64.0)), ((18.7, 23.3), (33.6, 100.9), (64.0, 109.7)),
    ((26.7, 21.8), (48.8, 188.4), (91.2, 204.8)), ((42.7, 21.1), (79.2, 303.1), (145.6, 396.4)),
    ((41.6, 23.3), (73.5, 50.5), (106.4, 54.9)), ((33.5, 21.8), (57.2, 94.2), (133.6, 102.4)),
    ((49.5, 21.1), (87.6, 182.3), (188.0, 198.2)), ((81.5, 20.7), (148.4, 298.3), (296.8, 390.1)),
    ((81.6, 21.8), (141.5, 47.1), (218.4, 51.2)), ((63.1, 21.1), (104.4, 91.2), (272.8, 99.1)),
    ((95.1, 20.7), (165.2, 179.4), (381.6, 195.0)), ((159.1, 20.6), (286.8, 295.9), (599.2, 387.0)),
    ((161.6, 21.1), (277.5, 45.6), (442.4, 49.5)), ((122.3, 20.7), (198.8, 89.7), (551.2, 97.5)),
    ((186.3, 20.6), (320.4, 178.0), (768.8, 193.5)), ((314.3, 20.5), (563.6, 294.8), (1204.0, 385.5)),
)
_AR_TREE = (
    ((16.8, 9.3), (31.0, 31.2), (36.4, 35.2)), ((18.0, 16.6), (33.5, 62.4), (44.4, 70.4)),
    ((20.4, 16.6), (38.5, 124.8), (60.4, 140.8)), ((25.2, 16.6), (48.5, 124.8), (92.4, 140.8)),
    ((26.8, 4.9), (48.0, 17.6), (64.4, 18.8)), ((28.0, 8.7), (50.5, 35.2), (72.4, 37.5)),
    ((30.4, 8.7), (55.5, 70.4), (88.4, 75.1)), ((35.2, 8.7), (65.5, 98.6), (120.4, 122.4)),
    ((36.8, 4.9), (65.0, 17.6), (92.4, 18.8)), ((38.0, 8.7), (67.5, 35.2), (100.4, 37.5)),
    ((40.4, 8.7), (72.5, 70.4), (116.4, 75.1)), ((45.2, 8.7), (82.5, 98.6), (148.4, 122.4)),
    ((46.8, 4.9), (82.0, 17.6), (120.4, 18.8)), ((48.0, 8.7), (84.5, 35.2), (128.4, 37.5)),
    ((50.4, 8.7), (89.5, 70.4), (144.4, 75.1)), ((55.2, 8.7), (99.5, 98.6), (176.4, 122.4)),
    ((56.8, 4.9), (99.0, 17.6), (148.4, 18.8)), ((58.0, 8.7), (101.5, 35.2), (156.4, 37.5)),
    ((60.4, 8.7), (106.5, 70.4), (172.4, 75.1)), ((65.2, 8.7), (116.5, 98.6), (204.4, 122.4)),
)
# nvls-tree (Simple only), ppn 4 and 8 per node count: (lat, bw)
_AR_NVLS_TREE = {
    (2, 4): (53.0, 160.0), (2, 8): (53.0, 266.7), (4, 4): (81.0, 80.0), (4, 8): (81.0, 160.0),
    (8, 4): (109.0, 80.0), (8, 8): (109.0, 160.0), (16, 4): (137.0, 80.0), (16, 8): (137.0, 160.0),
    (32, 4): (165.0, 80.0), (32, 8): (165.0, 160.0),
}


def _row(table, n_nodes: int, ppn: int):
    if n_nodes in _NODES and ppn in _PPN:
        return table[_NODES.index(n_nodes) * 4 + _PPN.index(ppn)]
    return None


@dataclass
class NcclConfig:
    arch: int
    num_nodes: int
    gpus_per_node: int
    bw_intra: float
    bw_inter: float
    num_channels: Optional[int] = None
    has_nvswitch: bool = False
    has_collnet: bool = False
    net_latency: float = 0.0


@dataclass
class DimTopo:
    n_ranks: int
    n_nodes: int
    ppn: int
    bw_intra: float
    bw_inter: float
    n_channels: int


def a100_config(num_nodes=1, gpus_per_node=8, bw_inter=25.0, **kw) -> NcclConfig:
    return NcclConfig(AMPERE, num_nodes, gpus_per_node, 87.7, bw_inter, **kw)


def h100_config(num_nodes=1, gpus_per_node=8, bw_inter=50.0, has_nvswitch=True, **kw) -> NcclConfig:
    return NcclConfig(HOPPER, num_nodes, gpus_per_node, 320.0, bw_inter, has_nvswitch=has_nvswitch, **kw)


def gb200_config(num_nodes=1, gpus_per_node=72, bw_inter=50.0, has_nvswitch=True, **kw) -> NcclConfig:
    return NcclConfig(BLACKWELL, num_nodes, gpus_per_node, 640.0, bw_inter, has_nvswitch=has_nvswitch, **kw)


def node_bucket(n_nodes: int) -> int:
    return 0 if n_nodes <= 1 else (1 if n_nodes <= 2 else 2)


def log2i(n: int) -> int:
    return 0 if n <= 0 else n.bit_length() - 1


def derive_dim_topo(cfg: NcclConfig, mesh_shape: Sequence[int], dim: int) -> DimTopo:
    size = mesh_shape[dim]
    inner = math.prod(mesh_shape[dim + 1:])
    ppn = max(1, min(cfg.gpus_per_node // inner, size))
    nch = cfg.num_channels if cfg.num_channels is not None else DEFAULT_CHANNELS[cfg.arch]
    return DimTopo(size, size // ppn, ppn, cfg.bw_intra / nch, cfg.bw_inter / nch, nch)


def interp_correction(table: Sequence[float], n_bytes: int, shift: int = 6) -> float:
    shifted = n_bytes >> shift
    if shifted <= 0:
        return table[0]
    lv = math.log2(shifted)
    lo = int(lv)
    hi = lo + 1
    if hi >= len(table) or lo >= len(table):
        return table[-1]
    frac = lv - lo
    return table[lo] * (1 - frac) + table[hi] * frac


@functools.lru_cache(maxsize=None)
def depth_scaled_ring_table(n_nodes: int) -> Tuple[float, ...]:
    e = 1.0 + 0.2 * (log2i(n_nodes) - 2)
    out: List[float] = []
    for i, c in enumerate(RING_CORR):
        if c < 1.0:
            c = c ** e
        if i > 0:
            c = min(c, 2.0 * out[i - 1])
        out.append(c)
    return tuple(out)


def interp_clamped(points, x: int) -> float:
    if x <= points[0][0]:
        return points[0][1]
    if x >= points[-1][0]:
        return points[-1][1]
    for (x0, y0), (x1, y1) in zip(points, points[1:]):
        if x <= x1:
            t = (x - x0) / (x1 - x0)
            return y0 + t * (y1 - y0)
    return points[-1][1]


def algo_bw(func: int, algo: int, proto: int, t: DimTopo, cfg: NcclConfig) -> float:
    nsteps = 2 * (t.n_ranks - 1) if func == AR else t.n_ranks - 1
    nb = node_bucket(t.n_nodes)
    nch, ppn = t.n_channels, t.ppn
    if proto != SIMPLE and algo in (NVLS, NVLS_TREE, COLLNET_DIRECT, COLLNET_CHAIN):
        return 0.0
    if cfg.has_nvswitch and t.n_nodes > 1:
        inter_agg = min(t.bw_intra, t.bw_inter * ppn)
    else:
        inter_agg = t.bw_inter
    link = t.bw_intra if t.n_nodes <= 2 else inter_agg

    if algo == RING:
        bus = nch * link
    elif algo == TREE:
        if func != AR:
            return 0.0
        bus = nch * link
    elif algo == NVLS:
        if nch < 2:
            return 0.0
        if func in (AG, RS) and t.n_nodes > 1 and not cfg.has_collnet:
            return 0.0
        intra = t.bw_intra * NVLS_EFF[cfg.arch] * (nch - 1) / nch
        if func == AR:
            intra *= 2.0
        else:
            intra *= (ppn - 1) / ppn
        bus = nch * (min(intra, t.bw_inter) if t.n_nodes > 1 else intra)
    elif algo == NVLS_TREE:
        if func != AR:
            return 0.0
        if nch < 2:
            return 0.0
        intra = t.bw_intra * NVLS_EFF[cfg.arch] * (nch - 1) / nch
        intra *= 2.0
        inter = inter_agg * (2 if t.n_nodes <= 2 else 1)
        bus = nch * min(intra, inter, MAX_NVLS_TREE_BW[cfg.arch][nb])
    elif algo == COLLNET_DIRECT:
        if func in (AG, RS):
            return ppn * min(t.bw_intra * nch, t.bw_inter * nch * 0.9)
        bus = nch * link
        factor = ppn / nch
        factor -= (factor - 1) / 2
        bus /= factor
        if cfg.arch in (HOPPER, BLACKWELL):
            bus *= 0.85
    elif algo == COLLNET_CHAIN:
        if func != AR:
            return 0.0
        bus = nch * link
    else:
        return 0.0

    ll_max = LL_MAX_BW[cfg.arch][nb]
    if algo == RING and proto == LL:
        bus = min(ll_max, bus * 0.5)
    if algo == RING and proto == LL128:
        bus = min(bus * 0.92, nch * MAX_RING_LL128_BW[cfg.arch][nb])
    if algo == TREE and func == AR:
        bus = min(bus * 0.92, nch * MAX_TREE_BW[cfg.arch][nb])
    if algo == TREE and proto == LL:
        bus = min(bus / 3.8, ll_max)
    if algo == TREE and proto == LL128:
        bus = min(bus * (7.0 / 9.0 if t.n_nodes == 1 else 120.0 / 128.0), nch * MAX_TREE_LL128_BW[cfg.arch][nb])

    if algo == RING or func not in (AG, RS):
        if algo in (RING, NVLS, NVLS_TREE):
            bus *= t.n_ranks / nsteps
        else:
            bus *= 0.5
    return bus


def algo_latency(func: int, algo: int, proto: int, t: DimTopo, cfg: NcclConfig) -> float:
    base = BASE_LAT[algo][proto]
    intra = HW_LAT_NVLINK[algo][proto]
    inter = HW_LAT_NET[TREE if t.ppn == 1 else algo][proto] + cfg.net_latency
    if proto == SIMPLE:
        inter += cfg.net_latency
    nsteps = 2 * (t.n_ranks - 1) if func == AR else t.n_ranks - 1
    if algo == RING:
        if t.n_nodes > 1:
            overhead = NET_OVERHEAD
            if proto == SIMPLE:
                overhead *= 3
        else:
            overhead = 0.0
        intra = max(intra, overhead)
        if t.n_nodes == 1:
            n_inter = 0
        elif func == AR:
            n_inter = 2 * (t.n_nodes - 1)
        else:
            n_inter = t.n_nodes - 1
        lat = base + (nsteps - n_inter) * intra + n_inter * inter
        if t.n_nodes > 1:
            sync = RING_SYNC_PER_NODE * t.n_nodes
            if t.n_nodes > 4:
                sync *= (t.n_nodes / 4) ** 0.65
            lat += sync
        return lat
    if algo == TREE:
        return base + 2 * ((t.n_ranks // t.n_nodes - 1) * intra + log2i(t.n_nodes) * inter)
    if algo == COLLNET_DIRECT:
        return base + 2 * (min(1, t.ppn - 1) * intra + (t.ppn - 1) * 0.4) + inter
    if algo == COLLNET_CHAIN:
        return base + 2 * (t.ppn - 1) * intra + inter
    if algo == NVLS:
        return intra + (inter if t.n_nodes > 1 else 0.0)
    if algo == NVLS_TREE:
        return base + intra + 2 * log2i(t.n_nodes) * inter
    return 0.0


def algo_time(func: int, algo: int, proto: int, n_bytes: int, t: DimTopo, cfg: NcclConfig) -> float:
    bw = algo_bw(func, algo, proto, t, cfg)
    lat = algo_latency(func, algo, proto, t, cfg)
    if bw <= 0:
        return INF
    ls = log2i(n_bytes >> 6)
    if algo == TREE and func == AR and 0 <= ls < 23:
        bw *= TREE_CORR[proto][ls]
    if algo == NVLS_TREE and func == AR and cfg.arch == BLACKWELL and 0 <= ls < 24:
        bw *= TREE_CORR[proto][ls]
    if algo == RING and t.n_nodes > 1:
        table = depth_scaled_ring_table(t.n_nodes) if t.n_nodes > 4 else RING_CORR
        bw *= interp_correction(table, n_bytes // t.n_ranks)
    if algo == RING and proto == SIMPLE and t.n_nodes > 1 and func == AR and n_bytes / (t.n_channels * t.n_ranks) >= 64:
        lat *= 1.4
    return lat + n_bytes / (1000.0 * bw)


def eligible_algos(func: int, cfg: NcclConfig, n_nodes: int) -> List[int]:
    hopper_switch = cfg.has_nvswitch and cfg.arch in (HOPPER, BLACKWELL)
    if func in (AG, RS):
        out = [RING]
        if hopper_switch:
            out.append(NVLS)
        if cfg.has_collnet:
            out.append(COLLNET_DIRECT)
        return out
    out = [RING, TREE]
    if cfg.has_collnet:
        out += [COLLNET_DIRECT, COLLNET_CHAIN]
    if hopper_switch:
        out.append(NVLS)
        if n_nodes > 1:
            out.append(NVLS_TREE)
    return out


def eligible_protos(algo: int) -> List[int]:
    return [LL, LL128, SIMPLE] if algo in (TREE, RING) else [SIMPLE]


def table_algo_time(algo, proto, lat, bw, func, n_bytes, t: DimTopo, full_mesh=False) -> float:
    if algo == TREE and func == AR:
        ls = log2i(n_bytes >> 6)
        if 0 <= ls < 23:
            bw *= TREE_CORR[proto][ls]
    if algo == NVLS_TREE:
        bw *= interp_correction(NVLS_TREE_RAMP, n_bytes // t.n_ranks)
    if algo == RING and t.n_nodes > 1 and full_mesh:
        per_gpu = n_bytes // t.n_ranks
        lg = log2i(per_gpu >> 6)
        if 0 <= lg < len(FULL_MESH_RING_RAMP):
            bw *= interp_correction(FULL_MESH_RING_RAMP, per_gpu)
        elif lg < 0:
            bw *= FULL_MESH_RING_RAMP[0]
    if algo == RING and proto == SIMPLE and func == AR and n_bytes / (t.n_channels * t.n_ranks) >= 64:
        lat *= 1.4
    if bw <= 0:
        return INF
    return lat + n_bytes / (1000.0 * bw)


def table_collective_time(func: int, n_bytes: int, t: DimTopo, cfg: NcclConfig) -> Optional[float]:
    scale = BLACKWELL_BW_SCALE if cfg.arch == BLACKWELL else 1.0
    full_mesh = t.ppn == cfg.gpus_per_node
    best = INF
    if func in (AG, RS):
        row = _row(_AGRS_RING, t.n_nodes, t.ppn)
        if row is None:
            return None
        for p in (LL, LL128, SIMPLE):
            lat, bw = row[p]
            best = min(best, table_algo_time(RING, p, lat, bw * scale, func, n_bytes, t, full_mesh))
        return best
    found = False
    row = _row(_AR_TREE, t.n_nodes, t.ppn)
    if row is not None:
        found = True
        for p in (LL, LL128, SIMPLE):
            lat, bw = row[p]
            best = min(best, table_algo_time(TREE, p, lat, bw * scale, func, n_bytes, t))
    nv = _AR_NVLS_TREE.get((t.n_nodes, t.ppn))
    if nv is not None:
        found = True
        best = min(best, table_algo_time(NVLS_TREE, SIMPLE, nv[0], nv[1] * scale, func, n_bytes, t))
    return best if found else None


def collective_time(func: int, n_bytes: int, t: DimTopo, cfg: NcclConfig) -> float:
    switch = cfg.arch in (HOPPER, BLACKWELL) and cfg.has_nvswitch
    if switch and t.n_nodes == 1:
        bw = interp_clamped(NVSWITCH_BW[func], t.n_ranks)
        if cfg.arch == BLACKWELL:
            bw *= BLACKWELL_BW_SCALE
        lat = interp_clamped(NVSWITCH_LAT[func], t.n_ranks)
        return lat + n_bytes / (1000.0 * bw)
    if switch and t.n_nodes > 1:
        r = table_collective_time(func, n_bytes, t, cfg)
        if r is not None:
            if func in (AG, RS):
                return r
            best = r
            for p in eligible_protos(RING):
                best = min(best, algo_time(func, RING, p, n_bytes, t, cfg))
            return best
    best = INF
    for a in eligible_algos(func, cfg, t.n_nodes):
        for p in eligible_protos(a):
            v = algo_time(func, a, p, n_bytes, t, cfg)
            if v < best:
                best = v
    return best


def all_to_all_time(n_bytes: int, t: DimTopo, cfg: NcclConfig) -> float:
    if cfg.arch in (HOPPER, BLACKWELL) and cfg.has_nvswitch and t.n_nodes == 1:
        return A2A_CE_LAT + n_bytes / (1000.0 * A2A_CE_BW[cfg.arch])
    if t.n_nodes > 1 and cfg.has_nvswitch:
        lat = interp_clamped(A2A_MULTI_NODE_LAT, t.n_nodes)
        remote = (t.n_ranks - t.ppn) / t.n_ranks
        nic = cfg.bw_inter * (1.0 - A2A_NIC_OVERHEAD / t.n_nodes)
        if nic <= 0:
            return INF
        lg = log2i((n_bytes // t.n_ranks) >> 6)
        if 0 <= lg < 24:
            corr = A2A_NIC_RAMP[lg]
        elif lg < 0:
            corr = A2A_NIC_RAMP[0]
        else:
            corr = 1.0
        ln = log2i(t.n_nodes)
        if ln > 1 and corr < 1.0:
            corr = 1.0 - (1.0 - corr) / ln
        if corr <= 0:
            return INF
        return lat + n_bytes * remote / (1000.0 * nic * corr)
    bw = t.bw_intra if t.n_nodes <= 2 else t.bw_inter
    bus = t.n_channels * bw * A2A_SM_BW_CORR
    if bus <= 0:
        return INF
    base = BASE_LAT[RING][SIMPLE]
    intra = HW_LAT_NVLINK[RING][SIMPLE]
    inter = HW_LAT_NET[TREE if t.ppn == 1 else RING][SIMPLE] + cfg.net_latency
    inter += cfg.net_latency
    overhead = NET_OVERHEAD * 3 if t.n_nodes > 1 else 0.0
    intra = max(intra, overhead)
    n_inter = 0 if t.n_nodes == 1 else t.n_nodes - 1
    lat = base + (t.n_ranks - n_inter) * intra + n_inter * inter
    return lat + n_bytes / (1000.0 * bus)


def comm_cost(collective: str, n_bytes: int, mesh_shape: Sequence[int], dim: int, cfg: NcclConfig) -> float:
    t = derive_dim_topo(cfg, tuple(mesh_shape), dim)
    if collective == "allgather":
        return collective_time(AG, n_bytes, t, cfg)
    if collective == "allreduce":
        return collective_time(AR, n_bytes, t, cfg)
    if collective == "reduce_scatter":
        return collective_time(RS, n_bytes, t, cfg)
    if collective == "all_to_all":
        return all_to_all_time(n_bytes, t, cfg)
    return 0.0
