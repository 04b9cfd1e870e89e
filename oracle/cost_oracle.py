"""CPU oracle for the sharding-search cost engine.  TEST INFRASTRUCTURE ONLY.

Nothing under ``autoparallel_amd/`` may import this module: it is the checker
for the HIP path (tests, the smoke check, and the ``cpu_baseline`` leg of the
benchmark), never the thing shipped or measured as the product.

It restates, per entry and in the reference's evaluation order, on plain
Python ints and floats (IEEE binary64, no fused operations):

  topology            torch/distributed/tensor/_collective_utils.py:246-278
  allgather/allreduce/reduce_scatter cost            same file :281-313
  all_to_all_cost     autoparallel/cost_models/collective_runtime_estimation.py:100-110
  redistribute_cost   autoparallel/cost_models/collective_runtime_estimation.py:115-229
  estimate_strategy_comms_cost (order rule + memo)   same file :239-262
  contiguity          torch/_prims_common/__init__.py:252-293
  compute_read_write_time   autoparallel/cost_models/compute_estimation.py:391-403
  _get_sharded_shape_stride                          same file :300-318
  estimate_strategy_runtime_cost (roofline part)     same file :438-493
  remove_invalid_configs / _create_all_options
                      autoparallel/shardings/propagation_rules.py:127-201
  _build_decision_vars / _compute_edge_costs
                      autoparallel/optimize_sharding.py:446-552
  add_inf_cost_constraint / _set_objective / apply_prefetch_discount
                      autoparallel/optimize_sharding.py:803-885
  _compute_solution_cost                              same file :1056-1111
  NCCL collective model (selected by Topo.nccl)       oracle/nccl_oracle.py

Pinning (what each function is checked against, see tests/test_oracle_*.py):
  * redistribute_cost, estimate_strategy_comms_cost, compute_read_write_time,
    _get_sharded_shape_stride: golden vectors written by
    tests/golden/make_cost_vectors.py from the reference's own functions, plus
    hand-derived closed forms and invariants.
  * collectives / topology: closed forms evaluated independently with
    ``fractions.Fraction`` and the installed torch functions.
  * flop programs: ``torch.utils.flop_counter.FlopCounterMode`` on meta tensors.
  * decision-var assembly, scorer: algebraic identities and the reference
    tests' mock DecisionVar sums (tests/test_log_formatting.py:57-148 there).
  * sample_feasible: no counterpart in the reference (which has no sampler); it
    restates this library's own definition, and is pinned by what that definition
    implies: no forbidden variable selected unless a node is counted as a
    fallback, every allowed strategy of a node reached, and the frequencies of a
    node's choices flat over many assignments (tests/test_oracle_closed_forms.py).
"""
from __future__ import annotations

import itertools
import math
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

# placement byte encoding (same as the packed format)
PLC_R = 0x00
PLC_SHARD = 0x40
PLC_PARTIAL = 0x80
KIND = 0xC0
ARG = 0x3F
PARTIAL_SUM = 0x80

INF = float("inf")

# MI355X row of the reference's device table (compute_estimation.py:226-239)
MI355X_GMEM_BW = 8.0 * (1024**4)
# dtype code -> TFLOPS   (codes: 0 f64, 1 f32, 2 f16, 3 bf16, 4 int8)
MI355X_TFLOPS = {0: 78.6, 1: 157.3, 2: 2516.6, 3: 2516.6, 4: 5033.2}


# The whole table (compute_estimation.py:66-255), in its order: name ->
# (bytes/s, {dtype code: TFLOPS}); the halves are integer halves there.  Pinned row by
# row, with the substring matching and its order, by tests/golden/device_table_vectors.json:
# what the reference's own lookups answer for 38 device names (tests/test_device_table_golden.py).
DEVICE_TABLE = (
    ("H100", 3.35 * (1024**4), {0: 67, 1: 989 // 2, 2: 1979 // 2, 3: 1979 // 2, 4: 3958 // 2}),
    ("B200", 7.7 * (1024**4), {0: 37, 1: 2200 // 2, 2: 4500 // 2, 3: 4500 // 2, 4: 9000 // 2}),
    ("A100", 2 * (1024**4), {0: 19.5, 1: 156, 2: 312, 3: 312, 4: 624}),
    ("A30", 933 * (1024**3), {0: 10.3, 1: 82, 2: 165, 3: 165, 4: 330}),
    ("A10G", 933 * (1024**3), {1: 31.2, 2: 125, 3: 125, 4: 250}),
    ("T4", 300 * (1024**3), {1: 8.1, 2: 65, 4: 130}),
    ("V100", 900 * (1024**3), {0: 7.8, 1: 15.7, 2: 125}),
    ("P100", 732 * (1024**3), {0: 5.3, 1: 10.6, 2: 21.2}),
    ("AMD Instinct MI200X", 1.6 * (1024**4), {0: 45.3, 1: 45.3, 2: 181.0, 3: 181.0, 4: 181.0}),
    ("AMD Instinct MI300X", 5.3 * (1024**4), {0: 163.4, 1: 653.7, 2: 1307.4, 3: 1307.4, 4: 2614.9}),
    ("AMD Instinct MI325X", 6.0 * (1024**4), {0: 163.4, 1: 653.7, 2: 1307.4, 3: 1307.4, 4: 2614.9}),
    ("AMD Instinct MI350X", 8.0 * (1024**4), {0: 72.1, 1: 144.2, 2: 2309.6, 3: 2309.6, 4: 4614.0}),
    ("AMD Instinct MI355X", MI355X_GMEM_BW, MI355X_TFLOPS),
    ("Max 1550", 3.3 * (1024**4), {0: 46, 1: 46, 2: 367, 3: 367, 4: 734}),
)


class DeviceLimit:
    def __init__(self, gmem_bandwidth=MI355X_GMEM_BW, tflops=None):
        self.gmem_bandwidth = gmem_bandwidth
        self.tflops = dict(MI355X_TFLOPS if tflops is None else tflops)

    @classmethod
    def named(cls, device_name: str) -> "DeviceLimit":
        """First row whose name occurs in device_name; PG509 boards are A100s
        (compute_estimation.py:258-275)."""
        for name, bw, tf in DEVICE_TABLE:
            if name in device_name or (name == "A100" and "PG509" in device_name):
                return cls(bw, {k: float(v) for k, v in tf.items()})
        raise ValueError(f"Unsupported device: {device_name}")


class Topo:
    """MeshTopoInfo (torch _collective_utils.py:236-278)."""

    def __init__(self, mesh_shape: Sequence[int], devices_per_host: int, nccl=None, xgmi=None):
        ndim = len(mesh_shape)
        self.nccl = nccl  # oracle.nccl_oracle.NcclConfig selects the NCCL model
        self.a2a_bw = None  # per dim, where all_to_all sees another bandwidth (xgmi)
        base_bw = 87.7
        self.mesh_shape = tuple(int(x) for x in mesh_shape)
        self.bw = [base_bw] * ndim
        self.lat = [0.6] * ndim
        self.devices = [1] * ndim
        total = 1
        for d in reversed(range(ndim)):
            n = self.mesh_shape[d]
            self.devices[d] = n
            total *= n
            if total > devices_per_host:
                self.bw[d] *= 0.22
                self.lat[d] = 2.7
        if xgmi is not None:
            # Not in the reference (an extension of this build, outside the parity
            # claim): nodes of GPUs joined pairwise by xGMI links.  xgmi: an object
            # with gpus_per_node, links_per_gpu, link_gbps (both directions), nic_gbps,
            # lat_intra_us, lat_inter_us.  A ring moves every byte over one link per
            # direction; an all_to_all among n ranks drives min(n - 1, links) links.
            one_way = xgmi.link_gbps / 2.0
            self.a2a_bw = [0.0] * ndim
            total = 1
            for d in reversed(range(ndim)):
                n = self.mesh_shape[d]
                total *= n
                if total <= xgmi.gpus_per_node:
                    self.bw[d] = one_way
                    self.a2a_bw[d] = one_way * float(max(1, min(n - 1, xgmi.links_per_gpu)))
                    self.lat[d] = xgmi.lat_intra_us
                else:
                    self.bw[d] = self.a2a_bw[d] = xgmi.nic_gbps
                    self.lat[d] = xgmi.lat_inter_us


def allgather_cost(bytes_gb: float, topo: Topo, dim: int) -> float:
    n = topo.devices[dim]
    hops = n - 1
    latency = 6.6 + hops * topo.lat[dim]
    bw = (bytes_gb * hops / n) / topo.bw[dim]
    return latency + bw * 1e6


def allreduce_cost(bytes_gb: float, topo: Topo, dim: int) -> float:
    n = topo.devices[dim]
    hops = 2 * (n - 1)
    latency = 6.6 + hops * topo.lat[dim]
    bw = (bytes_gb * hops / n) / topo.bw[dim]
    return latency + bw * 1e6


def reduce_scatter_cost(bytes_gb: float, topo: Topo, dim: int) -> float:
    n = topo.devices[dim]
    hops = n - 1
    latency = 6.6 + hops * topo.lat[dim]
    bw = (bytes_gb * hops / n) / topo.bw[dim]
    return latency + bw * 1e6


def all_to_all_cost(bytes_gb: float, topo: Topo, dim: int) -> float:
    n = topo.devices[dim]
    hops = n - 1
    latency = 6.6 + hops * topo.lat[dim]
    dim_bw = topo.a2a_bw[dim] if topo.a2a_bw is not None and topo.a2a_bw[dim] > 0 else topo.bw[dim]
    bw = (bytes_gb * hops / n) / dim_bw
    total = latency + bw * 1e6
    total *= 5
    return total


def collective_comm_cost(collective: str, comm_bytes: int, topo: Topo, dim: int) -> float:
    """collective_runtime_estimation.py:65-97: NCCL model when a topology
    config is set (:85-86), otherwise the alpha-beta functions."""
    if topo.nccl is not None:
        from . import nccl_oracle

        return nccl_oracle.comm_cost(collective, comm_bytes, topo.mesh_shape, dim, topo.nccl)
    g = comm_bytes / 1024**3
    if collective == "allgather":
        return allgather_cost(g, topo, dim)
    if collective == "allreduce":
        return allreduce_cost(g, topo, dim)
    if collective == "reduce_scatter":
        return reduce_scatter_cost(g, topo, dim)
    if collective == "all_to_all":
        return all_to_all_cost(g, topo, dim)
    return 0.0


def compute_read_write_time(nbytes, dev: DeviceLimit):
    t = nbytes / dev.gmem_bandwidth * 1e6
    return max(t / 0.70, 7)


def check_contiguous(sizes: Sequence[int], strides: Sequence[int]) -> bool:
    expected = 1
    expected_max = 1
    for x, y in reversed(tuple(zip(sizes, strides))):
        if x == 1:
            continue
        if y != expected and y != expected_max:
            return False
        expected_max *= max(x, 1)
        expected *= x
    return True


def _is_shard(p):
    return (p & KIND) == PLC_SHARD


def _is_partial(p):
    return (p & KIND) == PLC_PARTIAL


def redistribute_cost(
    src_plc: Sequence[int],
    shape: Sequence[int],
    stride: Sequence[int],
    itemsize: int,
    tgt_plc: Sequence[int],
    topo: Topo,
    dev: DeviceLimit,
    order: Sequence[int],
) -> float:
    if all(p == PLC_R for p in src_plc):
        if any(_is_partial(p) for p in tgt_plc):
            return INF
        return 0.0
    cost = 0.0
    num_shards = 1
    for i, p in enumerate(src_plc):
        if _is_shard(p):
            num_shards *= topo.mesh_shape[i]
    comm_bytes_gb = itemsize * math.prod(shape) / num_shards / 1024 / 1024 / 1024
    is_contiguous = check_contiguous(shape, stride)
    for i in order:
        current, target = src_plc[i], tgt_plc[i]
        if current == target:
            continue
        n = topo.devices[i]
        if not is_contiguous:
            cost += compute_read_write_time(comm_bytes_gb * 2 * 1024**3, dev)
        if _is_shard(current) and target == PLC_R:
            comm_bytes_gb *= n
            cost += collective_comm_cost("allgather", int(comm_bytes_gb * 1024**3), topo, i)
            if (current & ARG) != 0:
                cost += compute_read_write_time(comm_bytes_gb * 2 * 1024**3, dev)
        elif _is_shard(current) and _is_shard(target):
            cost += collective_comm_cost("all_to_all", int(comm_bytes_gb * 1024**3), topo, i)
            num_copies = 0
            if (current & ARG) != 0:
                num_copies += 1
            if (target & ARG) != 0:
                num_copies += 1
            cost += num_copies * compute_read_write_time(comm_bytes_gb * 2 * 1024**3, dev)
        elif _is_partial(current) and target == PLC_R:
            cost += collective_comm_cost("allreduce", int(comm_bytes_gb * 1024**3), topo, i)
        elif _is_partial(current) and _is_shard(target):
            cost += collective_comm_cost("reduce_scatter", int(comm_bytes_gb * 1024**3), topo, i)
            if (target & ARG) != 0:
                cost += compute_read_write_time(comm_bytes_gb * 2 * 1024**3, dev)
            comm_bytes_gb /= n
        elif _is_shard(current) and _is_partial(target):
            return INF
        elif current == PLC_R and _is_partial(target):
            return INF
        is_contiguous = True
    return cost


def comms_order(src_plc: Sequence[int], tgt_plc: Sequence[int]) -> List[int]:
    """estimate_strategy_comms_cost's order rule (:253-258)."""
    order = list(range(len(src_plc)))
    if tuple(src_plc) == (PARTIAL_SUM, PARTIAL_SUM) and all(_is_shard(p) for p in tgt_plc):
        order = [1, 0]
    return order


def estimate_strategy_comms_cost(src_plc, shape, stride, itemsize, tgt_plc, topo, dev) -> float:
    return redistribute_cost(
        src_plc, shape, stride, itemsize, tgt_plc, topo, dev, comms_order(src_plc, tgt_plc)
    )


def sharded_shape_stride(shape, stride, plc, mesh_shape):
    """_get_sharded_shape_stride (compute_estimation.py:300-318)."""
    new_shape = list(shape)
    new_stride = list(stride)
    for mesh_size, p in zip(mesh_shape, plc):
        if _is_shard(p):
            dim = p & ARG
            new_shape[dim] = (new_shape[dim] + mesh_size - 1) // mesh_size
            if dim - 1 > 0:
                new_stride[dim - 1] = (new_stride[dim - 1] + mesh_size - 1) // mesh_size
    return new_shape, new_stride


def is_valid_spec(shape, plc, mesh_shape) -> bool:
    """Per-spec test of remove_invalid_configs (propagation_rules.py:143-154)."""
    shape = list(shape)
    for mesh_size, p in zip(mesh_shape, plc):
        if _is_shard(p):
            dim = p & ARG
            if shape[dim] >= mesh_size:
                shape[dim] = (shape[dim] + mesh_size - 1) // mesh_size
            else:
                return False
    return True


def create_all_options(shape, mesh_shape) -> List[Tuple[int, ...]]:
    """_create_all_options (propagation_rules.py:184-201): placement tuples, in
    itertools.product order, that survive remove_invalid_configs."""
    options = [PLC_R] + [PLC_SHARD | i for i in range(len(shape))]
    out = []
    for plc in itertools.product(*[options for _ in mesh_shape]):
        if is_valid_spec(shape, plc, mesh_shape):
            out.append(plc)
    return out


def roofline_cost(flops: int, nbytes: int, dtype: int, dev: DeviceLimit):
    """Tail of estimate_strategy_runtime_cost (compute_estimation.py:474-489)."""
    rw = compute_read_write_time(nbytes, dev)
    if flops == 0:
        return rw
    if dtype not in dev.tflops:
        raise ValueError(f"dtype code {dtype} has no tflops entry")
    gpu_flops = dev.tflops[dtype] * 10**12
    compute_time = flops / gpu_flops * 1e6
    compute_time = compute_time / 0.70
    return max(compute_time, rw)


# ---------------------------------------------------------------------------
# Compute programs (see autoparallel_amd/packed.py for the encoding)
# ---------------------------------------------------------------------------
DIM_CONST, DIM_ARG, DIM_BCAST, DIM_ARGNUMEL = 0, 1, 2, 3


def run_program(prog: Sequence[int], local_shapes: List[Optional[List[int]]], itemsizes: List[int]):
    """Evaluate a compute program on the local input shapes.

    Returns (flops, bytes): flops as the flop counter reports them for the
    sharded op, bytes as compute_memory_cost does (inputs read + outputs
    written, compute_estimation.py:321-331)."""
    p = 0
    n_terms, n_outs = int(prog[0]), int(prog[1])
    p = 2
    flops = 0
    for _ in range(n_terms):
        coeff, nfac = int(prog[p]), int(prog[p + 1])
        p += 2
        term = coeff
        for _ in range(nfac):
            a, d = int(prog[p]), int(prog[p + 1])
            p += 2
            term *= local_shapes[a][d]
        flops += term
    nbytes = 0
    for shp, isz in zip(local_shapes, itemsizes):
        if shp is None:
            continue
        nbytes += math.prod(shp) * isz
    for _ in range(n_outs):
        isz, rank = int(prog[p]), int(prog[p + 1])
        p += 2
        numel = 1
        for _ in range(rank):
            kind, a, b = int(prog[p]), int(prog[p + 1]), int(prog[p + 2])
            p += 3
            if kind == DIM_CONST:
                size = a
            elif kind == DIM_ARG:
                size = local_shapes[a][b]
            elif kind == DIM_ARGNUMEL:
                size = math.prod(local_shapes[a])
            else:
                size = 1
                for shp in local_shapes:
                    if shp is None or a >= len(shp):
                        continue
                    s = shp[len(shp) - 1 - a]
                    if s != 1:
                        size = s
            numel *= size
        nbytes += numel * isz
    return flops, nbytes


# ---------------------------------------------------------------------------
# Drivers over a PackedGraph (duck-typed: only its numpy arrays are used)
# ---------------------------------------------------------------------------
class GraphOracle:
    """Per-entry build of all coefficients, mirroring the loop nest and the two
    memo caches of the reference (optimize_sharding.py:481-552;
    collective_runtime_estimation.py:239-262; compute_estimation.py:449-492)."""

    def __init__(self, g, dev: Optional[DeviceLimit] = None, nccl=None, xgmi=None):
        self.g = g
        self.dev = dev or DeviceLimit()
        self.topo = Topo([int(x) for x in g.mesh_shape], g.devices_per_host, nccl=nccl, xgmi=xgmi)
        self.ndim = len(self.topo.mesh_shape)
        self._comm_cache: Dict[tuple, float] = {}
        self._compute_cache: Dict[tuple, float] = {}
        # plain-Python views so the timed loop does no numpy.  A spec is a
        # 32-bit word: meta id in the high 20 bits, placement-tuple id below.
        self._tuple_plc = [tuple(int(x) for x in row[: self.ndim]) for row in g.tuple_plc]
        self._meta = []
        for m in range(g.meta_rank.shape[0]):
            r = int(g.meta_rank[m])
            self._meta.append(
                (
                    tuple(int(x) for x in g.meta_shape[m, :r]),
                    tuple(int(x) for x in g.meta_stride[m, :r]),
                    int(g.meta_itemsize[m]),
                    int(g.meta_dtype[m]),
                )
            )
        self._lists = [(-1 if int(x) == 0xFFFFFFFF else int(x)) for x in g.lists]

    def reset_caches(self):
        self._comm_cache.clear()
        self._compute_cache.clear()

    # -- per-entry pieces ----------------------------------------------------
    def comm_cost(self, src_id: int, tgt_id: int) -> float:
        # (placements, tensor meta) of both sides, as the reference's memo key
        key = (src_id, tgt_id)
        c = self._comm_cache.get(key)
        if c is not None:
            return c
        shape, stride, itemsize, _ = self._meta[src_id >> 12]
        c = estimate_strategy_comms_cost(
            self._tuple_plc[src_id & 0xFFF], shape, stride, itemsize,
            self._tuple_plc[tgt_id & 0xFFF], self.topo, self.dev
        )
        self._comm_cache[key] = c
        return c

    def node_compute_cost(self, v: int, o: int):
        g = self.g
        op = int(g.node_op[v])
        if op == 0:
            return 0
        e0, e1 = int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])
        in_ids = tuple(self._lists[int(g.edge_dst_list[e]) + o] for e in range(e0, e1))
        if op == 2:
            idx = int(g.node_comp_off[v]) + o
            flops, nbytes = int(g.explicit_flops[idx]), int(g.explicit_bytes[idx])
            dtype = self._first_dtype(in_ids)
            return roofline_cost(flops, nbytes, dtype, self.dev)
        po = int(g.node_prog_off[v])
        key = (po if po < 0 else self._prog_key(po), in_ids)
        c = self._compute_cache.get(key)
        if c is not None:
            return c
        shapes, isz = [], []
        for sid in in_ids:
            if sid < 0:
                shapes.append(None)
                isz.append(0)
                continue
            shape, stride, itemsize, _ = self._meta[sid >> 12]
            ls, _ = sharded_shape_stride(shape, stride, self._tuple_plc[sid & 0xFFF], self.topo.mesh_shape)
            shapes.append(ls)
            isz.append(itemsize)
        flops, nbytes = run_program(self._prog_slice(po), shapes, isz)
        c = roofline_cost(flops, nbytes, self._first_dtype(in_ids), self.dev)
        self._compute_cache[key] = c
        return c

    def _first_dtype(self, in_ids) -> int:
        for sid in in_ids:
            if sid >= 0:
                return self._meta[sid >> 12][3]
        return 1  # torch.float32 default (compute_estimation.py:418-419)

    def _prog_len(self, po: int) -> int:
        prog = self.g.prog
        n_terms, n_outs = int(prog[po]), int(prog[po + 1])
        p = po + 2
        for _ in range(n_terms):
            p += 2 + 2 * int(prog[p + 1])
        for _ in range(n_outs):
            p += 2 + 3 * int(prog[p + 1])
        return p - po

    def _prog_slice(self, po: int):
        return self.g.prog[po : po + self._prog_len(po)]

    def _prog_key(self, po: int):
        if not hasattr(self, "_prog_keys"):
            self._prog_keys = {}
        k = self._prog_keys.get(po)
        if k is None:
            k = tuple(int(x) for x in self._prog_slice(po))
            self._prog_keys[po] = k
        return k

    # -- the build -----------------------------------------------------------
    def build(self, nodes: Optional[Sequence[int]] = None, out: Optional[dict] = None):
        """Returns dict of numpy arrays in entry order:
        comm f64[slots], transition u8[slots], cost f64[slots] (before the inf clamp),
        compute f64[sum S] (the per-strategy estimate, not divided).
        ``nodes`` restricts the build to some nodes; ``out`` reuses arrays."""
        g = self.g
        E = g.num_slots  # entry arrays are indexed by slot; padding stays zero
        if out is None:
            out = {
                "comm": np.zeros(E, np.float64),
                "transition": np.zeros(E, np.uint8),
                "cost": np.zeros(E, np.float64),
                "compute": np.zeros(g.num_compute, np.float64),
            }
        comm, trans, cost, compute = out["comm"], out["transition"], out["cost"], out["compute"]
        lists = self._lists
        tuple_plc = self._tuple_plc
        node_range = range(g.num_nodes) if nodes is None else nodes
        for v in node_range:
            S = int(g.node_nstrat[v])
            nargs = int(g.node_nargs[v])
            e0, e1 = int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])
            c0 = int(g.node_comp_off[v])
            for o in range(S):
                cc = self.node_compute_cost(v, o)
                compute[c0 + o] = cc
                per_arg = cc / nargs
                for e in range(e0, e1):
                    ssrc = int(g.edge_ssrc[e])
                    base = int(g.edge_off[e]) + o * ssrc
                    flags = int(g.edge_flags[e])
                    tgt_id = lists[int(g.edge_dst_list[e]) + o]
                    src_list = int(g.edge_src_list[e])
                    doff = int(g.edge_default_off[e])
                    for j in range(ssrc):
                        t = 0
                        src_id = lists[src_list + j] if (flags & 1) else -1
                        if src_id >= 0 and tgt_id >= 0:
                            c = self.comm_cost(src_id, tgt_id)
                            if tuple_plc[src_id & 0xFFF] != tuple_plc[tgt_id & 0xFFF]:
                                t = 1
                        else:
                            c = float(g.default_vals[doff + o * ssrc + j])
                        comm[base + j] = c
                        trans[base + j] = t
                        cost[base + j] = c + per_arg + t
        return out


def clamp_inf(cost: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """add_inf_cost_constraint (optimize_sharding.py:803-812): non-finite cost
    -> 10000.0 and the variable forced to 0.  Returns (cost, forbidden mask)."""
    out = cost.copy()
    bad = np.zeros(cost.shape[0], np.uint8)
    for i in range(cost.shape[0]):
        if not math.isfinite(out[i]):
            out[i] = 10000.0
            bad[i] = 1
    return out, bad


def prefetch_discount(g, comm, transition, compute, cost, scale: float):
    """apply_prefetch_discount (optimize_sharding.py:824-875) on entry arrays.
    ``compute`` is the per-strategy vector; per-arg value is recomputed."""
    comm = comm.copy()
    cost = cost.copy()
    n_modified = 0
    for e in range(g.num_edges):
        if not g.edge_prefetchable[e] or g.edge_src_node[e] < 0:
            continue
        v = int(g.edge_node[e])
        ssrc = int(g.edge_ssrc[e])
        for o in range(int(g.edge_sdst[e])):
            per_arg = compute[int(g.node_comp_off[v]) + o] / int(g.node_nargs[v])
            for j in range(ssrc):
                i = int(g.edge_off[e]) + o * ssrc + j
                c = comm[i]
                if c > 0 and math.isfinite(c):
                    c = c * scale
                    comm[i] = c
                    cost[i] = c + per_arg + float(transition[i])
                    n_modified += 1
    return comm, cost, n_modified


def score_assignment(g, comm, transition, compute, assign: Sequence[int]):
    """_compute_solution_cost (optimize_sharding.py:1056-1111) for one
    assignment (out_idx per node).  Returns (total, compute, comm, transition)."""
    total_compute = 0.0
    total_comm = 0.0
    total_transition = 0.0
    for v in range(g.num_nodes):
        o = int(assign[v])
        nargs = int(g.node_nargs[v])
        per_arg = compute[int(g.node_comp_off[v]) + o] / nargs
        total_compute += per_arg * max(nargs, 1)
        for e in range(int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])):
            u = int(g.edge_src_node[e])
            if u < 0:
                continue
            j = int(assign[u])
            i = int(g.edge_off[e]) + o * int(g.edge_ssrc[e]) + j
            c = comm[i]
            if math.isfinite(c):
                total_comm += c
            if (int(g.edge_flags[e]) & 2) and transition[i]:
                total_transition += 1
    return (total_compute + total_comm + total_transition, total_compute, total_comm, total_transition)


def ilp_objective(g, cost_clamped, forbidden, assign: Sequence[int]):
    """Value of the ILP objective (optimize_sharding.py:879-885) at the point
    an assignment induces (x=1 on (v, a, assign[v], assign[producer])), and the
    number of selected variables pinned to zero by the inf-cost rows."""
    obj = 0.0
    viol = 0
    for v in range(g.num_nodes):
        o = int(assign[v])
        mult = int(g.node_multiplier[v])
        for e in range(int(g.node_edge_off[v]), int(g.node_edge_off[v + 1])):
            u = int(g.edge_src_node[e])
            j = int(assign[u]) if u >= 0 else 0
            i = int(g.edge_off[e]) + o * int(g.edge_ssrc[e]) + j
            obj += cost_clamped[i] * mult
            viol += int(forbidden[i])
    return obj, viol


# ---------------------------------------------------------------------------
# Candidate assignments without a forbidden variable
# ---------------------------------------------------------------------------
_M32 = 0xFFFFFFFF


def _finalise32(h: int) -> int:
    h ^= h >> 16
    h = (h * 0x85EBCA6B) & _M32
    h ^= h >> 13
    h = (h * 0xC2B2AE35) & _M32
    h ^= h >> 16
    return h


def _assignment_hash(seed: int, a: int) -> int:
    seed &= 0xFFFFFFFFFFFFFFFF
    a &= 0xFFFFFFFFFFFFFFFF
    h = (seed & _M32) ^ (((seed >> 32) * 0x27D4EB2F) & _M32)
    h ^= ((a & _M32) * 0x9E3779B1) & _M32
    h ^= ((a >> 32) * 0x85EBCA77) & _M32
    return h


def plain_draw(seed: int, a: int, gid: int, nstrat: int) -> int:
    """Uniform draw of the scorers: a 32-bit mix of (seed, assignment, node)
    scaled to [0, nstrat) by a multiply-high."""
    h = _finalise32(_assignment_hash(seed, a) ^ (((gid + 1) * 0xC2B2AE3D) & _M32))
    return (h * nstrat) >> 32


def sample_rank(seed: int, a: int, gid: int, count: int) -> int:
    """Which of the ``count`` allowed strategies of node gid is taken, counted in
    out_idx order: a 32-bit mix of (seed, assignment, node) of its own, scaled to
    [0, count) by a multiply-high."""
    h = _finalise32(_assignment_hash(seed, a) ^ (((gid + 1) * 0xC2B2AE3D) & _M32) ^ 0x68E31DA4)
    return (h * count) >> 32


def sample_feasible(g, forbidden, seed: int, a: int, node_gid=None, first_node: int = 0, given=None,
                    row_filter=None):
    """One assignment, node by node in graph order: node v gets, uniformly, one of
    its strategies whose entries against the choices of its producers are all
    allowed (``forbidden``: uint8 per slot, the non-finite costs that
    add_inf_cost_constraint pins to zero, optimize_sharding.py:803-812); a node
    without one takes the plain draw and is counted.  ``given``: the choices of
    the nodes below first_node.  ``row_filter``: {node: bool per strategy}, the
    strategies a node may take at all.  Returns (choices per node, number of
    fallbacks)."""
    N = g.num_nodes
    assign = [0] * N
    for v in range(first_node):
        assign[v] = int(given[v])
    fallbacks = 0
    for v in range(first_node, N):
        gid = int(node_gid[v]) if node_gid is not None else v
        S = int(g.node_nstrat[v])
        edges = range(int(g.node_edge_off[v]), int(g.node_edge_off[v + 1]))
        allowed = []
        keep = row_filter.get(v) if row_filter else None
        for o in range(S):
            ok = keep is None or bool(keep[o])
            for e in edges:
                if not ok:
                    break
                u = int(g.edge_src_node[e])
                j = assign[u] if u >= 0 else 0
                if forbidden[int(g.edge_off[e]) + o * int(g.edge_ssrc[e]) + j]:
                    ok = False
                    break
            if ok:
                allowed.append(o)
        count, pick = len(allowed), 0
        if count:
            pick = allowed[sample_rank(seed, a, gid, count)]
        if count == 0:
            pick = plain_draw(seed, a, gid, S)
            fallbacks += 1
        assign[v] = pick
    return assign, fallbacks
