"""Runtime and memory metrics of a lowered (sharded) graph, for one order or for
a batch of candidate orders, evaluated on the device.

``estimate_graph_metrics(gm, runtime_estimator)`` keeps the reference's
interface (autoparallel/graph_passes/estimate_graph_metrics.py:30-89): a compute
stream and one stream per communication group, 1 us of launch overhead per
node, ``wait_tensor`` stalls, and torch's liveness-based peak memory.  The walk
itself runs in ``apc_schedule_metrics``; this module flattens the FX graph into
the arrays that kernel reads (``PackedSchedule``) and, because the walk is a
serial chain per order, offers what the reference cannot do cheaply:
``ScheduleEstimator.evaluate(orders)`` prices thousands of candidate orders of
the same nodes in one launch, one lane per order.
"""
from __future__ import annotations

import ctypes as C
import dataclasses
from typing import Callable, List, Optional

import numpy as np
import torch
import torch.fx as fx

from . import _lib

SCHED_COMM, SCHED_WAIT, SCHED_SYNC, SCHED_NO_MEM = 1, 2, 4, 8
MAX_STREAMS = 8

# _dtensor ops that are collectives although they are not _c10d_functional ops
# (reference: graph_passes/debug_helpers.py:104-107)
_DTENSOR_COLLECTIVE_OPS = frozenset({"shard_dim_alltoall"})


@dataclasses.dataclass
class GraphMetrics:
    """Same fields as the reference's GraphMetrics (estimate_graph_metrics.py:21-27)."""

    total_time: float  # critical-path time (max across all streams), microseconds
    compute_time: float  # sum of compute node durations, microseconds
    communication_time: float  # sum of comm node durations (excl. wait_tensor), microseconds
    exposed_comm_time: float  # time the compute stream stalls at wait_tensor nodes, microseconds
    peak_memory: int  # peak live tensor memory in bytes


# -- node predicates (reference: graph_passes/debug_helpers.py:110-133, 250-255)
def is_communication_node(node: fx.Node) -> bool:
    if node.op != "call_function" or not isinstance(node.target, torch._ops.OpOverload):
        return False
    ns = node.target.namespace
    if ns in ("_c10d_functional", "c10d_functional"):
        return True
    return ns == "_dtensor" and node.target._opname in _DTENSOR_COLLECTIVE_OPS


def is_sync_collective(node: fx.Node) -> bool:
    return is_communication_node(node) and node.target.namespace == "_dtensor"


def is_wait_tensor(node: fx.Node) -> bool:
    return is_communication_node(node) and node.target._opname == "wait_tensor"


def stream_key(node: fx.Node):
    if is_communication_node(node) and not is_wait_tensor(node):
        return f"group-{node.args[-1]}"
    return 0


def resolve_comm_node(node: fx.Node, in_flight) -> object:
    """The collective a wait_tensor waits for: through chained waits and
    wrappers such as control_deps, preferring an argument that is in flight
    (reference: debug_helpers.py:135-167)."""
    arg = node.args[0]
    while isinstance(arg, fx.Node) and is_wait_tensor(arg):
        arg = arg.args[0]
    while (isinstance(arg, fx.Node) and arg not in in_flight and arg.op == "call_function"
           and not is_communication_node(arg)):
        nxt = next((a for a in arg.args if isinstance(a, fx.Node) and a in in_flight), None)
        if nxt is None:
            nxt = next((a for a in arg.args if isinstance(a, fx.Node)), None)
            if nxt is None:
                break
        arg = nxt
    return arg


@dataclasses.dataclass
class PackedSchedule:
    dur: np.ndarray  # float64[N]
    stream: np.ndarray  # int32[N]
    flags: np.ndarray  # uint8[N]
    wait_src: np.ndarray  # int32[N]
    n_stream: int
    st_bytes: np.ndarray  # int64[S]
    st_freeable: np.ndarray  # uint8[S]
    st_users: np.ndarray  # int32[S]
    alloc_off: np.ndarray  # int32[N+1]
    alloc_st: np.ndarray  # int32[...]
    use_off: np.ndarray  # int32[N+1]
    use_st: np.ndarray  # int32[...]
    initial_bytes: int
    node_names: Optional[List[str]] = None
    # producers of every node (CSR), for drawing valid orders
    dep_off: Optional[np.ndarray] = None
    dep_node: Optional[np.ndarray] = None

    @property
    def n_node(self) -> int:
        return int(self.dur.shape[0])

    @property
    def n_storage(self) -> int:
        return int(self.st_bytes.shape[0])

    def validate(self) -> None:
        """Every index the kernel dereferences, checked on the host."""
        N, S = self.n_node, self.n_storage
        assert 1 <= self.n_stream <= MAX_STREAMS
        for a in (self.stream, self.flags, self.wait_src):
            assert a.shape == (N,)
        assert ((self.stream >= 0) & (self.stream < self.n_stream)).all()
        assert ((self.wait_src >= -1) & (self.wait_src < N)).all()
        assert self.st_freeable.shape == (S,) and self.st_users.shape == (S,)
        for off, idx in ((self.alloc_off, self.alloc_st), (self.use_off, self.use_st)):
            assert off.shape == (N + 1,) and off[0] == 0 and (np.diff(off) >= 0).all()
            assert int(off[-1]) == idx.shape[0]
            assert idx.shape[0] == 0 or ((idx >= 0) & (idx < S)).all()
        # a storage's reader count is the number of use lists it appears in
        assert (np.bincount(self.use_st, minlength=S) == self.st_users).all()

    def random_orders(self, n: int, seed: int = 0) -> np.ndarray:
        """int32[n, N]: valid orders (every node after its producers) drawn by a
        randomised topological sort; order 0 is the graph's own."""
        N = self.n_node
        rng = np.random.default_rng(seed)
        users: List[List[int]] = [[] for _ in range(N)]
        for v in range(N):
            for u in self.dep_node[self.dep_off[v]:self.dep_off[v + 1]]:
                users[int(u)].append(v)
        out = np.empty((n, N), np.int32)
        out[0] = np.arange(N)
        for b in range(1, n):
            need = np.diff(self.dep_off).astype(np.int64)
            ready = [v for v in range(N) if need[v] == 0]
            for t in range(N):
                k = int(rng.integers(len(ready)))
                ready[k], ready[-1] = ready[-1], ready[k]
                v = ready.pop()
                out[b, t] = v
                for w in users[v]:
                    need[w] -= 1
                    if need[w] == 0:
                        ready.append(w)
        return out


def pack_schedule(
    gm: fx.GraphModule,
    runtime_estimator: Callable[[fx.Node], float],
    is_releasable: Optional[Callable[[fx.Node], bool]] = None,
    device_filter: Optional[Callable[[torch.device], bool]] = None,
) -> PackedSchedule:
    """Flatten ``gm`` for the schedule kernel.  ``is_releasable`` /
    ``device_filter`` as torch's MemoryTracker takes them (defaults: every node
    but ``primals*``; every device but the CPU)."""
    from torch._inductor.fx_passes.memory_estimator import GraphAliasTracker

    nodes = list(gm.graph.nodes)
    index = {n: i for i, n in enumerate(nodes)}
    N = len(nodes)
    if is_releasable is None:
        is_releasable = lambda n: not n.name.startswith("primals")  # noqa: E731
    if device_filter is None:
        device_filter = lambda d: d.type != "cpu"  # noqa: E731

    dur = np.zeros(N, np.float64)
    stream = np.zeros(N, np.int32)
    flags = np.zeros(N, np.uint8)
    wait_src = np.full(N, -1, np.int32)
    streams = {0: 0}
    in_flight = set()  # which collectives global_time holds, in the graph's own order
    for i, node in enumerate(nodes):
        dur[i] = float(runtime_estimator(node))
        key = stream_key(node)
        if key not in streams:
            if len(streams) == MAX_STREAMS:
                raise ValueError(f"more than {MAX_STREAMS - 1} communication groups in one graph")
            streams[key] = len(streams)
        stream[i] = streams[key]
        f = 0
        if node.op in ("placeholder", "get_attr", "output"):
            f |= SCHED_NO_MEM
        if is_communication_node(node):
            f |= SCHED_COMM
            if stream[i] == 0 and is_wait_tensor(node) and node.args[0].op != "placeholder":
                f |= SCHED_WAIT
                src = resolve_comm_node(node, in_flight)
                if isinstance(src, fx.Node):
                    wait_src[i] = index[src]
                    in_flight.discard(src)
            if is_sync_collective(node):
                f |= SCHED_SYNC
        if stream[i] != 0:
            in_flight.add(node)
        flags[i] = f

    alias = GraphAliasTracker(nodes)
    st_index = {}
    st_bytes: List[int] = []
    st_free: List[int] = []

    def sid(key):
        if key not in st_index:
            st_index[key] = len(st_bytes)
            st_bytes.append(int(key.storage.nbytes()))
            st_free.append(1 if is_releasable(alias.storage_to_allocator[key]) else 0)
        return st_index[key]

    initial = 0
    alloc_off, alloc_st, use_off, use_st = [0], [], [0], []
    for node in nodes:
        fresh = [k for k in alias.get_fresh_allocations(node) if device_filter(k.device)]
        if node.op in ("placeholder", "get_attr"):
            initial += sum(int(k.storage.nbytes()) for k in fresh)
            for k in fresh:
                sid(k)
        elif node.op != "output":
            alloc_st.extend(sid(k) for k in fresh)
        alloc_off.append(len(alloc_st))
        use_st.extend(sid(k) for k in alias.get_storage_uses(node) if device_filter(k.device))
        use_off.append(len(use_st))
    S = len(st_bytes)
    use_arr = np.asarray(use_st, np.int32)
    dep_off, dep_node = [0], []
    for node in nodes:
        dep_node.extend(index[u] for u in node.all_input_nodes)
        dep_off.append(len(dep_node))
    ps = PackedSchedule(
        dur=dur, stream=stream, flags=flags, wait_src=wait_src, n_stream=len(streams),
        st_bytes=np.asarray(st_bytes, np.int64), st_freeable=np.asarray(st_free, np.uint8),
        st_users=np.bincount(use_arr, minlength=S).astype(np.int32),
        alloc_off=np.asarray(alloc_off, np.int32), alloc_st=np.asarray(alloc_st, np.int32),
        use_off=np.asarray(use_off, np.int32), use_st=use_arr, initial_bytes=int(initial),
        node_names=[n.name for n in nodes],
        dep_off=np.asarray(dep_off, np.int32), dep_node=np.asarray(dep_node, np.int32))
    ps.validate()
    return ps


def synthetic_schedule(n_layers: int = 32, seed: int = 0) -> PackedSchedule:
    """A lowered decoder-like schedule built straight in the packed form, for
    benchmarks: per layer an all-gather of the weights on group 1 issued one
    layer ahead, its wait, four compute nodes, and a reduce-scatter on group 2
    waited for two layers later; one storage per node, read by the next node
    on its stream of data and freed after its last reader."""
    rng = np.random.default_rng(seed)
    dur, stream, flags, wait_src, deps, nbytes = [], [], [], [], [], []

    def node(d, st=0, fl=0, src=-1, dep=(), size=0):
        dur.append(float(d)); stream.append(st); flags.append(fl); wait_src.append(src)
        deps.append(list(dep)); nbytes.append(int(size))
        return len(dur) - 1

    x = node(0.0, fl=SCHED_NO_MEM, size=1 << 24)  # activations in
    weights = [node(0.0, fl=SCHED_NO_MEM, size=1 << 22) for _ in range(n_layers)]
    gathers = {0: node(rng.uniform(20, 60), 1, SCHED_COMM, dep=[weights[0]], size=1 << 25)}
    scatters = {}
    for layer in range(n_layers):
        if layer + 1 < n_layers:
            gathers[layer + 1] = node(rng.uniform(20, 60), 1, SCHED_COMM, dep=[weights[layer + 1]], size=1 << 25)
        w = node(0.0, 0, SCHED_COMM | SCHED_WAIT, src=gathers[layer], dep=[gathers[layer]], size=1 << 25)
        for k in range(4):
            x = node(rng.uniform(15, 120), dep=[x, w] if k == 0 else [x], size=1 << 24)
        scatters[layer] = node(rng.uniform(10, 40), 2, SCHED_COMM, dep=[x], size=1 << 21)
        if layer - 2 in scatters:
            node(0.0, 0, SCHED_COMM | SCHED_WAIT, src=scatters[layer - 2], dep=[scatters[layer - 2]], size=1 << 21)
    node(0.0, fl=SCHED_NO_MEM, dep=[x])  # output
    N = len(dur)
    n_in = 1 + n_layers
    use_off, use_st = [0], []
    for v in range(N):
        use_st.extend(sorted(set(deps[v])))  # storage k is the output of node k
        use_off.append(len(use_st))
    alloc_off, alloc_st = [0], []
    for v in range(N):
        if not flags[v] & SCHED_NO_MEM:
            alloc_st.append(v)
        alloc_off.append(len(alloc_st))
    use_arr = np.asarray(use_st, np.int32)
    dep_off = np.concatenate([[0], np.cumsum([len(d) for d in deps])]).astype(np.int32)
    ps = PackedSchedule(
        dur=np.asarray(dur), stream=np.asarray(stream, np.int32), flags=np.asarray(flags, np.uint8),
        wait_src=np.asarray(wait_src, np.int32), n_stream=3, st_bytes=np.asarray(nbytes, np.int64),
        st_freeable=np.asarray([0 if 1 <= v < n_in else 1 for v in range(N)], np.uint8),  # weights stay
        st_users=np.bincount(use_arr, minlength=N).astype(np.int32),
        alloc_off=np.asarray(alloc_off, np.int32), alloc_st=np.asarray(alloc_st, np.int32),
        use_off=np.asarray(use_off, np.int32), use_st=use_arr,
        initial_bytes=int(sum(nbytes[:n_in])),
        dep_off=dep_off, dep_node=np.asarray([u for d in deps for u in d], np.int32))
    ps.validate()
    return ps


class ScheduleEstimator:
    """A packed schedule resident on the device."""

    def __init__(self, ps: PackedSchedule, device: str = "cuda"):
        self.lib = _lib.load()
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise _lib.ApcError("ScheduleEstimator needs a HIP device; there is no CPU path")
        ps.validate()
        self.ps = ps
        self._keep = {}

        def up(name, arr):
            t = torch.from_numpy(np.ascontiguousarray(arr)).to(self.device)
            self._keep[name] = t
            return t.data_ptr() if t.numel() else None

        s = _lib.ApcSchedule()
        s.n_node, s.n_stream, s.n_storage = ps.n_node, ps.n_stream, ps.n_storage
        s.initial_bytes = ps.initial_bytes
        for name in ("dur", "stream", "flags", "wait_src", "st_bytes", "st_freeable", "st_users",
                     "alloc_off", "alloc_st", "use_off", "use_st"):
            setattr(s, name, up(name, getattr(ps, name)))
        # the nodes whose end time the walk keeps (those on a stream of their own), numbered
        on_stream = ps.stream != 0
        slot = np.where(on_stream, np.cumsum(on_stream) - 1, -1).astype(np.int32)
        s.comm_slot, s.n_comm = up("comm_slot", slot), int(on_stream.sum())
        self.sched = s

    def evaluate(self, orders: Optional[np.ndarray] = None):
        """(times float64[B, 4], peak int64[B]); ``orders`` int32[B, N] (each row
        a valid order of the nodes) or None for the graph's own order."""
        ps = self.ps
        N, S = ps.n_node, ps.n_storage
        if orders is None:
            B, order_ptr = 1, None
        else:
            orders = np.ascontiguousarray(orders, np.int32)
            assert orders.ndim == 2 and orders.shape[1] == N
            B = orders.shape[0]
            d_orders = torch.from_numpy(orders).to(self.device)
            # each row a permutation: the kernel indexes node arrays with it (checked on the
            # device, where sorting the rows of a large batch takes a fraction of the host's time)
            rows_sorted = torch.sort(d_orders, dim=1).values
            assert bool((rows_sorted == torch.arange(N, dtype=torch.int32, device=self.device)).all().item()), \
                "not permutations"
            del rows_sorted
            order_ptr = C.c_void_p(d_orders.data_ptr())
        end = torch.empty(max(B * N, 1), dtype=torch.float64, device=self.device)
        rem = torch.empty(max(B * S, 1), dtype=torch.int32, device=self.device)
        times = torch.empty((B, 4), dtype=torch.float64, device=self.device)
        peak = torch.empty(B, dtype=torch.int64, device=self.device)
        stream = C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)
        _lib.check(
            self.lib.apc_schedule_metrics(
                C.byref(self.sched), order_ptr, B, C.c_void_p(end.data_ptr()), C.c_void_p(rem.data_ptr()),
                C.c_void_p(times.data_ptr()), C.c_void_p(peak.data_ptr()), stream),
            "apc_schedule_metrics")
        return times.cpu().numpy(), peak.cpu().numpy()


def estimate_graph_metrics(
    gm: fx.GraphModule,
    runtime_estimator: Callable[[fx.Node], float],
    is_releasable: Optional[Callable[[fx.Node], bool]] = None,
    device_filter: Optional[Callable[[torch.device], bool]] = None,
) -> GraphMetrics:
    """Drop-in for the reference's estimate_graph_metrics
    (graph_passes/estimate_graph_metrics.py:30-89)."""
    ps = pack_schedule(gm, runtime_estimator, is_releasable, device_filter)
    times, peak = ScheduleEstimator(ps).evaluate()
    return GraphMetrics(
        total_time=float(times[0, 0]), compute_time=float(times[0, 1]),
        communication_time=float(times[0, 2]), exposed_comm_time=float(times[0, 3]),
        peak_memory=int(peak[0]))


def make_custom_runtime_estimation(mesh):
    """The runtime estimator the reference hands to its lowered-graph passes
    (graph_passes/debug_helpers.py:170-224): a collective is priced with
    ``collective_comm_cost`` on the mesh dim its process group belongs to (the
    flattened mesh when the group is none of the mesh's own; all-gather volume
    is the input shard times the group size), ``wait_tensor`` and unknown
    collectives cost nothing, and every other operator gets the unsharded
    compute estimate.  ``override_size`` (GiB) replaces the traced volume."""
    from torch._inductor.fx_passes.overlap_scheduling import get_group_name
    from torch.distributed.tensor._collective_utils import MeshTopoInfo

    from .cost_models.collective_runtime_estimation import collective_comm_cost
    from .cost_models.compute_estimation import estimate_strategy_runtime_cost

    c10d, dt = torch.ops._c10d_functional, torch.ops._dtensor
    kinds = {
        c10d.all_gather_into_tensor.default: "allgather",
        c10d.all_gather_into_tensor_out.default: "allgather",
        c10d.reduce_scatter_tensor.default: "reduce_scatter",
        c10d.all_reduce.default: "allreduce",
        dt.shard_dim_alltoall.default: "all_to_all",
    }

    def custom_runtime_estimation(node: fx.Node, override_size=None):
        if node.op != "call_function" or not isinstance(node.target, torch._ops.OpOverload):
            return 0
        if not is_communication_node(node):
            return estimate_strategy_runtime_cost(node, None)
        kind = kinds.get(node.target)
        if kind is None:  # wait_tensor and collectives the cost model does not know
            return 0
        group = get_group_name(node)
        names = tuple(g.group_name for g in mesh.get_all_groups())
        if group in names:
            cost_mesh, dim = mesh, names.index(group)
        elif mesh.ndim > 1:
            cost_mesh, dim = mesh._flatten(), 0
        else:
            return 0
        t = node.args[0].meta["val"]
        nbytes = t.numel() * t.itemsize if override_size is None else int(override_size * 2**30)
        if kind == "allgather":
            nbytes *= cost_mesh.shape[dim]
        return collective_comm_cost(kind, nbytes, tuple(cost_mesh.shape), dim, MeshTopoInfo.build_from_mesh(cost_mesh))

    return custom_runtime_estimation
