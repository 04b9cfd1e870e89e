"""Host driver of the HIP cost engine: holds a packed problem in HBM and runs
the kernels through the C ABI.  PyTorch is used only for device memory and the
current HIP stream."""
from __future__ import annotations

import ctypes as C
import threading
from typing import Dict, Optional

import numpy as np
import torch

from . import _lib
from .packed import CHUNK_SHIFT, ITEM_ENTRIES, MAX_MESH_DIMS, PackedGraph

_LARGE_BLOCKS_FROM = 8192  # mean entries per edge block
_UPLOAD_ARENA_BYTES = 8 << 20  # descriptor arrays of one problem that go up in one copy
_UPLOAD_ARENA_MAX_ARRAY = 2 << 20
_SCORE_LANES_FROM = 32768  # assignments: below, one wavefront per assignment (entry arrays as they are)
_SCORE_FROM_TABLE = True  # the three ways of scoring a graph with large blocks can be switched off (tests do)
_SCORE_COMPACT = True
# Matrices of up to this many LDS tiles (64 KB each) go through LDS in the table scorer, larger
# ones are read in place.  Measured on a 3 000-node window of the stress DAG, 2^20 assignments:
# 17.9 ms with 1, 17.4 with 2, 18.0 with 4, 18.35 with 8 or 16.  (A lower bound, small matrices
# read in place to save their barrier, only cost time: 17.4 -> 18.9 ms at 1 024 doubles.)
_SCORE_STAGE_TILES = 2
# The table scorer pays about 2 us per edge whatever the batch (a matrix copied into LDS on every CU), the
# walks over records about 14 ns per edge and assignment: from this many assignments on the table wins
# (measured on a 3 000-node window of the stress DAG: 18 ms per window from the table for any batch up to
# 2^20, 78 ms from compact records for 2^20)
_SCORE_TABLE_FROM = 131072
_SCORE_PER_LANE = 0  # assignments per lane of the compact scorer; 0: the library chooses
_READBACK_PINNED = True  # results() copies into pinned host memory (else pageable)
_LUT_TABLE_FROM = 2048  # table units: larger tables are built tile by tile with per-source terms in LDS


def xgmi_config_struct(cfg) -> _lib.ApcXgmiConfig:
    """apc_xgmi_config from any object with XGMITopoConfig's fields."""
    if isinstance(cfg, _lib.ApcXgmiConfig):
        return cfg
    c = _lib.ApcXgmiConfig()
    c.gpus_per_node, c.links_per_gpu = int(cfg.gpus_per_node), int(cfg.links_per_gpu)
    c.link_gbps, c.nic_gbps = float(cfg.link_gbps), float(cfg.nic_gbps)
    c.lat_intra_us, c.lat_inter_us = float(cfg.lat_intra_us), float(cfg.lat_inter_us)
    return c


def make_model(mesh_shape, devices_per_host: int, device_name: str, order_mode: int = 0,
               topo_config=None) -> _lib.ApcModel:
    """Cost-model constants for a mesh on a named device (raises ApcError for a
    device the reference's table does not know either).  ``topo_config``: an
    XGMITopoConfig whose link constants replace the reference's NVLink-era ones
    (then ``devices_per_host`` is not used)."""
    lib = _lib.load()
    m = _lib.ApcModel()
    nd = len(mesh_shape)
    assert 1 <= nd <= MAX_MESH_DIMS
    m.ndim = nd
    m.order_mode = int(order_mode)
    shape = (C.c_int32 * MAX_MESH_DIMS)(*([int(x) for x in mesh_shape] + [1] * (MAX_MESH_DIMS - nd)))
    m.mesh_shape = shape
    bw = (C.c_double * MAX_MESH_DIMS)()
    lat = (C.c_double * MAX_MESH_DIMS)()
    _lib.check(
        lib.apc_mesh_topology(C.addressof(shape), nd, int(devices_per_host), C.addressof(bw), C.addressof(lat)),
        "apc_mesh_topology",
    )
    if topo_config is not None:
        a2a = (C.c_double * MAX_MESH_DIMS)()
        xc = xgmi_config_struct(topo_config)
        _lib.check(
            lib.apc_xgmi_topology(C.byref(xc), C.addressof(shape), nd, C.addressof(bw), C.addressof(lat),
                                  C.addressof(a2a)),
            "apc_xgmi_topology")
        m.mesh_a2a_bw = a2a
    m.mesh_bw = bw
    m.mesh_lat = lat
    _lib.check(lib.apc_device_limits(device_name.encode(), C.byref(m)), "apc_device_limits")
    return m


def nccl_config_struct(cfg) -> _lib.ApcNcclConfig:
    """apc_nccl_config from any object with NCCLTopoConfig's fields
    (autoparallel/cost_models/nccl_cost_model.py:67-82); ``arch`` may be an
    int or an enum with an int ``value``."""
    if isinstance(cfg, _lib.ApcNcclConfig):
        return cfg
    c = _lib.ApcNcclConfig()
    c.arch = int(getattr(cfg.arch, "value", cfg.arch))
    c.num_nodes = int(cfg.num_nodes)
    c.gpus_per_node = int(cfg.gpus_per_node)
    c.num_channels = int(cfg.num_channels) if cfg.num_channels is not None else 0
    c.has_nvswitch = int(bool(cfg.has_nvswitch))
    c.has_collnet = int(bool(cfg.has_collnet))
    c.bw_intra = float(cfg.bw_intra)
    c.bw_inter = float(cfg.bw_inter)
    c.net_latency = float(cfg.net_latency)
    return c


def build_nccl_plan(cfg, mesh_shape) -> _lib.ApcNcclPlan:
    """Host plan of the NCCL-tuning model for a mesh (apc_nccl_plan_build)."""
    lib = _lib.load()
    nd = len(mesh_shape)
    shape = (C.c_int32 * MAX_MESH_DIMS)(*([int(x) for x in mesh_shape] + [1] * (MAX_MESH_DIMS - nd)))
    plan = _lib.ApcNcclPlan()
    c = nccl_config_struct(cfg)
    _lib.check(lib.apc_nccl_plan_build(C.byref(c), C.addressof(shape), nd, C.byref(plan)), "apc_nccl_plan_build")
    return plan


def upload_nccl_plan(model: _lib.ApcModel, cfg, device) -> torch.Tensor:
    """Build the plan for model's mesh, copy it to ``device`` and point
    ``model.nccl_plan`` at the copy.  The caller keeps the returned tensor alive
    for as long as the model is used."""
    plan = build_nccl_plan(cfg, [model.mesh_shape[i] for i in range(model.ndim)])
    raw = np.frombuffer(bytes(plan), dtype=np.uint8).copy()
    t = torch.from_numpy(raw).to(device)
    model.nccl_plan = t.data_ptr()
    return t


_stage = threading.local()  # .buffer: this thread's pinned staging buffer


def _upload_stage(nbytes: int) -> torch.Tensor:
    """Pinned staging buffer of the upload arena, kept between the engines a
    thread makes (pinning memory costs more than the copy it serves); an engine
    is done with it when its copy has run, before its constructor returns."""
    buf = getattr(_stage, "buffer", None)
    if buf is None or buf.numel() < nbytes:
        buf = _stage.buffer = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, pin_memory=True)
    return buf


def detect_device_name(device=None) -> str:
    """Marketing name of the HIP device, as the reference's device table keys
    on it (autoparallel/cost_models/compute_estimation.py:258-275).  Hosts
    without the amdgpu id database report every card as "AMD Radeon Graphics";
    the architecture name then decides (gfx950 is MI355X)."""
    name = torch.cuda.get_device_name(device)
    if "Instinct" not in name:
        arch = getattr(torch.cuda.get_device_properties(device), "gcnArchName", "")
        if arch.startswith("gfx950"):
            return "AMD Instinct MI355X"
        if arch.startswith("gfx942"):
            return "AMD Instinct MI300X"
    return name


class CostEngine:
    def __init__(
        self,
        g: PackedGraph,
        device: str = "cuda",
        device_name: Optional[str] = None,
        use_table: Optional[bool] = None,
        order_mode: int = 0,
        nccl_config=None,
        table_mode: Optional[str] = None,
        item_entries: Optional[int] = None,
        topo_config=None,
        allocate_results: bool = True,
        lut: Optional[bool] = None,
    ):
        """``table_mode``: "full" (one S_dst x S_src matrix per distinct pair of
        runs), "compressed" (matrices by distinct spec word, read by gather),
        "direct" (no table: every entry evaluated), or None: the first of the
        three whose table is small against the entry count.  ``topo_config``:
        an XGMITopoConfig for the alpha-beta constants (make_model).
        ``allocate_results=False``: only the problem is uploaded (for the node
        hashes, which are taken before it is decided which edges get entries);
        such an engine cannot build.  ``lut``: build the block table (or, without
        one, the entries) with the lookup-table kernels; None: for tables of
        more than 2 048 units and for direct evaluation.  ``use_table`` is
        the older switch: True = "full", False = "direct".  ``item_entries``:
        entries per work item of the entry kernel, 256 or 512 (512 needs a
        table); None: by problem size."""
        self.lib = _lib.load()
        self.g = g
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise _lib.ApcError("CostEngine needs a HIP device; there is no CPU path")
        if device_name is None:
            device_name = detect_device_name(self.device)
        self.device_name = device_name
        g.validate()
        sizes = g.edge_sdst.astype(np.int64) * g.edge_ssrc
        assert g.num_edges == 0 or int(sizes.max()) < 2**31, "edge block too large for 32-bit local index"

        self._keep: Dict[str, torch.Tensor] = {}

        # The problem is some thirty arrays, most of them a few kilobytes: they go up in
        # one copy.  An array is laid into a pinned staging buffer and gets its address
        # inside a device arena at once (the struct fields below need it); the arena is
        # filled by _flush_uploads when all of them are known.  Large arrays (and what
        # does not fit any more) are copied on their own.
        arena_bytes = int(min(_UPLOAD_ARENA_BYTES, (256 << 10) + 32 * g.lists.shape[0] + 160 * g.num_edges
                              + 320 * g.num_nodes + 8 * g.default_vals.shape[0]))
        stage = _upload_stage(arena_bytes)
        arena = torch.empty(arena_bytes, dtype=torch.uint8, device=self.device)
        stage_np = stage.numpy()
        used = [0]

        def up(name, arr, dtype=None):
            a = np.ascontiguousarray(arr if dtype is None else arr.astype(dtype))
            if a.dtype == np.uint32:
                a = a.view(np.int32)
            raw = a.reshape(-1).view(np.uint8) if a.dtype.fields is None else a.view(np.uint8).reshape(-1)
            n = raw.shape[0]
            off = (used[0] + 255) & ~255
            if n == 0 or n > _UPLOAD_ARENA_MAX_ARRAY or off + n > arena_bytes:
                t = torch.from_numpy(raw if a.dtype.fields is not None else a).to(self.device)
            else:
                stage_np[off:off + n] = raw
                used[0] = off + n
                t = arena[off:off + n]
                if a.dtype.fields is None:
                    t = t.view(torch.from_numpy(a[:0].reshape(-1)).dtype).view(a.shape)
            self._keep[name] = t
            return t.data_ptr() if t.numel() else None

        def flush_uploads():
            if used[0]:
                arena[:used[0]].copy_(stage[:used[0]], non_blocking=True)
                # the staging buffer is let go once the copy has run
                torch.cuda.current_stream(self.device).synchronize()
            self._keep["upload_arena"] = arena

        p = _lib.ApcProblem()
        model = make_model([int(x) for x in g.mesh_shape], g.devices_per_host, device_name, order_mode,
                           topo_config=topo_config)
        if nccl_config is not None:  # NCCL-tuning collectives instead of alpha-beta
            self._keep["nccl_plan"] = upload_nccl_plan(model, nccl_config, self.device)
        p.model = model
        p.n_meta = g.meta_rank.shape[0]
        p.meta_rank = up("meta_rank", g.meta_rank)
        p.meta_shape = up("meta_shape", g.meta_shape)
        p.meta_stride = up("meta_stride", g.meta_stride)
        p.meta_itemsize = up("meta_itemsize", g.meta_itemsize)
        p.meta_dtype = up("meta_dtype", g.meta_dtype)
        p.n_tuple = g.tuple_plc.shape[0]
        p.tuple_plc = up("tuple_plc", g.tuple_plc)
        p.n_list = g.lists.shape[0]
        p.lists = up("lists", g.lists)
        p.n_node = g.num_nodes
        p.node_nstrat = up("node_nstrat", g.node_nstrat)
        p.node_nargs = up("node_nargs", g.node_nargs)
        p.node_op = up("node_op", g.node_op)
        p.node_comp_off = up("node_comp_off", g.node_comp_off)
        p.node_edge_off = up("node_edge_off", g.node_edge_off)
        p.node_prog_off = up("node_prog_off", g.node_prog_off)
        p.node_prog_len = up("node_prog_len", g.node_prog_len)
        p.max_node_args = g.max_node_args
        p.max_rank = g.max_rank
        p.n_compute = g.num_compute
        p.n_comp_node = g.comp_nodes.shape[0]
        p.comp_nodes = up("comp_nodes", g.comp_nodes)
        p.comp_recs = up("comp_recs", g.comp_records())
        terms, _ = g.program_terms()
        p.n_prog_term = terms.shape[0]
        p.prog_terms = up("prog_terms", terms)
        p.spec_recs = up("spec_recs", g.spec_records())
        p.max_nstrat = int(g.node_nstrat[g.comp_nodes].max()) if g.comp_nodes.shape[0] else 1
        mult = g.node_multiplier if g.node_multiplier is not None else np.ones(g.num_nodes, np.int32)
        p.node_multiplier = up("node_multiplier", mult)
        p.n_prog = g.prog.shape[0]
        p.prog = up("prog", g.prog)
        p.explicit_flops = up("explicit_flops", g.explicit_flops) if g.explicit_flops is not None else None
        p.explicit_bytes = up("explicit_bytes", g.explicit_bytes) if g.explicit_bytes is not None else None
        p.n_edge = g.num_edges
        p.n_entry = g.num_entries
        p.n_slot = g.num_slots
        chunk_edge = g.chunk_edge_index()
        p.n_chunk = chunk_edge.shape[0]
        assert p.n_chunk == g.num_slots >> CHUNK_SHIFT
        p.chunk_edge = up("chunk_edge", chunk_edge)
        signed_defaults = bool(np.signbit(g.default_vals).any())
        if table_mode is None and use_table is not None:
            table_mode = "full" if use_table else "direct"
        if table_mode is None:
            table_mode = g.default_table_mode()
        if table_mode not in ("direct", "full", "compressed"):
            raise ValueError(f"unknown table_mode {table_mode!r}")
        if table_mode != "direct" and signed_defaults:
            raise ValueError("a block table needs default values with a clear sign bit")
        self.table_mode = table_mode
        squeezed = table_mode == "compressed"
        p.edges = up("edges", g.edge_records(squeezed))
        self.item_entries = g.default_item_entries(table_mode) if item_entries is None else int(item_entries)
        items = g.work_items(squeezed, self.item_entries)
        p.item_entries = self.item_entries
        p.n_item = items.shape[0]
        p.items = up("items", items)
        p.n_default = g.default_vals.shape[0]
        p.default_vals = up("default_vals", g.default_vals)
        block_edge, block_off, unit_block, _, _, block_udst = g.block_table(squeezed)
        if squeezed:
            uidx, ufirst, _ = g.run_unique_index()
            p.list_uidx = up("list_uidx", uidx)
            p.list_ufirst = up("list_ufirst", ufirst)
            p.block_udst = up("block_udst", block_udst)
        p.n_block = block_edge.shape[0]
        p.block_edge = up("block_edge", block_edge)
        p.block_off = up("block_off", block_off)
        p.table_size = int(block_off[-1])
        p.n_table_unit = unit_block.shape[0]
        p.table_unit_block = up("table_unit_block", unit_block)
        p.table_units = up("table_units", g.table_unit_records(squeezed))
        self.problem = p
        # Large tables, and direct evaluation, go through the lookup-table kernels:
        # tiles of whole matrices instead of one element per lane.
        # The library takes that route by itself when the problem carries the tile list.
        self._lut_tiles = None
        self.lut = lut if lut is not None else (table_mode == "direct" or p.n_table_unit > _LUT_TABLE_FROM)
        if self.lut and g.num_entries > 0:
            tiles = g.lut_tiles(squeezed, entries=(table_mode == "direct"))
            self._lut_tiles = (up("lut_tiles", tiles), int(tiles.shape[0]))
            if table_mode == "direct":
                p.lut_entry_tiles, p.n_lut_entry_tile = self._lut_tiles
            else:
                p.lut_table_tiles, p.n_lut_table_tile = self._lut_tiles
        flush_uploads()

        E, NC = (g.num_slots, g.num_compute) if allocate_results else (0, 0)
        self.can_build = bool(allocate_results)
        # entry arrays hold num_slots elements; padding slots stay zero
        self.compute = torch.zeros(NC, dtype=torch.float64, device=self.device)
        self.per_arg = torch.zeros(NC, dtype=torch.float64, device=self.device)
        self.comm = torch.zeros(E, dtype=torch.float64, device=self.device)
        self.cost = torch.zeros(E, dtype=torch.float64, device=self.device)
        self.flags = torch.zeros(E, dtype=torch.uint8, device=self.device)
        self.status = torch.zeros(1, dtype=torch.int32, device=self.device)
        tsize = int(self.lib.apc_pair_table_size(C.byref(p)))
        self.use_table = table_mode != "direct"
        self.table = (
            torch.empty(tsize, dtype=torch.float64, device=self.device)
            if self.use_table and allocate_results else None
        )
        self.built = False
        self._build_args = None
        # Batches of _SCORE_LANES_FROM assignments and more are scored from something
        # denser than the three entry arrays: the block table itself when the blocks
        # are large (_score_packed), else records made from the arrays on first use,
        # stale after anything rewrites the arrays.
        self.packed_scoring = g.num_edges > 0 and g.num_entries > 0
        self.large_blocks = g.num_edges > 0 and g.num_entries / g.num_edges >= _LARGE_BLOCKS_FROM
        self._recs: Optional[torch.Tensor] = None
        self._recs_valid = False
        self._recs_compact = False
        # clamp_inf of the build whose table path wrote the entry arrays as they are now,
        # None once anything else has written them: then scoring cannot read the table instead
        self._table_clamp: Optional[int] = None
        self.last_score_backend = "entry_arrays"  # what the last large batch was scored from

    def synchronize(self) -> None:
        torch.cuda.synchronize(self.device)

    # -- raw stream -----------------------------------------------------------
    def _stream(self):
        return C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)

    @staticmethod
    def _ptr(t: Optional[torch.Tensor]):
        return None if t is None or t.numel() == 0 else C.c_void_p(t.data_ptr())

    # -- kernels --------------------------------------------------------------
    def build_pair_table(self):
        if self.table is not None:
            _lib.check(
                self.lib.apc_build_pair_table(C.byref(self.problem), self._ptr(self.table), self._stream()),
                "apc_build_pair_table",
            )

    def node_compute(self):
        _lib.check(
            self.lib.apc_node_compute_costs(
                C.byref(self.problem), self._ptr(self.compute), self._ptr(self.per_arg),
                self._ptr(self.status), self._stream()),
            "apc_node_compute_costs",
        )

    def mark_results_edited(self) -> None:
        """To be called by a caller that has written into comm / cost / flags / per_arg
        itself: scoring then reads the arrays as they are (records are made again on the
        next large batch, and the block table no longer stands for the arrays)."""
        self._recs_valid = False
        self._table_clamp = None

    def edge_costs(self, clamp_inf: bool = True, want_comm: bool = True, want_flags: bool = True):
        self._recs_valid = False
        self._table_clamp = None
        _lib.check(
            self.lib.apc_edge_costs(
                C.byref(self.problem), self._ptr(self.table), self._ptr(self.per_arg),
                self._ptr(self.comm) if want_comm else None, self._ptr(self.cost),
                self._ptr(self.flags) if want_flags else None, int(bool(clamp_inf)), self._stream()),
            "apc_edge_costs",
        )

    def edge_costs_timed(self, timer, slot: int, clamp_inf: bool = True):
        """edge_costs with HIP events at the kernel's begin and end (a timer from
        apc_timer_create); the launch is otherwise identical."""
        self._recs_valid = False
        self._table_clamp = None
        _lib.check(
            self.lib.apc_edge_costs_timed(
                C.byref(self.problem), self._ptr(self.table), self._ptr(self.per_arg), self._ptr(self.comm),
                self._ptr(self.cost), self._ptr(self.flags), int(bool(clamp_inf)), timer, int(slot),
                self._stream()),
            "apc_edge_costs_timed",
        )

    def prepare(self):
        """Pair table and node compute vectors, as build() makes them: one launch,
        or, with the lookup-table kernels, the table by tiles and the node launch."""
        _lib.check(
            self.lib.apc_prepare(
                C.byref(self.problem), self._ptr(self.table), self._ptr(self.compute),
                self._ptr(self.per_arg), self._ptr(self.status), self._stream()),
            "apc_prepare",
        )

    def build_args(self):
        if not self.can_build:
            raise _lib.ApcError("this engine holds the problem only (allocate_results=False)")
        if self._build_args is None:
            self._build_args = (
                C.byref(self.problem), self._ptr(self.table), self._ptr(self.compute), self._ptr(self.per_arg),
                self._ptr(self.status), self._ptr(self.comm), self._ptr(self.cost), self._ptr(self.flags))
        return self._build_args

    def build(self, clamp_inf: bool = True):
        """All coefficients: pair table and node compute vectors, then the entry
        arrays (apc_build_all: two launches, three when the table is built by tiles)."""
        self._recs_valid = False
        # the argument list is the same from call to call apart from the stream:
        # made once, so that issuing a step costs less host time than the step takes
        args = self._build_args or self.build_args()
        stream = torch.cuda.current_stream(self.device).cuda_stream
        rc = self.lib.apc_build_all(*args, 1 if clamp_inf else 0, stream)
        if rc:
            _lib.check(rc, "apc_build_all")
        self.built = True
        self._table_clamp = (1 if clamp_inf else 0) if self.table is not None else None
        return self

    def build_timed(self, timer, slot: int, clamp_inf: bool = True):
        """build() with HIP events at the begin and end of the kernel that writes
        the entries (a timer from apc_timer_create); the launches are otherwise
        identical."""
        self.build_args()
        stream = torch.cuda.current_stream(self.device).cuda_stream
        clamp = 1 if clamp_inf else 0
        rc = self.lib.apc_build_all_timed(*self._build_args, clamp, timer, int(slot), stream)
        if rc:
            _lib.check(rc, "apc_build_all_timed")
        self._recs_valid = False
        self.built = True
        self._table_clamp = clamp if self.table is not None else None
        return self

    def set_node_multiplier(self, mult: np.ndarray) -> None:
        """Replace the objective multiplier per node (cluster multiplicity)."""
        t = self._keep["node_multiplier"]
        assert len(mult) == t.numel()
        t.copy_(torch.from_numpy(np.ascontiguousarray(mult, np.int32)))

    def load_results(self, comm, cost, flags, compute, per_arg):
        """Adopt coefficient arrays computed earlier (a saved optimizer): host
        arrays of num_slots / num_compute elements are copied to the device and
        the engine counts as built.  Nothing is recomputed."""
        g = self.g
        assert len(comm) == len(cost) == len(flags) == g.num_slots and len(compute) == len(per_arg) == g.num_compute
        self.comm.copy_(torch.from_numpy(np.ascontiguousarray(comm, np.float64)))
        self.cost.copy_(torch.from_numpy(np.ascontiguousarray(cost, np.float64)))
        self.flags.copy_(torch.from_numpy(np.ascontiguousarray(flags, np.uint8)))
        self.compute.copy_(torch.from_numpy(np.ascontiguousarray(compute, np.float64)))
        self.per_arg.copy_(torch.from_numpy(np.ascontiguousarray(per_arg, np.float64)))
        self.built = True
        self._recs_valid = False
        self._table_clamp = None
        return self

    def capture_build(self, clamp_inf: bool = True) -> "torch.cuda.CUDAGraph":
        """The launches of build() recorded in a HIP graph, for callers that
        replay a whole planning step from a graph.  On its own a replay is no
        faster than the eager launches (measured on the headline graph: 29.8 us
        a replay against 25.8 us for the two launches issued eagerly with cached
        argument lists).  The graph holds kernel nodes only (no memset nodes);
        it is valid while this engine's buffers live.  build() is run once
        eagerly first so that one-time function attributes are set outside the
        capture."""
        self.build(clamp_inf)
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.build(clamp_inf)
        return graph

    def check_status(self):
        if int(self.status.item()) != 0:
            raise ValueError(
                "a node with flops has an input dtype without a tflops entry on "
                f"{self.device_name} (the reference raises ValueError for it)"
            )

    def apply_prefetch_discount(self, scale: float = 0.0) -> int:
        assert self.built
        self._recs_valid = False
        self._table_clamp = None
        n = torch.zeros(1, dtype=torch.int64, device=self.device)
        _lib.check(
            self.lib.apc_apply_prefetch_discount(
                C.byref(self.problem), self._ptr(self.per_arg), float(scale), self._ptr(self.comm),
                self._ptr(self.cost), self._ptr(self.flags), self._ptr(n), self._stream()),
            "apc_apply_prefetch_discount",
        )
        return int(n.item())

    def objective_coeffs(self) -> torch.Tensor:
        assert self.built
        obj = torch.zeros_like(self.cost)
        _lib.check(
            self.lib.apc_objective_coeffs(C.byref(self.problem), self._ptr(self.cost), self._ptr(obj), self._stream()),
            "apc_objective_coeffs",
        )
        return obj

    def score(self, assign: torch.Tensor) -> torch.Tensor:
        """assign: uint16/int16 [n_node, n_assign] on the device -> float64 [n_assign, 6]."""
        assert self.built
        assert assign.dim() == 2 and assign.shape[0] == self.g.num_nodes and assign.is_contiguous()
        assert assign.dtype in (torch.int16, torch.uint16) and assign.device == self.comm.device
        A = assign.shape[1]
        out = torch.empty((A, 6), dtype=torch.float64, device=self.device)
        if self.packed_scoring and A >= _SCORE_LANES_FROM:
            return self._score_packed(assign, 0, 0, A, None, 0, None, out)
        _lib.check(
            self.lib.apc_score_assignments(
                C.byref(self.problem), self._ptr(self.per_arg), self._ptr(self.comm), self._ptr(self.cost),
                self._ptr(self.flags), self._ptr(assign), A, self._ptr(out), self._stream()),
            "apc_score_assignments",
        )
        return out

    def _score_packed(self, assign, seed, first, count, d_gid, first_node, init, out) -> torch.Tensor:
        """Scoring of a large batch.  A graph with large blocks: from the block
        table while the entry arrays are what the last build made of it
        (apc_score_table, 5x the rate of any walk over records there).  Else,
        and for graphs with small blocks (where the records win: 15.6 ms against
        18.0 ms from the table and 31.2 ms from the three arrays for 2^20
        assignments of the Llama-3-8B graph), from records made here if the entry
        arrays changed since: compact 16-byte
        records, several assignments per lane (apc_score_compact), while every
        cost is (comm + per_arg) + transition or its clamp (checked on the device
        when the records are made); else the 32-byte records that carry the cost
        (apc_score_packed)."""
        if (self._table_clamp is not None and _SCORE_FROM_TABLE and (self.large_blocks or not _SCORE_COMPACT)
                and count >= _SCORE_TABLE_FROM):
            aux = self._score_edge_aux(d_gid)
            _lib.check(
                self.lib.apc_score_table(
                    C.byref(self.problem), self._ptr(self.per_arg), self._ptr(self.table),
                    C.c_void_p(aux.data_ptr()), self._ptr(assign),
                    int(seed), int(first), int(count), self._ptr(d_gid), int(first_node), self.g.num_nodes,
                    self._table_clamp, min(_SCORE_PER_LANE, 4),
                    self._ptr(init), self._ptr(out), self._stream()),
                "apc_score_table")
            self.last_score_backend = "block_table"
            return out
        if not self._recs_valid:
            self._recs = None  # one kind at a time: either is as large as the entry arrays
            recs = None
            self._recs_compact = False
            if _SCORE_COMPACT:
                recs = torch.empty(self.g.num_slots * 2, dtype=torch.float64, device=self.device)
                mismatch = torch.empty(1, dtype=torch.int32, device=self.device)
                _lib.check(
                    self.lib.apc_pack_score_records16(
                        C.byref(self.problem), self._ptr(self.per_arg), self._ptr(self.comm), self._ptr(self.cost),
                        self._ptr(self.flags), self._ptr(recs), self._ptr(mismatch), self._stream()),
                    "apc_pack_score_records16")
                self._recs_compact = int(mismatch.item()) == 0
            if not self._recs_compact:
                del recs
                recs = torch.empty(self.g.num_slots * 4, dtype=torch.float64, device=self.device)
                _lib.check(
                    self.lib.apc_pack_score_records(
                        C.byref(self.problem), self._ptr(self.comm), self._ptr(self.cost), self._ptr(self.flags),
                        self._ptr(recs), self._stream()),
                    "apc_pack_score_records")
            self._recs = recs
            self._recs_valid = True
        if self._recs_compact:
            _lib.check(
                self.lib.apc_score_compact(
                    C.byref(self.problem), self._ptr(self.per_arg), self._ptr(self._recs), self._ptr(assign),
                    int(seed), int(first), int(count), self._ptr(d_gid), int(first_node), self.g.num_nodes,
                    _SCORE_PER_LANE, self._ptr(init), self._ptr(out), self._stream()),
                "apc_score_compact")
            self.last_score_backend = "compact_records"
            return out
        _lib.check(
            self.lib.apc_score_packed(
                C.byref(self.problem), self._ptr(self.per_arg), self._ptr(self._recs), self._ptr(assign),
                int(seed), int(first), int(count), self._ptr(d_gid), int(first_node), self._ptr(init),
                self._ptr(out), self._stream()),
            "apc_score_packed")
        self.last_score_backend = "records"
        return out

    def _score_msize(self) -> np.ndarray:
        """int32[num_edges]: the padded size of an edge's matrix in the block table
        if it is worth taking through LDS (_SCORE_STAGE_TILES tiles at most), else 0."""
        g = self.g
        _, block_off, _, edge_table_off, _, _ = g.block_table(self.table_mode == "compressed")
        msize = np.zeros(g.num_edges, np.int32)
        has = edge_table_off >= 0
        b = np.searchsorted(block_off, edge_table_off[has], side="right") - 1
        size = (block_off[b + 1] - block_off[b]).astype(np.int64)
        limit = _SCORE_STAGE_TILES * int(self.lib.apc_score_table_tile())
        msize[has] = np.where(size <= limit, size, 0).astype(np.int32)
        return msize

    def _score_edge_aux(self, d_gid: Optional[torch.Tensor]) -> torch.Tensor:
        """apc_score_edge_aux records of apc_score_table (int32[num_edges + 1, 4] on
        the device): what does not depend on the call is made once; the producers'
        ids for the draw follow the call's node ids."""
        g = self.g
        base = self._keep.get("score_edge_aux")
        if base is None:
            msize = self._score_msize()
            idx = np.where(msize > 0, np.arange(g.num_edges), g.num_edges)
            nxt = np.minimum.accumulate(np.concatenate([idx, [g.num_edges]])[::-1])[::-1]
            aux = np.zeros((g.num_edges + 1, 4), np.int32)
            aux[:-1, 0] = msize
            aux[:, 1] = np.where(nxt < g.num_edges, nxt, -1)
            aux[:-1, 2] = g.edge_src_node
            base = self._keep["score_edge_aux"] = torch.from_numpy(aux).to(self.device)
            self._keep["score_edge_src"] = torch.from_numpy(
                np.maximum(g.edge_src_node, 0).astype(np.int64)).to(self.device)
        if d_gid is None:
            return base
        aux = base.clone()
        aux[:-1, 2] = d_gid[self._keep["score_edge_src"]]
        return aux

    def node_hashes(self, node_phase: Optional[np.ndarray] = None) -> np.ndarray:
        """uint64[n_node] structural hash of every node (the clustering key).
        Needs only the uploaded problem, not the coefficients."""
        g = self.g
        out_list = torch.from_numpy(np.ascontiguousarray(g.node_out_list, np.int64)).to(self.device)
        phase = None
        if node_phase is not None:
            phase = torch.from_numpy(np.ascontiguousarray(node_phase, np.int32)).to(self.device)
        out = torch.empty(g.num_nodes, dtype=torch.int64, device=self.device)
        _lib.check(
            self.lib.apc_node_hashes(C.byref(self.problem), self._ptr(out_list), self._ptr(phase), self._ptr(out),
                                     self._stream()),
            "apc_node_hashes",
        )
        return out.cpu().numpy().view(np.uint64)

    def export_decision_vars(self):
        """(keys int32[E, 4], vals float64[E, 3]) on the device: the packed twin
        of the reference's ``decision_vars`` in its insertion order."""
        assert self.built
        if "export_row_base" not in self._keep:
            base, stride = self.g.export_rows()
            self._keep["export_row_base"] = torch.from_numpy(base).to(self.device)
            self._keep["export_row_stride"] = torch.from_numpy(stride).to(self.device)
        E = self.g.num_entries
        keys = torch.empty((E, 4), dtype=torch.int32, device=self.device)
        vals = torch.empty((E, 3), dtype=torch.float64, device=self.device)
        _lib.check(
            self.lib.apc_export_decision_vars(
                C.byref(self.problem), self._ptr(self.per_arg), self._ptr(self.comm), self._ptr(self.flags),
                self._ptr(self._keep["export_row_base"]), self._ptr(self._keep["export_row_stride"]),
                self._ptr(keys), self._ptr(vals), self._stream()),
            "apc_export_decision_vars",
        )
        return keys, vals

    def solution_terms(self, assign: torch.Tensor):
        """assign: int16/uint16 [n_node] on the device -> (terms float64
        [n_edge, 4] = compute, comm, transition, cost of each edge's selected
        entry; slot int64[n_edge])."""
        assert self.built
        assert assign.dim() == 1 and assign.shape[0] == self.g.num_nodes and assign.is_contiguous()
        assert assign.dtype in (torch.int16, torch.uint16) and assign.device == self.comm.device
        terms = torch.empty((self.g.num_edges, 4), dtype=torch.float64, device=self.device)
        slot = torch.empty(self.g.num_edges, dtype=torch.int64, device=self.device)
        _lib.check(
            self.lib.apc_solution_terms(
                C.byref(self.problem), self._ptr(self.per_arg), self._ptr(self.comm), self._ptr(self.cost),
                self._ptr(self.flags), self._ptr(assign), self._ptr(terms), self._ptr(slot), self._stream()),
            "apc_solution_terms",
        )
        return terms, slot

    def score_random(self, seed: int, first: int, count: int) -> torch.Tensor:
        assert self.built
        out = torch.empty((count, 6), dtype=torch.float64, device=self.device)
        if self.packed_scoring and count >= _SCORE_LANES_FROM:
            return self._score_packed(None, seed, first, count, None, 0, None, out)
        _lib.check(
            self.lib.apc_score_random_assignments(
                C.byref(self.problem), self._ptr(self.per_arg), self._ptr(self.comm), self._ptr(self.cost),
                self._ptr(self.flags), int(seed), int(first), int(count), self._ptr(out), self._stream()),
            "apc_score_random_assignments",
        )
        return out

    def score_random_window(self, seed: int, first: int, count: int, node_gid: np.ndarray, first_node: int,
                            init: Optional[torch.Tensor] = None) -> torch.Tensor:
        """score_random for a window of a larger graph (apc_score_random_window):
        draws by global node id, skips the first ``first_node`` stand-in nodes and
        continues the sums of ``init`` (the previous window's result)."""
        assert self.built
        gid = np.ascontiguousarray(node_gid, np.int32)
        assert gid.shape == (self.g.num_nodes,) and 0 <= first_node <= self.g.num_nodes
        assert init is None or (init.shape == (count, 6) and init.dtype == torch.float64 and init.is_contiguous())
        d_gid = torch.from_numpy(gid).to(self.device)
        out = torch.empty((count, 6), dtype=torch.float64, device=self.device)
        if self.packed_scoring and count >= _SCORE_LANES_FROM:
            return self._score_packed(None, seed, first, count, d_gid, first_node, init, out)
        self.last_score_backend = "entry_arrays"
        _lib.check(
            self.lib.apc_score_random_window(
                C.byref(self.problem), self._ptr(self.per_arg), self._ptr(self.comm), self._ptr(self.cost),
                self._ptr(self.flags), int(seed), int(first), int(count), self._ptr(d_gid), int(first_node),
                self._ptr(init), self._ptr(out), self._stream()),
            "apc_score_random_window",
        )
        return out

    def score_window(self, assign: torch.Tensor, first_node: int, init: Optional[torch.Tensor] = None) -> torch.Tensor:
        """score() for a window of a larger graph: explicit assignments (uint16
        [n_node, n_assign], stand-in nodes included), the first ``first_node``
        nodes contribute nothing, and the sums continue from ``init``."""
        assert self.built
        assert assign.dim() == 2 and assign.shape[0] == self.g.num_nodes and assign.is_contiguous()
        assert assign.dtype in (torch.int16, torch.uint16) and assign.device == self.comm.device
        count = assign.shape[1]
        assert 0 <= first_node <= self.g.num_nodes
        assert init is None or (init.shape == (count, 6) and init.dtype == torch.float64 and init.is_contiguous())
        out = torch.empty((count, 6), dtype=torch.float64, device=self.device)
        if self.packed_scoring and count >= _SCORE_LANES_FROM:
            return self._score_packed(assign, 0, 0, count, None, first_node, init, out)
        _lib.check(
            self.lib.apc_score_assignments_window(
                C.byref(self.problem), self._ptr(self.per_arg), self._ptr(self.comm), self._ptr(self.cost),
                self._ptr(self.flags), self._ptr(assign), count, int(first_node), self._ptr(init), self._ptr(out),
                self._stream()),
            "apc_score_assignments_window")
        self.last_score_backend = "entry_arrays"
        return out

    def _allowed_columns(self):
        """(colbits, col_off, max_words) of apc_pack_allowed_columns for the flags as they
        are now: the layout is made once per engine, the bits on every call (one pass over
        the flags; any build or pass may have rewritten them)."""
        g = self.g
        lay = self._keep.get("column_layout")
        if lay is None:
            words = (g.edge_sdst.astype(np.int64) + 63) >> 6
            size = g.edge_ssrc.astype(np.int64) * ((words + 1) & ~1)  # a column: whole pairs of words
            own = np.ones(g.num_edges, bool) if g.edge_alias is None else g.priced
            off = np.zeros(g.num_edges, np.int64)
            off[own] = np.cumsum(size[own]) - size[own]
            if g.edge_alias is not None:  # an edge without a block of its own reads its root's columns
                off[~own] = off[g.edge_alias[~own]]
            total = int(size[own].sum())
            lay = self._keep["column_layout"] = (
                torch.from_numpy(off).to(self.device), max(int(words.max()) if g.num_edges else 1, 1),
                torch.empty(max(total, 1), dtype=torch.int64, device=self.device))
        d_off, max_words, colbits = lay
        _lib.check(
            self.lib.apc_pack_allowed_columns(
                C.byref(self.problem), self._ptr(self.flags), self._ptr(d_off), int(max_words), self._ptr(colbits),
                self._stream()),
            "apc_pack_allowed_columns")
        return colbits, d_off, max_words

    def sample_feasible(self, seed: int, first: int, count: int, node_gid: Optional[np.ndarray] = None,
                        first_node: int = 0, assign: Optional[torch.Tensor] = None,
                        row_filter: Optional[dict] = None):
        """``count`` assignments drawn node by node among the strategies that select
        no forbidden (non-finite) entry against the choices made for the node's
        producers (apc_pack_allowed_columns, then apc_sample_feasible).  Returns
        (assign uint16[n_node, count] on the device, n_fallback int32[count]: nodes
        that had no such strategy and took the plain draw).  ``assign``/``first_node``:
        rows below first_node are given (a window of a larger graph); ``node_gid``:
        ids for the hashes; ``row_filter``: {node: bool per strategy}, the strategies a
        node may take at all, or "plan" for the filters feasible_plan.plan_filters makes
        for this graph (made once per engine)."""
        assert self.built
        if isinstance(row_filter, str):
            assert row_filter == "plan" and first_node == 0
            if "row_filter_plan" not in self._keep:
                from . import feasible_plan

                self._keep["row_filter_plan"] = feasible_plan.plan_filters(feasible_plan.window_masks(self.g))[0]
            row_filter = self._keep["row_filter_plan"]
        N = self.g.num_nodes
        if assign is None:
            assert first_node == 0
            assign = torch.empty((N, count), dtype=torch.uint16, device=self.device)
        assert assign.shape == (N, count) and assign.dtype == torch.uint16 and assign.is_contiguous()
        d_gid = None
        if node_gid is not None:
            d_gid = torch.from_numpy(np.ascontiguousarray(node_gid, np.int32)).to(self.device)
        fallback = torch.empty(count, dtype=torch.int32, device=self.device)
        colbits, d_off, _ = self._allowed_columns()
        d_keep = d_keep_off = None
        if row_filter:
            # bit out_idx mod 64 of word out_idx / 64, the words of the filtered nodes one after the other
            keep_off = np.full(N, -1, np.int64)
            words = []
            at = 0
            for v in sorted(row_filter):
                keep = np.asarray(row_filter[v], bool)
                assert keep.shape == (int(self.g.node_nstrat[v]),)
                padded = np.zeros(-(-keep.shape[0] // 64) * 64, np.uint8)
                padded[: keep.shape[0]] = keep
                w = np.packbits(padded, bitorder="little").view(np.uint64)
                keep_off[v] = at
                at += w.shape[0]
                words.append(w)
            d_keep = torch.from_numpy(np.concatenate(words).view(np.int64)).to(self.device)
            d_keep_off = torch.from_numpy(keep_off).to(self.device)
        _lib.check(
            self.lib.apc_sample_feasible(
                C.byref(self.problem), self._ptr(colbits), self._ptr(d_off), int(seed), int(first), int(count),
                self._ptr(d_gid), int(first_node), self._ptr(d_keep), self._ptr(d_keep_off), self._ptr(assign),
                self._ptr(fallback), self._stream()),
            "apc_sample_feasible")
        return assign, fallback

    def random_assignment(self, seed: int, a: int) -> np.ndarray:
        """The out_idx per node that score_random draws for assignment a."""
        g = self.g
        return np.asarray(
            [self.lib.apc_random_assignment(int(seed), int(a), v, int(g.node_nstrat[v])) for v in range(g.num_nodes)],
            dtype=np.int64,
        )

    # -- results on host --------------------------------------------------------
    def compact_entries(self):
        """(comm, cost, flags) on the device with one element per decision variable:
        the entry arrays without the padding between edge blocks
        (apc_compact_entries), in the order of the ILP's columns."""
        assert self.built
        g = self.g
        if "var_start" not in self._keep:
            start = np.zeros(g.num_edges + 1, np.int64)
            np.cumsum(g.block_sizes(), out=start[1:])
            self._keep["var_start"] = torch.from_numpy(start).to(self.device)
        E = g.num_entries
        comm = torch.empty(E, dtype=torch.float64, device=self.device)
        cost = torch.empty(E, dtype=torch.float64, device=self.device)
        flags = torch.empty(E, dtype=torch.uint8, device=self.device)
        _lib.check(
            self.lib.apc_compact_entries(
                C.byref(self.problem), self._ptr(self._keep["var_start"]), self._ptr(self.comm), self._ptr(self.cost),
                self._ptr(self.flags), self._ptr(comm), self._ptr(cost), self._ptr(flags), self._stream()),
            "apc_compact_entries")
        return comm, cost, flags

    def results(self, compact: bool = False) -> Dict[str, np.ndarray]:
        """The five result arrays on the host.  ``compact``: comm, cost and flags
        per decision variable (padding taken out on the device) instead of per
        slot.  They are copied into pinned memory (torch keeps freed pinned
        blocks, so only a process's first call pays for pinning) by copies that
        run back to back; the arrays returned own it."""
        self.check_status()
        src = {name: getattr(self, name) for name in ("comm", "cost", "flags", "compute", "per_arg")}
        if compact and self.g.num_slots != self.g.num_entries:
            src["comm"], src["cost"], src["flags"] = self.compact_entries()
        out = {}
        for name, t in src.items():
            dst = torch.empty(t.shape, dtype=t.dtype, pin_memory=_READBACK_PINNED)
            dst.copy_(t, non_blocking=_READBACK_PINNED)
            out[name] = dst
        torch.cuda.current_stream(self.device).synchronize()
        return {k: v.numpy() for k, v in out.items()}
