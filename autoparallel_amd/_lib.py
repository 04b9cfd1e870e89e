"""ctypes binding of libapc_hip.so (the C ABI declared in include/apc.h).

There is no fallback: if the library is missing, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libapc_hip.so")

MAX_MESH_DIMS = 4
NUM_DTYPES = 8


class ApcModel(C.Structure):
    _fields_ = [
        ("ndim", C.c_int32),
        ("mesh_shape", C.c_int32 * MAX_MESH_DIMS),
        ("mesh_bw", C.c_double * MAX_MESH_DIMS),
        ("mesh_lat", C.c_double * MAX_MESH_DIMS),
        ("gmem_bw", C.c_double),
        ("tflops", C.c_double * NUM_DTYPES),
        ("order_mode", C.c_int32),
        ("reserved", C.c_int32),
        ("nccl_plan", C.c_void_p),
        ("mesh_a2a_bw", C.c_double * MAX_MESH_DIMS),
    ]


class ApcXgmiConfig(C.Structure):
    _fields_ = [
        ("gpus_per_node", C.c_int32),
        ("links_per_gpu", C.c_int32),
        ("link_gbps", C.c_double),
        ("nic_gbps", C.c_double),
        ("lat_intra_us", C.c_double),
        ("lat_inter_us", C.c_double),
    ]


NCCL_MAX_CAND = 10
NCCL_TABLE_LEN = 24


class ApcNcclConfig(C.Structure):
    _fields_ = [
        ("arch", C.c_int32),
        ("num_nodes", C.c_int32),
        ("gpus_per_node", C.c_int32),
        ("num_channels", C.c_int32),
        ("has_nvswitch", C.c_int32),
        ("has_collnet", C.c_int32),
        ("bw_intra", C.c_double),
        ("bw_inter", C.c_double),
        ("net_latency", C.c_double),
    ]


class ApcNcclCand(C.Structure):
    _fields_ = [("lat", C.c_double), ("bw", C.c_double), ("flags", C.c_int32), ("proto", C.c_int32)]


class ApcNcclDim(C.Structure):
    _fields_ = [
        ("n_ranks", C.c_int32),
        ("n_nodes", C.c_int32),
        ("ppn", C.c_int32),
        ("n_channels", C.c_int32),
        ("bw_intra", C.c_double),
        ("bw_inter", C.c_double),
        ("n_cand", C.c_int32 * 4),
        ("cand", (ApcNcclCand * NCCL_MAX_CAND) * 4),
        ("ring_corr", C.c_double * NCCL_TABLE_LEN),
        ("a2a_remote", C.c_double),
        ("a2a_log_nodes", C.c_int32),
        ("reserved", C.c_int32),
    ]


class ApcNcclPlan(C.Structure):
    _fields_ = [
        ("ndim", C.c_int32),
        ("reserved", C.c_int32),
        ("dim", ApcNcclDim * MAX_MESH_DIMS),
        ("tree_corr", (C.c_double * NCCL_TABLE_LEN) * 3),
        ("nvls_tree_ramp", C.c_double * NCCL_TABLE_LEN),
        ("full_mesh_ramp", C.c_double * NCCL_TABLE_LEN),
        ("a2a_nic_ramp", C.c_double * NCCL_TABLE_LEN),
    ]


class ApcProblem(C.Structure):
    _fields_ = [
        ("model", ApcModel),
        ("n_meta", C.c_int32),
        ("meta_rank", C.c_void_p),
        ("meta_shape", C.c_void_p),
        ("meta_stride", C.c_void_p),
        ("meta_itemsize", C.c_void_p),
        ("meta_dtype", C.c_void_p),
        ("n_tuple", C.c_int32),
        ("tuple_plc", C.c_void_p),
        ("n_list", C.c_int64),
        ("lists", C.c_void_p),
        ("n_node", C.c_int32),
        ("node_nstrat", C.c_void_p),
        ("node_nargs", C.c_void_p),
        ("node_op", C.c_void_p),
        ("node_comp_off", C.c_void_p),
        ("node_edge_off", C.c_void_p),
        ("node_prog_off", C.c_void_p),
        ("node_prog_len", C.c_void_p),
        ("max_node_args", C.c_int32),
        ("max_rank", C.c_int32),
        ("n_compute", C.c_int64),
        ("n_comp_node", C.c_int32),
        ("max_nstrat", C.c_int32),
        ("comp_nodes", C.c_void_p),
        ("node_multiplier", C.c_void_p),
        ("n_prog", C.c_int64),
        ("prog", C.c_void_p),
        ("explicit_flops", C.c_void_p),
        ("explicit_bytes", C.c_void_p),
        ("n_edge", C.c_int32),
        ("edges", C.c_void_p),
        ("n_entry", C.c_int64),
        ("n_slot", C.c_int64),
        ("n_chunk", C.c_int64),
        ("chunk_edge", C.c_void_p),
        ("n_item", C.c_int32),
        ("items", C.c_void_p),
        ("n_default", C.c_int64),
        ("default_vals", C.c_void_p),
        ("n_block", C.c_int32),
        ("block_edge", C.c_void_p),
        ("block_off", C.c_void_p),
        ("table_size", C.c_int64),
        ("n_table_unit", C.c_int32),
        ("table_unit_block", C.c_void_p),
        ("list_uidx", C.c_void_p),
        ("list_ufirst", C.c_void_p),
        ("block_udst", C.c_void_p),
        ("comp_recs", C.c_void_p),
        ("item_entries", C.c_int32),
        ("table_units", C.c_void_p),
        ("spec_recs", C.c_void_p),
        ("n_prog_term", C.c_int64),
        ("prog_terms", C.c_void_p),
        ("lut_table_tiles", C.c_void_p),
        ("n_lut_table_tile", C.c_int64),
        ("lut_entry_tiles", C.c_void_p),
        ("n_lut_entry_tile", C.c_int64),
    ]


class ApcSchedule(C.Structure):
    """apc_schedule of include/apc.h."""

    _fields_ = [
        ("n_node", C.c_int32),
        ("n_stream", C.c_int32),
        ("dur", C.c_void_p),
        ("stream", C.c_void_p),
        ("flags", C.c_void_p),
        ("wait_src", C.c_void_p),
        ("n_storage", C.c_int32),
        ("st_bytes", C.c_void_p),
        ("st_freeable", C.c_void_p),
        ("st_users", C.c_void_p),
        ("alloc_off", C.c_void_p),
        ("alloc_st", C.c_void_p),
        ("use_off", C.c_void_p),
        ("use_st", C.c_void_p),
        ("initial_bytes", C.c_int64),
        ("comm_slot", C.c_void_p),
        ("n_comm", C.c_int32),
    ]


_SIGNATURES = {
    "apc_version": (C.c_int, []),
    "apc_last_error": (C.c_char_p, []),
    "apc_mesh_topology": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]),
    "apc_device_limits": (C.c_int, [C.c_char_p, C.POINTER(ApcModel)]),
    "apc_xgmi_topology": (
        C.c_int, [C.POINTER(ApcXgmiConfig), C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_nccl_plan_build": (C.c_int, [C.POINTER(ApcNcclConfig), C.c_void_p, C.c_int32, C.POINTER(ApcNcclPlan)]),
    "apc_nccl_plan_for_topo": (
        C.c_int,
        [C.POINTER(ApcNcclConfig), C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_double, C.c_double,
         C.POINTER(ApcNcclPlan)]),
    "apc_pair_table_size": (C.c_int64, [C.POINTER(ApcProblem)]),
    "apc_build_pair_table": (C.c_int, [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p]),
    "apc_node_compute_costs": (
        C.c_int, [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_edge_costs": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_int32, C.c_void_p]),
    "apc_timer_create": (C.c_int, [C.c_int32, C.POINTER(C.c_void_p)]),
    "apc_timer_destroy": (C.c_int, [C.c_void_p]),
    "apc_timer_elapsed_ms": (C.c_int, [C.c_void_p, C.c_int32, C.POINTER(C.c_float)]),
    "apc_edge_costs_timed": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_int32, C.c_void_p, C.c_int32, C.c_void_p]),
    "apc_prepare": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_build_all": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]),
    "apc_build_all_noalloc": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_int32, C.c_void_p]),
    "apc_build_pair_table_lut": (C.c_int, [C.POINTER(ApcProblem), C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]),
    "apc_edge_costs_lut": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32,
         C.c_void_p]),
    "apc_edge_costs_lut_timed": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32,
         C.c_void_p, C.c_int32, C.c_void_p]),
    "apc_calibration_copy": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
    "apc_apply_prefetch_discount": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_double, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_void_p]),
    "apc_objective_coeffs": (C.c_int, [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_node_hashes": (C.c_int, [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_export_decision_vars": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_void_p]),
    "apc_compact_entries": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_void_p]),
    "apc_solution_terms": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_void_p]),
    "apc_score_assignments": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_int64, C.c_void_p, C.c_void_p]),
    "apc_score_random_assignments": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64,
         C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]),
    "apc_score_assignments_window": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32,
         C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_random_assignment": (C.c_uint32, [C.c_uint64, C.c_int64, C.c_int32, C.c_int32]),
    "apc_pack_allowed_columns": (
        C.c_int, [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p]),
    "apc_sample_feasible": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_uint64, C.c_int64, C.c_int64, C.c_void_p, C.c_int32,
         C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_sample_rank": (C.c_uint32, [C.c_uint64, C.c_int64, C.c_int32, C.c_uint32]),
    "apc_local_shapes": (
        C.c_int,
        [C.POINTER(ApcModel), C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_void_p]),
    "apc_collective_costs": (
        C.c_int,
        [C.POINTER(ApcModel), C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_rw_times": (C.c_int, [C.POINTER(ApcModel), C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_filter_strategies": (
        C.c_int,
        [C.POINTER(ApcModel), C.c_int32, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p,
         C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_enumerate_input_options": (
        C.c_int,
        [C.POINTER(ApcModel), C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_void_p]),
    "apc_build_all_timed": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_int32, C.c_void_p, C.c_int32, C.c_void_p]),
    "apc_score_random_window": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_int64, C.c_int64,
         C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_pack_score_records": (
        C.c_int, [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_score_packed": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_int64, C.c_int64, C.c_void_p,
         C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_pack_score_records16": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_score_compact": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_int64, C.c_int64, C.c_void_p,
         C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_score_table": (
        C.c_int,
        [C.POINTER(ApcProblem), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_int64,
         C.c_int64, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "apc_score_table_tile": (C.c_int, []),
    "apc_schedule_metrics": (
        C.c_int,
        [C.POINTER(ApcSchedule), C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None


ABI_VERSION = 5  # apc_version() of the library whose struct layouts this module mirrors


class ApcError(RuntimeError):
    pass


def load() -> C.CDLL:
    """Load libapc_hip.so; raise (never fall back) if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ApcError(
            f"{LIB_PATH} is missing: build it with `python -m autoparallel_amd.csrc.build` "
            "(hipcc, gfx950). There is no CPU fallback."
        )
    lib = C.CDLL(LIB_PATH)
    lib.apc_version.restype = C.c_int
    if lib.apc_version() != ABI_VERSION:
        # the structs mirrored here are the ones of include/apc.h at this version: a library
        # built from other sources would read them wrongly
        raise ApcError(f"{LIB_PATH} has ABI version {lib.apc_version()}, this package needs {ABI_VERSION}: "
                       "rebuild it with `python -m autoparallel_amd.csrc.build`")
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _warn_if_stale()
    _lib = lib
    return lib


def _warn_if_stale() -> None:
    """A library older than a source next to it runs kernels those sources no
    longer describe (an edited kernel, a record laid out differently): say so."""
    here = os.path.dirname(LIB_PATH)
    srcs = [os.path.join(here, "csrc", f) for f in os.listdir(os.path.join(here, "csrc"))
            if f.endswith((".hip", ".cpp", ".h"))] if os.path.isdir(os.path.join(here, "csrc")) else []
    header = os.path.join(os.path.dirname(here), "include", "apc.h")
    if os.path.exists(header):
        srcs.append(header)
    built = os.path.getmtime(LIB_PATH)
    newer = [os.path.basename(f) for f in srcs if os.path.getmtime(f) > built]
    if newer:
        import warnings

        warnings.warn(f"{LIB_PATH} is older than {', '.join(sorted(newer))}: rebuild it with "
                      "`python -m autoparallel_amd.csrc.build`", RuntimeWarning, stacklevel=3)


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().apc_last_error().decode(errors="replace")
        raise ApcError(f"{what} failed ({rc}): {msg}")
