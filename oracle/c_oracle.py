"""ctypes wrapper of oracle/cost_oracle.c.  TEST INFRASTRUCTURE ONLY (tests and
the cpu_baseline leg of the benchmark); nothing under autoparallel_amd/ may
import it.  Build the library with ``make -C oracle``."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libcost_oracle.so")

MI355X_GMEM_BW = 8.0 * (1024**4)
MI355X_TFLOPS = [78.6, 157.3, 2516.6, 2516.6, 5033.2, 0.0, 0.0, 0.0]


class Model(C.Structure):
    _fields_ = [("ndim", C.c_int32), ("mesh", C.c_int32 * 4), ("bw", C.c_double * 4), ("lat", C.c_double * 4),
                ("gmem_bw", C.c_double), ("tflops", C.c_double * 8)]


_PTRS = ["meta_rank", "meta_shape", "meta_stride", "meta_itemsize", "meta_dtype", "tuple_plc", "lists"]
_NODE = ["node_nstrat", "node_nargs", "node_op", "node_comp_off", "node_edge_off", "node_prog_off", "prog",
         "explicit_flops", "explicit_bytes"]
_EDGE = ["edge_src_node", "edge_ssrc", "edge_sdst", "edge_dst_list", "edge_src_list", "edge_off", "edge_flags",
         "edge_default_off", "default_vals"]


class Graph(C.Structure):
    _fields_ = ([("m", Model)] + [(n, C.c_void_p) for n in _PTRS] + [("n_node", C.c_int32)]
                + [(n, C.c_void_p) for n in _NODE] + [(n, C.c_void_p) for n in _EDGE])


def load(build: bool = True) -> C.CDLL:
    if build and (not os.path.exists(LIB) or os.path.getmtime(LIB) < os.path.getmtime(os.path.join(HERE, "cost_oracle.c"))):
        subprocess.run(["make", "-C", HERE], check=True, capture_output=True)
    lib = C.CDLL(LIB)
    lib.oc_build.restype = C.c_int
    lib.oc_build.argtypes = [C.POINTER(Graph), C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.oc_redistribute.restype = C.c_double
    lib.oc_topology.restype = None
    return lib


_DTYPES = {"meta_rank": np.int32, "meta_shape": np.int64, "meta_stride": np.int64, "meta_itemsize": np.int32,
           "meta_dtype": np.int32, "tuple_plc": np.uint8, "lists": np.uint32, "node_nstrat": np.int32,
           "node_nargs": np.int32, "node_op": np.int32, "node_comp_off": np.int64, "node_edge_off": np.int32,
           "node_prog_off": np.int64, "prog": np.int64, "explicit_flops": np.int64, "explicit_bytes": np.int64,
           "edge_src_node": np.int32, "edge_ssrc": np.int32, "edge_sdst": np.int32, "edge_dst_list": np.int64,
           "edge_src_list": np.int64, "edge_off": np.int64, "edge_flags": np.int32, "edge_default_off": np.int64,
           "default_vals": np.float64}


class COracle:
    """Holds the packed graph's arrays for the C library."""

    def __init__(self, g):
        self.lib = load()
        self.g = g
        self._keep = {}
        cg = Graph()
        nd = len(g.mesh_shape)
        cg.m.ndim = nd
        mesh = (C.c_int32 * 4)(*([int(x) for x in g.mesh_shape] + [1] * (4 - nd)))
        cg.m.mesh = mesh
        bw, lat = (C.c_double * 4)(), (C.c_double * 4)()
        self.lib.oc_topology(mesh, nd, int(g.devices_per_host), bw, lat)
        cg.m.bw, cg.m.lat = bw, lat
        cg.m.gmem_bw = MI355X_GMEM_BW
        cg.m.tflops = (C.c_double * 8)(*MI355X_TFLOPS)
        cg.n_node = g.num_nodes
        for name, dt in _DTYPES.items():
            a = getattr(g, name)
            if a is None:
                setattr(cg, name, None)
                continue
            a = np.ascontiguousarray(a, dt)
            self._keep[name] = a
            setattr(cg, name, a.ctypes.data if a.size else None)
        self.cg = cg

    def build(self, v0: int = 0, v1: int = -1, threads: int = 1, out=None):
        g = self.g
        v1 = g.num_nodes if v1 < 0 else v1
        if out is None:
            out = {"comm": np.zeros(g.num_slots), "cost": np.zeros(g.num_slots),
                   "transition": np.zeros(g.num_slots, np.uint8), "compute": np.zeros(g.num_compute)}
        rc = self.lib.oc_build(C.byref(self.cg), int(v0), int(v1), int(threads), out["comm"].ctypes.data,
                               out["cost"].ctypes.data, out["transition"].ctypes.data, out["compute"].ctypes.data)
        if rc != 0:
            raise ValueError("a node with flops has an input dtype without a tflops entry")
        return out
