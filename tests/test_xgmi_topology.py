"""The xGMI node topology for the alpha-beta model (an extension: the reference
has no preset for AMD systems and detects none on an MI355X): the per-dim
constants against their definition, and the two closed forms that motivate
them: a ring collective inside a node is bound by one link per direction, an
all-to-all drives all seven links of a GPU."""
import ctypes as C

import pytest

from autoparallel_amd import _lib, cost_models as cm
from oracle import cost_oracle as O

LINK = 153.6  # GB/s of one MI355X Infinity Fabric link, both directions
ONE_WAY = LINK / 2


def test_per_dim_constants():
    bw, lat, a2a = cm.mi355x_topo((8, 8), 8)
    assert bw == [50.0, ONE_WAY] and lat == [2.7, 0.6] and a2a == [50.0, 7 * ONE_WAY]
    bw, lat, a2a = cm.mi355x_topo((2, 4), 8)  # both dims inside one node
    assert bw == [ONE_WAY, ONE_WAY] and lat == [0.6, 0.6] and a2a == [1 * ONE_WAY, 3 * ONE_WAY]
    bw, lat, a2a = cm.mi355x_topo((4, 8, 8), 8)
    assert bw == [50.0, 50.0, ONE_WAY] and a2a == [50.0, 50.0, 7 * ONE_WAY]
    bw, lat, a2a = cm.mi355x_topo((16,), 8)  # a dim that spans nodes goes over the NICs
    assert bw == [50.0] and lat == [2.7] and a2a == [50.0]
    bw, _, a2a = cm.mi355x_topo((8,), 8, cm.mi300x_topo_config(nic_gbps=25.0))
    assert bw == [64.0] and a2a == [7 * 64.0]
    # the oracle's restatement of the same rule
    for mesh in ((8, 8), (2, 4), (4, 8, 8), (16,), (2, 2, 2, 8)):
        t = O.Topo(mesh, 8, xgmi=cm.mi355x_topo_config())
        assert (t.bw, t.lat, t.a2a_bw) == tuple(cm.mi355x_topo(mesh, 8))


def test_ring_is_bound_by_one_link_and_all_to_all_uses_all_seven():
    topo = O.Topo((8,), 8, xgmi=cm.mi355x_topo_config())
    nbytes = 1 << 30
    gb = nbytes / 1024**3
    n = 8
    # allreduce = reduce-scatter + allgather around a ring: 2 (n - 1) steps of 1/n of the bytes,
    # each over one link in one direction
    want_ar = 6.6 + 2 * (n - 1) * 0.6 + (gb * 2 * (n - 1) / n) / ONE_WAY * 1e6
    assert O.collective_comm_cost("allreduce", nbytes, topo, 0) == want_ar
    want_ag = 6.6 + (n - 1) * 0.6 + (gb * (n - 1) / n) / ONE_WAY * 1e6
    assert O.collective_comm_cost("allgather", nbytes, topo, 0) == want_ag
    assert O.collective_comm_cost("reduce_scatter", nbytes, topo, 0) == want_ag
    # all_to_all: the same (n - 1)/n of the bytes, spread over the 7 direct links at once
    # (and the reference's factor of 5 on the whole term, which this preset keeps)
    want_a2a = (6.6 + (n - 1) * 0.6 + (gb * (n - 1) / n) / (7 * ONE_WAY) * 1e6) * 5
    assert O.collective_comm_cost("all_to_all", nbytes, topo, 0) == want_a2a
    # for a large message: seven times less wire time than the allgather of the same bytes
    wire = lambda t, scale: t / scale - 6.6 - (n - 1) * 0.6
    assert wire(want_ag, 1) / wire(want_a2a, 5) == pytest.approx(7.0, rel=1e-12)
    # without a config: the reference's constants, all_to_all on the same bandwidth
    ref = O.Topo((8,), 8)
    assert ref.a2a_bw is None and ref.bw == [87.7]


def test_detection_and_selection():
    assert cm.detect_mesh_topo_config("AMD Instinct MI355X") == cm.mi355x_topo_config()
    assert cm.detect_mesh_topo_config("AMD Instinct MI350X").link_gbps == 153.6
    assert cm.detect_mesh_topo_config("AMD Instinct MI300X").link_gbps == 128.0
    assert cm.detect_mesh_topo_config("NVIDIA H100") is None
    assert cm.get_mesh_topo_config() is None
    cm.set_mesh_topo_config(cm.mi355x_topo_config())
    try:
        assert cm.get_mesh_topo_config().links_per_gpu == 7
    finally:
        cm.set_mesh_topo_config(None)
    assert cm.get_mesh_topo_config() is None


def test_bad_config_is_refused():
    lib = _lib.load()
    cfg = _lib.ApcXgmiConfig(8, 7, 0.0, 50.0, 0.6, 2.7)
    shape = (C.c_int32 * 4)(8, 1, 1, 1)
    out = [(C.c_double * 4)() for _ in range(3)]
    rc = lib.apc_xgmi_topology(C.byref(cfg), C.addressof(shape), 1, *[C.addressof(o) for o in out])
    assert rc == -1 and b"positive" in lib.apc_last_error()
