"""The Python oracle against vectors written by the reference's own functions
(tests/golden/make_cost_vectors.py).  Bit-exact: the oracle restates the same
binary64 operations in the same order."""
import json

import numpy as np
import pytest

from oracle import cost_oracle as O


def _cases(golden):
    return range(int(golden["comm_ncases"][0]))


def test_comm_vectors_bit_exact(golden):
    dev = O.DeviceLimit()
    total = 0
    for k in _cases(golden):
        mesh = [int(x) for x in golden[f"comm_{k}_mesh"]]
        topo = O.Topo(mesh, int(golden[f"comm_{k}_dph"][0]))
        shape = [int(x) for x in golden[f"comm_{k}_shape"]]
        stride = [int(x) for x in golden[f"comm_{k}_stride"]]
        itemsize = int(golden[f"comm_{k}_itemsize"][0])
        src, tgt = golden[f"comm_{k}_src"], golden[f"comm_{k}_tgt"]
        want, want_fwd = golden[f"comm_{k}_cost"], golden[f"comm_{k}_cost_fwd"]
        for i in range(src.shape[0]):
            s = tuple(int(x) for x in src[i])
            t = tuple(int(x) for x in tgt[i])
            got = O.estimate_strategy_comms_cost(s, shape, stride, itemsize, t, topo, dev)
            got_fwd = O.redistribute_cost(s, shape, stride, itemsize, t, topo, dev, list(range(len(mesh))))
            assert got == want[i] or (np.isinf(got) and np.isinf(want[i])), (k, s, t, got, want[i])
            assert got_fwd == want_fwd[i] or (np.isinf(got_fwd) and np.isinf(want_fwd[i]))
            total += 1
    assert total > 20000


def test_order_rule_matters(golden):
    # the (P,P)->all-Shard reorder must be visible in the vectors, otherwise
    # they would not pin it
    k = 2
    diff = golden[f"comm_{k}_cost"] != golden[f"comm_{k}_cost_fwd"]
    assert diff.any()
    src = golden[f"comm_{k}_src"][diff]
    assert (src == 0x80).all()


def test_rw_time(golden):
    dev = O.DeviceLimit()
    for b, t in zip(golden["rw_bytes"], golden["rw_time"]):
        assert float(O.compute_read_write_time(int(b), dev)) == t
    for b, t in zip(golden["rw_fbytes"], golden["rw_ftime"]):
        assert float(O.compute_read_write_time(float(b), dev)) == t


def test_sharded_shape_stride(golden):
    mesh = [int(x) for x in golden["shard_mesh"]]
    for i in range(golden["shard_rank"].shape[0]):
        r = int(golden["shard_rank"][i])
        shape = [int(x) for x in golden["shard_shape"][i, :r]]
        stride = [int(x) for x in golden["shard_stride"][i, :r]]
        plc = [int(x) for x in golden["shard_plc"][i]]
        ns, nst = O.sharded_shape_stride(shape, stride, plc, mesh)
        assert ns == [int(x) for x in golden["shard_out_shape"][i, :r]]
        assert nst == [int(x) for x in golden["shard_out_stride"][i, :r]]
