"""The device table (apc_device_limits and the oracle's DEVICE_TABLE) against what
the reference's own lookups answer for driver-style device names:
tests/golden/device_table_vectors.json, written by
tests/golden/make_device_table_vectors.py from
autoparallel/cost_models/compute_estimation.py:257-289."""
import ctypes
import json
import os

import pytest

from oracle import cost_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
DTYPES = ("float64", "float32", "float16", "bfloat16", "int8")  # order of apc_model.tflops


@pytest.fixture(scope="module")
def vectors():
    with open(os.path.join(HERE, "golden", "device_table_vectors.json")) as f:
        return json.load(f)


def test_fixture_covers_every_row(vectors):
    # every row of the table is reached by at least one name, and so are the three special cases:
    # a board name (PG509), a name that two rows match, a name that none matches
    reached = {(v["gmem_bandwidth"], tuple(sorted(v["tflops"].items()))) for v in vectors.values() if "error" not in v}
    assert len(reached) == len(O.DEVICE_TABLE)  # the rows are pairwise different
    assert "error" in vectors["NVIDIA GeForce RTX 4090"] and "error" not in vectors["NVIDIA PG509-210"]
    assert vectors["NVIDIA H100 and A100"] == vectors["H100"] == vectors["NVIDIA A100 and H100"]


def test_oracle_table_matches_reference_lookups(vectors):
    for name, want in vectors.items():
        if "error" in want:
            with pytest.raises(ValueError, match="Unsupported device"):
                O.DeviceLimit.named(name)
            continue
        got = O.DeviceLimit.named(name)
        assert got.gmem_bandwidth == float.fromhex(want["gmem_bandwidth"]), name
        for code, label in enumerate(DTYPES):
            ref = want["tflops"][label]
            if ref is None:
                assert code not in got.tflops, (name, label)
            else:
                assert float(got.tflops[code]) == float.fromhex(ref), (name, label)


def test_library_table_matches_reference_lookups(vectors):
    from autoparallel_amd import _lib

    lib = _lib.load()
    m = _lib.ApcModel()
    for name, want in vectors.items():
        rc = lib.apc_device_limits(name.encode(), ctypes.byref(m))
        if "error" in want:
            assert rc != 0 and b"Unsupported device" in lib.apc_last_error(), name
            continue
        assert rc == 0, name
        assert m.gmem_bw == float.fromhex(want["gmem_bandwidth"]), name
        for code, label in enumerate(DTYPES):
            ref = want["tflops"][label]
            # a dtype the reference refuses on this device is 0 in the model (the host mirror raises for it)
            assert m.tflops[code] == (0.0 if ref is None else float.fromhex(ref)), (name, label)
