"""Writes tests/golden/schedule_vectors.json from the reference's own
``estimate_graph_metrics``.

Run in the build container only (the reference tree is not present anywhere
else):   python tests/golden/make_schedule_vectors.py

The reference's tests for this function (tests/test_estimate_graph_metrics.py)
assert inequalities and one sum; no test pins a timeline with collectives.
These vectors do: seeded lowered-graph descriptions (tests/schedule_graphs.py:
compute nodes, views, asynchronous collectives on three groups, the blocking
_dtensor collective, waits that are late, doubled, chained, behind a wrapper
node or on a graph input) and, for each, the five numbers the reference returns.
The two graph_passes modules are loaded by file path under a stub parent package,
as tests/golden/make_cost_vectors.py loads cost_models.

The output holds inputs (descriptions) and expected outputs only.
"""
import importlib.util
import json
import os
import sys
import types

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
sys.path.insert(0, os.path.dirname(HERE))

import make_cost_vectors as M  # noqa: E402
import schedule_graphs as SG  # noqa: E402

REF = "/root/reference/autoparallel"
OUT = os.path.join(HERE, "schedule_vectors.json")


def load_reference_estimator():
    M.load_reference_cost_models()  # imported by debug_helpers; nothing here evaluates a cost
    sub = types.ModuleType("autoparallel.graph_passes")
    sub.__path__ = [REF + "/graph_passes"]
    sys.modules["autoparallel.graph_passes"] = sub
    mods = {}
    for name in ("debug_helpers", "estimate_graph_metrics"):
        spec = importlib.util.spec_from_file_location(
            "autoparallel.graph_passes." + name, f"{REF}/graph_passes/{name}.py")
        m = importlib.util.module_from_spec(spec)
        sys.modules[spec.name] = m
        spec.loader.exec_module(m)
        mods[name] = m
    return mods["estimate_graph_metrics"].estimate_graph_metrics


def main():
    estimate = load_reference_estimator()
    cases = []
    for seed in range(48):
        desc = SG.random_description(seed, n_ops=12 + 3 * seed)
        gm, estimator = SG.build_graph(desc)
        m = estimate(gm, estimator)
        cases.append({"seed": seed, "desc": desc,
                      "metrics": [m.total_time, m.compute_time, m.communication_time, m.exposed_comm_time,
                                  int(m.peak_memory)]})
    with open(OUT, "w") as f:
        json.dump({"group_size": SG.GROUP_SIZE, "cases": cases}, f, separators=(",", ":"))
    n_wait = sum(sum(nd["kind"] == "wait" for nd in c["desc"]["nodes"]) for c in cases)
    exposed = sum(c["metrics"][3] > 0 for c in cases)
    print(f"wrote {OUT}: {len(cases)} graphs, {n_wait} waits, {exposed} with exposed communication, "
          f"{os.path.getsize(OUT)} bytes")


if __name__ == "__main__":
    main()
