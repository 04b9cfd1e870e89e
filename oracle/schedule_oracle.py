"""CPU restatement of the lowered-graph estimator on the packed schedule.

TEST INFRASTRUCTURE ONLY: tests, the smoke check and the benchmark's CPU
baseline may import this; the product (autoparallel_amd) never does.

Follows, statement by statement, the loop of ``estimate_graph_metrics``
(reference: autoparallel/graph_passes/estimate_graph_metrics.py:45-81; the same
timeline as ``create_execution_trace``, graph_passes/debug_helpers.py:336-388)
and ``MemoryTracker.schedule_node`` of torch
(torch/_inductor/fx_passes/memory_estimator.py, ``_update_memory_for_node`` and
``_get_storages_freed_by_node``), with Python floats, ints, dicts and sets as the
reference uses them.  Input is the PackedSchedule the kernel reads, plus an
order (a permutation of the nodes; None = the graph's own).

Pinned by tests/test_oracle_schedule.py: vectors written by the reference's own
function on generated lowered graphs (tests/golden/make_schedule_vectors.py),
hand-derived timelines, and torch's MemoryTracker driven in permuted orders.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

SCHED_COMM, SCHED_WAIT, SCHED_SYNC, SCHED_NO_MEM = 1, 2, 4, 8


def schedule_metrics(ps, order: Optional[Sequence[int]] = None) -> Tuple[float, float, float, float, int]:
    """(total_time, compute_time, communication_time, exposed_comm_time, peak_memory)."""
    N = ps.n_node
    order = range(N) if order is None else [int(v) for v in order]
    launch_overhead = 1.0

    curr_time = {0: 0.0}  # estimate_graph_metrics.py:43
    global_time = {}
    compute_time = 0.0
    communication_time = 0.0
    exposed_comm_time = 0.0

    # MemoryTracker.__init__: inputs and attributes are live from the start
    scheduled = set()
    current = int(ps.initial_bytes)
    peak = current
    live_freed = set()
    readers = [set() for _ in range(ps.n_storage)]
    for v in range(N):
        for q in range(int(ps.use_off[v]), int(ps.use_off[v + 1])):
            readers[int(ps.use_st[q])].add(v)

    for v in order:
        # ---- tracker.schedule_node(node)
        scheduled.add(v)
        flags = int(ps.flags[v])
        if not flags & SCHED_NO_MEM:
            for q in range(int(ps.alloc_off[v]), int(ps.alloc_off[v + 1])):
                current += int(ps.st_bytes[int(ps.alloc_st[q])])
            peak = max(current, peak)
            for q in range(int(ps.use_off[v]), int(ps.use_off[v + 1])):
                k = int(ps.use_st[q])
                if not ps.st_freeable[k] or k in live_freed:
                    continue
                if all(u in scheduled for u in readers[k]):
                    live_freed.add(k)
                    current -= int(ps.st_bytes[k])

        # ---- timeline (estimate_graph_metrics.py:51-81)
        dur = float(ps.dur[v])
        tid = int(ps.stream[v])
        if tid not in curr_time:
            curr_time[tid] = curr_time[0]
        if flags & SCHED_COMM:
            if tid == 0 and flags & SCHED_WAIT:
                src = int(ps.wait_src[v])
                if src in global_time:
                    comm_end_time = global_time.pop(src)
                else:
                    comm_end_time = curr_time[0]
                stall = max(0.0, comm_end_time - curr_time[0])
                exposed_comm_time += stall
                curr_time[tid] = max(curr_time[tid], comm_end_time)
            else:
                curr_time[tid] = max(curr_time[0], curr_time[tid])
                communication_time += dur
        else:
            compute_time += dur
        curr_time[tid] += dur + launch_overhead
        if tid != 0:
            curr_time[0] += launch_overhead
            global_time[v] = curr_time[tid]
            if flags & SCHED_SYNC:
                stall = max(0.0, curr_time[tid] - curr_time[0])
                exposed_comm_time += stall
                curr_time[0] = max(curr_time[0], curr_time[tid])

    return (max(curr_time.values()), compute_time, communication_time, exposed_comm_time, peak)
