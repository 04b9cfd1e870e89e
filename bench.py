"""Benchmark of the sharding-search cost engine on one MI355X.

A step is one build of every ILP coefficient of the workload graph, with the
packed problem already resident in HBM: pair table, node compute vectors, and
the entry kernel that writes comm / cost / flags for all E decision variables.
``value`` is that resident rebuild (``value_is``); ``end_to_end_cold`` is the same
work from a fresh packed problem on the host to the coefficients back on the host
(validation, layout, descriptor upload, one build, read-back;
``end_to_end_warm_layout``: with the layout kept from an earlier engine), and
``cpu_baseline`` the per-entry Python oracle on this box's host, which pays its
memoisation inside its timed region as the reference does.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Prints one JSON line (see the keys below).  A step issues the two launches
(``--launch graph`` replays a HIP graph of them instead: measured slower on
this stack, 29.8 us against 25.8 us per step); ``roofline`` is for the dominant
kernel (edge_cost_kernel), timed with HIP events on the launch stream inside the
timed steps (on a sample of them, launched with the event pair attached to the
kernel's dispatch: every 6th step of a short region, 25 steps of a long one).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak


def workloads():
    from autoparallel_amd import graphgen as G

    return {
        # the configuration the metric is quoted on
        "llama3_8b_fwd_bwd_mesh8x8": lambda: G.config_llama3_8b(),
        # configs[0]
        "gpt2_small_fwd_bwd_mesh8": lambda: G.config_gpt2_small(),
        # configs[2] at reduced depth fits a quick run; full depth via --layers
        "llama3_70b_fwd_bwd_mesh4x8x8": lambda: G.config_llama3_70b(),
        # configs[3] and a seeded slice of configs[4] (3 000 of its 200 000 nodes)
        "moe_16l_fwd_bwd_mesh8x8": lambda: G.config_moe(),
        "stress_3k_mesh4x8x8": lambda: G.stress_graph(3000, (4, 8, 8), seed=0),
    }


def read_traffic(workload):
    """HBM bytes per launch of the entry kernel from the committed rocprofv3
    counter summary (profiles/edge_cost_item_kernel_<workload>_traffic.txt), if any."""
    path = os.path.join(ROOT, "profiles", f"edge_cost_item_kernel_{workload}_traffic.txt")
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("traffic_bytes_per_launch="):
            return float(line.split("=", 1)[1])
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="llama3_8b_fwd_bwd_mesh8x8")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--score-assignments", type=int, default=1 << 20,
                    help="also score this many on-device generated assignments (0 = skip)")
    ap.add_argument("--schedules", type=int, default=16384,
                    help="also price this many candidate orders of a lowered 32-layer schedule (0 = skip)")
    ap.add_argument("--fx-layers", type=int, default=32,
                    help="also plan the traced transformers Llama-3-8B with this many layers through "
                         "ShardingOptimizer and report its host time (0 = skip)")
    ap.add_argument("--fx-solve", action="store_true",
                    help="also solve the two clustered problems of the FX figure (input pinned to "
                         "(Shard(0), Replicate()), parameter-memory budget 1/64): minutes of one host core")
    ap.add_argument("--launch", choices=["graph", "eager"], default="eager",
                    help="how a step is issued: replay of a HIP graph of its launches, or the launches themselves")
    ap.add_argument("--direct", action="store_true", help="evaluate every entry directly (no block table)")
    ap.add_argument("--table-mode", choices=["full", "compressed", "direct"], default=None,
                    help="force the block-table layout (default: chosen from the table sizes)")
    ap.add_argument("--windowed", type=int, default=2048, metavar="ASSIGNMENTS",
                    help="also build and score configs[4] at its full 200 000 nodes window by window with this many "
                         "assignments, plain and feasible draws (about 30 s of wall time with 14 host workers; 0 = skip)")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="after the timed steps, also launch the plain copy kernel on this many MiB "
                         "(the known-traffic reference for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path needs no second one); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from autoparallel_amd.engine import CostEngine

    t0 = time.perf_counter()
    g = workloads()[args.workload]()
    t_gen = time.perf_counter() - t0
    E = g.num_entries

    t0 = time.perf_counter()
    eng = CostEngine(g, table_mode="direct" if args.direct else args.table_mode)
    torch.cuda.synchronize()
    t_first_engine = time.perf_counter() - t0  # includes the creation of the HIP context

    # End to end, on a warm process (HIP context up, pinned buffers allocated before
    # the clock starts): an engine from the packed problem on the host (validation,
    # layout records, descriptor upload), one build, and the five result arrays copied
    # into pinned host memory.  "cold": from a fresh PackedGraph, whose block-table
    # layout, work items, record arrays and validation are all made inside the clock,
    # as for a problem seen for the first time.  "warm_layout": from the graph the first
    # engine was made from, which keeps those layouts.
    import dataclasses

    pinned = {k: torch.empty(t.shape, dtype=t.dtype, pin_memory=True)
              for k, t in (("comm", eng.comm), ("cost", eng.cost), ("flags", eng.flags),
                           ("compute", eng.compute), ("per_arg", eng.per_arg))}

    def end_to_end(fresh: bool) -> dict:
        runs = {"engine_construct": [], "build": [], "readback": []}
        for _ in range(5):
            gg = dataclasses.replace(g) if fresh else g  # a copy of the fields only: none of the cached layouts
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            eng2 = CostEngine(gg, table_mode=args.table_mode if fresh else eng.table_mode)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            eng2.build(clamp_inf=True)
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            for k, dst in pinned.items():
                dst.copy_(getattr(eng2, k), non_blocking=True)
            torch.cuda.synchronize()
            t3 = time.perf_counter()
            runs["engine_construct"].append(t1 - t0)
            runs["build"].append(t2 - t1)
            runs["readback"].append(t3 - t2)
            del eng2
        best = int(np.argmin([sum(x) for x in zip(*runs.values())]))
        return {k: v[best] for k, v in runs.items()}

    e2e = end_to_end(False)
    e2e_cold = end_to_end(True)
    t_e2e, t_e2e_cold = sum(e2e.values()), sum(e2e_cold.values())

    # before the timed region: the prepare kernel bracketed the same way, for the report
    pe = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(20)]
    for a, b in pe:
        a.record()
        eng.prepare()
        b.record()
        eng.edge_costs(clamp_inf=True)
    torch.cuda.synchronize()

    for _ in range(args.warmup):
        eng.build()
    torch.cuda.synchronize()
    graph = eng.capture_build(clamp_inf=True) if args.launch == "graph" else None
    if graph is not None:
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()

    # HIP events on the launch stream (torch's current stream is the one the
    # engine launches on), recorded at the begin and end of the dominant kernel
    # (apc_build_all_timed: the events are attached to the kernel's own dispatch,
    # so dispatch latency is not counted).
    import ctypes as C

    # The event pair costs about 30 us of host time per launch on this stack, more
    # than the whole step: on every launch it would make the loop host-bound.  So
    # a sample of the timed region's steps carries events: the last step of every
    # full group of `stride` steps (10 in a short region, 1/25 of a long one), when the
    # queue holds the steps issued ahead and the pair's host time hides behind them.
    # Measured at --steps 20: 24.9-25.2 us per step without any pair, 25.5-26.0 with two,
    # 26.2-26.9 with four.
    stride = max(1, min(max(10, args.steps // 25), args.steps))
    n_timed = max(1, args.steps // stride)
    timer = C.c_void_p()
    assert eng.lib.apc_timer_create(n_timed, C.byref(timer)) == 0
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        if k % stride == stride - 1:
            eng.build_timed(timer, k // stride, clamp_inf=True)
        elif graph is not None:
            graph.replay()
        else:
            eng.build(clamp_inf=True)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    eng.check_status()
    ms = C.c_float()
    t_edge = 0.0
    for k in range(n_timed):
        assert eng.lib.apc_timer_elapsed_ms(timer, k, C.byref(ms)) == 0
        t_edge += ms.value
    t_edge = t_edge / n_timed * 1e-3
    eng.lib.apc_timer_destroy(timer)
    # a larger sample of the same launch, after the clock has stopped (not part of
    # `value`): every step carries the event pair, issued behind a queue of plain steps
    n_after = 32
    assert eng.lib.apc_timer_create(n_after, C.byref(timer)) == 0
    for k in range(n_after):
        for _ in range(4):
            eng.build(clamp_inf=True)
        eng.build_timed(timer, k, clamp_inf=True)
    torch.cuda.synchronize()
    after = []
    for k in range(n_after):
        assert eng.lib.apc_timer_elapsed_ms(timer, k, C.byref(ms)) == 0
        after.append(ms.value * 1e-3)
    eng.lib.apc_timer_destroy(timer)
    t_edge_after = float(np.mean(after))
    # and the same launch 100 times back to back between two events on the stream: no event
    # pair inside, so no launch carries the system-scope release a timed one ends with
    # (the entry kernel alone: table and per-arg terms are those of the last build)
    n_b2b = 100
    ev_a, ev_b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(5):
        eng.edge_costs(clamp_inf=True)
    ev_a.record()
    for _ in range(n_b2b):
        eng.edge_costs(clamp_inf=True)
    ev_b.record()
    torch.cuda.synchronize()
    t_edge_b2b = ev_a.elapsed_time(ev_b) * 1e-3 / n_b2b

    if args.calibration_copy_mib > 0:
        nbytes = args.calibration_copy_mib << 20
        a = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        b = torch.empty_like(a)
        for _ in range(5):
            eng.lib.apc_calibration_copy(C.c_void_p(a.data_ptr()), C.c_void_p(b.data_ptr()), nbytes, eng._stream())
        torch.cuda.synchronize()

    t_prep = sum(a.elapsed_time(b) for a, b in pe) / len(pe) * 1e-3
    ms_per_step = elapsed / args.steps * 1e3

    # algorithmic bytes of one edge_cost_kernel launch: per entry one fp64 comm,
    # one fp64 cost and one flag byte written (17 B); per edge its S_dst + S_src
    # spec words (4 B each) and its 64-byte record read once.  Table rows and
    # per-arg terms are re-read from cache and not counted.
    desc_bytes = int((g.edge_sdst.astype(np.int64) + g.edge_ssrc).sum()) * 4 + 64 * g.num_edges
    algo_bytes = 17 * E + desc_bytes
    achieved = algo_bytes / t_edge / 1e9

    out = {
        "metric": "cost entries/sec (all ILP coefficients of the graph built per step)",
        "value": E / (elapsed / args.steps),
        "value_is": "resident_rebuild: packed problem, block-table layout and work items already in HBM; "
                    "see end_to_end_cold for the figure from host arrays to host arrays",
        "launch": args.launch,
        "unit": "entries/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": {
            "workload": args.workload,
            "mesh": [int(x) for x in g.mesh_shape],
            "devices_per_host": g.devices_per_host,
            "nodes": g.num_nodes,
            "edges": g.num_edges,
            "entries": E,
            "strategies": int(g.node_nstrat.sum()),
            "tensor_metas": int(g.meta_rank.shape[0]),
            "placement_tuples": int(g.tuple_plc.shape[0]),
            "block_table": bool(eng.use_table),
            "table_mode": eng.table_mode,
            "block_table_doubles": int(eng.table.numel()) if eng.table is not None else 0,
            "compute_slots": g.num_compute,
            "evaluated_nodes": int(g.comp_nodes.shape[0]),
            "device": eng.device_name,
        },
        "coefficient_build_wall_s": elapsed / args.steps,
        "kernel_s": {"prepare(pair_table+node_compute)": t_prep, "edge_cost": t_edge},
        "host_s": {"graph_generation_and_pack": t_gen, "first_engine_with_hip_context": t_first_engine,
                   "engine_construct_cold": e2e_cold["engine_construct"],
                   "engine_construct_warm_layout": e2e["engine_construct"],
                   "single_build_synchronised": e2e_cold["build"],
                   "readback_to_pinned_host": e2e_cold["readback"]},
        "end_to_end_cold": {
            "what": "from a fresh PackedGraph (no cached layout, not validated yet) on the host: CostEngine(...) "
                    "+ one build + copy of comm, cost, flags, compute, per_arg to pinned host memory; HIP context "
                    "up and pinned buffers allocated beforehand; best of 5",
            "seconds": t_e2e_cold,
            "entries_per_s": E / t_e2e_cold,
            "phases_s": e2e_cold,
        },
        "end_to_end_warm_layout": {
            "what": "the same from the PackedGraph the first engine was made from, which keeps its block-table "
                    "layout, work items, record arrays and validation; best of 5",
            "seconds": t_e2e,
            "entries_per_s": E / t_e2e,
            "phases_s": e2e,
        },
        "roofline": {
            "kernel": "edge_cost_item_kernel" if eng.use_table else
                      ("edge_cost_kernel<0,4>" if eng._lut_tiles is None else "lut_kernel<entries>"),
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "algorithmic_bytes_per_launch": algo_bytes,
            "bytes_per_entry": 17,
            "avg_launch_s": t_edge,
            "timed_launches": n_timed,
            "avg_launch_s_after_region": t_edge_after,
            "timed_launches_after_region": n_after,
            "avg_launch_s_back_to_back": t_edge_b2b,
            "launches_back_to_back": n_b2b,
            "frac_back_to_back": algo_bytes / t_edge_b2b / 1e9 / HBM_PEAK_GBS,
            # the same bytes over the whole step (prepare launch included), and both
            # with 8 B per entry (the cost alone) instead of the 17 B this build writes
            "step_frac": algo_bytes / (elapsed / args.steps) / 1e9 / HBM_PEAK_GBS,
            "frac_at_8B": (8 * E + desc_bytes) / t_edge / 1e9 / HBM_PEAK_GBS,
            "step_frac_at_8B": (8 * E + desc_bytes) / (elapsed / args.steps) / 1e9 / HBM_PEAK_GBS,
            "traffic": read_traffic(args.workload),
            "traffic_source": "profiles/edge_cost_item_kernel_%s_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                              "runs of this command, scaled by the copy kernel; not a quantity of this run)"
                              % args.workload,
        },
    }

    if args.score_assignments > 0:
        # batch scoring of candidate assignments against the objective (secondary
        # figure; the assignments are generated on the device, nothing is uploaded)
        n = args.score_assignments
        eng.score_random(1, 0, min(n, 4096))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        scores = eng.score_random(1, 0, n)
        torch.cuda.synchronize()
        t_score = time.perf_counter() - t0
        out["scoring"] = {
            "assignments": n,
            "scored_from": eng.last_score_backend,
            "seconds": t_score,
            "assignments_per_s": n / t_score,
            "edge_terms_per_s": n * g.num_edges / t_score,
            "algorithmic_bytes_per_assignment": 8 * g.num_nodes + 17 * g.num_edges,
            "assignments_are": "independent uniform draws of one strategy per node (flow-consistent by "
                               "construction: each edge's inp_idx is its producer's draw), not ILP-feasible plans",
            "fraction_without_forbidden_entry": float((scores[:, 5] == 0).double().mean().item()),
        }
        # The bound that applies to this launch.  Its inputs are the 16-byte records of the
        # entries (one per slot) and 48 B of sums per assignment: that is all HBM has to
        # deliver, once.  An assignment then reads one record per edge at a position its
        # draws decide: random 16-byte reads served by L2 and the memory-side cache, at
        # the rate at which a CU gets cache misses served.  Counted against HBM the
        # requested bytes exceed the peak, which is why no HBM fraction is claimed.
        reads = n * g.num_edges
        hbm_bytes = 16 * g.num_slots + 48 * n
        out["scoring"]["roofline"] = {
            "kernel": "score_compact_kernel" if eng.last_score_backend == "compact_records" else eng.last_score_backend,
            "bound": "cache-miss service rate (random 16-byte reads of records resident in L2 and the "
                     "memory-side cache); not HBM, not MFMA",
            "achieved": reads / t_score,
            "unit": "random reads/s",
            "per_cu_per_ns": reads / t_score / 256 / 1e9,
            "peak": None,
            "requested_bytes_per_s": 16 * reads / t_score,
            "requested_bytes_over_hbm_peak": 16 * reads / t_score / (HBM_PEAK_GBS * 1e9),
            "hbm_bytes_per_launch": hbm_bytes,
            "hbm_frac": hbm_bytes / t_score / (HBM_PEAK_GBS * 1e9),
        }
        # the same batch drawn so that no forbidden (non-finite) entry is selected where the
        # graph allows it: node by node, uniformly among the strategies allowed against the
        # producers' choices (apc_sample_feasible), then scored from the assignment matrix
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        assign, fallbacks = eng.sample_feasible(1, 0, n)
        torch.cuda.synchronize()
        t_sample = time.perf_counter() - t0
        t0 = time.perf_counter()
        fscores = eng.score(assign)
        torch.cuda.synchronize()
        t_fscore = time.perf_counter() - t0
        out["scoring"]["feasible_draws"] = {
            "assignments": n,
            "sample_seconds": t_sample,
            "score_seconds": t_fscore,
            "scored_from": eng.last_score_backend,
            "assignments_per_s_sampled_and_scored": n / (t_sample + t_fscore),
            "fraction_without_forbidden_entry": float((fscores[:, 5] == 0).double().mean().item()),
            "fraction_without_fallback_node": float((fallbacks == 0).double().mean().item()),
            "mean_fallback_nodes_per_assignment": float(fallbacks.double().mean().item()),
            "objective_min": float(fscores[:, 4].min().item()),
            "objective_mean": float(fscores[:, 4].mean().item()),
            "objective_mean_of_the_plain_draws": float(scores[:, 4].mean().item()),
        }
        del assign, fscores

    if args.schedules > 0:
        # next row of the path: the lowered-graph estimator as a batch scorer of
        # candidate orders (secondary figure)
        from autoparallel_amd import schedule_metrics as SM

        ps = SM.synthetic_schedule(32, seed=0)
        base = ps.random_orders(256, seed=1)
        orders = np.tile(base, ((args.schedules + 255) // 256, 1))[:args.schedules]
        est = SM.ScheduleEstimator(ps)
        est.evaluate(orders[:256])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        times, peak = est.evaluate(orders)
        t_sched = time.perf_counter() - t0
        out["schedule_estimator"] = {
            "nodes": ps.n_node, "orders": int(orders.shape[0]), "seconds_including_upload_and_readback": t_sched,
            "orders_per_s": orders.shape[0] / t_sched,
            "best_total_time_us": float(times[:, 0].min()), "graph_order_total_time_us": float(times[0, 0]),
        }
        if not args.no_cpu_baseline:
            from oracle import schedule_oracle as SO

            t0 = time.perf_counter()
            for o in base[:64]:
                SO.schedule_metrics(ps, o)
            out["schedule_estimator"]["cpu_port_orders_per_s"] = 64 / (time.perf_counter() - t0)

    if not args.no_cpu_baseline:
        from oracle import cost_oracle as O

        orc = O.GraphOracle(g)
        orc.reset_caches()
        # bounded sample: whole nodes in graph order until ~25 s of CPU time
        budget = 25.0
        done_entries = 0
        t0 = time.perf_counter()
        nodes_done = 0
        chunk = max(1, g.num_nodes // 64)
        arrays = None
        while nodes_done < g.num_nodes and time.perf_counter() - t0 < budget:
            hi = min(g.num_nodes, nodes_done + chunk)
            arrays = orc.build(nodes=range(nodes_done, hi), out=arrays)
            e_lo = int(g.node_edge_off[nodes_done])
            e_hi = int(g.node_edge_off[hi])
            done_entries += int((g.edge_sdst[e_lo:e_hi].astype(np.int64) * g.edge_ssrc[e_lo:e_hi]).sum())
            nodes_done = hi
        t_cpu = time.perf_counter() - t0
        out["cpu_baseline"] = {
            "value": done_entries / t_cpu,
            "unit": "entries/s",
            "cores": 1,
            "host_cores_available": os.cpu_count(),
            "kind": "port",
            "sample": f"first {nodes_done} of {g.num_nodes} nodes in graph order "
                      f"({done_entries} of {E} entries), memo caches cleared first",
            "seconds": t_cpu,
        }
        out["speedup_vs_cpu_baseline"] = out["value"] / out["cpu_baseline"]["value"]
        out["speedup_vs_cpu_baseline_end_to_end"] = out["end_to_end_cold"]["entries_per_s"] / out["cpu_baseline"]["value"]
        # also reported, and not the reference: the compiled (C, no memo cache)
        # restatement on the same graph, one thread and all cores of the box's share
        try:
            from oracle import c_oracle

            co = c_oracle.COracle(g)
            arrays_c = co.build(threads=1)  # warm-up, and the output buffers to reuse
            res = {}
            for label, threads in (("1_thread", 1), ("all_cores", min(os.cpu_count() or 1, 16))):
                reps, t0 = 0, time.perf_counter()
                while reps < 3 or (time.perf_counter() - t0 < 2.0 and reps < 50):
                    co.build(threads=threads, out=arrays_c)
                    reps += 1
                res[label] = {"threads": threads, "entries_per_s": E * reps / (time.perf_counter() - t0)}
            out["cpu_baseline"]["compiled_port"] = res
        except Exception as exc:  # the checker library is optional for the benchmark
            out["cpu_baseline"]["compiled_port"] = {"error": str(exc)}
    if args.windowed > 0:
        # configs[4] at full size: 2.4e10 entries, built and scored in windows of 3 000 nodes
        from autoparallel_amd import windowed

        legs = {}
        # the third leg: the same generator with another seed, a DAG of the same size whose every node
        # can be served (seed 0, the configuration's, has one that cannot)
        for label, feasible, dag_seed in (("plain_draws", False, 0), ("feasible_draws", True, 0),
                                          ("feasible_draws_dag_seed_1", True, 1)):
            scores, st = windowed.score_in_windows(200000, 3000, args.windowed, workers=14, feasible=feasible,
                                                   seed=dag_seed)
            st.update({
                "assignments": int(scores.shape[0]),
                "entries_per_s_device_build": st["entries"] * st["assignment_batches"] / st["build_device_s"],
                "edge_terms_per_s_scoring": scores.shape[0] * st["edges"] / st["score_device_s"],
                "fraction_without_forbidden_entry": float((scores[:, 5] == 0).mean()),
                "forbidden_entries_per_assignment_mean": float(scores[:, 5].mean()),
                "objective_min": float(scores[:, 4].min()), "objective_mean": float(scores[:, 4].mean()),
            })
            if feasible and st.get("unservable_nodes"):
                st["note"] = ("unservable_nodes: none of their strategies finds, for every argument, a strategy of "
                              "the producer that offers the Partial placements it asks for; they select a forbidden "
                              "entry in every assignment of this DAG, so no assignment of it is free of them")
            legs[label] = st
        out["windowed_stress_dag_200k"] = legs
    if args.fx_layers > 0 and args.workload == "llama3_8b_fwd_bwd_mesh8x8":
        # secondary figure: the same model through the reference-shaped interface, from
        # the traced joint graph to coefficients and ILP rows (strategy sets of the
        # installed torch, so fewer entries than the generator's graph above)
        try:
            out["fx_path"] = _fx_path_figure(args.fx_layers, not args.no_cpu_baseline, args.fx_solve)
        except Exception as exc:  # transformers or the fake process group unavailable
            out["fx_path"] = {"error": f"{type(exc).__name__}: {exc}"[:300]}
    print(json.dumps(out))


def _fx_path_figure(n_layers: int, cpu_port: bool, solve: bool = False) -> dict:
    import contextlib

    import torch
    import torch.distributed as dist
    import transformers
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.device_mesh import init_device_mesh
    from torch.testing._internal.distributed.fake_pg import FakeStore

    from autoparallel_amd.optimize_sharding import ShardingOptimizer
    from autoparallel_amd.shardings import placement_options as PO

    class Wrap(torch.nn.Module):
        def __init__(self, lm):
            super().__init__()
            self.lm = lm

        def forward(self, ids):
            m = self.lm.model
            x = m.embed_tokens(ids)
            pos = torch.arange(ids.shape[1], device=ids.device)[None]
            pe = m.rotary_emb(x, pos)
            for layer in m.layers:
                o = layer(x, attention_mask=None, position_ids=pos, position_embeddings=pe)
                x = o[0] if isinstance(o, tuple) else o
            logits = self.lm.lm_head(m.norm(x))
            return torch.nn.functional.cross_entropy(
                logits[:, :-1].reshape(-1, logits.shape[-1]).float(), ids[:, 1:].reshape(-1))

    cfg = transformers.LlamaConfig(
        vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_hidden_layers=n_layers,
        num_attention_heads=32, num_key_value_heads=8, max_position_embeddings=8192, rope_theta=500000.0,
        attention_dropout=0.0, use_cache=False, attn_implementation="sdpa")
    t0 = time.perf_counter()
    with FakeTensorMode():
        torch.set_default_dtype(torch.bfloat16)
        try:
            with torch.device("cuda"):
                m = Wrap(transformers.LlamaForCausalLM(cfg))
        finally:
            torch.set_default_dtype(torch.float32)
        ids = torch.randint(0, cfg.vocab_size, (64, 8192), device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (ids,)).graph_module
    t_trace = time.perf_counter() - t0
    # as the reference prepares its joint graph before planning (autoparallel/api.py:208):
    # linear layers become einsums, so that batch and sequence can be sharded separately
    from autoparallel_amd.graph_utils import add_alias_nodes, replace_view_mm_view_with_einsum

    t0 = time.perf_counter()
    n_einsum = replace_view_mm_view_with_einsum(gm)
    t_rewrite = time.perf_counter() - t0
    # and every tensor gets an alias node, where a redistribution can sit (:209-211)
    t0 = time.perf_counter()
    add_alias_nodes(gm)
    t_alias = time.perf_counter() - t0
    own = not dist.is_initialized()
    if own:
        dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=64)
    try:
        mesh = init_device_mesh("cpu", (8, 8))
        PO.fallback_nodes.clear()
        PO.reset_placement_options_cache()
        def leg(repeated_subgraphs) -> dict:
            PO.fallback_nodes.clear()
            PO.reset_placement_options_cache()
            t0 = time.perf_counter()
            opt = ShardingOptimizer(gm, mesh, devices_per_host=8, device_name="AMD Instinct MI355X",
                                    repeated_subgraphs=repeated_subgraphs)
            t_opt = time.perf_counter() - t0
            g = opt._packed
            priced_nodes = sorted(set(int(v) for v in g.edge_node[g.priced]))
            res = {
                "nodes": g.num_nodes, "edges": g.num_edges, "priced_nodes": len(priced_nodes),
                # decision variables = entries the engine builds: every node's, or with
                # repeated_subgraphs those of one representative per repeated node
                "entries": g.num_entries,
                "sharding_optimizer_s": t_opt,
                # the split the reference logs for the same constructor
                # (autoparallel/optimize_sharding.py:249-291, 579-587)
                "phase_s": {k: round(v, 6) for k, v in opt.phase_s.items()},
                "entries_per_s_through_the_api": g.num_entries / t_opt,
                "strategy_queries": dict(PO.strategy_cache_stats), "replicate_stand_ins": len(PO.fallback_nodes),
                "ilp_rows": len(opt.prob.constraints),
            }
            if cpu_port:
                # the per-entry Python port on this same packed problem and the same set of
                # nodes: what the reference's _build_decision_vars loop costs after strategy
                # enumeration
                from oracle import cost_oracle as O

                orc = O.GraphOracle(g)
                orc.reset_caches()
                t0 = time.perf_counter()
                orc.build(nodes=priced_nodes)
                t_cpu = time.perf_counter() - t0
                coeff_s = sum(opt.phase_s.get(k, 0.0) for k in ("pack", "engine_construct", "device_build", "readback"))
                device_s = sum(opt.phase_s.get(k, 0.0) for k in ("engine_construct", "device_build", "readback"))
                res["cpu_baseline"] = {
                    "kind": "port", "cores": 1, "seconds": t_cpu, "entries_per_s": g.num_entries / t_cpu,
                    "what": "oracle.cost_oracle.GraphOracle(opt._packed).build(nodes=priced nodes), memo caches "
                            "cleared first",
                    "pack_plus_device_phases_s": coeff_s, "device_phases_s": device_s,
                    "speedup_of_device_phases": t_cpu / device_s if device_s > 0 else None,
                }
            if solve and repeated_subgraphs:
                res["solve"] = _timed_solve(opt, mesh)
            return res

        return {
            "workload": f"transformers LlamaForCausalLM, Llama-3-8B dimensions, {n_layers} layers, bf16, "
                        f"batch 64 x 8192, joint graph, mesh (8,8)",
            "trace_s": t_trace,
            "linear_layers_as_einsums": n_einsum,
            "einsum_rewrite_s": t_rewrite,
            "alias_nodes_s": t_alias,
            "all_nodes": leg(False),
            "cluster_roots_only": leg(True),
            # the duplicates that the reference's pass drops clustered too (no counterpart in the reference)
            "cluster_roots_only_extended_pass": leg("extended"),
        }
    finally:
        if own:
            dist.destroy_process_group()


def _timed_solve(opt, mesh) -> dict:
    """The problem a caller of the reference's example poses (examples/example_llama3.py:226-236):
    batch-sharded input, parameters within 1/mesh size of their bytes; solved by the library's
    solver hand-off.  A line goes to stderr every minute: the solver itself prints nothing."""
    import threading

    from torch.distributed.tensor.placement_types import Replicate, Shard

    opt.add_sharded_input_constraint([(Shard(0),) + (Replicate(),) * (mesh.ndim - 1)])
    opt.add_parameter_memory_constraint(0.0, 1.0 / mesh.size())
    done = threading.Event()
    t0 = time.perf_counter()

    def beat():
        while not done.wait(60):
            print(f"[bench] solving, {time.perf_counter() - t0:.0f} s", file=sys.stderr, flush=True)

    threading.Thread(target=beat, daemon=True).start()
    try:
        plan = opt.get_solution()
    finally:
        done.set()
    dt = time.perf_counter() - t0
    params = [n for n in opt.nodes if n.op == "placeholder" and n in plan]
    fully = sum(all(pl.is_shard() for pl in plan[n].output_specs.placements) for n in params)
    return {"seconds": dt, "objective": opt._core.objective_value, "variables": opt._packed.num_entries,
            "rows": len(opt.prob.constraints), "solver": "HiGHS through scipy.optimize.milp, one thread, gap 0",
            "placeholders_sharded_on_every_mesh_dim": f"{fully} of {len(params)}"}


if __name__ == "__main__":
    main()
