"""Coefficient build and batch scoring of a graph whose coefficients do not fit
the device at once, in windows of nodes.

The 200 000-node planner stress DAG has about 2.4e10 cost entries, 400 GB of
coefficients: more than one GPU's 288 GB.  Nothing in the build needs them all
at once.  The objective of an assignment is a sum over nodes, so the graph is
cut into windows of consecutive nodes; each window is a packed graph of its own
(producers outside it enter as stand-in input nodes carrying the producer's real
output specs), its coefficients are built and scored on the device, and the
running sums are handed to the next window (``apc_score_random_window``): the
result is bit-identical to one pass over the whole graph, which the tests check
at a size where that pass fits.  Windows are generated on the host by a pool of
worker processes (they never touch the GPU) while the device works on the
previous ones.

    python -m autoparallel_amd.windowed --nodes 200000 --window 3000 --assignments 1048576

prints one JSON line: sizes, wall time, device time of the builds and the
scoring, entries per second.
"""
from __future__ import annotations

import argparse
import json
import multiprocessing as mp
import os
import sys
import time
from typing import Optional

import numpy as np


def _make_window(task):
    import gc

    from autoparallel_amd import graphgen

    n_total, lo, hi, mesh, seed, s_min, s_max = task
    # millions of small objects that all live until the window is packed: the cyclic
    # collector only walks them over and over (a quarter of the time of a window)
    was = gc.isenabled()
    gc.disable()
    try:
        g, gid, n_standin = graphgen.stress_dag_window(n_total, lo, hi, mesh, seed, s_min, s_max)
        g.validate()
        # the layouts the engine derives on the host are cached on the graph and travel with
        # it: made here, in the worker, instead of in the one process that drives the device
        g.warm_host_layout()
    finally:
        if was:
            gc.enable()
    return lo, hi, g, gid, n_standin


def _window_masks(task):
    from autoparallel_amd import graphgen

    n_total, lo, hi, mesh, seed, s_min, s_max = task
    return graphgen.stress_dag_partial_masks(n_total, lo, hi, mesh, seed, s_min, s_max)


def score_in_windows(
    n_total: int,
    window: int,
    n_assign: int,
    mesh=(4, 8, 8),
    seed: int = 0,
    assign_seed: int = 1,
    s_min: int = 4,
    s_max: int = 512,
    workers: int = 8,
    max_windows: Optional[int] = None,
    progress=None,
    feasible: bool = False,
    plan: bool = True,
    first: int = 0,
    max_batch: Optional[int] = None,
):
    """Scores ``n_assign`` on-device drawn assignments of the n_total-node stress
    DAG, window by window.  Returns (scores float64[n_assign, 6] on the host,
    stats dict).  ``feasible``: the assignments are drawn node by node among the
    strategies that select no forbidden entry against the producers' choices
    (CostEngine.sample_feasible) instead of independently per node; the choices
    of all nodes are then kept on the device (2 bytes per node and assignment),
    since a later window's stand-in producers carry the choices of their nodes.
    ``plan`` (with ``feasible``): before the first window, the nodes that could run
    out of strategies are found from the spec words of the whole DAG and their
    producers confined to the strategies that serve them (feasible_plan), so that
    no node falls back to the plain draw.  ``first``: counter of the first assignment
    (assignment a is drawn from the counter first + a).  ``max_batch``: the largest
    number of assignments of a pass of feasible draws (default: what 45 % of the
    free device memory holds the choices of)."""
    import torch

    from autoparallel_amd.engine import CostEngine

    tasks = [(n_total, lo, min(lo + window, n_total), tuple(mesh), seed, s_min, s_max)
             for lo in range(0, n_total, window)]
    if max_windows is not None:
        tasks = tasks[:max_windows]
    stats = {"nodes": 0, "edges": 0, "entries": 0, "standin_nodes": 0, "windows": 0, "table_doubles": 0,
             "build_device_s": 0.0, "score_device_s": 0.0, "wait_for_window_s": 0.0, "engine_construct_s": 0.0,
             "modes": {}}
    # Feasible draws keep the choice of every node for every assignment on the device (a later
    # window's stand-ins carry them): a sample too large for that is taken in batches, each a
    # pass over all windows, which are kept on the host after the first pass.
    batch = n_assign
    if feasible:
        free = torch.cuda.mem_get_info()[0]
        cap = max(1, int(0.45 * free) // (2 * n_total))
        if max_batch is not None:
            cap = max(1, min(cap, int(max_batch)))
        if n_assign > cap:
            batch = 1 << (cap.bit_length() - 1)
        stats["sample_device_s"] = 0.0
    n_batches = -(-n_assign // batch)
    stats["assignment_batches"] = n_batches
    kept = [] if n_batches > 1 else None
    outs, fbs = [], []
    t_wall = time.perf_counter()
    pool = None
    if workers > 1 and len(tasks) > 1:
        pool = mp.get_context("spawn").Pool(min(workers, len(tasks)))
    filters = {}
    try:
        if feasible and plan:
            from autoparallel_amd import feasible_plan

            t_mark = time.perf_counter()
            masks = {}
            for part in (pool.imap_unordered(_window_masks, tasks) if pool else map(_window_masks, tasks)):
                masks.update(part)
            filters, stuck = feasible_plan.plan_filters(masks)
            stats["plan_s"] = time.perf_counter() - t_mark
            stats["plan_confined_nodes"] = len(filters)
            stats["plan_stuck_nodes"] = len(stuck)
            # nodes that no assignment of the graph can serve: none of their strategies finds,
            # for every argument, a producer's strategy that offers the Partials it asks for
            stats["unservable_nodes"] = [v for v in stuck if feasible_plan.unservable(masks, v)]
            del masks
        for b in range(n_batches):
            first_b, n_b = first + b * batch, min(batch, n_assign - b * batch)
            out = None
            choices = fallbacks = None
            if feasible:
                # int16 storage of the uint16 choices: torch gathers rows of int16, not of uint16
                choices = torch.zeros((n_total, n_b), dtype=torch.int16, device="cuda")
                fallbacks = torch.zeros(n_b, dtype=torch.int64, device="cuda")
            if b == 0:
                results = pool.imap(_make_window, tasks) if pool else map(_make_window, tasks)
            else:
                results = kept
            t_mark = time.perf_counter()
            for item in results:
                lo, hi, g, gid, n_standin = item
                if b == 0 and kept is not None:
                    kept.append(item)
                stats["wait_for_window_s"] += time.perf_counter() - t_mark  # the host's generation and packing
                t_mark = time.perf_counter()
                eng = CostEngine(g)
                stats["engine_construct_s"] += time.perf_counter() - t_mark  # layout of the problem and its upload
                ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
                ev[0].record()
                eng.build(clamp_inf=True)
                ev[1].record()
                if feasible:
                    # the stand-ins' rows are the choices made for their nodes in earlier windows
                    local = choices[torch.from_numpy(gid.astype(np.int64)).to(choices.device)].contiguous()
                    keep = {i: filters[int(gid[i])] for i in range(n_standin, g.num_nodes) if int(gid[i]) in filters}
                    _, fb = eng.sample_feasible(assign_seed, first_b, n_b, node_gid=gid, first_node=n_standin,
                                                assign=local.view(torch.uint16), row_filter=keep)
                    choices[lo:hi] = local[n_standin:]
                    fallbacks += fb
                    ev[2].record()
                    out = eng.score_window(local.view(torch.uint16), n_standin, init=out)
                    del local
                else:
                    ev[2].record()
                    out = eng.score_random_window(assign_seed, first_b, n_b, gid, n_standin, init=out)
                ev[3].record()
                torch.cuda.synchronize()
                eng.check_status()
                stats["build_device_s"] += ev[0].elapsed_time(ev[1]) * 1e-3
                if feasible:
                    stats["sample_device_s"] += ev[1].elapsed_time(ev[2]) * 1e-3
                stats["score_device_s"] += ev[2].elapsed_time(ev[3]) * 1e-3
                if b == 0:
                    real = g.edge_node >= n_standin  # the stand-ins' own input edges are not the DAG's
                    stats["nodes"] += hi - lo
                    stats["standin_nodes"] += n_standin
                    stats["edges"] += int(real.sum())
                    stats["entries"] += int((g.edge_sdst.astype(np.int64) * g.edge_ssrc)[real].sum())
                    stats["table_doubles"] += 0 if eng.table is None else int(eng.table.numel())
                    stats["modes"][eng.table_mode] = stats["modes"].get(eng.table_mode, 0) + 1
                    stats["windows"] += 1
                if progress:
                    progress(stats, time.perf_counter() - t_wall)
                del eng
                t_mark = time.perf_counter()
            outs.append(out.cpu().numpy())
            if feasible:
                fbs.append(fallbacks.cpu().numpy())
            del out, choices, fallbacks
    finally:
        if pool is not None:
            pool.terminate()
            pool.join()
    stats["wall_s"] = time.perf_counter() - t_wall
    if feasible:
        fb = np.concatenate(fbs)
        stats["fallback_nodes_per_assignment_mean"] = float(fb.mean())
        stats["fallback_nodes_per_assignment_min"] = int(fb.min())
        stats["assignments_without_fallback"] = int((fb == 0).sum())
    return np.concatenate(outs), stats


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--nodes", type=int, default=200000)
    ap.add_argument("--window", type=int, default=3000)
    ap.add_argument("--assignments", type=int, default=1 << 20)
    ap.add_argument("--workers", type=int, default=min(14, os.cpu_count() or 1))
    ap.add_argument("--max-windows", type=int, default=None)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--first", type=int, default=0, help="counter of the first assignment")
    ap.add_argument("--feasible", action="store_true",
                    help="draw the assignments node by node among the strategies without a forbidden entry")
    ap.add_argument("--no-plan", action="store_true",
                    help="with --feasible: do not confine the producers of the nodes that could run out of strategies")
    args = ap.parse_args()

    def progress(st, wall):
        print(f"window {st['windows']}: {st['nodes']} nodes, {st['entries']:.4g} entries, wall {wall:.0f} s, "
              f"device build {st['build_device_s']:.2f} s, scoring {st['score_device_s']:.2f} s",
              file=sys.stderr, flush=True)

    scores, st = score_in_windows(args.nodes, args.window, args.assignments, seed=args.seed,
                                  workers=args.workers, max_windows=args.max_windows, progress=progress,
                                  feasible=args.feasible, plan=not args.no_plan, first=args.first)
    obj = scores[:, 4]
    st.update({
        "workload": f"stress DAG, {args.nodes} nodes, mesh (4,8,8), windows of {args.window}",
        "assignments": int(scores.shape[0]),
        "entries_per_s_device_build": st["entries"] * st["assignment_batches"] / st["build_device_s"],
        "entries_per_s_wall": st["entries"] / st["wall_s"],
        "edge_terms_per_s_scoring": scores.shape[0] * st["edges"] / st["score_device_s"],
        "coefficient_bytes_if_resident": 17 * st["entries"],
        "objective_min": float(obj.min()), "objective_mean": float(obj.mean()),
        "feasible_fraction": float((scores[:, 5] == 0).mean()),
    })
    print(json.dumps(st))


if __name__ == "__main__":
    main()
