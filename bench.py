#!/usr/bin/env python3
"""Benchmark of one rank's MoE dispatch+combine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C4] [--rank 0] [--mode graph|eager]

A step is one pass of one rank's share of the job (rank 0 unless --rank says otherwise), everything on the
device and on one stream:

    dispatch_send -> [exchange leg r->r] -> dispatch_recv -> [expert stand-in]
      -> combine_send -> [exchange leg r->r] -> combine_recv

The bracketed launches are the stand-ins for what is outside this path (the xGMI exchange, the expert
GEMM). The seven peers' inbound segments are produced once, before timing, by running the peers' own
kernels on their seeded inputs; they stay resident where an exchange would have written them.

Prints ONE JSON line. `value` is the wall time of a whole step (stand-ins included) in microseconds, the
mean over exactly `--steps` graph replays between two synchronisations; `step_us_median` / `step_us_min`
are taken over batches of the same replays timed with events. `hot_path_us` is the time of the four path
launches by themselves: HIP events on the launch stream around a graph that holds `--kernel-reps` times
dispatch_send, dispatch_recv, combine_send, combine_recv and nothing else, every input resident where
the step leaves it; `hot_path_launch_floor_us` is the same graph on a job without rows (what four
launches cost when they move nothing). The cost of one of them is that time minus the time of the same graph without it;
`roofline` prices the slowest against HBM peak with the algorithmic bytes of its stage.
`hot_path_us_in_step` is the whole step minus a step of the three stand-ins alone. `ranks` repeats the
hot-path figure for every rank of the job (their received row counts differ); `cpu_baseline` is the
row-by-row torch-CPU statement of the same step timed on this box's
host cores, with the vectorised numpy statement beside it; `custom_kernel_wall_us` is one call of the
reference's entry point (which steps all ranks of the job on this one GPU). `expert_gemm` is the
grouped GEMM a model would run between the two halves, on this rank's expert-major rows and random
weights: one launch between HIP events, priced against HBM peak (it streams every weight once) with
its matrix rate beside it. `linear` is the per-rank product of the reference's gemm-rs task at the
largest shape of its benchmark list, priced against the dense bf16 matrix rate.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16/fp16 matrix rate, published
META_BYTES = 20
# HBM bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE, with the build they were measured on
TRAFFIC_FILE = ROOT / "profiles" / "hbm_traffic.json"
PATH = ("dispatch_send", "dispatch_recv", "combine_send", "combine_recv")


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="C4", choices=["C1", "C2", "C3", "C4", "C5", "C4x2", "C4x4", "C4x6", "W2x16"])
    ap.add_argument("--seed", type=int, default=2025)
    ap.add_argument("--rank", type=int, default=0, help="rank whose share of the job is the timed step")
    ap.add_argument("--mode", default="graph", choices=["graph", "eager"],
                    help="replay a captured HIP graph of the step (default) or launch eagerly")
    ap.add_argument("--kernel-reps", type=int, default=20,
                    help="repetitions of the launches inside each timing graph")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the cpu_baseline sample")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-gemm", action="store_true", help="skip the grouped GEMM and linear rows")
    ap.add_argument("--no-gemm-list", action="store_true",
                    help="skip the list of gemm-rs benchmark shapes inside the linear row (profiles of one shape)")
    ap.add_argument("--no-floor", action="store_true",
                    help="skip the launch-floor measurement (its launches without rows would count into a "
                         "profiler's per-kernel averages)")
    ap.add_argument("--no-rank-sweep", action="store_true", help="time only --rank, not every rank of the job")
    ap.add_argument("--no-placement-plan", action="store_true",
                    help="combine_send ranks its rows by scanning instead of using dispatch_recv's plan")
    ap.add_argument("--long-stream-rows", type=int, default=None,
                    help="row count above which the receive halves take the long-stream entry points "
                         "(default: the host class's own threshold)")
    ap.add_argument("--alone", action="store_true",
                    help="also time every kernel back to back with itself (warm inputs)")
    ap.add_argument("--dtype", default=None, choices=["fp16", "bf16"],
                    help="token type of the main workload (default: the workload's own, bf16; the reference "
                         "uses fp16, all2all/reference.py:16-17)")
    ap.add_argument("--weights", default=None, choices=["rand", "softmax"],
                    help="routing weights of the main workload (default: the workload's own, softmax; the "
                         "reference draws rand, all2all/reference.py:37-43)")
    ap.add_argument("--binding", default="ctypes", choices=["ctypes", "ext"],
                    help="how the host class reaches the C ABI: ctypes, or the torch extension built with load_inline")
    ap.add_argument("--no-extra-workloads", action="store_true",
                    help="skip the C5 block and the C4 block with the reference's input rules (fp16, rand weights)")
    ap.add_argument("--no-entry-points", action="store_true",
                    help="skip the timings of custom_kernel and of the class surface (they step every rank of the job)")
    return ap.parse_args()


def alg_bytes(T, K, H, R):
    """Algorithmic bytes of each stage for one rank: S = T*K rows sent, R rows received."""
    S, row = T * K, 2 * H
    return {
        "dispatch_send": 4 * S + T * row + S * (row + META_BYTES),
        "dispatch_recv": 2 * R * (row + META_BYTES),
        "combine_send": 2 * R * (row + META_BYTES),
        "combine_recv": S * (row + META_BYTES) + 4 * S + T * row,
    }


def measured_traffic(workload, seed, rank, kernel, build_id):
    """HBM bytes per launch of `kernel` from the committed counter summary, or None when that
    summary was taken on another build of the library, or on another workload or rank."""
    try:
        rec = json.loads(TRAFFIC_FILE.read_text())
    except (OSError, ValueError):
        return None
    if rec.get("build_id") != build_id:
        return None
    if (rec.get("workload"), rec.get("seed"), rec.get("rank")) != (workload, seed, rank):
        return None
    return rec.get("bytes_per_launch", {}).get(kernel)


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one rank on one GPU; --gpus {args.gpus} is not supported "
              "(the inter-GPU exchange is outside this build)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from amd_distributed_2025_amd import LocalWorld, WORKLOADS, generate_world, _lib
    from amd_distributed_2025_amd.all2all import exchange_leg
    from amd_distributed_2025_amd.task import dtype_name

    lib = _lib.load()
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    from amd_distributed_2025_amd.task import LARGE_WORKLOADS
    wl = dict({**WORKLOADS, **LARGE_WORKLOADS}[args.workload])
    if args.dtype:
        wl["dtype"] = args.dtype
    if args.weights:
        wl["weights"] = args.weights

    def set_up(workload, **layout):
        """The whole job once, so that every rank's inbound buffers hold the peers' segments."""
        world_ = generate_world(workload, args.seed)
        cfg_ = world_[0][0]
        data_ = [d.to(dev) for _, d, _, _ in world_]
        lw_ = LocalWorld(cfg_, len(world_), device=dev, reuse_placement=not args.no_placement_plan,
                         long_stream_rows=args.long_stream_rows, binding=args.binding, **layout)
        ys_ = [y.clone() for y in lw_.run(data_)]
        torch.cuda.synchronize()
        return world_, cfg_, data_, lw_, ys_

    world, cfg, data, lw, ys0 = set_up(wl)
    W, K, H = len(world), cfg.experts_per_token, cfg.hidden_dim
    if not 0 <= args.rank < W:
        print(f"--rank must be in [0, {W})", file=sys.stderr)
        sys.exit(2)

    def stages_of(r, lw=lw, data=data, cfg=cfg):
        """The seven launches of rank r's step, in order, as (name, callable)."""
        H = cfg.hidden_dim
        a, d, g = lw.ranks[r], data[r], lw.trace[r]
        T = d.num_tokens
        R = int(g["recv_counts"].sum().item())
        own_out = int(g["send_counts"][r].item())   # rows the rank sends to itself
        own_back = int(g["back_counts"][r].item())
        y = a._buf("y", (cfg.max_num_tokens, H), cfg.out_dtype)
        st = [
            ("dispatch_send", lambda: a.dispatch_send(d.x, d.indices)),
            ("exchange_out", lambda: exchange_leg(a, a, g["send_counts"], g["send_buf"], g["send_meta"],
                                                  g["recv_counts"], g["recv_buf"], g["recv_meta"], own_out)),
            ("dispatch_recv", lambda: a.dispatch_recv(g["recv_counts"], g["recv_buf"], g["recv_meta"], R)),
            ("expert_standin", lambda: a.expert_scale(g["expert_x"], g["expert_num_tokens"], R)),
            ("combine_send", lambda: a.combine_send(g["expert_meta"], g["expert_y"], g["expert_num_tokens"], R)),
            ("exchange_back", lambda: exchange_leg(a, a, g["back_counts"], g["back_buf"], g["back_meta"],
                                                   g["ret_counts"], g["ret_buf"], g["ret_meta"], own_back)),
            ("combine_recv", lambda: a.combine_recv(y, d.weights, g["ret_counts"], g["ret_buf"], g["ret_meta"],
                                                    accumulate=False)),
        ]
        return st, T, R, y

    def graph_of(fns, reps):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for fn in fns:
                fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            for _ in range(reps):
                for fn in fns:
                    fn()
        gr.replay()
        torch.cuda.synchronize()
        return gr

    def time_graph(gr, reps, rounds=9):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        samples = []
        for _ in range(rounds):
            e0.record()
            gr.replay()
            e1.record()
            e1.synchronize()
            samples.append(e0.elapsed_time(e1) * 1e3 / reps)
        return statistics.median(samples)

    # The path by itself: a graph of `reps` times the four path launches, timed with HIP events on the
    # launch stream. A kernel's cost is what the graph loses when the kernel is left out. (Leaving a
    # kernel out of the WHOLE step does not give a usable figure: with the small exchange stand-ins in
    # the graph the parts add up to between 3 us less and 1 us more than the whole, and the sum moves
    # by microseconds between builds whose whole step differs by half a microsecond.)
    def path_costs(stages, T, R, per_kernel=True, alone=False, K=K, H=H):
        reps = args.kernel_reps
        path = [(n, f) for n, f in stages if n in PATH]
        chain_us = time_graph(graph_of([f for _, f in path], reps), reps)
        kern = {}
        if per_kernel:
            for name, fn in path:
                without = time_graph(graph_of([f for n, f in path if n != name], reps), reps)
                kern[name] = {"us": round(chain_us - without, 3)}
                if alone:  # the kernel back to back with itself: inputs stay warm, no producer in between
                    kern[name]["us_alone_warm"] = round(time_graph(graph_of([fn], reps), reps), 3)
            ab = alg_bytes(T, K, H, R)
            for name in PATH:
                kern[name]["alg_bytes"] = ab[name]
                kern[name]["gbps"] = round(ab[name] / kern[name]["us"] * 1e-3, 1)
                kern[name]["frac"] = round(kern[name]["gbps"] / HBM_PEAK_GBPS, 4)
        for _, fn in stages:  # leave every buffer as a full step leaves it
            fn()
        torch.cuda.synchronize()
        return chain_us, kern, sum(alg_bytes(T, K, H, R).values())

    r0 = args.rank
    stages, T, R, y = stages_of(r0)

    def step():
        for _, fn in stages:
            fn()

    # ---- whole-step timing: exactly `steps` steps between two synchronisations
    if args.mode == "graph":
        graph = graph_of([fn for _, fn in stages], 1)
        run_step = graph.replay
    else:
        run_step = step
    for _ in range(args.warmup):
        run_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    y_after = y[:T].clone()
    same_as_setup = bool(torch.equal(y_after, ys0[r0]))
    # the same replays in batches between events: median and minimum of the batch means
    batch = max(1, min(10, args.steps))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    batches = []
    for _ in range(max(1, args.steps // batch)):
        e0.record()
        for _ in range(batch):
            run_step()
        e1.record()
        e1.synchronize()
        batches.append(e0.elapsed_time(e1) * 1e3 / batch)

    hot_us, kern, total_alg = path_costs(stages, T, R, alone=args.alone)
    reps = args.kernel_reps

    # What a launch of this path costs with nothing to move: the same four entry points in the same
    # kind of graph on a job without rows (no tokens sent, zero counts everywhere). It is the part of
    # a small workload's time that no kernel change can win back.
    def launch_floor():
        a, g = lw.ranks[r0], lw.trace[r0]
        zc = torch.zeros(W, dtype=torch.int32, device=dev)
        zn = torch.zeros(a.num_local_experts, dtype=torch.int32, device=dev)
        d0 = data[r0]
        fns = [
            lambda: a.dispatch_send(d0.x[:0], d0.indices[:0]),
            lambda: a.dispatch_recv(zc, g["recv_buf"], g["recv_meta"], 0),
            lambda: a.combine_send(g["expert_meta"], g["expert_y"], zn, 0),
            lambda: a.combine_recv(y, d0.weights[:1], zc, g["ret_buf"], g["ret_meta"], accumulate=True),
        ]
        us = time_graph(graph_of(fns, reps), reps)
        for _, fn in stages:  # put every buffer back as a full step leaves it
            fn()
        torch.cuda.synchronize()
        return us

    floor_us = None if args.no_floor else launch_floor()
    full_us = time_graph(graph_of([fn for _, fn in stages], reps), reps)
    standins_us = time_graph(graph_of([fn for n, fn in stages if n not in PATH], reps), reps)
    dominant = max(PATH, key=lambda n: kern[n]["us"])
    build_id = lib.moe_a2a_build_id().decode()

    out = {
        "metric": "us_per_dispatch_combine",
        "value": round(ms_per_step * 1e3, 3),
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if cfg.in_dtype == torch.bfloat16 else "f16",
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: rank {r0} of world_size={W}, num_experts={cfg.num_experts}, "
                        f"experts_per_token={K}, hidden_dim={H}, num_tokens={T}, routing={wl['routing']}, "
                        f"weights={wl['weights']}, seed={args.seed}",
            "rows_sent": T * K, "rows_received": R, "mode": args.mode,
            "binding": args.binding,
            "value_includes": "exchange and expert stand-ins",
        },
        "step_us_median": round(statistics.median(batches), 3),
        "step_us_min": round(min(batches), 3),
        "step_us_graph_of_steps": round(full_us, 3),
        "hot_path_us": round(hot_us, 3),
        "hot_path_measure": f"graph of {reps} x the four path launches, HIP events, median of 9",
        "hot_path_us_in_step": round(full_us - standins_us, 3),
        "hot_path_launch_floor_us": None if floor_us is None else round(floor_us, 3),
        "hot_path_launch_floor_measure": "the same graph of the four entry points on a job without rows",
        "hot_path_kernel_sum_us": round(sum(kern[n]["us"] for n in PATH), 3),
        "hot_path_alg_bytes": total_alg,
        "hot_path_gbps": round(total_alg / hot_us * 1e-3, 1),
        "hot_path_frac_of_hbm_peak": round(total_alg / hot_us * 1e-3 / HBM_PEAK_GBPS, 4),
        "kernels": kern,
        "roofline": {
            "bound": "hbm", "kernel": dominant,
            "achieved": kern[dominant]["gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": kern[dominant]["frac"],
            "traffic": measured_traffic(args.workload, args.seed, r0, dominant, build_id),
        },
        "library": {"version": lib.moe_a2a_version().decode(), "build_id": build_id},
        "result_identical_to_setup_run": same_as_setup,
    }

    # ---- the same hot-path figure for every rank of the job
    if W > 1 and not args.no_rank_sweep:
        ranks = {}
        for r in range(W):
            if r == r0:
                hot_r, alg_r, rows_r = hot_us, total_alg, R
            else:
                st_r, T_r, R_r, _ = stages_of(r)
                hot_r, _, alg_r = path_costs(st_r, T_r, R_r, per_kernel=False)
                rows_r = R_r
            ranks[str(r)] = {"rows_received": rows_r, "hot_path_us": round(hot_r, 3),
                             "frac": round(alg_r / hot_r * 1e-3 / HBM_PEAK_GBPS, 4)}
        fr = [v["frac"] for v in ranks.values()]
        out["ranks"] = ranks
        out["hot_path_frac_min_over_ranks"] = min(fr)
        out["hot_path_frac_mean_over_ranks"] = round(sum(fr) / len(fr), 4)

    # ---- the same path on the skewed workload of this shape (C5: Zipf-skewed routing;
    # rank 0 and the ranks that receive the most and the fewest rows, with their realised row
    # counts) and on C4 with the reference's own input rules (fp16 tokens and `rand` weights,
    # all2all/reference.py:16-17,37-43). One job each, set up like the main one.
    def hot_path_of(workload, pick_ranks, **layout):
        world_, cfg_, data_, lw_, _ = set_up(workload, **layout)
        W_ = len(world_)
        rows = [int(lw_.trace[r]["recv_counts"].sum().item()) for r in range(W_)]
        res = {}
        for r in pick_ranks(rows):
            if str(r) in res:
                continue
            st_r, T_r, R_r, _ = stages_of(r, lw_, data_, cfg_)
            hot_r, _, alg_r = path_costs(st_r, T_r, R_r, per_kernel=False, K=cfg_.experts_per_token,
                                         H=cfg_.hidden_dim)
            res[str(r)] = {"rows_sent": T_r * cfg_.experts_per_token, "rows_received": R_r,
                           "hot_path_us": round(hot_r, 3), "hot_path_alg_bytes": alg_r,
                           "frac": round(alg_r / hot_r * 1e-3 / HBM_PEAK_GBPS, 4)}
            if layout:
                res[str(r)]["workspace_bytes"] = lw_.ranks[r].workspace_bytes()
        del lw_, data_
        torch.cuda.empty_cache()
        return res, rows

    if args.workload == "C4" and not args.no_extra_workloads and not (args.dtype or args.weights):
        res, rows = hot_path_of(WORKLOADS["C5"], lambda n: [0, n.index(max(n)), n.index(min(n))])
        hot, cold = rows.index(max(rows)), rows.index(min(rows))
        out["c5"] = {
            "workload": f"C5: the C4 shape with routing=zipf (s=1.2), seed={args.seed}",
            "rows_received_per_rank": rows,
            "rank0": res["0"], "hottest_rank": hot, "hottest": res[str(hot)],
            "coldest_rank": cold, "coldest": res[str(cold)],
            "hot_path_frac_of_hbm_peak": res["0"]["frac"],
        }
        res, _ = hot_path_of(dict(WORKLOADS["C4"], dtype="fp16", weights="rand"), lambda n: [r0])
        out["c4_fp16_rand"] = dict(res[str(r0)], workload=f"C4 with dtype=fp16, weights=rand (the reference's "
                                   f"input rules), rank {r0}, seed={args.seed}",
                                   hot_path_frac_of_hbm_peak=res[str(r0)]["frac"])
        # the same job with the expert-major buffers in the compact layout (rows of an expert at its
        # offset, room for 2560 rows instead of 32 x 2048): the same four stages, a twentieth of the memory
        res, _ = hot_path_of(WORKLOADS["C4"], lambda n: [r0], layout="compact", compact_rows=2560)
        out["c4_compact_layout"] = dict(res[str(r0)], compact_rows=2560,
                                        workspace_bytes_padded_layout=lw.ranks[r0].workspace_bytes(),
                                        hot_path_frac_of_hbm_peak=res[str(r0)]["frac"])

    # ---- the reference's entry point: one call steps the whole job on this GPU (all ranks' kernels and
    # one gathering exchange launch per rank and direction). The first call of a job runs launch by
    # launch, the second captures it, later ones replay the capture.
    from amd_distributed_2025_amd import HIPAllToAll, custom_kernel, custom_kernel_job, run_lockstep, set_peer_inputs

    # (both entry-point sections make workspaces of their own for every rank of the job: they are for
    # the task's sizes and are left out for the larger row counts, and each frees what it made)
    entry_points = args.workload in WORKLOADS and not args.no_entry_points
    world_dev = [(c, d, r, w) for (c, _, r, w), d in zip(world, data)]
    set_peer_inputs(world_dev)

    def wall_of(fn, calls=9, skip=3):
        walls = []
        for _ in range(calls):
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            res = fn()
            torch.cuda.synchronize()
            walls.append((time.perf_counter() - t1) * 1e6)
        return statistics.median(walls[skip:]), walls, res

    if entry_points:
        from amd_distributed_2025_amd import submission

        ck_us, ck_walls, yk = wall_of(lambda: custom_kernel(world_dev[r0]))
        job_us, _, yjob = wall_of(lambda: custom_kernel_job(world_dev))
        out["custom_kernel_wall_us"] = round(ck_us, 1)
        out["custom_kernel_first_call_us"] = round(ck_walls[0], 1)
        out["custom_kernel_job_wall_us"] = round(job_us, 1)
        out["custom_kernel_job_wall_us_per_rank"] = round(job_us / W, 1)
        out["custom_kernel_matches_step"] = bool(torch.equal(yk, ys0[r0]) and
                                                 all(torch.equal(a_, b_) for a_, b_ in zip(yjob, ys0)))
        del yk, yjob
        submission._worlds.clear()
        torch.cuda.empty_cache()
    set_peer_inputs(None)

    # ---- the reference's class surface, launch by launch: every rank of the job in a thread of its own
    # calls dispatch() and combine() (all2all/reference.py:259-272 with the stand-in expert), through
    # each binding; wall time of the whole job, nothing read back from the device in between
    def class_surface(binding):
        objs = {}

        def rank_main(r, exchange):
            a = objs.get(r)
            if a is None:
                a = objs[r] = HIPAllToAll(cfg, r, W, exchange=exchange, device=dev, binding=binding)
            a.exchange = exchange  # (every job gets a new exchange object from run_lockstep)
            d = data[r]
            num, ex, em = a.dispatch(d.x, d.indices)
            ey = a.expert_scale(ex, num)
            y_ = a._buf("y_surface", (cfg.max_num_tokens, H), cfg.out_dtype)
            y_.zero_()
            a.combine(y_, d.weights, em, ey, num)
            return y_[: d.num_tokens]

        us, _, ys_ = wall_of(lambda: run_lockstep(W, rank_main, device=dev), calls=7, skip=2)
        same = bool(all(torch.equal(a_, b_) for a_, b_ in zip(ys_, ys0)))
        del ys_
        objs.clear()
        torch.cuda.empty_cache()
        return us, same

    if W > 1 and entry_points:
        surf = {}
        for b_name in ("ctypes", "ext"):
            us, same = class_surface(b_name)
            surf[b_name] = {"job_wall_us": round(us, 1), "per_rank_us": round(us / W, 1), "matches_step": same}
        out["class_surface_eager"] = dict(surf, measure="dispatch() + expert stand-in + combine() of every rank, one "
                                          "thread per rank, loose launch sizes, median wall time of 5 jobs")
        # The threads of that job spend most of their time meeting each other (eight Python threads at
        # four barriers); what the calls of ONE rank cost its process is seen on a job of a single rank
        # with the rank's share of the shape (its local experts, the same tokens, rows and row length):
        # time until the last launch is issued, and until the GPU has finished.
        from amd_distributed_2025_amd.task import MoEConfig, RankTestData
        solo_cfg = MoEConfig(cfg.num_experts // W, min(K, cfg.num_experts // W), H, cfg.max_num_tokens,
                             cfg.in_dtype, cfg.out_dtype)
        d0 = data[r0]
        solo_idx = (d0.indices % solo_cfg.num_experts)[:, : solo_cfg.experts_per_token].contiguous()
        solo_w = d0.weights[:, : solo_cfg.experts_per_token].contiguous()
        solo = {}
        for b_name in ("ctypes", "ext"):
            a1 = HIPAllToAll(solo_cfg, 0, 1, device=dev, binding=b_name)
            y1 = torch.zeros(solo_cfg.max_num_tokens, H, dtype=cfg.out_dtype, device=dev)
            issued, done = [], []
            for i in range(25):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                num, ex, em = a1.dispatch(d0.x, solo_idx)
                ey = a1.expert_scale(ex, num)
                a1.combine(y1, solo_w, em, ey, num)
                t1 = time.perf_counter()
                torch.cuda.synchronize()
                t2 = time.perf_counter()
                if i >= 5:
                    issued.append((t1 - t0) * 1e6)
                    done.append((t2 - t0) * 1e6)
            solo[b_name] = {"issue_us": round(statistics.median(issued), 1), "wall_us": round(statistics.median(done), 1)}
            del a1, y1
            torch.cuda.empty_cache()
        out["class_surface_eager"]["one_rank_job"] = dict(
            solo, measure="dispatch() + stand-in + combine() on a job of one rank with this rank's share of the shape "
                          "(no exchange, no other thread): host time to issue the launches, and wall time with the GPU's work")

    # ---- the expert computation a model runs between the two halves: the grouped GEMM over this
    # rank's expert-major rows (random weights; the stand-in of the reference stays in the step above)
    if not args.no_gemm and H % 64 == 0 and cfg.in_dtype == cfg.out_dtype:
        a, g = lw.ranks[r0], lw.trace[r0]
        nle = a.num_local_experts
        gen = torch.Generator(device=dev).manual_seed(args.seed)
        wts = torch.empty(nle, H, H, dtype=cfg.in_dtype, device=dev)
        for le in range(nle):  # (one expert at a time: the fp32 draw of all of them would not be small)
            wts[le] = (torch.randn(H, H, generator=gen, device=dev) / H ** 0.5).to(cfg.in_dtype)
        ex, num = g["expert_x"], g["expert_num_tokens"]
        counts = num.cpu().tolist()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        times = []
        for i in range(12):
            ev[0].record()
            ey = a.expert_gemm(ex, num, wts, rows_hint=R)
            ev[1].record()
            ev[1].synchronize()
            if i >= 2:
                times.append(ev[0].elapsed_time(ev[1]) * 1e3)
        gemm_us = statistics.median(times)
        le = max(range(nle), key=lambda i: counts[i])
        want = ex[le, : counts[le]].float() @ wts[le].float().T
        err = (ey[le, : counts[le]].float() - want).abs().max().item()
        gemm_bytes = nle * H * H * 2 + 2 * R * H * 2   # every weight once, valid rows read and written
        gemm_flop = 2 * R * H * H
        out["expert_gemm"] = {
            "us": round(gemm_us, 1), "rows": R, "rows_per_expert_max": max(counts), "experts": nle,
            "weights_bytes": nle * H * H * 2, "alg_bytes": gemm_bytes, "flop": gemm_flop,
            "roofline": {"bound": "hbm", "achieved": round(gemm_bytes / gemm_us * 1e-3, 1), "peak": HBM_PEAK_GBPS,
                         "unit": "GB/s", "frac": round(gemm_bytes / gemm_us * 1e-3 / HBM_PEAK_GBPS, 4)},
            "tflops": round(gemm_flop / gemm_us * 1e-6, 1),
            "frac_of_mfma_peak": round(gemm_flop / gemm_us * 1e-6 / MFMA_PEAK_TFLOPS, 4),
            "mfma_peak_tflops": MFMA_PEAK_TFLOPS,
            "max_abs_err_vs_fp32_matmul": err,
            "measure": "HIP events around single launches, median of 10",
        }
        del wts

    # ---- the gemm-rs task's per-rank product (gemm-rs/reference.py:54-57) at the largest shape of
    # its benchmark list (m = n = 8192, k = 29568 over 8 ranks, no bias): matrix-core bound
    if not args.no_gemm:
        from amd_distributed_2025_amd import gemm_rs

        m, n, k_job = 8192, 8192, 29568
        lin = gemm_rs.generate_input(0, 8, m, n, k_job, False, 42, device=dev)
        lin_out = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]

        def timed(fn, n_runs=10):
            ts = []
            for i in range(n_runs + 3):
                ev[0].record()
                fn()
                ev[1].record()
                ev[1].synchronize()
                if i >= 3:
                    ts.append(ev[0].elapsed_time(ev[1]) * 1e3)
            return statistics.median(ts)

        lin_us = timed(lambda: gemm_rs.local_product(lin, out=lin_out))
        torch_us = timed(lambda: torch.matmul(lin[0], lin[1].T))
        k_loc = k_job // 8
        flop = 2 * m * n * k_loc
        rows = torch.arange(0, m, 257, device=dev)
        want = lin[0][rows].float() @ lin[1].float().T
        got = lin_out[rows].float()
        out["linear"] = {
            "shape": {"m": m, "n": n, "k_per_rank": k_loc, "bias": False},
            "us": round(lin_us, 1), "flop": flop,
            "roofline": {"bound": "mfma", "achieved": round(flop / lin_us * 1e-6, 1), "peak": MFMA_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(flop / lin_us * 1e-6 / MFMA_PEAK_TFLOPS, 4)},
            "torch_matmul_us": round(torch_us, 1),
            "torch_matmul_tflops": round(flop / torch_us * 1e-6, 1),
            "max_rel_err_vs_fp32_matmul": float(((got - want).abs() / (want.abs() + 1e-3)).max().item()),
            "measure": "HIP events around single launches, median of 10; torch.matmul (the vendor "
                       "library, what the reference calls) timed the same way beside it",
        }
        del lin, lin_out

        # the whole benchmark list of that task (gemm-rs/task.yml:80-85, ranked by the geometric
        # mean), each shape timed like the one above, beside the reference's own two statements
        rows_, ours_, theirs_ = [], [], []
        for (bm, bn, bk, has_bias, bseed) in ([] if args.no_gemm_list else gemm_rs.TASK_BENCHMARKS):
            d = gemm_rs.generate_input(0, 8, bm, bn, bk, has_bias, bseed, device=dev)
            o = torch.empty(bm, bn, dtype=torch.bfloat16, device=dev)

            def reference_statements():
                y = torch.matmul(d[0], d[1].T)
                return y if d[2] is None else y + d[2]

            a_us = timed(lambda: gemm_rs.local_product(d, out=o))
            r_us = timed(reference_statements)
            ours_.append(a_us)
            theirs_.append(r_us)
            rows_.append({"m": bm, "n": bn, "k_per_rank": bk // 8, "bias": has_bias, "us": round(a_us, 1),
                          "torch_us": round(r_us, 1)})
            del d, o
        geo = lambda v: math.exp(sum(math.log(x) for x in v) / len(v))
        if rows_:
            out["linear"]["task_benchmarks"] = {
                "shapes": rows_, "geomean_us": round(geo(ours_), 1), "torch_geomean_us": round(geo(theirs_), 1),
                "note": "per-rank product only (the reduce-scatter between GPUs is not part of either figure)",
            }

    # ---- CPU baseline: the row-by-row torch statement of the same step on the host cores
    if not args.no_cpu:
        from oracle import moe_a2a_oracle as orc
        from oracle import rowwise_torch as rw

        a, d0, g = lw.ranks[r0], data[r0], lw.trace[r0]
        nle, max_recv = a.num_local_experts, a.max_recv
        x_c, idx_c, w_c = d0.x.cpu(), d0.indices.cpu(), d0.weights.cpu()
        recv_b, recv_m = g["recv_buf"][:R].cpu(), g["recv_meta"][:R].cpu()
        ret_b, ret_m = g["ret_buf"][: T * K].cpu(), g["ret_meta"][: T * K].cpu()

        def cpu_step():
            t = [time.perf_counter()]
            rw.send_side(x_c, idx_c, r0, W, nle); t.append(time.perf_counter())
            n_per, ex, em = rw.place_rows(recv_b, recv_m, nle, max_recv); t.append(time.perf_counter())
            ey = rw.simulated_expert(ex, r0, cfg.out_dtype); t.append(time.perf_counter())
            rw.return_side(ey, em, n_per, W); t.append(time.perf_counter())
            yc = torch.zeros(cfg.max_num_tokens, H, dtype=cfg.out_dtype)
            rw.accumulate(yc, w_c, ret_b, ret_m); t.append(time.perf_counter())
            return yc[:T], [b - a_ for a_, b in zip(t, t[1:])]

        runs, spent = [], 0.0
        while spent < args.cpu_seconds and len(runs) < 200:
            yc, parts = cpu_step()
            runs.append(parts)
            spent += sum(parts)
        med = [statistics.median(r[i] for r in runs) for i in range(5)]
        cpu_path_us = (med[0] + med[1] + med[3] + med[4]) * 1e6

        # the vectorised numpy statement of the same share (stable argsort / bincount, explicit rounding)
        dt_in, dt_out = dtype_name(cfg.in_dtype), dtype_name(cfg.out_dtype)
        as_bits = lambda t16: t16.contiguous().view(torch.int16).numpy().view(np.uint16)
        inp = orc.RankInput(x=as_bits(x_c), indices=idx_c.numpy(), weights=w_c.numpy())
        rb, rm, tb, tm = as_bits(recv_b), recv_m.numpy(), as_bits(ret_b), ret_m.numpy()

        def vec_step():
            t = [time.perf_counter()]
            orc.dispatch_send(inp, r0, W, nle); t.append(time.perf_counter())
            cnt, local, pos, order = orc.expert_placement(rm, nle)
            rows, metas = rb[order], rm[order]; t.append(time.perf_counter())
            ey = orc.expert_scale(rows, r0, dt_in, dt_out); t.append(time.perf_counter())
            _, back = orc.return_order(metas, W)
            ey[back], metas[back]; t.append(time.perf_counter())
            yv = orc.combine_recv(tb, tm, inp.weights, T, dt_out); t.append(time.perf_counter())
            return yv, [b - a_ for a_, b in zip(t, t[1:])]

        vruns, vspent = [], 0.0
        while vspent < args.cpu_seconds / 3 and len(vruns) < 100:
            yv, parts = vec_step()
            vruns.append(parts)
            vspent += sum(parts)
        vmed = [statistics.median(r[i] for r in vruns) for i in range(5)]
        out["cpu_baseline"] = {
            "value": round(sum(med) * 1e6, 1), "unit": "us", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{len(runs)} full steps of rank {r0}'s share of {args.workload} "
                      f"({spent:.1f} s of CPU), median per phase",
            "hot_path_us": round(cpu_path_us, 1),
            "expert_standin_us": round(med[2] * 1e6, 1),
            "host_cpus": os.cpu_count(),
            "matches_gpu_bits": bool(torch.equal(yc, y_after.cpu())),
            "vectorised": {
                "value": round(sum(vmed) * 1e6, 1), "unit": "us", "cores": 1,
                "hot_path_us": round((vmed[0] + vmed[1] + vmed[3] + vmed[4]) * 1e6, 1),
                "sample": f"{len(vruns)} steps of the numpy statement ({vspent:.1f} s of CPU), valid rows only",
                "matches_gpu_bits": bool(np.array_equal(yv, as_bits(y_after.cpu()))),
            },
        }

    print(json.dumps(out))


if __name__ == "__main__":
    main()
