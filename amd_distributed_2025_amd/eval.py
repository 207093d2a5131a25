"""Runner for the task's test and benchmark lists on one GPU.

The reference names an `eval.py` as the main program of the task
(all2all/task.yml:8,14) without shipping it; what it has to do follows from the
task file: run every entry of `tests:` through `custom_kernel` on every rank and
compare with `check_implementation` (all2all/reference.py:275-283), time every
entry of `benchmarks:` and rank by the geometric mean (all2all/task.yml:34,68).
This module does that for one GPU, where the ranks of a job are stepped in
lockstep by `LocalWorld` instead of running as one process per GPU.

    python -m amd_distributed_2025_amd.eval benchmark [--spec task.yml] [--repeats 50]
    python -m amd_distributed_2025_amd.eval test --reference package.module:function

`test` needs a reference implementation to compare with (a callable
`data -> output`, the role of `ref_kernel`); this package ships none, so the
caller names one. Without `--reference` only the structural checks run (shape,
dtype, device, finite values).
"""
from __future__ import annotations

import argparse
import importlib
import json
import math
import sys
import time
from pathlib import Path
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch
import yaml

from .task import generate_input, input_t, output_t

SPEC_FILE = Path(__file__).resolve().parent / "task.yml"
JOB_KEYS = ("num_experts", "experts_per_token", "hidden_dim", "max_num_tokens", "seed", "world_size")
# tolerances of the reference's comparison (all2all/reference.py:279)
RTOL, ATOL = 1e-2, 5e-3


def load_spec(path=SPEC_FILE) -> Dict:
    """Parse a task file: `tests` and `benchmarks` become lists of job dicts with
    exactly JOB_KEYS (all integers); `ranking_by` defaults to "geom"."""
    with open(path) as f:
        raw = yaml.safe_load(f) or {}
    spec = {"ranking_by": raw.get("ranking_by", "geom")}
    if spec["ranking_by"] != "geom":
        raise ValueError(f"{path}: ranking_by={spec['ranking_by']!r} is not supported (only 'geom')")
    for section in ("tests", "benchmarks"):
        jobs = raw.get(section) or []
        out = []
        for n, job in enumerate(jobs):
            missing = [k for k in JOB_KEYS if k not in job]
            extra = [k for k in job if k not in JOB_KEYS]
            if missing or extra:
                raise ValueError(f"{path}: {section}[{n}]: missing {missing}, unknown {extra}")
            if any(not isinstance(job[k], int) or isinstance(job[k], bool) for k in JOB_KEYS):
                raise ValueError(f"{path}: {section}[{n}]: every field must be an integer")
            if job["num_experts"] % job["world_size"]:
                raise ValueError(f"{path}: {section}[{n}]: num_experts must be a multiple of world_size")
            out.append({k: job[k] for k in JOB_KEYS})
        spec[section] = out
    return spec


def job_inputs(job: Dict, device, **input_rules) -> List[input_t]:
    """`generate_input` for every rank of a job (all2all/reference.py:237-253)."""
    shape = {k: job[k] for k in JOB_KEYS if k not in ("seed", "world_size")}
    W = job["world_size"]
    return [generate_input(seed=job["seed"], rank=r, world_size=W, device=device, **shape, **input_rules)
            for r in range(W)]


def check_implementation(expected: Optional[output_t], output: output_t, data: input_t) -> Tuple[bool, str]:
    """The reference's comparison (all2all/reference.py:275-283) with the expected
    tensor handed in, preceded by the checks that need no reference."""
    cfg, rank_data, _, _ = data
    want_shape = (rank_data.num_tokens, cfg.hidden_dim)
    if tuple(output.shape) != want_shape:
        return False, f"Output shape mismatch: {tuple(output.shape)} != {want_shape}"
    if output.dtype != cfg.out_dtype:
        return False, f"Output dtype mismatch: {output.dtype} != {cfg.out_dtype}"
    if output.device != rank_data.x.device:
        return False, f"Output device mismatch: {output.device} != {rank_data.x.device}"
    if not bool(torch.isfinite(output.float()).all()):
        return False, "Output holds non-finite values"
    if expected is None:
        return True, ""
    expected = expected.to(output.device)
    if not torch.allclose(output, expected, rtol=RTOL, atol=ATOL):
        worst = (output.float() - expected.float()).abs().max().item()
        return False, f"Output values mismatch, largest absolute difference {worst:g}"
    return True, ""


def geometric_mean(values: Sequence[float]) -> float:
    if not values or any(v <= 0 for v in values):
        raise ValueError("geometric mean needs positive values")
    return math.exp(sum(math.log(v) for v in values) / len(values))


def run_tests(spec: Dict, device, reference: Optional[Callable[[input_t], output_t]] = None,
              log=print) -> bool:
    """Every job of the test list: the job is stepped once (all ranks together, as the
    reference's harness has all ranks call `custom_kernel` at the same time) and every rank's
    output is checked; rank 0 is also asked for through `custom_kernel` itself."""
    from .submission import custom_kernel, custom_kernel_job, set_peer_inputs

    all_ok = True
    for n, job in enumerate(spec["tests"]):
        world = job_inputs(job, device)
        outs = custom_kernel_job(world)
        job_ok = True
        for data, out in zip(world, outs):
            ok, msg = check_implementation(None if reference is None else reference(data), out, data)
            if not ok:
                job_ok = False
                log(f"test {n} {job} rank {data[2]}: FAIL {msg}")
        set_peer_inputs(world)
        try:
            if not torch.equal(custom_kernel(world[0]), outs[0]):
                job_ok = False
                log(f"test {n} {job} rank 0: FAIL custom_kernel(data) differs from the job's step")
        finally:
            set_peer_inputs(None)
        log(f"test {n} {job}: {'checked' if job_ok else 'see failures above'}")
        all_ok = all_ok and job_ok
    return all_ok


def run_benchmarks(spec: Dict, device, repeats: int = 50, warmup: int = 5, log=print) -> Dict:
    """Times one dispatch+combine of every rank of each job, stepped on this one
    GPU (`LocalWorld.run`), and the geometric mean over the jobs. The job is
    captured once into a HIP graph and replayed, so the figure is device time,
    not Python launch overhead; launches are sized from the counts of one eager run.
    It includes the stand-ins (W*W exchange legs per direction, W expert
    kernels). `us_per_rank` divides by world_size: the ranks run one after the
    other here."""
    from .all2all import LocalWorld

    rows = []
    for n, job in enumerate(spec["benchmarks"]):
        world = job_inputs(job, device)
        lw = LocalWorld(world[0][0], job["world_size"], device=device)
        data = [d for _, d, _, _ in world]
        side = torch.cuda.Stream(device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(side):  # allocates the workspaces and reads the row counts back once
            lw.run(data)
        torch.cuda.current_stream(device).wait_stream(side)
        torch.cuda.synchronize(device)
        lw.exact_hints = "last"  # the replayed job is the same job: launch sizes from that run
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            lw.run(data)
        for _ in range(warmup):
            graph.replay()
        torch.cuda.synchronize(device)
        t0 = time.perf_counter()
        for _ in range(repeats):
            graph.replay()
        torch.cuda.synchronize(device)
        us = (time.perf_counter() - t0) * 1e6 / repeats
        rows.append({**job, "us_all_ranks": us, "us_per_rank": us / job["world_size"]})
        log(f"benchmark {n} {job}: {us:.1f} us for all ranks, {us / job['world_size']:.1f} us per rank")
        del graph, lw
    result = {"benchmarks": rows, "ranking_by": spec["ranking_by"]}
    if rows:
        result["geom_mean_us_per_rank"] = geometric_mean([r["us_per_rank"] for r in rows])
        log(f"geometric mean: {result['geom_mean_us_per_rank']:.1f} us per rank")
    return result


def _resolve(dotted: str) -> Callable:
    module, _, name = dotted.partition(":")
    if not name:
        raise ValueError("--reference takes package.module:function")
    return getattr(importlib.import_module(module), name)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m amd_distributed_2025_amd.eval")
    ap.add_argument("mode", choices=["test", "benchmark"])
    ap.add_argument("--spec", default=str(SPEC_FILE))
    ap.add_argument("--reference", help="package.module:function returning the expected output of one rank")
    ap.add_argument("--repeats", type=int, default=50)
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    spec = load_spec(args.spec)
    if not torch.cuda.is_available():
        print("this runner needs a GPU (the path has no CPU fallback)", file=sys.stderr)
        return 2
    device = torch.device(args.device)
    torch.cuda.set_device(device)
    if args.mode == "test":
        ok = run_tests(spec, device, _resolve(args.reference) if args.reference else None)
        print("pass" if ok else "fail")
        return 0 if ok else 1
    print(json.dumps(run_benchmarks(spec, device, repeats=args.repeats)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
