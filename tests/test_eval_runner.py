"""The runner of the task's test/benchmark lists (amd_distributed_2025_amd/eval.py):
spec parsing, the reference's comparison rule, the ranking rule on the CPU; a real
pass over a short spec, with the oracle as the reference implementation, on the GPU."""
import json
import textwrap

import numpy as np
import pytest
import torch

from amd_distributed_2025_amd import eval as runner
from amd_distributed_2025_amd.task import (TASK_YML_BENCHMARKS, TASK_YML_TESTS, MoEConfig, generate_input)
from tests.helpers import from_bits, run_oracle


def write(tmp_path, text):
    p = tmp_path / "task.yml"
    p.write_text(textwrap.dedent(text))
    return p


def test_shipped_spec_is_the_reference_lists():
    spec = runner.load_spec()
    assert spec["tests"] == TASK_YML_TESTS          # all2all/task.yml:48-57
    assert spec["benchmarks"] == TASK_YML_BENCHMARKS  # all2all/task.yml:60-65
    assert spec["ranking_by"] == "geom"             # all2all/task.yml:68


def test_spec_errors_are_reported(tmp_path):
    good = '{"num_experts": 8, "experts_per_token": 2, "hidden_dim": 64, "max_num_tokens": 4, "seed": 1, "world_size": 2}'
    assert runner.load_spec(write(tmp_path, f"tests:\n  - {good}\n"))["tests"][0]["hidden_dim"] == 64
    assert runner.load_spec(write(tmp_path, "lang: py\n")) == {"ranking_by": "geom", "tests": [], "benchmarks": []}
    for bad in (good.replace('"seed": 1, ', ""),                       # missing key
                good.replace('"seed": 1', '"seed": 1, "flavour": 3'),  # unknown key
                good.replace('"seed": 1', '"seed": 1.5'),              # not an integer
                good.replace('"seed": 1', '"seed": true'),
                good.replace('"world_size": 2', '"world_size": 3')):   # experts do not divide
        with pytest.raises(ValueError):
            runner.load_spec(write(tmp_path, f"benchmarks:\n  - {bad}\n"))
    with pytest.raises(ValueError):
        runner.load_spec(write(tmp_path, 'ranking_by: "mean"\n'))


def test_comparison_rule():
    data = generate_input(8, 2, 16, 4, seed=3, rank=0, world_size=1)
    cfg, rd, _, _ = data
    T = rd.num_tokens
    good = torch.ones(T, 16, dtype=cfg.out_dtype)
    assert runner.check_implementation(None, good, data) == (True, "")
    assert runner.check_implementation(good.clone(), good, data) == (True, "")
    # rtol 1e-2, atol 5e-3 (all2all/reference.py:279): 1.0 vs 1.0146 passes, 1.0 vs 1.0156 does not
    near = torch.full_like(good, 1.0146)
    far = torch.full_like(good, 1.0166)
    assert runner.check_implementation(near, good, data)[0]
    ok, msg = runner.check_implementation(far, good, data)
    assert not ok and "mismatch" in msg
    assert not runner.check_implementation(None, good[:-1] if T > 1 else good[:, :-1], data)[0]
    assert not runner.check_implementation(None, good.float(), data)[0]
    bad = good.clone(); bad[0, 0] = float("nan")
    assert not runner.check_implementation(None, bad, data)[0]


def test_ranking_rule():
    assert runner.geometric_mean([2.0, 8.0]) == pytest.approx(4.0)
    assert runner.geometric_mean([5.0]) == pytest.approx(5.0)
    for bad in ([], [1.0, 0.0], [1.0, -2.0]):
        with pytest.raises(ValueError):
            runner.geometric_mean(bad)


def test_runner_refuses_to_run_without_a_gpu(capsys):
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    assert runner.main(["benchmark"]) == 2
    assert "GPU" in capsys.readouterr().err


# ------------------------------------------------------------------ on the GPU

SHORT = {"ranking_by": "geom",
         "tests": [dict(num_experts=8, experts_per_token=2, hidden_dim=6144, max_num_tokens=4, seed=1236, world_size=8),
                   dict(num_experts=64, experts_per_token=6, hidden_dim=2048, max_num_tokens=8, seed=542, world_size=8)],
         "benchmarks": [dict(num_experts=8, experts_per_token=2, hidden_dim=512, max_num_tokens=16, seed=6, world_size=4),
                        dict(num_experts=64, experts_per_token=6, hidden_dim=256, max_num_tokens=32, seed=7, world_size=8)]}


class OracleReference:
    """`ref_kernel` stand-in: the oracle's result for the rank of `data`; the job's other ranks
    are regenerated from the job shape and seed the way the runner does."""

    def __init__(self, spec):
        self.expected = {}
        for job in spec["tests"]:
            world = runner.job_inputs(job, "cpu")
            for r, t in enumerate(run_oracle(world)):
                self.expected[(job["seed"], job["hidden_dim"], job["max_num_tokens"], r)] = from_bits(t.y, world[0][0].out_dtype)
        self.calls = 0

    def __call__(self, data):
        cfg, rd, rank, _ = data
        self.calls += 1
        return self.expected[(self.seed_of(cfg), cfg.hidden_dim, cfg.max_num_tokens, rank)]

    def seed_of(self, cfg):
        for job in SHORT["tests"]:
            if (job["hidden_dim"], job["max_num_tokens"]) == (cfg.hidden_dim, cfg.max_num_tokens):
                return job["seed"]
        raise KeyError


@pytest.mark.gpu
def test_short_spec_passes_against_the_oracle_and_fails_against_a_wrong_reference():
    lines = []
    ref = OracleReference(SHORT)
    assert runner.run_tests(SHORT, torch.device("cuda:0"), ref, log=lines.append)
    assert ref.calls == 16 and all("FAIL" not in l for l in lines)
    lines.clear()
    assert not runner.run_tests(SHORT, torch.device("cuda:0"), lambda data: ref(data) + 1.0, log=lines.append)
    assert any("FAIL" in l for l in lines)
    assert runner.run_tests(SHORT, torch.device("cuda:0"), None, log=lines.append)  # structural checks only


@pytest.mark.gpu
def test_benchmark_mode_reports_the_geometric_mean():
    out = runner.run_benchmarks(SHORT, torch.device("cuda:0"), repeats=5, warmup=1, log=lambda s: None)
    rows = out["benchmarks"]
    assert [r["world_size"] for r in rows] == [4, 8] and all(r["us_all_ranks"] > 0 for r in rows)
    assert out["geom_mean_us_per_rank"] == pytest.approx(
        runner.geometric_mean([r["us_per_rank"] for r in rows]))
    json.dumps(out)
