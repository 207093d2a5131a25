"""Task contract of the all2all path: config, per-rank inputs, test specs.

Mirrors the names of the reference's task files so code written against them
reads the same here: `MoEConfig` (all2all/reference.py:10-17), `RankTestData`
(:21-51), `generate_input` (:237-253), `TestSpec` (all2all/task.py:12-17),
`input_t = (MoEConfig, RankTestData, rank, world_size)` (all2all/task.py:8).

Differences, all by necessity:
  * the reference draws its inputs from a CUDA generator on `cuda:{rank}`;
    here they come from a numpy PCG64 stream seeded `seed + rank`, on the host,
    and are then moved to the requested device, so the same inputs exist with
    and without a GPU;
  * the reference fixes fp16, `rand` weights, uniform routing and
    `num_tokens ~ randint(1, max_num_tokens)` (upper end exclusive); those are
    the defaults of `generate_input`'s extra keyword arguments, which also
    offer bf16, softmax weights, Zipf-skewed routing and other token-count
    rules.
"""
from __future__ import annotations

import dataclasses
from typing import Optional, Tuple, TypedDict

import numpy as np
import torch


@dataclasses.dataclass
class MoEConfig:
    num_experts: int
    experts_per_token: int
    hidden_dim: int
    max_num_tokens: int
    in_dtype: torch.dtype = torch.float16
    out_dtype: torch.dtype = torch.float16


class TestSpec(TypedDict):
    num_experts: int
    experts_per_token: int
    hidden_dim: int
    max_num_tokens: int
    seed: int


TestSpec.__test__ = False  # not a pytest class

DTYPES = {"fp16": torch.float16, "bf16": torch.bfloat16}


def dtype_name(dt: torch.dtype) -> str:
    for k, v in DTYPES.items():
        if v == dt:
            return k
    raise ValueError(f"unsupported token dtype {dt}")


def _draw_num_tokens(rng: np.random.Generator, max_num_tokens: int, rule: str) -> int:
    if rule == "reference":  # randint(1, max) with the upper end exclusive (reference.py:24-28)
        return int(rng.integers(1, max(max_num_tokens, 2)))
    if rule == "uniform":    # uniform on [1, max]
        return int(rng.integers(1, max_num_tokens + 1))
    if rule == "full":
        return int(max_num_tokens)
    raise ValueError(rule)


def _draw_indices(rng, T: int, E: int, K: int, routing: str, zipf_s: float, popularity_seed: int):
    if routing == "uniform":  # first K entries of a random permutation per token (reference.py:33-35)
        keys = rng.random((T, E))
    elif routing == "zipf":
        # expert popularity ~ 1/rank^s over a seeded permutation of the experts (shared by all
        # ranks of a job); K distinct experts per token drawn by those probabilities without
        # replacement (Gumbel top-K == sequential sampling without replacement)
        perm = np.random.default_rng(popularity_seed).permutation(E)
        p = 1.0 / np.arange(1, E + 1, dtype=np.float64) ** zipf_s
        logp = np.empty(E)
        logp[perm] = np.log(p / p.sum())
        keys = logp[None, :] + rng.gumbel(size=(T, E))
    else:
        raise ValueError(routing)
    top = np.argsort(-keys, axis=1, kind="stable")[:, :K]
    return np.ascontiguousarray(top, dtype=np.int32)


class RankTestData:
    """Inputs of one rank: `num_tokens`, `indices [T,K] int32`, `weights [T,K] f32`,
    `x [T,H] in_dtype` (reference: all2all/reference.py:21-51; same draw order)."""

    def __init__(
        self,
        cfg: MoEConfig,
        rng: np.random.Generator,
        rank: int,
        device: Optional[torch.device] = None,
        *,
        num_tokens: str = "reference",
        routing: str = "uniform",
        weights: str = "rand",
        zipf_s: float = 1.2,
        popularity_seed: int = 0,
    ):
        device = torch.device("cpu") if device is None else torch.device(device)
        T = _draw_num_tokens(rng, cfg.max_num_tokens, num_tokens)
        self.num_tokens = T
        idx = _draw_indices(rng, T, cfg.num_experts, cfg.experts_per_token, routing, zipf_s, popularity_seed)
        if weights == "rand":  # uniform [0,1), not normalised (reference.py:37-43)
            w = rng.random((T, cfg.experts_per_token), dtype=np.float32)
        elif weights == "softmax":
            logits = rng.standard_normal((T, cfg.experts_per_token)).astype(np.float32)
            w = torch.softmax(torch.from_numpy(logits), dim=1).numpy()
        else:
            raise ValueError(weights)
        x = rng.standard_normal((T, cfg.hidden_dim), dtype=np.float32)
        self.indices = torch.from_numpy(idx).to(device)
        self.weights = torch.from_numpy(np.ascontiguousarray(w, dtype=np.float32)).to(device)
        self.x = torch.from_numpy(x).to(cfg.in_dtype).to(device)
        self.rank = rank

    def to(self, device) -> "RankTestData":
        other = object.__new__(RankTestData)
        other.num_tokens, other.rank = self.num_tokens, self.rank
        other.indices = self.indices.to(device)
        other.weights = self.weights.to(device)
        other.x = self.x.to(device)
        return other


input_t = Tuple[MoEConfig, RankTestData, int, int]
output_t = torch.Tensor


def generate_input(
    num_experts: int,
    experts_per_token: int,
    hidden_dim: int,
    max_num_tokens: int,
    seed: int,
    rank: int,
    world_size: int,
    *,
    device=None,
    dtype: str = "fp16",
    num_tokens: str = "reference",
    routing: str = "uniform",
    weights: str = "rand",
    zipf_s: float = 1.2,
) -> input_t:
    """Same positional signature and return tuple as all2all/reference.py:237-253.
    The generator of rank r is seeded `seed + r`."""
    rng = np.random.default_rng(seed + rank)
    cfg = MoEConfig(
        num_experts=num_experts,
        experts_per_token=experts_per_token,
        hidden_dim=hidden_dim,
        max_num_tokens=max_num_tokens,
        in_dtype=DTYPES[dtype],
        out_dtype=DTYPES[dtype],
    )
    data = RankTestData(
        cfg, rng, rank, device,
        num_tokens=num_tokens, routing=routing, weights=weights, zipf_s=zipf_s, popularity_seed=seed,
    )
    return cfg, data, rank, world_size


# The five workloads this build is measured and checked on. C1 is the reference's own
# CPU-runnable case; C4 is the one the headline metric is quoted on.
WORKLOADS = {
    "C1": dict(world_size=1, num_experts=8, experts_per_token=2, hidden_dim=256, max_num_tokens=16,
               num_tokens="uniform", routing="uniform", weights="softmax", dtype="bf16"),
    "C2": dict(world_size=8, num_experts=8, experts_per_token=2, hidden_dim=2048, max_num_tokens=16,
               num_tokens="full", routing="uniform", weights="softmax", dtype="bf16"),
    "C3": dict(world_size=8, num_experts=64, experts_per_token=6, hidden_dim=2048, max_num_tokens=128,
               num_tokens="uniform", routing="uniform", weights="softmax", dtype="bf16"),
    "C4": dict(world_size=8, num_experts=256, experts_per_token=8, hidden_dim=7168, max_num_tokens=256,
               num_tokens="full", routing="uniform", weights="softmax", dtype="bf16"),
    "C5": dict(world_size=8, num_experts=256, experts_per_token=8, hidden_dim=7168, max_num_tokens=256,
               num_tokens="full", routing="zipf", weights="softmax", dtype="bf16"),
}


# The C4 shape with two, four and six times the tokens per rank (4096 to 12288 rows sent per rank):
# not part of the task's lists; bench.py times them to show how the path scales with the row count.
LARGE_WORKLOADS = {
    "C4x2": dict(WORKLOADS["C4"], max_num_tokens=512),
    "C4x4": dict(WORKLOADS["C4"], max_num_tokens=1024),
    "C4x6": dict(WORKLOADS["C4"], max_num_tokens=1536),
    # 32768 rows per rank: two ranks with C4's 32 local experts each and 4096 tokens
    "W2x16": dict(WORKLOADS["C4"], world_size=2, num_experts=64, max_num_tokens=4096),
}


def generate_world(workload: dict, seed: int, device=None):
    """Inputs of every rank of one job: list of `input_t`, one per rank."""
    spec = dict(workload)
    W = spec.pop("world_size")
    return [generate_input(seed=seed, rank=r, world_size=W, device=device, **spec) for r in range(W)]


# Shapes of the reference's own test and benchmark lists (all2all/task.yml:48-65).
TASK_YML_TESTS = [
    dict(num_experts=8, experts_per_token=2, hidden_dim=6144, max_num_tokens=4, seed=1236, world_size=8),
    dict(num_experts=64, experts_per_token=6, hidden_dim=2048, max_num_tokens=4, seed=1234, world_size=8),
    dict(num_experts=64, experts_per_token=6, hidden_dim=2048, max_num_tokens=8, seed=542, world_size=8),
    dict(num_experts=128, experts_per_token=4, hidden_dim=2880, max_num_tokens=16, seed=347, world_size=8),
    dict(num_experts=128, experts_per_token=4, hidden_dim=2880, max_num_tokens=32, seed=51, world_size=8),
    dict(num_experts=128, experts_per_token=8, hidden_dim=4096, max_num_tokens=64, seed=175, world_size=8),
    dict(num_experts=128, experts_per_token=8, hidden_dim=4096, max_num_tokens=128, seed=534, world_size=8),
    dict(num_experts=256, experts_per_token=8, hidden_dim=7168, max_num_tokens=64, seed=897, world_size=8),
    dict(num_experts=256, experts_per_token=8, hidden_dim=7168, max_num_tokens=128, seed=4, world_size=8),
]
TASK_YML_BENCHMARKS = [
    dict(num_experts=8, experts_per_token=2, hidden_dim=6144, max_num_tokens=16, seed=6635, world_size=8),
    dict(num_experts=64, experts_per_token=6, hidden_dim=2048, max_num_tokens=32, seed=1234, world_size=8),
    dict(num_experts=128, experts_per_token=4, hidden_dim=2880, max_num_tokens=128, seed=51, world_size=8),
    dict(num_experts=128, experts_per_token=8, hidden_dim=4096, max_num_tokens=256, seed=175, world_size=8),
    dict(num_experts=256, experts_per_token=8, hidden_dim=7168, max_num_tokens=256, seed=4, world_size=8),
]
