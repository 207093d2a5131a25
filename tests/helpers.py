"""Shared glue for the tests: conversions between the package's torch inputs and
the numpy oracle's bit-pattern arrays."""
from __future__ import annotations

import numpy as np
import torch

from oracle import moe_a2a_oracle as orc


def bits(t: torch.Tensor) -> np.ndarray:
    """16-bit float tensor -> uint16 bit patterns (host)."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(a: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(dtype)


def oracle_inputs(world):
    """list of input_t -> list of oracle RankInput"""
    return [
        orc.RankInput(x=bits(d.x), indices=d.indices.cpu().numpy().astype(np.int32),
                      weights=d.weights.cpu().numpy().astype(np.float32))
        for (_, d, _, _) in world
    ]


def run_oracle(world, expert=None):
    from amd_distributed_2025_amd.task import dtype_name

    cfg = world[0][0]
    return orc.run_world(oracle_inputs(world), cfg.num_experts, cfg.max_num_tokens,
                         dtype_name(cfg.in_dtype), dtype_name(cfg.out_dtype), expert=expert)
