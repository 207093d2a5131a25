"""Writes the golden fixtures of this directory.

    python tests/golden/make_golden.py

Each `<case>.npz` holds, for every rank r of one small job, the inputs
(`r{r}_x` as uint16 bit patterns, `r{r}_indices`, `r{r}_weights`) and the
outputs of every step of the path as computed by the row-by-row torch-CPU
statement in `oracle/rowwise_torch.py` (the producer), stored as plain arrays:
counts, meta rows, expert counts, result rows `y` as bit patterns. The large row
buffers are pure row permutations of `x` (scaled after the expert), so they are
stored as one CRC32 per buffer over their bytes plus their meta rows, which
name every row.

The reference ships no vectors for this path; these fixtures pin this build's
own statements of it against each other and against later changes.
"""
from __future__ import annotations

import sys
import zlib
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent.parent))

from amd_distributed_2025_amd.task import WORKLOADS, generate_world  # noqa: E402
from oracle import rowwise_torch as rw  # noqa: E402

CASES = {
    # name: (workload dict, seed)
    "c1_w1_e8_k2_h256": (WORKLOADS["C1"], 11),
    "c2_w8_e8_k2_h2048": (WORKLOADS["C2"], 12),
    "ref_style_fp16_w4_e8_k3_h64": (
        dict(world_size=4, num_experts=8, experts_per_token=3, hidden_dim=64, max_num_tokens=12,
             num_tokens="reference", routing="uniform", weights="rand", dtype="fp16"), 13),
    "zipf_w8_e64_k6_h128": (
        dict(world_size=8, num_experts=64, experts_per_token=6, hidden_dim=128, max_num_tokens=24,
             num_tokens="uniform", routing="zipf", weights="softmax", dtype="bf16"), 14),
}


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def crc(a: np.ndarray) -> np.uint32:
    return np.uint32(zlib.crc32(np.ascontiguousarray(a).tobytes()))


def valid_rows(padded: torch.Tensor, n_per: torch.Tensor) -> torch.Tensor:
    return torch.cat([padded[le, : int(n_per[le])] for le in range(padded.shape[0])], dim=0)


def build(workload: dict, seed: int) -> dict:
    world = generate_world(workload, seed)
    cfg = world[0][0]
    out = rw.run_world_rowwise([d.x for _, d, _, _ in world], [d.indices for _, d, _, _ in world],
                               [d.weights for _, d, _, _ in world], cfg.num_experts,
                               cfg.max_num_tokens, cfg.out_dtype)
    z = dict(world_size=np.int32(len(world)), num_experts=np.int32(cfg.num_experts),
             experts_per_token=np.int32(cfg.experts_per_token), hidden_dim=np.int32(cfg.hidden_dim),
             max_num_tokens=np.int32(cfg.max_num_tokens), dtype=np.str_(workload["dtype"]),
             seed=np.int32(seed))
    for r, ((_, d, _, _), o) in enumerate(zip(world, out)):
        p = f"r{r}_"
        z[p + "x"] = bits(d.x)
        z[p + "indices"] = d.indices.numpy()
        z[p + "weights"] = d.weights.numpy()
        for name in ("send_counts", "recv_counts", "back_counts", "ret_counts"):
            z[p + name] = o[name].numpy().astype(np.int64)
        for name in ("send_meta", "recv_meta", "back_meta", "ret_meta"):
            z[p + name] = o[name].numpy()
        z[p + "expert_num_tokens"] = o["expert_num_tokens"].numpy()
        z[p + "expert_meta_rows"] = valid_rows(o["expert_meta"], o["expert_num_tokens"]).numpy()
        for name in ("send_buf", "recv_buf", "back_buf", "ret_buf"):
            z[p + name + "_crc"] = crc(bits(o[name]))
        z[p + "expert_rows_crc"] = crc(bits(valid_rows(o["expert_x"], o["expert_num_tokens"])))
        z[p + "expert_y_rows_crc"] = crc(bits(valid_rows(o["expert_y"], o["expert_num_tokens"])))
        z[p + "y"] = bits(o["y"])
    return z


if __name__ == "__main__":
    for name, (workload, seed) in CASES.items():
        np.savez_compressed(HERE / f"{name}.npz", **build(workload, seed))
        print("wrote", name, (HERE / f"{name}.npz").stat().st_size, "bytes")
