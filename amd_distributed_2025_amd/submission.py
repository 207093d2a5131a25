"""`custom_kernel(data)` — the entry point the reference's harness calls
(all2all/submission.py:339-356, all2all/hipv8.py:375-394; contract in
all2all/task.py:8-9): `data = (cfg, rank_data, rank, world_size)` in, the
rank's `[num_tokens, hidden_dim]` result of `cfg.out_dtype` out.

On one GPU the other ranks of the job do not exist as processes. Their inputs
are registered once with `set_peer_inputs` (they are synthesised from the same
seeds the harness would give those ranks); `custom_kernel` then steps the whole
job through `LocalWorld` on the caller's device and returns the caller's rows.
With `world_size == 1` nothing has to be registered.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence, Tuple

import torch

from .all2all import HIPAllToAll, LocalWorld
from .task import MoEConfig, input_t, output_t

_peers: Optional[Sequence[input_t]] = None
_worlds: Dict[Tuple, LocalWorld] = {}


def set_peer_inputs(inputs: Optional[Sequence[input_t]]) -> None:
    """Register the inputs of every rank of the job (index = rank). The entry of
    the calling rank is ignored: its data comes with the call."""
    global _peers
    _peers = inputs


def _world_for(cfg: MoEConfig, world_size: int, device: torch.device) -> LocalWorld:
    key = (cfg.num_experts, cfg.experts_per_token, cfg.hidden_dim, cfg.max_num_tokens,
           cfg.in_dtype, cfg.out_dtype, world_size, str(device))
    w = _worlds.get(key)
    if w is None:
        _worlds.clear()  # one job shape at a time keeps the workspaces bounded
        w = _worlds[key] = LocalWorld(cfg, world_size, device=device)
    return w


def custom_kernel_job(inputs: Sequence[input_t]) -> list:
    """Every rank's `custom_kernel` result from ONE step of the job: what W processes calling
    `custom_kernel` at the same time produce together. `inputs[r]` is rank r's tuple."""
    cfg, first, _, world_size = inputs[0]
    device = first.x.device
    if device.type != "cuda":
        raise RuntimeError("custom_kernel needs its inputs on a GPU; this path has no CPU fallback")
    if len(inputs) != world_size:
        raise ValueError(f"a job of world_size={world_size} needs {world_size} inputs, got {len(inputs)}")
    with torch.cuda.device(device):
        ys = _world_for(cfg, world_size, device).run([d[1].to(device) for d in inputs])
        return [y.clone() for y in ys]


def custom_kernel(data: input_t) -> output_t:
    cfg, rank_data, rank, world_size = data
    device = rank_data.x.device
    if device.type != "cuda":
        raise RuntimeError("custom_kernel needs its inputs on a GPU; this path has no CPU fallback")
    if world_size == 1:
        everyone = [rank_data]
    else:
        if _peers is None or len(_peers) != world_size:
            raise RuntimeError(
                f"world_size={world_size}: register the job's per-rank inputs with set_peer_inputs() first"
            )
        everyone = [rank_data if r == rank else _peers[r][1].to(device) for r in range(world_size)]
    with torch.cuda.device(device):
        ys = _world_for(cfg, world_size, device).run(everyone)
        return ys[rank].clone()
