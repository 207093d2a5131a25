"""`custom_kernel(data)` — the entry point the reference's harness calls
(all2all/submission.py:339-356, all2all/hipv8.py:375-394; contract in
all2all/task.py:8-9): `data = (cfg, rank_data, rank, world_size)` in, the
rank's `[num_tokens, hidden_dim]` result of `cfg.out_dtype` out.

On one GPU the other ranks of the job do not exist as processes. Their inputs
are registered once with `set_peer_inputs` (they are synthesised from the same
seeds the harness would give those ranks); `custom_kernel` then steps the whole
job through `LocalWorld` on the caller's device and returns the caller's rows.
With `world_size == 1` nothing has to be registered.

A harness calls the entry point again and again on jobs of one shape. The first
call of a job (a shape and the token counts of its ranks) runs launch by launch
and reads the exchanged counts back to size its launches; from the second call
on the job is a HIP graph captured once (one per rank asked for: a call needs
every rank's dispatch, experts and send-back, but only the caller's return
exchange and weighted sum): the inputs are copied into buffers the
graph reads, the graph is replayed, the result is copied out. The graph's
launches are sized by the counts of the first call; sizes are a matter of speed
only, every kernel moves what the device-side counts of the call at hand say.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .all2all import LocalWorld
from .task import MoEConfig, RankTestData, input_t, output_t

_peers: Optional[Sequence[input_t]] = None
_worlds: Dict[Tuple, "_World"] = {}
MAX_CAPTURED_JOBS = 18  # graphs kept per job shape (each holds only launches; the buffers are the world's)


def set_peer_inputs(inputs: Optional[Sequence[input_t]]) -> None:
    """Register the inputs of every rank of the job (index = rank). The entry of
    the calling rank is ignored: its data comes with the call."""
    global _peers
    _peers = inputs


class _World:
    """A `LocalWorld` of one job shape with the buffers its captured jobs read their inputs from."""

    def __init__(self, cfg: MoEConfig, world_size: int, device: torch.device):
        self.lw = LocalWorld(cfg, world_size, device=device)
        T, K, H = cfg.max_num_tokens, cfg.experts_per_token, cfg.hidden_dim
        self.x = [torch.empty(T, H, dtype=cfg.in_dtype, device=device) for _ in range(world_size)]
        self.indices = [torch.empty(T, K, dtype=torch.int32, device=device) for _ in range(world_size)]
        self.weights = [torch.empty(T, K, dtype=torch.float32, device=device) for _ in range(world_size)]
        self.seen: Dict[Tuple[int, ...], int] = {}
        self.graphs: Dict[Tuple, Tuple[torch.cuda.CUDAGraph, List[torch.Tensor]]] = {}

    def _staged(self, tokens: Tuple[int, ...]) -> List[RankTestData]:
        """Views of the input buffers cut to the job's token counts, as rank inputs."""
        out = []
        for r, t in enumerate(tokens):
            d = object.__new__(RankTestData)
            d.num_tokens, d.rank = t, r
            d.x, d.indices, d.weights = self.x[r][:t], self.indices[r][:t], self.weights[r][:t]
            out.append(d)
        return out

    def run(self, everyone: Sequence[RankTestData], only: Optional[int] = None) -> List[torch.Tensor]:
        """One step of the job; `only=r` leaves out what only the other ranks' results need (their
        return exchange and weighted sum) and returns None in their places."""
        tokens = tuple(int(d.num_tokens) for d in everyone)
        calls = self.seen.get(tokens, 0)
        self.seen[tokens] = calls + 1
        if calls == 0:  # launch by launch, reading the counts back: they size the later launches
            self.lw.exact_hints = True
            return self.lw.run(everyone, only=only)
        staged = self._staged(tokens)
        torch._foreach_copy_([d.x for d in staged] + [d.indices for d in staged] + [d.weights for d in staged],
                             [d.x for d in everyone] + [d.indices for d in everyone] + [d.weights for d in everyone])
        key = (tokens, only)
        if key not in self.graphs:
            while len(self.graphs) >= MAX_CAPTURED_JOBS:
                self.graphs.pop(next(iter(self.graphs)))
            # the counts sizing the launches are those the latest launch-by-launch run of this world
            # read back; a job of other token counts came in between only if it ran that way too
            self.lw.exact_hints = True
            self.lw.run(staged, only=only)  # (also leaves every workspace buffer allocated before the capture)
            self.lw.exact_hints = "last"
            torch.cuda.synchronize(self.lw.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                ys = self.lw.run(staged, only=only)
            self.graphs[key] = (graph, ys)
        graph, ys = self.graphs[key]
        graph.replay()
        return ys


def _world_for(cfg: MoEConfig, world_size: int, device: torch.device) -> _World:
    key = (cfg.num_experts, cfg.experts_per_token, cfg.hidden_dim, cfg.max_num_tokens,
           cfg.in_dtype, cfg.out_dtype, world_size, str(device))
    w = _worlds.get(key)
    if w is None:
        _worlds.clear()  # one job shape at a time keeps the workspaces bounded
        w = _worlds[key] = _World(cfg, world_size, device)
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
        ys = _world_for(cfg, world_size, device).run(everyone, only=rank)
        return ys[rank].clone()
