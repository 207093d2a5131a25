"""The one-GPU part of the reference's gemm-rs task: `input @ weight.T (+ bias)`.

The reference's `ref_kernel` (gemm-rs/reference.py:36-60) multiplies this rank's
[M, local_K] slice of the activations with its [N, local_K] slice of the weight,
adds the bias, and reduce-scatters the [M, N] partial products over the ranks.
`local_product` is everything up to the reduce-scatter, on the matrix cores of
one MI355X through `moe_a2a_linear`; the reduce-scatter is an exchange between
GPUs and is not part of this package. `custom_kernel` therefore serves a job of
one rank (where the reduce-scatter is the identity) and refuses larger ones.

`generate_input` restates gemm-rs/reference.py:5-33 (uniform values in
[-0.01, 0.01), bias drawn from the job seed so that all ranks share it).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from . import _binding
from .all2all import _stream

input_t = Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]

# (m, n, k of the 8-rank job, has_bias, seed): gemm-rs/task.yml:66-76 (tests) and :80-85 (benchmarks,
# ranked by their geometric mean, task.yml:62)
TASK_TESTS = [(64, 2880, 2880, True, 2035), (64, 3584, 14336, True, 13), (512, 3584, 14336, True, 4297),
              (512, 4608, 36864, False, 1597), (2048, 4096, 7168, False, 716), (2048, 8192, 30720, False, 20201),
              (4096, 2880, 2880, True, 136), (4096, 8192, 2048, True, 138), (8192, 3584, 14336, True, 748),
              (8192, 4608, 36864, True, 4422), (8192, 8192, 28672, False, 1536)]
TASK_BENCHMARKS = [(64, 7168, 18432, False, 1234), (512, 4096, 12288, True, 663), (2048, 2880, 2880, True, 166),
                   (4096, 4096, 4096, False, 1371), (8192, 4096, 14336, True, 7168), (8192, 8192, 29568, False, 42)]


def generate_input(rank: int, world_size: int, m: int, n: int, k: int, has_bias: bool, seed: int,
                   device=None) -> input_t:
    device = torch.device(device if device is not None else f"cuda:{rank}")
    gen = torch.Generator(device=device)
    gen.manual_seed(seed + rank)
    if m % world_size or k % world_size:
        raise ValueError("m and k must be divisible by world_size")
    local_k = k // world_size
    inp = (torch.rand((m, local_k), dtype=torch.bfloat16, device=device, generator=gen) * 2 - 1) * 0.01
    weight = (torch.rand((n, local_k), dtype=torch.bfloat16, device=device, generator=gen) * 2 - 1) * 0.01
    bias = None
    if has_bias:
        gen.manual_seed(seed)
        bias = (torch.rand((n,), dtype=torch.bfloat16, device=device, generator=gen) * 2 - 1) * 0.01
    return inp, weight, bias


def local_product(data: input_t, out: Optional[torch.Tensor] = None, binding: str = "ctypes") -> torch.Tensor:
    """`matmul(input, weight.T)` rounded to the 16-bit type, then `+ bias` rounded again
    (gemm-rs/reference.py:54-57), as one launch. Returns [M, N]."""
    inp, weight, bias = data
    if inp.dim() != 2 or weight.dim() != 2 or inp.shape[1] != weight.shape[1]:
        raise ValueError(f"input [M, K] and weight [N, K] expected, got {tuple(inp.shape)} and {tuple(weight.shape)}")
    if inp.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError(f"input: expected float16 or bfloat16, got {inp.dtype}")
    if not inp.is_cuda:
        raise ValueError("input: expected a GPU tensor (there is no CPU path)")
    tensors = [("weight", weight)] + ([("bias", bias)] if bias is not None else [])
    for what, t in [("input", inp)] + tensors:
        if t.dtype != inp.dtype or t.device != inp.device or not t.is_contiguous():
            raise ValueError(f"{what}: must be contiguous, {inp.dtype}, on {inp.device}")
    m, n = inp.shape[0], weight.shape[0]
    if bias is not None and tuple(bias.shape) != (n,):
        raise ValueError(f"bias must be [{n}], got {tuple(bias.shape)}")
    if out is None:
        out = torch.empty((m, n), dtype=inp.dtype, device=inp.device)
    elif tuple(out.shape) != (m, n) or out.dtype != inp.dtype or out.device != inp.device or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous [{m}, {n}] {inp.dtype} tensor on {inp.device}")
    stream = _stream(inp.device)
    _binding.get(binding).linear(inp, weight, bias, out, stream)
    return out


def custom_kernel(data: input_t) -> torch.Tensor:
    """The reference's entry point (gemm-rs/submission.py:9-29) for a job of one rank."""
    world_size = torch.distributed.get_world_size() if torch.distributed.is_initialized() else 1
    if world_size != 1:
        raise NotImplementedError("the reduce-scatter over several GPUs is outside this package; "
                                  "local_product() gives this rank's [M, N] partial product")
    return local_product(data)


def reduce_scatter_local(partials: Sequence[torch.Tensor], rank: int) -> torch.Tensor:
    """Stand-in, on one GPU, for the `reduce_scatter_tensor` that ends the reference's kernel
    (gemm-rs/reference.py:58-59): rank `rank`'s [M / W, N] slice of the sum of all W ranks'
    [M, N] partial products. The sum is formed in float32 in rank order and rounded once; the
    collective's own order and intermediate roundings are the library's, so results agree with
    it within the task's tolerance (rtol = atol = 1e-2, reference.py:66), not to the bit."""
    world_size = len(partials)
    m, n = partials[0].shape
    if m % world_size:
        raise ValueError("m must be divisible by world_size")
    rows = slice(rank * (m // world_size), (rank + 1) * (m // world_size))
    total = partials[0][rows].float()
    for p in partials[1:]:
        total += p[rows].float()
    return total.to(partials[0].dtype)


def run_job(world: Sequence[input_t], binding: str = "ctypes") -> List[torch.Tensor]:
    """All ranks of a job on one GPU: every rank's local product through `moe_a2a_linear`, then
    the stand-in reduce-scatter. Returns the ranks' [M / W, N] outputs. (As in the reference,
    every rank adds the bias before the sum, so the result holds it W times.)"""
    partials = [local_product(data, binding=binding) for data in world]
    return [reduce_scatter_local(partials, r) for r in range(len(world))]
