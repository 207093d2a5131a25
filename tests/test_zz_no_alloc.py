"""`moe_a2a_dispatch_recv_static`, the entry point that allocates nothing, against
`moe_a2a_dispatch_recv`, through the C ABI on a real GPU: same counts, same valid
rows of the expert-major buffers, same plan ints, and the plan address it hands
out drives `moe_a2a_combine_send` to the same send-back stream. Two calls in a
row, the second on a smaller job, because both share the library's one buffer."""
import ctypes as C

import numpy as np
import pytest
import torch

from amd_distributed_2025_amd import LocalWorld, _lib, generate_world
from oracle import moe_a2a_oracle as orc
from tests.helpers import bits, run_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

BIG = dict(world_size=8, num_experts=64, experts_per_token=6, hidden_dim=2048, max_num_tokens=128,
           num_tokens="uniform", routing="zipf", weights="softmax", dtype="bf16")
SMALL = dict(world_size=4, num_experts=8, experts_per_token=2, hidden_dim=264, max_num_tokens=16,
             num_tokens="full", routing="uniform", weights="rand", dtype="fp16")


class _RawInts:
    """n int32 at a raw device address, for torch.as_tensor (the array interface torch reads)."""

    def __init__(self, address: int, n: int):
        self.__cuda_array_interface__ = {"shape": (n,), "typestr": "<i4", "data": (address, False), "version": 2}


def device_ints(address: int, n: int) -> np.ndarray:
    """n int32 from a raw device address on the host (the plan lives in memory torch does not own):
    read through a tensor view of that address, by the runtime torch itself has loaded."""
    return torch.as_tensor(_RawInts(address, n), device=DEV).clone().cpu().numpy()


def one_job(spec, seed):
    """Rank 1's receive side of a job, once through each entry point; compares everything."""
    world = generate_world(spec, seed)
    cfg, W = world[0][0], len(world)
    lw = LocalWorld(cfg, W, device=DEV)
    lw.run([d.to(DEV) for _, d, _, _ in world])  # fills rank 1's receive buffers; plan from the existing entry point
    torch.cuda.synchronize()
    a, g = lw.ranks[1], lw.trace[1]
    nle, E = a.num_local_experts, cfg.num_experts
    R = int(g["recv_counts"].sum().item())
    cap = min(g["recv_buf"].shape[0], g["recv_meta"].shape[0])
    p = lambda t: C.c_void_p(t.data_ptr())
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    lib = _lib.load()

    # ---- the existing entry point, plan in a caller-owned buffer
    num0 = torch.full((nle,), -1, dtype=torch.int32, device=DEV)
    ex0, em0 = torch.zeros_like(g["expert_x"]), torch.full_like(g["expert_meta"], -9)
    plan0 = torch.full((2 * E,), -1, dtype=torch.int32, device=DEV)
    _lib.call("moe_a2a_dispatch_recv", C.byref(a.shape), p(g["recv_buf"]), p(g["recv_meta"]), p(g["recv_counts"]),
              R, cap, p(num0), p(ex0), p(em0), p(plan0), st)

    # ---- the entry point that allocates nothing
    before = torch.cuda.memory_allocated(DEV)
    num1 = torch.full((nle,), -1, dtype=torch.int32, device=DEV)
    ex1, em1 = torch.zeros_like(g["expert_x"]), torch.full_like(g["expert_meta"], -9)
    held = torch.cuda.memory_allocated(DEV)
    where = C.c_void_p()

    def call_static(stream):
        rc = lib.moe_a2a_dispatch_recv_static(C.byref(a.shape), p(g["recv_buf"]), p(g["recv_meta"]),
                                              p(g["recv_counts"]), R, cap, p(num1), p(ex1), p(em1),
                                              C.byref(where), stream)
        assert rc == 0, lib.moe_a2a_strerror(rc)
        assert where.value, "no plan address came back"

    call_static(st)  # (the first call on a GPU also looks the buffer's address up)
    assert torch.cuda.memory_allocated(DEV) == held > before  # torch's pool saw no allocation by the call
    torch.cuda.synchronize()
    # The same call while the stream is being captured: a device allocation or free by anyone
    # (hipMalloc, hipFree, torch's allocator) is refused during a capture and would fail it, so a
    # capture that ends well shows that the call made none. The replay then has to do the work.
    first_address = where.value
    num1.fill_(-1); ex1.zero_(); em1.fill_(-9)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call_static(C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert where.value == first_address
    assert bool((num1 == -1).all())  # captured, not run
    graph.replay()
    torch.cuda.synchronize()
    del graph

    cnt = num0.cpu().numpy()
    assert np.array_equal(cnt, run_oracle(world)[1].expert_num_tokens)
    assert torch.equal(num1, num0)
    for le in range(nle):
        n = int(cnt[le])
        assert torch.equal(ex1[le, :n], ex0[le, :n]) and torch.equal(em1[le, :n], em0[le, :n]), le
        assert bool((em1[le, n:] == -9).all()), le
    plan1 = device_ints(where.value, 2 * E)
    assert np.array_equal(plan1, plan0.cpu().numpy())

    # ---- the plan address drives combine_send like a caller-owned plan
    ey = a.expert_scale(ex0, num0, R)
    outs = []
    for plan_arg in (p(plan0), where):
        bc = torch.full((W,), -1, dtype=torch.int32, device=DEV)
        bb = torch.zeros(cap, cfg.hidden_dim, dtype=cfg.out_dtype, device=DEV)
        bm = torch.full((cap, 5), -9, dtype=torch.int32, device=DEV)
        _lib.call("moe_a2a_combine_send", C.byref(a.shape), p(ey), p(em0), p(num0), R, cap, p(bb), p(bm), p(bc),
                  plan_arg, st)
        outs.append((bc, bb, bm))
    torch.cuda.synchronize()
    for x, y in zip(outs[0], outs[1]):
        assert torch.equal(x, y)
    want = run_oracle(world)[1]
    assert np.array_equal(outs[1][0].cpu().numpy(), want.back_counts)
    assert np.array_equal(outs[1][2].cpu().numpy()[:R], want.back_meta)
    assert np.array_equal(bits(outs[1][1][:R]), want.back_buf)
    return where.value, 2 * E, plan1


def test_static_plan_entry_point_matches_dispatch_recv_twice_in_a_row():
    print("no-alloc entry point: big job", flush=True)
    addr_big, n_big, plan_big = one_job(BIG, 41)
    print("no-alloc entry point: smaller job on the same buffer", flush=True)
    addr_small, n_small, plan_small = one_job(SMALL, 42)
    assert addr_small == addr_big  # one buffer per GPU
    assert n_small < n_big
    # the smaller call rewrote its own ints and left the rest of the buffer as the first call wrote it
    after = device_ints(addr_big, n_big)
    assert np.array_equal(after[:n_small], plan_small)
    assert np.array_equal(after[n_small:], plan_big[n_small:])


def test_shapes_beyond_the_static_buffer_are_refused():
    lib = _lib.load()
    one = C.c_void_p(256)  # never dereferenced
    where = C.c_void_p(1)
    big = _lib.Shape(2, 0, 2 * 65, 2, 64, 4)
    assert lib.moe_a2a_dispatch_recv_static(C.byref(big), one, one, one, 0, 0, one, one, one, C.byref(where), None) == -4
    assert where.value is None
