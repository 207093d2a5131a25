"""The long-stream entry points (moe_a2a_dispatch_recv_long, moe_a2a_combine_recv_long): positions
from a planning launch instead of a scan in every workgroup. They must give what the one-launch
entry points give and what the oracle says, bit for bit, at every size; `long_stream_rows=0`
sends every receive half through them, however short its stream."""
import numpy as np
import pytest
import torch

from amd_distributed_2025_amd import LocalWorld, WORKLOADS, generate_world
from amd_distributed_2025_amd.all2all import LONG_STREAM_ROWS
from tests.helpers import bits, run_oracle
from tests.test_gpu_parity import DEV, EDGE, assert_rank_matches, to_dev

pytestmark = pytest.mark.gpu


def run_long(world, long_stream_rows=0, exact_hints=True, accumulate=False, reuse_placement=True,
             binding="ctypes", lw=None):
    cfg = world[0][0]
    if lw is None:
        lw = LocalWorld(cfg, len(world), device=DEV, exact_hints=exact_hints, reuse_placement=reuse_placement,
                        binding=binding, long_stream_rows=long_stream_rows)
    ys = lw.run([d for _, d, _, _ in to_dev(world)], accumulate=accumulate)
    torch.cuda.synchronize()
    tr = run_oracle(world)
    for r in range(len(world)):
        T = world[r][1].num_tokens
        assert_rank_matches(lw.trace[r], tr[r], T, cfg.experts_per_token, f"rank {r}")
        assert np.array_equal(bits(ys[r]), tr[r].y)
    return lw


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_workloads_through_the_long_stream_entry_points(name):
    print(f"long-stream workload {name}", flush=True)
    run_long(generate_world(WORKLOADS[name], 2025))


@pytest.mark.parametrize("name", sorted(EDGE))
def test_edge_shapes_through_the_long_stream_entry_points(name):
    print(f"long-stream edge {name}", flush=True)
    spec = dict(routing="uniform", weights="rand")
    spec.update(EDGE[name])
    run_long(generate_world(spec, 77))


def test_extension_binding_and_loose_hints():
    world = generate_world(WORKLOADS["C3"], 5)
    run_long(world, binding="ext")
    run_long(world, exact_hints=False, accumulate=True, reuse_placement=False)


def test_streams_above_the_threshold_take_them_by_default():
    """20480 rows sent and about as many received per rank, many planning tiles, skewed
    routing; nothing forced: the host class picks the long-stream entry points from the row
    count."""
    spec = dict(world_size=4, num_experts=64, experts_per_token=8, hidden_dim=264, max_num_tokens=2560,
                num_tokens="full", routing="zipf", weights="softmax", dtype="bf16")
    world = generate_world(spec, 4)
    assert spec["max_num_tokens"] * spec["experts_per_token"] > max(LONG_STREAM_ROWS.values())
    lw = run_long(world, long_stream_rows=None)
    assert any("row_position" in a._ws for a in lw.ranks)  # (skewed routing: not every rank receives that many)
    assert all("entry_row" in a._ws for a in lw.ranks)
    # and the one-launch entry points agree on the same job
    short = LocalWorld(world[0][0], 4, device=DEV, long_stream_rows=1 << 30)
    ys = short.run([d for _, d, _, _ in to_dev(world)])
    torch.cuda.synchronize()
    assert not any("row_position" in a._ws or "entry_row" in a._ws for a in short.ranks)
    for r in range(4):
        assert torch.equal(ys[r], lw.trace[r]["y"][: world[r][1].num_tokens])


def test_repeated_expert_ids_and_many_ranks():
    """Entries of a token that name the same expert keep their k order, also through the
    long-stream entry points; a job of 16 ranks."""
    spec = dict(world_size=16, num_experts=32, experts_per_token=6, hidden_dim=136, max_num_tokens=200,
                num_tokens="full", routing="uniform", weights="rand", dtype="bf16")
    world = generate_world(spec, 99)
    rng = np.random.default_rng(5)
    for _, d, r, _ in world:
        ids = rng.integers(0, 32, tuple(d.indices.shape)).astype(np.int32)
        ids[r] = 7
        ids[r + 4, :3] = 31
        d.indices = torch.from_numpy(ids)
    run_long(world)
    run_long(world, reuse_placement=False, exact_hints=False)


def test_tables_left_by_an_earlier_job_do_no_harm():
    """The (token, k) -> row table and the position table are never cleared. A second, smaller
    job on the same objects finds the first job's entries in them and must not use any."""
    spec = dict(world_size=4, num_experts=16, experts_per_token=4, hidden_dim=264, max_num_tokens=96,
                num_tokens="full", routing="uniform", weights="rand", dtype="fp16")
    lw = run_long(generate_world(spec, 1))
    small = dict(spec, num_tokens="uniform")
    for seed in (2, 3):
        run_long(generate_world(small, seed), lw=lw)


def test_random_small_jobs_through_the_long_stream_entry_points():
    rng = np.random.default_rng(777)
    for case in range(24):
        W = int(rng.choice([1, 2, 3, 4, 8, 16]))
        nle = int(rng.choice([1, 2, 5, 32, 65, 130, 300]))  # (300: beyond the planner's tables, scans instead)
        E = W * nle
        K = int(rng.integers(1, min(E, 9) + 1))
        H = int(rng.choice([8, 24, 100, 256, 520, 1032, 4104]))
        max_T = int(rng.integers(1, 300))
        spec = dict(world_size=W, num_experts=E, experts_per_token=K, hidden_dim=H, max_num_tokens=max_T,
                    num_tokens=str(rng.choice(["uniform", "full", "reference"])),
                    routing=str(rng.choice(["uniform", "zipf"])),
                    weights=str(rng.choice(["rand", "softmax"])),
                    dtype=str(rng.choice(["bf16", "fp16"])))
        print(f"long-stream random job {case}: {spec}", flush=True)
        run_long(generate_world(spec, 500 + case), exact_hints=bool(case % 2))


def test_overflowing_expert_drops_the_same_rows():
    """Every entry routed to expert 0: positions reach past max_recv and those rows are not
    stored, exactly as with the scanning movers."""
    spec = dict(world_size=2, num_experts=4, experts_per_token=4, hidden_dim=64, max_num_tokens=6,
                num_tokens="full", routing="uniform", weights="rand", dtype="bf16")
    world = generate_world(spec, 11)
    cfg = world[0][0]
    outs = []
    for long_rows in (0, 1 << 30):
        lw = LocalWorld(cfg, len(world), device=DEV, long_stream_rows=long_rows)
        data = [d.to(DEV) for _, d, _, _ in world]
        for d in data:
            d.indices = torch.zeros_like(d.indices)
        ys = lw.run(data)
        torch.cuda.synchronize()
        tr = lw.trace[0]
        assert int(tr["expert_num_tokens"][0]) > lw.ranks[0].max_recv
        n = int(tr["back_counts"].sum())
        outs.append([tr["expert_num_tokens"].cpu().numpy(), tr["back_counts"].cpu().numpy(),
                     tr["back_meta"][:n].cpu().numpy(), bits(tr["back_buf"][:n])] + [bits(y) for y in ys])
    for a, b in zip(*outs):
        assert np.array_equal(a, b)


def test_graph_replays_of_the_long_stream_step():
    world = generate_world(WORKLOADS["C3"], 12)
    cfg = world[0][0]
    dev = [d.to(DEV) for _, d, _, _ in world]
    lw = LocalWorld(cfg, 8, device=DEV, long_stream_rows=0)
    eager = [y.clone() for y in lw.run(dev)]
    a, d0, g = lw.ranks[0], dev[0], lw.trace[0]
    R = int(g["recv_counts"].sum().item())
    y = a._buf("y", (cfg.max_num_tokens, cfg.hidden_dim), cfg.out_dtype)

    def step():
        a.dispatch_send(d0.x, d0.indices)
        a.dispatch_recv(g["recv_counts"], g["recv_buf"], g["recv_meta"], R)
        a.expert_scale(g["expert_x"], g["expert_num_tokens"], R)
        a.combine_send(g["expert_meta"], g["expert_y"], g["expert_num_tokens"], R)
        a.combine_recv(y, d0.weights, g["ret_counts"], g["ret_buf"], g["ret_meta"], accumulate=False)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for i in range(3):
        y.fill_(float(i))
        a._ws["entry_row"].fill_(i)      # whatever the tables hold before a replay
        a._ws["row_position"].fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y[: d0.num_tokens], eager[0]), f"replay {i}"


def test_counts_beyond_capacity_are_cut_off_by_the_long_stream_entry_points():
    """Device-side counts that claim more rows than the caller says its buffers hold, through the
    C ABI: the planner, the table builder and the movers stop at the stated capacity, whatever the
    hint. Tensors are allocated with 64 rows and pre-filled with a sentinel; the calls are told 24."""
    import ctypes as C
    from amd_distributed_2025_amd import HIPAllToAll, _lib
    from amd_distributed_2025_amd.task import MoEConfig
    from oracle import moe_a2a_oracle as orc
    from tests.test_gpu_parity import valid_rows

    W, nle, K, H, max_T = 4, 2, 2, 72, 32
    cfg = MoEConfig(W * nle, K, H, max_T, in_dtype=torch.bfloat16, out_dtype=torch.bfloat16)
    a = HIPAllToAll(cfg, 0, W, device=DEV)
    max_recv = max_T * W
    rng = np.random.default_rng(78)
    ALLOC, CAP, SENT = 64, 24, -12345
    p = lambda t: C.c_void_p(t.data_ptr())
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    shape = C.byref(a.shape)
    meta_np = np.zeros((ALLOC, 5), np.int32)
    meta_np[:, 0] = rng.integers(0, nle, ALLOC)
    meta_np[:, 1] = np.minimum(np.arange(ALLOC) // 10, W - 1)
    pairs = rng.permutation(max_T * K)[:ALLOC]          # every (token, k) at most once
    meta_np[:, 2], meta_np[:, 3] = pairs // K, pairs % K
    recv_buf = torch.from_numpy(rng.integers(0, 0x4400, (ALLOC, H), dtype=np.int16)).view(torch.bfloat16).to(DEV)
    recv_meta = torch.from_numpy(meta_np).to(DEV)
    counts40 = torch.tensor([10, 10, 10, 10], dtype=torch.int32, device=DEV)

    num = torch.full((nle,), SENT, dtype=torch.int32, device=DEV)
    ex = torch.zeros(nle, max_recv, H, dtype=torch.bfloat16, device=DEV)
    em = torch.full((nle, max_recv, 5), SENT, dtype=torch.int32, device=DEV)
    pos = torch.full((ALLOC,), SENT, dtype=torch.int32, device=DEV)
    for hint in (0, 7, CAP, 40, 1000):
        num.fill_(SENT); em.fill_(SENT); pos.fill_(SENT)
        _lib.call("moe_a2a_dispatch_recv_long", shape, p(recv_buf), p(recv_meta), p(counts40), hint, CAP,
                  p(num), p(ex), p(em), None, p(pos), st)
        torch.cuda.synchronize()
        cnt, local, where, order = orc.expert_placement(meta_np[:CAP], nle)
        assert np.array_equal(num.cpu().numpy(), cnt), hint
        assert np.array_equal(valid_rows(em, cnt).numpy(), meta_np[:CAP][order]), hint
        assert np.array_equal(bits(valid_rows(ex, cnt)), bits(recv_buf[:CAP])[order]), hint
        assert bool((pos[CAP:] == SENT).all()), hint          # the planner wrote no position past the capacity
        for le in range(nle):
            assert bool((em[le, int(cnt[le]):] == SENT).all()), hint

    weights = torch.from_numpy(rng.random((max_T, K), dtype=np.float32)).to(DEV)
    y = torch.zeros(max_T, H, dtype=torch.bfloat16, device=DEV)
    table = torch.full((max_T * K,), 63, dtype=torch.int32, device=DEV)  # stale entries that name a row past the capacity
    for hint in (0, CAP, 40, 1000):
        _lib.call("moe_a2a_combine_recv_long", shape, p(recv_buf), p(recv_meta), p(counts40), hint, CAP,
                  p(weights), max_T, p(y), 0, _lib.BF16, p(table), st)
        torch.cuda.synchronize()
        want = orc.combine_recv(bits(recv_buf[:CAP]), meta_np[:CAP], weights.cpu().numpy(), max_T, "bf16")
        assert np.array_equal(bits(y), want), hint
    # null workspaces are refused before anything is launched
    lib = _lib.load()
    assert lib.moe_a2a_dispatch_recv_long(shape, p(recv_buf), p(recv_meta), p(counts40), CAP, CAP, p(num), p(ex), p(em),
                                          None, None, st) == -1
    assert lib.moe_a2a_combine_recv_long(shape, p(recv_buf), p(recv_meta), p(counts40), CAP, CAP, p(weights), max_T,
                                         p(y), 0, _lib.BF16, None, st) == -1


def test_a_pair_that_arrives_twice_is_added_twice_only_when_the_caller_says_pairs_may_repeat():
    """The reference adds every arriving row (all2all/reference.py:227-232). A stream out of a
    dispatch has every (src_token, src_k) pair once; a caller-made stream in which one repeats is
    served by the scan (`unique_pairs=False`), which adds both rows whatever the length. The table of
    the long-stream entry point holds one row per pair: by default, above its threshold, exactly one
    of the two rows is added."""
    from amd_distributed_2025_amd import HIPAllToAll
    from amd_distributed_2025_amd.task import MoEConfig
    from oracle import moe_a2a_oracle as orc

    T, K, H, W = 640, 8, 64, 1
    cfg = MoEConfig(8, K, H, T, torch.bfloat16, torch.bfloat16)
    a = HIPAllToAll(cfg, 0, W, device=DEV)
    rng = np.random.default_rng(5)
    S = T * K
    assert S > LONG_STREAM_ROWS["combine"]
    order = rng.permutation(S)
    meta = np.zeros((S + 1, 5), np.int32)
    meta[:S, 2], meta[:S, 3] = order // K, order % K
    dup = 1234
    meta[S] = meta[dup]                              # the pair of row `dup` arrives again at the end
    rows = torch.from_numpy(rng.standard_normal((S + 1, H)).astype(np.float32)).to(torch.bfloat16)
    weights = torch.from_numpy(rng.random((T, K), dtype=np.float32))
    counts = torch.tensor([S + 1], dtype=torch.int32, device=DEV)
    y = torch.empty(T, H, dtype=torch.bfloat16, device=DEV)
    args = (weights.to(DEV), counts, rows.to(DEV), torch.from_numpy(meta).to(DEV))
    both = orc.combine_recv(bits(rows), meta, weights.numpy(), T, "bf16")
    a.combine_recv(y, *args, accumulate=False, unique_pairs=False)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), both)
    a.combine_recv(y, *args, accumulate=False)       # by default: the table, one row per pair
    torch.cuda.synchronize()
    keep_first, keep_last = np.ones(S + 1, bool), np.ones(S + 1, bool)
    keep_first[S], keep_last[dup] = False, False
    one_of = [orc.combine_recv(bits(rows)[k], meta[k], weights.numpy(), T, "bf16") for k in (keep_first, keep_last)]
    assert any(np.array_equal(bits(y), w) for w in one_of)
    assert not np.array_equal(bits(y), both)


@pytest.mark.parametrize("hidden_dim,tokens", [(2304, 640), (4608, 520), (7168, 513), (1024, 800)])
def test_stage_one_above_4096_entries_with_long_rows(hidden_dim, tokens):
    """Above 4096 entries per rank stage 1 ranks all of a token's entries in one pass over the keys
    (two at a time below): rows of more than 256, more than 512 and of at most 256 vectors take the
    three shapes of that kernel. Every buffer and `y` against the oracle, both kinds of receive half."""
    print(f"stage 1, {tokens * 8} entries of {hidden_dim} elements", flush=True)
    spec = dict(world_size=2, num_experts=16, experts_per_token=8, hidden_dim=hidden_dim,
                max_num_tokens=tokens, num_tokens="full", routing="uniform", weights="softmax", dtype="bf16")
    assert tokens * 8 > 4096
    world = generate_world(spec, 31)
    run_long(world, long_stream_rows=None)
    run_long(world, long_stream_rows=0)
