"""Parity of the HIP path with the CPU oracle, through the C ABI, on a real GPU.

Integer outputs (counts, meta rows, slots) and row buffers must match bit for
bit; the combined result `y` is compared bit for bit too, because the kernel
reproduces the reference's per-addend rounding (the documented tolerance of the
task, rtol 1e-2 / atol 5e-3 from all2all/reference.py:279, is therefore met
with zero error)."""
from pathlib import Path

import numpy as np
import pytest
import torch

from amd_distributed_2025_amd import LocalWorld, WORKLOADS, generate_world
from amd_distributed_2025_amd.task import (DTYPES, MoEConfig, RankTestData, TASK_YML_TESTS,
                                           dtype_name)
from oracle import moe_a2a_oracle as orc
from tests.helpers import bits, from_bits, oracle_inputs, run_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLDEN = Path(__file__).resolve().parent / "golden"


def to_dev(world):
    return [(c, d.to(DEV), r, w) for (c, d, r, w) in world]


def valid_rows(padded: torch.Tensor, counts: np.ndarray) -> np.ndarray:
    parts = [padded[le, : int(counts[le])] for le in range(padded.shape[0])]
    return torch.cat(parts, dim=0).cpu()


def assert_rank_matches(tr_gpu: dict, t: orc.RankTrace, T: int, K: int, tag: str):
    S = T * K
    R = int(t.recv_counts.sum())
    eq = np.array_equal
    assert eq(tr_gpu["send_counts"].cpu().numpy(), t.send_counts), tag
    assert eq(tr_gpu["send_meta"].cpu().numpy()[:S], t.send_meta), tag
    assert eq(bits(tr_gpu["send_buf"][:S]), t.send_buf), tag
    inv = np.empty(S, np.int64); inv[t.send_order] = np.arange(S)
    assert eq(tr_gpu["send_slot"].cpu().numpy()[:S], inv), tag
    assert eq(tr_gpu["recv_counts"].cpu().numpy(), t.recv_counts), tag
    assert eq(tr_gpu["recv_meta"].cpu().numpy()[:R], t.recv_meta), tag
    assert eq(bits(tr_gpu["recv_buf"][:R]), t.recv_buf), tag
    cnt = tr_gpu["expert_num_tokens"].cpu().numpy()
    assert eq(cnt, t.expert_num_tokens), tag
    assert eq(bits(valid_rows(tr_gpu["expert_x"], cnt)), t.expert_rows), tag
    assert eq(valid_rows(tr_gpu["expert_meta"], cnt).numpy(), t.expert_meta_rows), tag
    assert eq(bits(valid_rows(tr_gpu["expert_y"], cnt)), t.expert_y_rows), tag
    assert eq(tr_gpu["back_counts"].cpu().numpy(), t.back_counts), tag
    assert eq(tr_gpu["back_meta"].cpu().numpy()[:R], t.back_meta), tag
    assert eq(bits(tr_gpu["back_buf"][:R]), t.back_buf), tag
    assert eq(tr_gpu["ret_counts"].cpu().numpy(), t.ret_counts), tag
    assert eq(tr_gpu["ret_meta"].cpu().numpy()[:S], t.ret_meta), tag
    assert eq(bits(tr_gpu["ret_buf"][:S]), t.ret_buf), tag
    assert eq(bits(tr_gpu["y"][:T]), t.y), tag


def run_and_compare(world, exact_hints=True, accumulate=False, reuse_placement=True):
    cfg = world[0][0]
    lw = LocalWorld(cfg, len(world), device=DEV, exact_hints=exact_hints, reuse_placement=reuse_placement)
    dev = to_dev(world)
    ys = lw.run([d for _, d, _, _ in dev], accumulate=accumulate)
    torch.cuda.synchronize()
    tr = run_oracle(world)
    for r in range(len(world)):
        T = world[r][1].num_tokens
        assert_rank_matches(lw.trace[r], tr[r], T, cfg.experts_per_token, f"rank {r}")
        assert np.array_equal(bits(ys[r]), tr[r].y)
    return lw, tr


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_workloads_match_oracle(name):
    print(f"workload {name}", flush=True)
    run_and_compare(generate_world(WORKLOADS[name], 2025))


@pytest.mark.parametrize("case", sorted(p.stem for p in GOLDEN.glob("*.npz")))
def test_golden_fixtures(case):
    """Inputs and expected outputs both come from the committed fixture."""
    print(f"golden {case}", flush=True)
    z = np.load(GOLDEN / f"{case}.npz")
    W, dt = int(z["world_size"]), DTYPES[str(z["dtype"])]
    cfg = MoEConfig(int(z["num_experts"]), int(z["experts_per_token"]), int(z["hidden_dim"]),
                    int(z["max_num_tokens"]), dt, dt)
    data = []
    for r in range(W):
        d = object.__new__(RankTestData)
        d.indices = torch.from_numpy(z[f"r{r}_indices"]).to(DEV)
        d.weights = torch.from_numpy(z[f"r{r}_weights"]).to(DEV)
        d.x = from_bits(z[f"r{r}_x"], dt).to(DEV)
        d.num_tokens, d.rank = d.indices.shape[0], r
        data.append(d)
    lw = LocalWorld(cfg, W, device=DEV)
    ys = lw.run(data)
    torch.cuda.synchronize()
    for r in range(W):
        g, p = lw.trace[r], f"r{r}_"
        S = data[r].num_tokens * cfg.experts_per_token
        R = int(z[p + "recv_counts"].sum())
        for name in ("send_counts", "recv_counts", "back_counts", "ret_counts"):
            assert np.array_equal(g[name].cpu().numpy(), z[p + name]), (r, name)
        assert np.array_equal(g["send_meta"].cpu().numpy()[:S], z[p + "send_meta"])
        assert np.array_equal(g["recv_meta"].cpu().numpy()[:R], z[p + "recv_meta"])
        assert np.array_equal(g["back_meta"].cpu().numpy()[:R], z[p + "back_meta"])
        assert np.array_equal(g["ret_meta"].cpu().numpy()[:S], z[p + "ret_meta"])
        cnt = g["expert_num_tokens"].cpu().numpy()
        assert np.array_equal(cnt, z[p + "expert_num_tokens"])
        assert np.array_equal(valid_rows(g["expert_meta"], cnt).numpy(), z[p + "expert_meta_rows"])
        assert np.array_equal(bits(ys[r]), z[p + "y"])


@pytest.mark.parametrize("i", range(len(TASK_YML_TESTS)))
def test_reference_test_shapes_fp16(i):
    """The nine shapes of all2all/task.yml:48-57 with the reference's input rules
    (fp16, uniform weights, num_tokens ~ randint(1, max))."""
    spec = dict(TASK_YML_TESTS[i])
    seed = spec.pop("seed")
    print(f"task.yml test {i} {spec}", flush=True)
    run_and_compare(generate_world(spec, seed))


EDGE = {
    "odd_hidden_2byte_path": dict(world_size=4, num_experts=8, experts_per_token=2, hidden_dim=100,
                                  max_num_tokens=9, num_tokens="uniform", dtype="bf16"),
    "hidden_dim_odd": dict(world_size=2, num_experts=4, experts_per_token=2, hidden_dim=37,
                           max_num_tokens=5, num_tokens="full", dtype="fp16"),
    "hidden_dim_one": dict(world_size=2, num_experts=6, experts_per_token=3, hidden_dim=1,
                           max_num_tokens=7, num_tokens="full", dtype="bf16"),
    "hidden_16B_not_vec_multiple": dict(world_size=2, num_experts=4, experts_per_token=2, hidden_dim=2056,
                                        max_num_tokens=5, num_tokens="full", dtype="fp16"),
    "single_token_single_k": dict(world_size=8, num_experts=8, experts_per_token=1, hidden_dim=64,
                                  max_num_tokens=1, num_tokens="full", dtype="bf16"),
    "one_rank_all_experts_local": dict(world_size=1, num_experts=256, experts_per_token=8, hidden_dim=512,
                                       max_num_tokens=64, num_tokens="full", dtype="bf16"),
    "k_equals_e": dict(world_size=2, num_experts=4, experts_per_token=4, hidden_dim=32,
                       max_num_tokens=7, num_tokens="full", dtype="fp16"),
    "wide_rows_two_chunks": dict(world_size=2, num_experts=4, experts_per_token=2, hidden_dim=16384,
                                 max_num_tokens=6, num_tokens="full", dtype="bf16"),
    "many_entries_several_key_batches": dict(world_size=2, num_experts=16, experts_per_token=10, hidden_dim=64,
                                             max_num_tokens=300, num_tokens="full", dtype="bf16"),
    "two_entries_per_token_several_key_batches": dict(world_size=2, num_experts=4, experts_per_token=2,
                                                      hidden_dim=32, max_num_tokens=2300, num_tokens="full",
                                                      dtype="fp16"),
    "many_tokens_sixteen_key_batches": dict(world_size=4, num_experts=32, experts_per_token=8, hidden_dim=264,
                                            max_num_tokens=2048, num_tokens="uniform", routing="zipf",
                                            dtype="bf16"),
    "wide_fanout_several_key_batches": dict(world_size=2, num_experts=8, experts_per_token=8, hidden_dim=2056,
                                            max_num_tokens=300, num_tokens="full", dtype="bf16"),
    "wide_fanout_two_byte_rows": dict(world_size=2, num_experts=4, experts_per_token=4, hidden_dim=1001,
                                      max_num_tokens=6, num_tokens="full", dtype="fp16"),
    "wide_fanout_twelve_entries": dict(world_size=2, num_experts=24, experts_per_token=12, hidden_dim=4104,
                                       max_num_tokens=9, num_tokens="uniform", dtype="bf16"),
    "wide_fanout_two_vectors_per_lane_two_chunks": dict(world_size=2, num_experts=8, experts_per_token=4,
                                                        hidden_dim=8200, max_num_tokens=7, num_tokens="full",
                                                        dtype="bf16"),
    "wide_fanout_odd_local_experts": dict(world_size=4, num_experts=12, experts_per_token=5, hidden_dim=7168,
                                          max_num_tokens=11, num_tokens="uniform", dtype="fp16"),
    "k_above_fast_list": dict(world_size=2, num_experts=160, experts_per_token=72, hidden_dim=64,
                              max_num_tokens=3, num_tokens="full", dtype="bf16"),
    "k_above_the_weights_kept_in_lds": dict(world_size=2, num_experts=320, experts_per_token=136, hidden_dim=40,
                                            max_num_tokens=2, num_tokens="full", dtype="fp16"),
    "three_entries_per_token_wave_per_entry": dict(world_size=4, num_experts=12, experts_per_token=3,
                                                   hidden_dim=7168, max_num_tokens=40, num_tokens="uniform",
                                                   dtype="bf16"),
    # more ranks than a wave has lanes: the per-rank vectors no longer fit one register per lane
    "sixty_five_ranks": dict(world_size=65, num_experts=130, experts_per_token=5, hidden_dim=72,
                             max_num_tokens=9, num_tokens="uniform", routing="zipf", dtype="bf16"),
    "one_hundred_and_thirty_ranks": dict(world_size=130, num_experts=130, experts_per_token=4, hidden_dim=100,
                                         max_num_tokens=7, num_tokens="full", dtype="fp16"),
}


@pytest.mark.parametrize("name", sorted(EDGE))
def test_edge_shapes(name):
    print(f"edge {name}", flush=True)
    spec = dict(routing="uniform", weights="rand")
    spec.update(EDGE[name])
    run_and_compare(generate_world(spec, 77))


def test_loose_hints_and_in_place_accumulate_give_the_same_bits():
    world = generate_world(WORKLOADS["C3"], 31)
    run_and_compare(world, exact_hints=False, accumulate=True)


def test_accumulate_adds_onto_existing_rows():
    wl = dict(world_size=1, num_experts=8, experts_per_token=2, hidden_dim=256, max_num_tokens=16,
              num_tokens="full", routing="uniform", weights="softmax", dtype="bf16")
    world = generate_world(wl, 5)
    cfg, d = world[0][0], world[0][1].to(DEV)
    lw = LocalWorld(cfg, 1, device=DEV)
    lw.run([d])
    g = lw.trace[0]
    init = torch.randn(16, 256, device=DEV).to(torch.bfloat16)
    y = init.clone()
    lw.ranks[0].combine_recv(y, d.weights, g["ret_counts"], g["ret_buf"], g["ret_meta"], accumulate=True)
    tr = run_oracle(world)[0]
    want = orc.combine_recv(tr.ret_buf, tr.ret_meta, world[0][1].weights.numpy(), 16, "bf16", y_init=bits(init))
    assert np.array_equal(bits(y), want)


def test_unaligned_rows_take_the_element_path():
    """Row buffers that are only 2-byte aligned must still give the same bits."""
    wl = dict(world_size=1, num_experts=4, experts_per_token=2, hidden_dim=64, max_num_tokens=8,
              num_tokens="full", routing="uniform", weights="rand", dtype="fp16")
    world = generate_world(wl, 8)
    cfg, d = world[0][0], world[0][1].to(DEV)
    lw = LocalWorld(cfg, 1, device=DEV)
    a = lw.ranks[0]
    flat = torch.empty(8 * 64 + 1, dtype=torch.float16, device=DEV)
    x_off = flat[1:].view(8, 64)
    x_off.copy_(d.x)
    assert x_off.data_ptr() % 16 != 0
    counts, buf, meta = a.dispatch_send(x_off, d.indices)
    torch.cuda.synchronize()
    tr = run_oracle(world)[0]
    assert np.array_equal(bits(buf), tr.send_buf)
    assert np.array_equal(meta.cpu().numpy(), tr.send_meta)


def test_results_do_not_depend_on_scheduling():
    world = generate_world(WORKLOADS["C5"], 99)
    cfg = world[0][0]
    dev = [d.to(DEV) for _, d, _, _ in world]
    lw = LocalWorld(cfg, 8, device=DEV)
    first = [y.clone() for y in lw.run(dev)]
    meta1 = [lw.trace[r]["expert_meta"].clone() for r in range(8)]
    for _ in range(3):
        again = lw.run(dev)
        for r in range(8):
            assert torch.equal(first[r], again[r])
            cnt = lw.trace[r]["expert_num_tokens"].cpu().numpy()
            assert torch.equal(valid_rows(lw.trace[r]["expert_meta"], cnt), valid_rows(meta1[r], cnt))


def test_full_size_properties_without_oracle():
    """C4 at full size through checks that need no oracle: every dispatched row
    lands exactly once, unchanged, on the expert its id names; with unit weights
    and K identical copies the result is the sum of owner scales times x."""
    world = generate_world(WORKLOADS["C4"], 4242)
    cfg = world[0][0]
    W, K, H = 8, cfg.experts_per_token, cfg.hidden_dim
    nle = cfg.num_experts // W
    dev = [d.to(DEV) for _, d, _, _ in world]
    lw = LocalWorld(cfg, W, device=DEV)
    lw.run(dev)
    total = 0
    for r in range(W):
        g = lw.trace[r]
        cnt = g["expert_num_tokens"].cpu().numpy()
        total += int(cnt.sum())
        for le in range(nle):
            n = int(cnt[le])
            m = g["expert_meta"][le, :n]
            assert bool((m[:, 0] == r * nle + le).all())
            # rows are in (src_rank, token) order inside an expert
            key = m[:, 1].long() * cfg.max_num_tokens + m[:, 2].long()
            assert bool((key[1:] > key[:-1]).all())
            # payload equals the source token row, and the id matches the source's indices
            for s in range(W):
                sel = m[:, 1] == s
                if bool(sel.any()):
                    tok, kk = m[sel, 2].long(), m[sel, 3].long()
                    assert torch.equal(g["expert_x"][le, :n][sel], dev[s].x[tok])
                    assert bool((dev[s].indices[tok, kk] == r * nle + le).all())
    assert total == sum(d.num_tokens for d in dev) * K


@pytest.mark.parametrize("name", ["bf16", "fp16"])
def test_rounding_of_every_bit_pattern_through_combine_and_expert(name):
    """All 65536 input bit patterns (infinities, NaNs, subnormals, ties included)
    as addends, with weights that force roundings: the kernel's hardware
    conversions must agree with the oracle's explicit round-to-nearest-even.
    NaN results must be NaN; bf16 NaNs must be torch's canonical 0x7fc0."""
    dt = DTYPES[name]
    H, T, K = 2048, 32, 2
    allbits = np.arange(65536, dtype=np.uint32).astype(np.uint16).reshape(T, H)
    rng = np.random.default_rng(3)
    second = orc.f32_to_b16(rng.standard_normal((T, H)).astype(np.float32) * 3, name)
    cfg = MoEConfig(2, K, H, T, dt, dt)
    a = LocalWorld(cfg, 1, device=DEV).ranks[0]
    ret_buf = torch.cat([from_bits(allbits, dt), from_bits(second, dt)]).to(DEV)
    meta = np.zeros((2 * T, 5), np.int32)
    meta[:T, 2] = np.arange(T); meta[T:, 2] = np.arange(T); meta[T:, 3] = 1
    w = (1 + rng.random((T, K), dtype=np.float32) * 2.0 ** -6).astype(np.float32)
    w[::4, 0] = 1.0
    counts = torch.tensor([2 * T], dtype=torch.int32, device=DEV)
    y = torch.empty(T, H, dtype=dt, device=DEV)
    a.combine_recv(y, torch.from_numpy(w).to(DEV), counts, ret_buf, torch.from_numpy(meta).to(DEV),
                   accumulate=False)
    torch.cuda.synchronize()
    want = orc.combine_recv(np.concatenate([allbits, second]), meta, w, T, name)
    got = bits(y)
    nan = np.isnan(orc.b16_to_f32(want, name))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(orc.b16_to_f32(got[nan], name)).all()
    if name == "bf16":
        assert (got[nan] == 0x7FC0).all()
    # the simulated expert on the same patterns, rank 2 of 3 (scale 3)
    cfg3 = MoEConfig(3, 1, H, T, dt, dt)
    b = LocalWorld(cfg3, 3, device=DEV).ranks[2]
    ex = torch.zeros(1, 3 * T, H, dtype=dt, device=DEV)
    ex[0, :T] = from_bits(allbits, dt).to(DEV)
    ey = b.expert_scale(ex, torch.tensor([T], dtype=torch.int32, device=DEV), T)
    torch.cuda.synchronize()
    want = orc.expert_scale(allbits, 2, name, name)
    got = bits(ey[0, :T])
    nan = np.isnan(orc.b16_to_f32(want, name))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(orc.b16_to_f32(got[nan], name)).all()


def every_pattern(H):
    """All 65536 bit patterns laid into rows of H elements (the last row wraps around)."""
    rows = -(-65536 // H)
    return (np.arange(rows * H, dtype=np.uint32) % 65536).astype(np.uint16).reshape(rows, H)


@pytest.mark.parametrize("name_in,name_out", [("bf16", "bf16"), ("fp16", "fp16"), ("fp16", "bf16"), ("bf16", "fp16")])
@pytest.mark.parametrize("H,nle", [(100, 1), (2048, 65), (520, 3)])
def test_expert_standin_on_every_bit_pattern_through_every_kernel(name_in, name_out, H, nle):
    """The simulated expert has three kernels: rows that are not a multiple of 16 bytes move element by
    element (H = 100), more than 64 local experts take a workgroup per row (nle = 65), the rest a wave
    per row. Every bit pattern, negative zero among them, times 1 (rank 0) and times 3, in every
    pairing of the two types, against the oracle."""
    print(f"expert stand-in, all patterns: {name_in}->{name_out} H={H} nle={nle}", flush=True)
    pats = every_pattern(H)
    rows = pats.shape[0]
    for rank, W in ((0, 1), (2, 3)):
        cfg = MoEConfig(W * nle, 1, H, rows, DTYPES[name_in], DTYPES[name_out])
        a = LocalWorld(cfg, W, device=DEV).ranks[rank]
        ex = torch.zeros(nle, rows * W, H, dtype=DTYPES[name_in], device=DEV)
        ex[nle - 1, :rows] = from_bits(pats, DTYPES[name_in]).to(DEV)
        counts = torch.zeros(nle, dtype=torch.int32, device=DEV)
        counts[nle - 1] = rows
        ey = a.expert_scale(ex, counts, rows)
        torch.cuda.synchronize()
        want = orc.expert_scale(pats, rank, name_in, name_out)
        got = bits(ey[nle - 1, :rows])
        nan = np.isnan(orc.b16_to_f32(want, name_out))
        assert np.array_equal(got[~nan], want[~nan]), f"scale {1 + rank}"
        assert np.isnan(orc.b16_to_f32(got[nan], name_out)).all()
        zero_in = (pats & 0x7FFF) == 0
        assert np.array_equal(got[zero_in], pats[zero_in]), "a zero keeps its sign"


@pytest.mark.parametrize("name", ["bf16", "fp16"])
def test_combine_on_every_bit_pattern_on_rows_moved_element_by_element(name):
    """The weighted sum on rows that are not a multiple of 16 bytes (H = 100): every bit pattern as
    first addend, a random second one, weights that force roundings."""
    dt = DTYPES[name]
    H, K = 100, 2
    pats = every_pattern(H)
    T = pats.shape[0]
    rng = np.random.default_rng(4)
    second = orc.f32_to_b16(rng.standard_normal((T, H)).astype(np.float32) * 3, name)
    cfg = MoEConfig(2, K, H, T, dt, dt)
    a = LocalWorld(cfg, 1, device=DEV).ranks[0]
    ret_buf = torch.cat([from_bits(pats, dt), from_bits(second, dt)]).to(DEV)
    meta = np.zeros((2 * T, 5), np.int32)
    meta[:T, 2] = np.arange(T); meta[T:, 2] = np.arange(T); meta[T:, 3] = 1
    w = (1 + rng.random((T, K), dtype=np.float32) * 2.0 ** -6).astype(np.float32)
    w[::4, 0] = 1.0
    counts = torch.tensor([2 * T], dtype=torch.int32, device=DEV)
    y = torch.empty(T, H, dtype=dt, device=DEV)
    a.combine_recv(y, torch.from_numpy(w).to(DEV), counts, ret_buf, torch.from_numpy(meta).to(DEV),
                   accumulate=False)
    torch.cuda.synchronize()
    want = orc.combine_recv(np.concatenate([pats, second]), meta, w, T, name)
    got = bits(y)
    nan = np.isnan(orc.b16_to_f32(want, name))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(orc.b16_to_f32(got[nan], name)).all()
    if name == "bf16":
        assert (got[nan] == 0x7FC0).all()


def test_custom_kernel_drop_in():
    """`custom_kernel(data)` with the reference's tuple, checked the way the
    reference's check_implementation does (allclose rtol 1e-2, atol 5e-3,
    all2all/reference.py:279) and bit for bit."""
    from amd_distributed_2025_amd import custom_kernel, set_peer_inputs

    spec = dict(TASK_YML_TESTS[3])
    seed = spec.pop("seed")
    world = generate_world(spec, seed)
    tr = run_oracle(world)
    dev = to_dev(world)
    set_peer_inputs(dev)
    try:
        for rank in (0, 5):
            out = custom_kernel(dev[rank])
            cfg, d = dev[rank][0], dev[rank][1]
            assert out.shape == (d.num_tokens, cfg.hidden_dim) and out.dtype == cfg.out_dtype
            assert out.device == d.x.device
            want = from_bits(tr[rank].y, cfg.out_dtype).to(DEV)
            assert torch.allclose(out, want, rtol=1e-2, atol=5e-3)
            assert torch.equal(out, want)
    finally:
        set_peer_inputs(None)
    # world_size 1 needs no registration
    solo = generate_world(WORKLOADS["C1"], 3)
    out = custom_kernel(to_dev(solo)[0])
    assert np.array_equal(bits(out), run_oracle(solo)[0].y)


def test_graph_replays_match_eager():
    """One rank's step captured in a HIP graph: every replay, with eager work
    and synchronisations in between, gives the eager result."""
    world = generate_world(WORKLOADS["C3"], 12)
    cfg = world[0][0]
    dev = [d.to(DEV) for _, d, _, _ in world]
    lw = LocalWorld(cfg, 8, device=DEV)
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
    for i in range(4):
        y.fill_(float(i))                       # eager work between replays
        g["expert_x"][0, 0].zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y[: d0.num_tokens], eager[0]), f"replay {i}"


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_send_plan_counts_offsets_and_maps(name):
    """The explicit plan (per-rank and per-expert counts, offsets, dst and src maps)
    equals the oracle's stable order, and the fused dispatch_send uses the same slots."""
    print(f"plan {name}", flush=True)
    world = generate_world(WORKLOADS[name], 606)
    cfg = world[0][0]
    W = len(world)
    nle = cfg.num_experts // W
    lw = LocalWorld(cfg, W, device=DEV)
    for r in (0, W - 1):
        d = world[r][1].to(DEV)
        rc, ro, ec, dst, src = lw.ranks[r].plan_send(d.indices)
        _, _, _, slots = lw.ranks[r].dispatch_send(d.x, d.indices, want_slots=True)
        torch.cuda.synchronize()
        counts, order = orc.send_order(d.indices.cpu().numpy(), nle, W)
        S = order.size
        inv = np.empty(S, np.int64); inv[order] = np.arange(S)
        assert np.array_equal(rc.cpu().numpy(), counts)
        assert np.array_equal(ro.cpu().numpy(), np.concatenate([[0], np.cumsum(counts)]))
        assert np.array_equal(ec.cpu().numpy(), np.bincount(d.indices.cpu().numpy().ravel(), minlength=cfg.num_experts))
        assert np.array_equal(src.cpu().numpy(), order)
        assert np.array_equal(dst.cpu().numpy(), inv)
        assert np.array_equal(slots.cpu().numpy(), inv)


def test_send_plan_many_tiles_and_ragged_tail():
    """More entries than one 1024-entry tile, a tail that does not fill a wave, 64 ranks."""
    cfg = MoEConfig(128, 7, 16, 333, torch.bfloat16, torch.bfloat16)
    a = LocalWorld(cfg, 64, device=DEV).ranks[5]
    rng = np.random.default_rng(8)
    idx = np.stack([rng.permutation(128)[:7] for _ in range(333)]).astype(np.int32)
    rc, ro, ec, dst, src = a.plan_send(torch.from_numpy(idx).to(DEV))
    torch.cuda.synchronize()
    counts, order = orc.send_order(idx, 2, 64)
    assert np.array_equal(rc.cpu().numpy(), counts)
    assert np.array_equal(src.cpu().numpy(), order)
    assert np.array_equal(ro.cpu().numpy()[-1:], [333 * 7])


def test_random_small_jobs():
    """A seeded sweep over small job shapes (world sizes 1..16, few to many local
    experts, row lengths on and off the 16-byte path, fp16 and bf16, all routing
    and token-count rules): every intermediate of every rank against the oracle."""
    rng = np.random.default_rng(20251125)
    for case in range(40):
        W = int(rng.choice([1, 2, 3, 4, 8, 16]))
        nle = int(rng.choice([1, 2, 5, 32, 65, 130]))
        E = W * nle
        K = int(rng.integers(1, min(E, 9) + 1))
        H = int(rng.choice([8, 24, 100, 256, 520, 1032, 4104]))
        max_T = int(rng.integers(1, 40))
        spec = dict(world_size=W, num_experts=E, experts_per_token=K, hidden_dim=H, max_num_tokens=max_T,
                    num_tokens=str(rng.choice(["uniform", "full", "reference"])),
                    routing=str(rng.choice(["uniform", "zipf"])),
                    weights=str(rng.choice(["rand", "softmax"])),
                    dtype=str(rng.choice(["bf16", "fp16"])))
        print(f"random job {case}: {spec}", flush=True)
        run_and_compare(generate_world(spec, 9000 + case), exact_hints=bool(case % 2))


def test_counts_beyond_capacity_are_cut_off():
    """Device-side counts that claim more rows than the caller says its buffers hold: every
    kernel stops at the stated capacity. The tensors here are really allocated with 64 rows and
    pre-filled with a sentinel, the calls are told 24 (or 40), and nothing past that may be read
    into a result or written."""
    import ctypes as C
    from amd_distributed_2025_amd import HIPAllToAll, _lib

    W, nle, K, H, max_T = 4, 2, 2, 72, 8
    cfg = MoEConfig(W * nle, K, H, max_T, in_dtype=torch.bfloat16, out_dtype=torch.bfloat16)
    a = HIPAllToAll(cfg, 0, W, device=DEV)
    max_recv = max_T * W
    rng = np.random.default_rng(77)
    ALLOC, CAP, SENT = 64, 24, -12345
    p = lambda t: C.c_void_p(t.data_ptr())
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    shape = C.byref(a.shape)

    def rows(n):
        return torch.from_numpy(rng.integers(0, 0x4400, (n, H), dtype=np.int16)).view(torch.bfloat16).to(DEV)

    # ---- dispatch_recv: counts claim 40 rows, the buffers are said to hold 24
    meta_np = np.zeros((ALLOC, 5), np.int32)
    meta_np[:, 0] = rng.integers(0, nle, ALLOC)
    meta_np[:, 1] = np.minimum(np.arange(ALLOC) // 10, W - 1)  # the source of a row is the segment it arrives in
    meta_np[:, 2] = rng.integers(0, max_T, ALLOC)
    meta_np[:, 3] = rng.integers(0, K, ALLOC)
    recv_buf, recv_meta = rows(ALLOC), torch.from_numpy(meta_np).to(DEV)
    counts40 = torch.tensor([10, 10, 10, 10], dtype=torch.int32, device=DEV)
    num = torch.full((nle,), SENT, dtype=torch.int32, device=DEV)
    ex = torch.zeros(nle, max_recv, H, dtype=torch.bfloat16, device=DEV)
    em = torch.full((nle, max_recv, 5), SENT, dtype=torch.int32, device=DEV)
    for hint in (0, 7, CAP, 40, 1000):
        num.fill_(SENT); em.fill_(SENT)
        _lib.call("moe_a2a_dispatch_recv", shape, p(recv_buf), p(recv_meta), p(counts40), hint, CAP,
                  p(num), p(ex), p(em), None, st)
        torch.cuda.synchronize()
        cnt, local, pos, order = orc.expert_placement(meta_np[:CAP], nle)
        assert np.array_equal(num.cpu().numpy(), cnt), hint
        assert np.array_equal(valid_rows(em, cnt).numpy(), meta_np[:CAP][order]), hint
        assert np.array_equal(bits(valid_rows(ex, cnt)), bits(recv_buf[:CAP])[order]), hint
        for le in range(nle):
            assert bool((em[le, int(cnt[le]):] == SENT).all()), hint

    # ---- combine_send: the experts hold 40 rows, the send buffers are said to hold 24
    cnt40, _, _, order40 = orc.expert_placement(meta_np[:40], nle)
    ey = torch.zeros(nle, max_recv, H, dtype=torch.bfloat16, device=DEV)
    em.fill_(SENT)
    stream_meta = meta_np[:40][order40]
    stream_rows = rows(40)
    at = 0
    for le in range(nle):
        n = int(cnt40[le])
        ey[le, :n] = stream_rows[at:at + n]
        em[le, :n] = torch.from_numpy(stream_meta[at:at + n]).to(DEV)
        at += n
    num40 = torch.from_numpy(cnt40).to(DEV)
    back_buf = torch.zeros(ALLOC, H, dtype=torch.bfloat16, device=DEV)
    back_meta = torch.full((ALLOC, 5), SENT, dtype=torch.int32, device=DEV)
    back_counts = torch.full((W,), SENT, dtype=torch.int32, device=DEV)
    # the plan of these 40 rows, as stage 2 writes it next to the same placement
    plan = torch.full((2 * W * nle,), SENT, dtype=torch.int32, device=DEV)
    num_b, ex_b, em_b = torch.empty_like(num), torch.empty_like(ex), torch.empty_like(em)
    _lib.call("moe_a2a_dispatch_recv", shape, p(recv_buf), p(recv_meta), p(counts40), 40, 40,
              p(num_b), p(ex_b), p(em_b), p(plan), st)
    torch.cuda.synchronize()
    assert np.array_equal(num_b.cpu().numpy(), cnt40)
    assert np.array_equal(valid_rows(em_b, cnt40).numpy(), stream_meta)
    for hint, use_plan in ((0, None), (CAP, None), (40, None), (1000, None), (0, plan), (40, plan)):
        back_meta.fill_(SENT); back_buf.zero_()
        _lib.call("moe_a2a_combine_send", shape, p(ey), p(em), p(num40), hint, CAP, p(back_buf),
                  p(back_meta), p(back_counts), None if use_plan is None else p(use_plan), st)
        torch.cuda.synchronize()
        bc, bo = orc.return_order(stream_meta, W)
        assert np.array_equal(back_counts.cpu().numpy(), bc), hint   # counts are the true ones
        assert np.array_equal(back_meta.cpu().numpy()[:CAP], stream_meta[bo][:CAP]), hint
        assert np.array_equal(bits(back_buf[:CAP]), bits(stream_rows)[bo][:CAP]), hint
        assert bool((back_meta[CAP:] == SENT).all()) and not bool(back_buf[CAP:].any()), hint

    # ---- exchange leg: the source's segment for rank 1 starts at row 30 of a buffer said to hold 40
    send_counts = torch.tensor([30, 30, 0, 0], dtype=torch.int32, device=DEV)
    recv_counts = torch.tensor([30, 30, 0, 0], dtype=torch.int32, device=DEV)
    dst_buf = torch.zeros(ALLOC, H, dtype=torch.bfloat16, device=DEV)
    dst_meta = torch.full((ALLOC, 5), SENT, dtype=torch.int32, device=DEV)
    for send_cap, recv_cap, moved in ((40, ALLOC, 10), (ALLOC, 5, 5), (ALLOC, ALLOC, 30), (20, ALLOC, 0)):
        dst_buf.zero_(); dst_meta.fill_(SENT)
        # source rank 0 -> destination rank 1: reads rows [30, 60) of the source, writes rows [0, 30)
        _lib.call("moe_a2a_exchange_local", W, H, p(recv_buf), p(recv_meta), p(send_counts), 1,
                  p(dst_buf), p(dst_meta), p(recv_counts), 0, 30, send_cap, recv_cap, st)
        torch.cuda.synchronize()
        assert torch.equal(dst_buf[:moved], recv_buf[30:30 + moved]), (send_cap, recv_cap)
        assert torch.equal(dst_meta[:moved], recv_meta[30:30 + moved]), (send_cap, recv_cap)
        assert bool((dst_meta[moved:] == SENT).all()) and not bool(dst_buf[moved:].any()), (send_cap, recv_cap)

    # ---- combine_recv: counts claim 40 arrivals, the buffers are said to hold 24
    weights = torch.from_numpy(rng.random((max_T, K), dtype=np.float32)).to(DEV)
    y = torch.zeros(max_T, H, dtype=torch.bfloat16, device=DEV)
    for hint in (0, CAP, 40, 1000):
        _lib.call("moe_a2a_combine_recv", shape, p(recv_buf), p(recv_meta), p(counts40), hint, CAP,
                  p(weights), max_T, p(y), 0, _lib.BF16, st)
        torch.cuda.synchronize()
        want = orc.combine_recv(bits(recv_buf[:CAP]), meta_np[:CAP], weights.cpu().numpy(), max_T, "bf16")
        assert np.array_equal(bits(y), want), hint


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C5"])
def test_without_placement_plan(name):
    """Stage 3 ranking its rows by scanning the origin column, as it does for a caller that
    passes no plan."""
    run_and_compare(generate_world(WORKLOADS[name], 31), reuse_placement=False)


def test_plan_is_set_aside_when_an_expert_overflows():
    """Every entry of every rank routed to expert 0: more rows than max_recv arrive for it, the
    surplus is dropped by stage 2 and the plan no longer describes the buffers. Stage 3 must
    notice and rank by scanning: both settings give the same bits."""
    spec = dict(world_size=2, num_experts=4, experts_per_token=4, hidden_dim=64, max_num_tokens=6,
                num_tokens="full", routing="uniform", weights="rand", dtype="bf16")
    world = generate_world(spec, 11)
    cfg = world[0][0]
    outs = []
    for reuse in (True, False):
        lw = LocalWorld(cfg, len(world), device=DEV, reuse_placement=reuse)
        data = [d.to(DEV) for _, d, _, _ in world]
        for d in data:
            d.indices = torch.zeros_like(d.indices)
        ys = lw.run(data)
        torch.cuda.synchronize()
        tr = lw.trace[0]
        assert int(tr["expert_num_tokens"][0]) > lw.ranks[0].max_recv  # the overflow is reported
        n = int(tr["back_counts"].sum())
        outs.append([tr["back_counts"].cpu().numpy(), tr["back_meta"][:n].cpu().numpy(), bits(tr["back_buf"][:n])]
                    + [bits(y) for y in ys])
    for a, b in zip(*outs):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("inp,out", [("bf16", "fp16"), ("fp16", "bf16")])
def test_different_input_and_output_types(inp, out):
    """Tokens travel in `in_dtype`, the expert converts to `out_dtype` (all2all/reference.py:262),
    the combine runs in `out_dtype`."""
    spec = dict(world_size=4, num_experts=16, experts_per_token=3, hidden_dim=264, max_num_tokens=20,
                num_tokens="uniform", routing="uniform", weights="softmax", dtype=inp)
    world = generate_world(spec, 123)
    cfg = world[0][0]
    mixed = MoEConfig(cfg.num_experts, cfg.experts_per_token, cfg.hidden_dim, cfg.max_num_tokens,
                      in_dtype=DTYPES[inp], out_dtype=DTYPES[out])
    run_and_compare([(mixed, d, r, w) for (_, d, r, w) in world])


def test_repeated_expert_ids_inside_a_token():
    """The reference draws distinct ids per token, but its loops are defined for any ids
    (all2all/reference.py:76-86): entries of a token that name the same expert keep their k
    order everywhere. Ids drawn with replacement, a few tokens with all entries equal."""
    spec = dict(world_size=4, num_experts=32, experts_per_token=6, hidden_dim=136, max_num_tokens=24,
                num_tokens="full", routing="uniform", weights="rand", dtype="bf16")
    world = generate_world(spec, 99)
    rng = np.random.default_rng(5)
    for _, d, r, _ in world:
        ids = rng.integers(0, 32, tuple(d.indices.shape)).astype(np.int32)
        ids[r] = 7          # one token per rank sends every entry to the same expert
        ids[r + 4, :3] = 31
        d.indices = torch.from_numpy(ids)
    for plan in (True, False):
        run_and_compare(world, reuse_placement=plan)


@pytest.mark.parametrize("long_rows", [None, 0], ids=["one_launch", "long_stream"])
@pytest.mark.parametrize("K", [2, 6])
def test_expert_ids_outside_the_range_are_set_aside(K, long_rows):
    """Ids below 0 or at/above E name no destination. Their rows must land behind all
    destinations' rows without disturbing them, and the result must equal the oracle's on a job
    where those entries point at a real expert with weight 0 (an addend of +0 changes nothing)."""
    from amd_distributed_2025_amd import HIPAllToAll

    E, W = 16, 4
    spec = dict(world_size=W, num_experts=E, experts_per_token=K, hidden_dim=72, max_num_tokens=18,
                num_tokens="full", routing="uniform", weights="rand", dtype="bf16")
    world = generate_world(spec, 17)
    rng = np.random.default_rng(8)
    substitute = [(c, d.to("cpu"), r, w) for (c, d, r, w) in world]   # separate tensors
    for (_, d, r, _), (_, ds, _, _) in zip(world, substitute):
        ids = d.indices.numpy().copy()
        stray = rng.random(ids.shape) < 0.2
        stray[0, 0] = True
        bad = np.where(rng.random(ids.shape) < 0.5, -1 - rng.integers(0, 5, ids.shape), E + rng.integers(0, 5, ids.shape))
        d.indices = torch.from_numpy(np.where(stray, bad, ids).astype(np.int32))
        ds.indices = torch.from_numpy(ids.astype(np.int32))
        ds.weights = torch.from_numpy(np.where(stray, np.float32(0), d.weights.numpy()).astype(np.float32))
        ds.x = d.x
    want = run_oracle(substitute)
    cfg = world[0][0]
    lw = LocalWorld(cfg, W, device=DEV, long_stream_rows=long_rows)
    ys = lw.run([d.to(DEV) for _, d, _, _ in world])
    torch.cuda.synchronize()
    nle = E // W
    for r in range(W):
        assert np.array_equal(bits(ys[r]), want[r].y), r
        ids = world[r][1].indices.numpy().ravel()
        ok = (ids >= 0) & (ids < E)
        counts = lw.trace[r]["send_counts"].cpu().numpy()
        assert np.array_equal(counts, np.bincount(ids[ok] // nle, minlength=W)), r
        n = int(counts.sum())
        meta = lw.trace[r]["send_meta"].cpu().numpy()
        sent = meta[:n]
        assert ((sent[:, 0] >= 0) & (sent[:, 0] < E)).all() and (np.diff(sent[:, 0] // nle) >= 0).all(), r
        behind = meta[n: ids.size]
        assert np.array_equal(behind[:, 0], ids[~ok]), r                      # in (t, k) order
        assert np.array_equal(behind[:, 2] * K + behind[:, 3], np.flatnonzero(~ok)), r


def test_send_back_rows_whose_meta_names_no_rank_go_last():
    """Stage 3 ranking by the origin column (no plan): origins outside [0, W) must not shift the
    segments of the real origins; such rows are counted for nobody and placed behind."""
    import ctypes as C
    from amd_distributed_2025_amd import HIPAllToAll, _lib

    W, nle, K, H, max_T = 4, 2, 2, 40, 4
    cfg = MoEConfig(W * nle, K, H, max_T, in_dtype=torch.bfloat16, out_dtype=torch.bfloat16)
    a = HIPAllToAll(cfg, 1, W, device=DEV)
    max_recv = max_T * W
    counts = np.array([5, 7], np.int32)
    origin = [np.array([0, 0, -3, 2, 3]), np.array([0, 1, 1, 9, 2, -1, 3])]
    rng = np.random.default_rng(2)
    ey = torch.zeros(nle, max_recv, H, dtype=torch.bfloat16, device=DEV)
    em = torch.full((nle, max_recv, 5), -7, dtype=torch.int32, device=DEV)
    stream_meta, stream_rows = [], []
    for le in range(nle):
        n = int(counts[le])
        m = np.zeros((n, 5), np.int32)
        m[:, 0] = 2 + le; m[:, 1] = origin[le]; m[:, 2] = rng.integers(0, max_T, n); m[:, 3] = rng.integers(0, K, n)
        rows = torch.from_numpy(rng.integers(0, 0x4400, (n, H), dtype=np.int16)).view(torch.bfloat16)
        ey[le, :n] = rows.to(DEV); em[le, :n] = torch.from_numpy(m).to(DEV)
        stream_meta.append(m); stream_rows.append(bits(rows))
    stream_meta, stream_rows = np.concatenate(stream_meta), np.concatenate(stream_rows)
    real = (stream_meta[:, 1] >= 0) & (stream_meta[:, 1] < W)
    want_counts, order = orc.return_order(stream_meta[real], W)
    n_real, n_all = int(real.sum()), int(counts.sum())
    back_buf = torch.zeros(n_all, H, dtype=torch.bfloat16, device=DEV)
    back_meta = torch.zeros(n_all, 5, dtype=torch.int32, device=DEV)
    back_counts = torch.zeros(W, dtype=torch.int32, device=DEV)
    p = lambda t: C.c_void_p(t.data_ptr())
    _lib.call("moe_a2a_combine_send", C.byref(a.shape), p(ey), p(em), p(torch.from_numpy(counts).to(DEV)),
              n_all, n_all, p(back_buf), p(back_meta), p(back_counts), None,
              C.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert np.array_equal(back_counts.cpu().numpy(), want_counts)
    assert np.array_equal(back_meta.cpu().numpy()[:n_real], stream_meta[real][order])
    assert np.array_equal(bits(back_buf[:n_real]), stream_rows[real][order])
    # the strays follow, ordered by their origin read as an unsigned number, then by stream position
    stray = np.flatnonzero(~real)
    stray = stray[np.argsort(stream_meta[stray, 1].astype(np.uint32), kind="stable")]
    assert np.array_equal(back_meta.cpu().numpy()[n_real:], stream_meta[stray])
