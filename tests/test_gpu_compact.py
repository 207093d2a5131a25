"""The compact expert-major layout (`moe_a2a_*_compact`): the experts' rows back to back instead of
the reference's padded `[nle, max_recv, H]` buffers (all2all/reference.py:123-136). The compact rows
are, in order, exactly the oracle's expert-major rows; expanded to the padded layout they are what
the padded entry points write; every later stage and `y` give the same bits in both layouts."""
import numpy as np
import pytest
import torch

from amd_distributed_2025_amd import HIPAllToAll, LocalWorld, WORKLOADS, generate_world, _binding
from amd_distributed_2025_amd.task import MoEConfig, dtype_name
from oracle import moe_a2a_oracle as orc
from tests.helpers import bits, run_oracle
from tests.test_gpu_expert_path import selection_layer, select_columns

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SENT = 0x7B7B


def on_gpu(name, seed, **over):
    world = generate_world(dict(WORKLOADS[name], **over), seed)
    return world, world[0][0], [d.to(DEV) for _, d, _, _ in world]


@pytest.mark.parametrize("plan", [True, False], ids=["plan", "scan"])
@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_compact_layout_matches_the_oracle_and_the_padded_layout(name, plan):
    print(f"compact layout {name} plan={plan}", flush=True)
    world, cfg, dev = on_gpu(name, 21)
    W = len(world)
    nle, max_recv = cfg.num_experts // W, cfg.max_num_tokens * W
    lw = LocalWorld(cfg, W, device=DEV, layout="compact", reuse_placement=plan)
    ys = lw.run(dev)
    torch.cuda.synchronize()
    want = run_oracle(world)
    ref = LocalWorld(cfg, W, device=DEV, reuse_placement=plan)  # the padded layout on the same job
    ys_ref = ref.run(dev)
    torch.cuda.synchronize()
    for r in range(W):
        g, a = lw.trace[r], lw.ranks[r]
        cnt = g["expert_num_tokens"].cpu().numpy()
        R = int(cnt.sum())
        assert np.array_equal(cnt, want[r].expert_num_tokens), r
        assert np.array_equal(a.expert_offsets.cpu().numpy(), np.concatenate([[0], np.cumsum(cnt)])), r
        assert g["expert_x"].dim() == 2 and g["expert_meta"].dim() == 2
        # the compact rows are the oracle's expert-major stream, row for row
        assert np.array_equal(bits(g["expert_x"][:R]), want[r].expert_rows), r
        assert np.array_equal(g["expert_meta"][:R].cpu().numpy(), want[r].expert_meta_rows), r
        assert np.array_equal(bits(g["expert_y"][:R]), want[r].expert_y_rows), r
        # expanded to the reference's padded layout: what the padded entry points wrote
        if name != "C4" and name != "C5" or r == 0:
            off = np.concatenate([[0], np.cumsum(cnt)])
            px, pm = ref.trace[r]["expert_x"], ref.trace[r]["expert_meta"]
            for le in range(nle):
                n = int(cnt[le])
                assert torch.equal(px[le, :n], g["expert_x"][off[le]:off[le] + n]), (r, le)
                assert torch.equal(pm[le, :n], g["expert_meta"][off[le]:off[le] + n]), (r, le)
        n_back = int(want[r].back_counts.sum())
        assert np.array_equal(g["back_counts"].cpu().numpy(), want[r].back_counts), r
        assert np.array_equal(bits(g["back_buf"][:n_back]), want[r].back_buf), r
        assert np.array_equal(g["back_meta"][:n_back].cpu().numpy(), want[r].back_meta), r
        assert np.array_equal(bits(ys[r]), want[r].y), r
        assert torch.equal(ys[r], ys_ref[r]), r


def _edge_shapes():
    from tests.test_gpu_parity import EDGE
    return EDGE


@pytest.mark.parametrize("name", sorted(_edge_shapes()))
def test_compact_layout_on_the_edge_shapes(name):
    """Rows that are not 16 bytes long, one local expert, 256 local experts (the prefix table in LDS
    instead of registers), K = E, tiny and wide rows: `y` and the compact rows equal the oracle's."""
    print(f"compact edge {name}", flush=True)
    spec = dict(dict(routing="uniform", weights="rand"), **_edge_shapes()[name])
    world = generate_world(spec, 31)
    cfg, W = world[0][0], len(world)
    dev = [d.to(DEV) for _, d, _, _ in world]
    want = run_oracle(world)
    for plan in (True, False):
        lw = LocalWorld(cfg, W, device=DEV, layout="compact", reuse_placement=plan)
        ys = lw.run(dev)
        torch.cuda.synchronize()
        for r in range(W):
            R = int(want[r].expert_num_tokens.sum())
            assert np.array_equal(bits(lw.trace[r]["expert_x"][:R]), want[r].expert_rows), (plan, r)
            assert np.array_equal(lw.trace[r]["expert_meta"][:R].cpu().numpy(), want[r].expert_meta_rows), (plan, r)
            assert np.array_equal(bits(ys[r]), want[r].y), (plan, r)


@pytest.mark.parametrize("binding", ["ctypes", "ext"])
def test_compact_layout_through_both_bindings(binding):
    world, cfg, dev = on_gpu("C3", 22)
    lw = LocalWorld(cfg, len(world), device=DEV, layout="compact", binding=binding)
    ys = lw.run(dev)
    torch.cuda.synchronize()
    want = run_oracle(world)
    for r in range(len(world)):
        assert np.array_equal(bits(ys[r]), want[r].y), r


@pytest.mark.parametrize("name,inter", [("C2", 1024), ("C3", 4096), ("C4", None)])
def test_grouped_gemm_on_compact_rows(name, inter):
    """The expert as layers of `expert_gemm` on the compact rows: the oracle's bits with selection
    weights (one or two layers, widths above and below hidden_dim), and the bits of the padded layout
    with random weights and a bias (which layout the rows lie in changes no bit)."""
    print(f"compact gemm {name} inter={inter}", flush=True)
    world, cfg, dev = on_gpu(name, 23)
    W, H, dt = len(world), cfg.hidden_dim, cfg.in_dtype
    nle = cfg.num_experts // W
    rng = np.random.default_rng(6)
    if inter is None:
        layers = [selection_layer(rng, nle, H, H, dt)]
    else:
        layers = [selection_layer(rng, nle, inter, H, dt), selection_layer(rng, nle, H, inter, dt)]

    def gpu_expert(a, ex, num, hint):
        h = ex
        for w, _, _ in layers:
            h = a.expert_gemm(h, num, w, None, hint)
        return h

    def oracle_expert(rank, rows, counts):
        for _, src, neg in layers:
            rows = select_columns(rows, counts, src, neg)
        return rows

    lw = LocalWorld(cfg, W, device=DEV, layout="compact")
    ys = lw.run(dev, expert=gpu_expert)
    torch.cuda.synchronize()
    want = run_oracle(world, expert=oracle_expert)
    for r in range(W):
        R = int(want[r].expert_num_tokens.sum())
        assert np.array_equal(bits(lw.trace[r]["expert_y"][:R]), want[r].expert_y_rows), r
        assert np.array_equal(bits(ys[r]), want[r].y), r
    del layers
    # random weights and a bias: compact against padded, bit for bit (every kernel: the row count picks it)
    gen = torch.Generator(device=DEV).manual_seed(4)
    wts = torch.empty(nle, H, H, dtype=dt, device=DEV)
    for le in range(nle):
        wts[le] = (torch.randn(H, H, generator=gen, device=DEV) / H ** 0.5).to(dt)
    bias = (torch.randn(nle, H, generator=gen, device=DEV) * 0.1).to(dt)
    ref = LocalWorld(cfg, W, device=DEV)
    for hint_scale in (0, 1, 16):
        expert = lambda a, ex, num, hint: a.expert_gemm(ex, num, wts, bias, None if hint is None else hint * hint_scale)
        ys_c = [y.clone() for y in lw.run(dev, expert=expert)]
        ys_p = [y.clone() for y in ref.run(dev, expert=expert)]
        torch.cuda.synchronize()
        for r in range(W):
            cnt = lw.trace[r]["expert_num_tokens"].cpu().tolist()
            padded = torch.cat([ref.trace[r]["expert_y"][le, :c] for le, c in enumerate(cnt)])
            assert torch.equal(lw.trace[r]["expert_y"][: sum(cnt)], padded), (hint_scale, r)
            assert torch.equal(ys_c[r], ys_p[r]), (hint_scale, r)


def test_rows_without_room_are_dropped_and_nothing_is_touched_past_the_buffers():
    """Compact buffers that hold fewer rows than arrive: the first rows of the (expert, position)
    order are stored, the counts still report every arrival, the expert and the send-back stage work
    on the stored rows only, and memory behind the stated rows keeps its contents."""
    world, cfg, dev = on_gpu("C3", 24, num_tokens="full")
    W, H, dt = len(world), cfg.hidden_dim, cfg.in_dtype
    nle = cfg.num_experts // W
    lw = LocalWorld(cfg, W, device=DEV)
    lw.run(dev)                                    # the padded job: rank 0's received stream is left in its buffers
    torch.cuda.synchronize()
    g, a = lw.trace[0], lw.ranks[0]
    want = run_oracle(world)[0]
    R = int(want.expert_num_tokens.sum())
    ROOM = R - 37                                   # not enough for the last rows
    b = _binding.get("ctypes")
    st = torch.cuda.current_stream().cuda_stream
    big_x = torch.empty(ROOM + 64, H, dtype=dt, device=DEV); big_x.view(torch.int16).fill_(SENT)
    big_y = torch.empty(ROOM + 64, H, dtype=dt, device=DEV); big_y.view(torch.int16).fill_(SENT)
    big_g = torch.empty(ROOM + 64, H, dtype=dt, device=DEV); big_g.view(torch.int16).fill_(SENT)
    big_m = torch.full((ROOM + 64, 5), -SENT, dtype=torch.int32, device=DEV)
    num = torch.empty(nle, dtype=torch.int32, device=DEV)
    off = torch.empty(nle + 1, dtype=torch.int32, device=DEV)
    plan = torch.empty(2 * cfg.num_experts, dtype=torch.int32, device=DEV)
    ex, ey, eg, em = big_x[:ROOM], big_y[:ROOM], big_g[:ROOM], big_m[:ROOM]
    b.dispatch_recv_compact(a.shape, g["recv_buf"], g["recv_meta"], g["recv_counts"], R, num, off, ex, em, plan, st)
    b.expert_scale_compact(a.shape, ex, num, R, ey, st)
    eye = torch.eye(H, dtype=dt, device=DEV).expand(nle, H, H).contiguous()
    for hint in (0, R, 64 * R):                     # the streaming kernel and both kinds of tiles
        eg.view(torch.int16).fill_(SENT)
        b.expert_gemm_compact(a.shape, ex, num, hint, eye, None, eg, st)
        torch.cuda.synchronize()
        assert torch.equal(eg, ex), hint
    back_buf = torch.zeros(R, H, dtype=dt, device=DEV)
    back_meta = torch.full((R, 5), -SENT, dtype=torch.int32, device=DEV)
    back_counts = torch.empty(W, dtype=torch.int32, device=DEV)
    for use_plan in (plan, None):
        back_meta.fill_(-SENT)
        b.combine_send_compact(a.shape, ey, em, num, R, back_buf, back_meta, back_counts, use_plan, st)
        torch.cuda.synchronize()
        kept_meta = want.expert_meta_rows[:ROOM]
        counts, order = orc.return_order(kept_meta, W)
        assert np.array_equal(back_counts.cpu().numpy(), counts), use_plan is None
        assert np.array_equal(back_meta[:ROOM].cpu().numpy(), kept_meta[order])
        assert np.array_equal(bits(back_buf[:ROOM]), want.expert_y_rows[:ROOM][order])
        assert bool((back_meta[ROOM:] == -SENT).all())
    assert np.array_equal(num.cpu().numpy(), want.expert_num_tokens)          # every arrival is reported
    assert np.array_equal(off.cpu().numpy(), np.concatenate([[0], np.cumsum(want.expert_num_tokens)]))
    assert np.array_equal(bits(ex), want.expert_rows[:ROOM])
    assert np.array_equal(em.cpu().numpy(), want.expert_meta_rows[:ROOM])
    assert np.array_equal(bits(ey), want.expert_y_rows[:ROOM])
    for big in (big_x, big_y, big_g):
        assert bool((big[ROOM:].view(torch.int16) == SENT).all())
    assert bool((big_m[ROOM:] == -SENT).all())


def test_compact_workspace_at_c4_is_a_fraction_of_the_padded_one():
    world, cfg, dev = on_gpu("C4", 25)
    W = len(world)
    rows = 2560  # a quarter more than balanced routing delivers (2048); the most any rank of this job gets is below 2100
    lw = LocalWorld(cfg, W, device=DEV, layout="compact", compact_rows=rows)
    ys = lw.run(dev)
    torch.cuda.synchronize()
    want = run_oracle(world)
    for r in range(W):
        assert np.array_equal(bits(ys[r]), want[r].y), r
    a = lw.ranks[0]
    expert_bytes = sum(a._ws[n].numel() * a._ws[n].element_size() for n in ("expert_x", "expert_y", "expert_meta"))
    padded_bytes = 2 * (cfg.num_experts // W) * cfg.max_num_tokens * W * cfg.hidden_dim * 2
    print(f"expert buffers: {expert_bytes / 1e6:.1f} MB compact, {padded_bytes / 1e6:.1f} MB padded; "
          f"whole workspace of a rank {a.workspace_bytes() / 1e6:.1f} MB", flush=True)
    assert expert_bytes < 100e6 and padded_bytes > 1.8e9
    assert a.workspace_bytes() < 250e6


@pytest.mark.parametrize("layout", ["compact", "padded"])
@pytest.mark.parametrize("factor", [0.0, 0.05, 0.4, 1.5])
def test_launch_sizes_below_and_above_the_row_counts(layout, factor):
    """`rows_hint` only sizes launches: every half must move the whole stream when the hint is far
    below the rows that arrive (and when it is above). The row counts that size the launches of a
    skewed job are scaled by `factor` before they reach the halves."""
    print(f"hints x {factor}, {layout}", flush=True)
    spec = dict(world_size=4, num_experts=32, experts_per_token=6, hidden_dim=24, max_num_tokens=95,
                num_tokens="full", routing="zipf", weights="rand", dtype="bf16")
    world = generate_world(spec, 90003)
    cfg, W = world[0][0], 4
    dev = [d.to(DEV) for _, d, _, _ in world]
    want = run_oracle(world)
    for plan in (True, False):
        lw = LocalWorld(cfg, W, device=DEV, layout=layout, reuse_placement=plan)
        counts_of = lw._exchange_hints
        lw._exchange_hints = lambda phase, sent: [[int(c * factor) for c in row] for row in counts_of(phase, sent)]
        ys = lw.run(dev)
        torch.cuda.synchronize()
        for r in range(W):
            g, n = lw.trace[r], int(want[r].expert_num_tokens.sum())
            assert np.array_equal(g["expert_num_tokens"].cpu().numpy(), want[r].expert_num_tokens), r
            if layout == "compact":
                assert np.array_equal(bits(g["expert_x"][:n]), want[r].expert_rows), r
                assert np.array_equal(g["expert_meta"][:n].cpu().numpy(), want[r].expert_meta_rows), r
                assert np.array_equal(bits(g["expert_y"][:n]), want[r].expert_y_rows), r
            assert np.array_equal(bits(g["back_buf"][:n]), want[r].back_buf), r
            assert np.array_equal(bits(ys[r]), want[r].y), r


@pytest.mark.parametrize("binding", ["ctypes", "ext"])
def test_class_surface_in_the_compact_layout_on_a_skewed_job(binding):
    """`dispatch()` / `combine()` without row counts on the host size their launches for the rows a
    rank sends; with skewed routing some ranks receive more than that (here 749 and 654 rows for
    570 sent)."""
    from amd_distributed_2025_amd import run_lockstep

    spec = dict(world_size=4, num_experts=32, experts_per_token=6, hidden_dim=24, max_num_tokens=95,
                num_tokens="full", routing="zipf", weights="rand", dtype="bf16")
    world = generate_world(spec, 90003)
    cfg, W = world[0][0], 4
    dev = [d.to(DEV) for _, d, _, _ in world]
    want = run_oracle(world)
    assert max(int(t.recv_counts.sum()) for t in want) > cfg.max_num_tokens * cfg.experts_per_token

    def rank_main(rank, exchange):
        ata = HIPAllToAll(cfg, rank, W, exchange=exchange, device=DEV, binding=binding, layout="compact")
        num, ex, em = ata.dispatch(dev[rank].x, dev[rank].indices)
        ey = ata.expert_scale(ex, num)
        y = torch.zeros(cfg.max_num_tokens, cfg.hidden_dim, dtype=cfg.out_dtype, device=DEV)
        ata.combine(y, dev[rank].weights, em, ey, num)
        torch.cuda.synchronize()
        return y[: dev[rank].num_tokens].clone(), ex.clone(), em.clone()

    for r, (y, ex, em) in enumerate(run_lockstep(W, rank_main, exact_hints=False, device=DEV)):
        n = int(want[r].expert_num_tokens.sum())
        assert np.array_equal(bits(ex[:n]), want[r].expert_rows), r
        assert np.array_equal(em[:n].cpu().numpy(), want[r].expert_meta_rows), r
        assert np.array_equal(bits(y), want[r].y), r
