"""The drop-in boundary on a real GPU: the reference's class surface
(`dispatch` / `combine`, all2all/reference.py:68,151) driven exactly as
`ref_kernel` drives it (reference.py:259-272), the torch-extension binding
against the ctypes binding, and the oracle's 16-bit arithmetic against torch's
own on the device the reference runs on."""
import numpy as np
import pytest
import torch

from amd_distributed_2025_amd import HIPAllToAll, LocalWorld, WORKLOADS, generate_world
from amd_distributed_2025_amd.all2all import LocalExchange, run_lockstep
from amd_distributed_2025_amd.task import DTYPES, MoEConfig
from oracle import moe_a2a_oracle as orc
from tests.helpers import bits, from_bits, run_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ref_kernel_body(ata, cfg, rank_data, rank, seen):
    """The statements of all2all/reference.py:259-272 with the class under test."""
    expert_num, expert_x, expert_meta = ata.dispatch(rank_data.x, rank_data.indices)
    seen.update(expert_num=expert_num, expert_x=expert_x, expert_meta=expert_meta)
    expert_y = expert_x.to(cfg.out_dtype) * (1 + rank)
    y = torch.zeros(cfg.max_num_tokens, cfg.hidden_dim, dtype=cfg.out_dtype, device=rank_data.x.device)
    ata.combine(y, rank_data.weights, expert_meta, expert_y, expert_num)
    return y[: rank_data.num_tokens]


@pytest.mark.parametrize("name,binding", [("C1", "ctypes"), ("C2", "ctypes"), ("C2", "ext"), ("C3", "ctypes")])
@pytest.mark.parametrize("exact_hints", [False, True])
def test_reference_class_surface_runs_ref_kernel(name, binding, exact_hints):
    """Only `dispatch(dp_x, indices)` and `combine(out_tokens, weights, expert_meta, expert_y,
    expert_num_tokens)` are called, one thread per rank as the reference has one process per
    rank; every rank's result and the three returned layouts are checked."""
    print(f"class surface {name} {binding} exact_hints={exact_hints}", flush=True)
    world = generate_world(WORKLOADS[name], 2025)
    cfg, W = world[0][0], len(world)
    nle, max_recv = cfg.num_experts // W, cfg.max_num_tokens * W
    dev = [d.to(DEV) for _, d, _, _ in world]
    seen = [dict() for _ in range(W)]

    def rank_main(rank, exchange):
        ata = HIPAllToAll(cfg, rank, W, exchange=exchange, device=DEV, binding=binding)
        y = ref_kernel_body(ata, cfg, dev[rank], rank, seen[rank])
        torch.cuda.synchronize()
        return y.clone(), {k: v.clone() for k, v in seen[rank].items()}

    results = run_lockstep(W, rank_main, exact_hints=exact_hints, device=DEV)
    want = run_oracle(world)
    for r, (y, layouts) in enumerate(results):
        num, ex, em = layouts["expert_num"], layouts["expert_x"], layouts["expert_meta"]
        # the layouts of all2all/reference.py:123-136,148
        assert num.shape == (nle,) and num.dtype == torch.int32
        assert ex.shape == (nle, max_recv, cfg.hidden_dim) and ex.dtype == cfg.in_dtype
        assert em.shape == (nle, max_recv, 5) and em.dtype == torch.int32
        assert y.shape == (dev[r].num_tokens, cfg.hidden_dim) and y.dtype == cfg.out_dtype
        cnt = num.cpu().numpy()
        assert np.array_equal(cnt, want[r].expert_num_tokens), r
        rows = torch.cat([ex[le, : int(cnt[le])] for le in range(nle)])
        metas = torch.cat([em[le, : int(cnt[le])] for le in range(nle)])
        assert np.array_equal(bits(rows), want[r].expert_rows), r
        assert np.array_equal(metas.cpu().numpy(), want[r].expert_meta_rows), r
        assert np.array_equal(bits(y), want[r].y), f"rank {r}: combined rows differ from the oracle"


def test_single_rank_job_needs_no_exchange_object():
    world = generate_world(WORKLOADS["C1"], 11)
    cfg, d = world[0][0], world[0][1].to(DEV)
    y = ref_kernel_body(HIPAllToAll(cfg, 0, 1, device=DEV), cfg, d, 0, {})
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), run_oracle(world)[0].y)


def test_several_ranks_without_exchange_say_what_is_missing():
    world = generate_world(WORKLOADS["C2"], 11)
    cfg, d = world[0][0], world[0][1].to(DEV)
    with pytest.raises(RuntimeError, match="exchange"):
        HIPAllToAll(cfg, 0, 8, device=DEV).dispatch(d.x, d.indices)


def test_a_failing_rank_does_not_leave_the_others_waiting():
    world = generate_world(WORKLOADS["C2"], 3)
    cfg, W = world[0][0], len(world)
    dev = [d.to(DEV) for _, d, _, _ in world]

    def rank_main(rank, exchange):
        if rank == 3:
            raise ValueError("rank 3 gives up")
        return HIPAllToAll(cfg, rank, W, exchange=exchange, device=DEV).dispatch(dev[rank].x, dev[rank].indices)

    with pytest.raises(ValueError, match="rank 3 gives up"):
        run_lockstep(W, rank_main, device=DEV)
    torch.cuda.synchronize()


TRACE_KEYS = ("send_counts", "send_buf", "send_meta", "send_slot", "recv_counts", "expert_num_tokens",
              "back_counts", "ret_counts")


@pytest.mark.parametrize("name", ["C2", "C3"])
def test_extension_binding_gives_the_bits_of_the_ctypes_binding(name):
    """The whole job through the torch extension (torch::Tensor wrappers built by load_inline)
    and through ctypes: every intermediate of every rank is identical, and equals the oracle."""
    print(f"extension vs ctypes {name}", flush=True)
    world = generate_world(WORKLOADS[name], 77)
    cfg, W = world[0][0], len(world)
    dev = [d.to(DEV) for _, d, _, _ in world]
    via_ext = LocalWorld(cfg, W, device=DEV, binding="ext")
    via_ctypes = LocalWorld(cfg, W, device=DEV, binding="ctypes")
    assert via_ext.ranks[0].binding.name == "ext" and via_ctypes.ranks[0].binding.name == "ctypes"
    ys_e = via_ext.run(dev)
    ys_c = via_ctypes.run(dev)
    torch.cuda.synchronize()
    want = run_oracle(world)
    for r in range(W):
        e, c = via_ext.trace[r], via_ctypes.trace[r]
        S = dev[r].num_tokens * cfg.experts_per_token
        R = int(c["recv_counts"].sum().item())
        for key in TRACE_KEYS:
            assert torch.equal(e[key], c[key]), (r, key)
        # buffers of which only the leading rows are written
        for key, n in (("recv_buf", R), ("recv_meta", R), ("back_buf", R), ("back_meta", R),
                       ("ret_buf", S), ("ret_meta", S), ("y", dev[r].num_tokens)):
            assert torch.equal(e[key][:n], c[key][:n]), (r, key)
        cnt = c["expert_num_tokens"].cpu().numpy()
        for le in range(cnt.size):
            n = int(cnt[le])
            for key in ("expert_x", "expert_meta", "expert_y"):
                assert torch.equal(e[key][le, :n], c[key][le, :n]), (r, key, le)
        assert torch.equal(ys_e[r], ys_c[r])
        assert np.array_equal(bits(ys_e[r]), want[r].y)
    # the explicit send plan through the extension
    rc, ro, ec, dst, src = via_ext.ranks[0].plan_send(dev[0].indices)
    rc2, ro2, ec2, dst2, src2 = via_ctypes.ranks[0].plan_send(dev[0].indices)
    torch.cuda.synchronize()
    for a, b in ((rc, rc2), (ro, ro2), (ec, ec2), (dst, dst2), (src, src2)):
        assert torch.equal(a, b)


def test_extension_checks_its_tensors_before_launching():
    from amd_distributed_2025_amd import _ext

    m = _ext.load()
    shape = [1, 0, 4, 2, 64, 8]
    T, K, H = 8, 2, 64
    x = torch.zeros(T, H, dtype=torch.bfloat16, device=DEV)
    idx = torch.zeros(T, K, dtype=torch.int32, device=DEV)
    buf = torch.zeros(T * K, H, dtype=torch.bfloat16, device=DEV)
    meta = torch.zeros(T * K, 5, dtype=torch.int32, device=DEV)
    counts = torch.zeros(1, dtype=torch.int32, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    m.a2a_dispatch_send(shape, x, idx, T, buf, meta, counts, None, st)  # the good call
    with pytest.raises(RuntimeError, match="indices: expected Int"):
        m.a2a_dispatch_send(shape, x, idx.long(), T, buf, meta, counts, None, st)
    with pytest.raises(RuntimeError, match="x: must be contiguous"):
        m.a2a_dispatch_send(shape, torch.zeros(H, T, dtype=torch.bfloat16, device=DEV).t(), idx, T, buf, meta,
                            counts, None, st)
    with pytest.raises(RuntimeError, match="send_buf: holds"):
        m.a2a_dispatch_send(shape, x, idx, T, buf[: T * K - 1], meta, counts, None, st)
    with pytest.raises(RuntimeError, match="send_buf: expected BFloat16"):
        m.a2a_dispatch_send(shape, x, idx, T, buf.to(torch.float16), meta, counts, None, st)
    with pytest.raises(RuntimeError, match="x: token rows must be float16 or bfloat16"):
        m.a2a_dispatch_send(shape, x.float(), idx, T, buf, meta, counts, None, st)
    with pytest.raises(RuntimeError, match="send_meta: must be a GPU tensor"):
        m.a2a_dispatch_send(shape, x, idx, T, buf, meta.cpu(), counts, None, st)
    with pytest.raises(RuntimeError, match="status -1"):  # the library's own argument check
        m.a2a_dispatch_send([1, 0, 4, 2, 64, 4], x, idx, T, buf, meta, counts, None, st)
    torch.cuda.synchronize()


# ----------------------------------------------------------------------------- arithmetic on the device


def halfway_cases(name: str, n: int, rng) -> tuple:
    """Pairs (a, b) of 16-bit values with a + b exactly halfway between two neighbours of a:
    only round-to-nearest-EVEN after the addition gives the reference's bits."""
    if name == "bf16":
        mant_bits, exps = 7, rng.integers(-20, 60, n)
    else:
        mant_bits, exps = 10, rng.integers(-8, 10, n)
    mant = rng.integers(0, 1 << mant_bits, n)
    a = (1.0 + mant / float(1 << mant_bits)) * np.exp2(exps.astype(np.float64))
    b = np.exp2(exps.astype(np.float64) - mant_bits - 1)  # half a unit in the last place of a
    a16 = orc.f32_to_b16(a.astype(np.float32), name)
    b16 = orc.f32_to_b16(b.astype(np.float32), name)
    assert np.array_equal(orc.b16_to_f32(a16, name), a.astype(np.float32))  # both exact in 16 bits
    assert np.array_equal(orc.b16_to_f32(b16, name), b.astype(np.float32))
    return a16, b16


def torch_accumulate_on_device(rows, meta, w, T, dt):
    """The loop of all2all/reference.py:227-232, executed by torch on the GPU."""
    recv = from_bits(rows, dt).to(DEV)
    weights = torch.from_numpy(w).to(DEV)
    y = torch.zeros(T, rows.shape[1], dtype=dt, device=DEV)
    for i in range(rows.shape[0]):
        src_token, src_k = int(meta[i, 2]), int(meta[i, 3])
        weight = weights[src_token, src_k]
        y[src_token] += recv[i].to(torch.float32) * weight
    torch.cuda.synchronize()
    return bits(y)


# Rows of at most 8192 elements: the range every hidden_dim of the task lies in (the longest is
# 7168, all2all/task.yml:48-65). For much longer rows (16384 elements and more) this torch build's
# GPU kernel for `y16 += f32` switches to a vectorised form that first rounds the float32 addend
# to 16 bits; the library and the oracle follow the rule torch applies to the task's row lengths.
ROW = 8192


@pytest.mark.parametrize("name", ["bf16", "fp16"])
def test_oracle_accumulate_equals_torch_on_the_device(name):
    """all2all/reference.py:232 as torch executes it on the GPU — `y16[t] += row.float() * w`
    in a 16-bit tensor — for every 16-bit pattern as first addend, random second addends,
    weights that force roundings, and exact ties, against the oracle's `combine_recv`."""
    dt = DTYPES[name]
    rng = np.random.default_rng(5)
    n, blocks = 65536, 65536 // ROW
    allbits = np.arange(n, dtype=np.uint32).astype(np.uint16)
    second = orc.f32_to_b16((rng.standard_normal(n) * 3).astype(np.float32), name)
    tie_a, tie_b = halfway_cases(name, n, rng)
    # token group 0: every pattern, then a random addend; group 1: ties with unit weights;
    # group 2: a single addend. A group is `blocks` tokens, one per block of ROW columns.
    addends = [(allbits, 0, 0), (second, 0, 1), (tie_a, 1, 0), (tie_b, 1, 1), (second, 2, 1)]
    w_group = np.array([[1.0 + 2.0 ** -7, 0.3], [1.0, 1.0], [0.0, 0.7]], np.float32)
    rows, meta = [], []
    for values, group, k in addends:
        for b in range(blocks):
            rows.append(values[b * ROW:(b + 1) * ROW])
            meta.append([0, 0, group * blocks + b, k, 0])
    rows, meta = np.stack(rows), np.array(meta, np.int32)
    w = np.repeat(w_group, blocks, axis=0)
    T = 3 * blocks
    want = orc.combine_recv(rows, meta, w, T, name)
    got = torch_accumulate_on_device(rows, meta, w, T, dt)
    nan = np.isnan(orc.b16_to_f32(want, name))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(orc.b16_to_f32(got[nan], name)).all()
    # the ties really are ties: the exact sum is not a 16-bit value
    exact = orc.b16_to_f32(tie_a, name) + orc.b16_to_f32(tie_b, name)
    assert (orc.b16_to_f32(want[blocks:2 * blocks].ravel(), name) != exact).all()


@pytest.mark.parametrize("name", ["bf16", "fp16"])
@pytest.mark.parametrize("hidden_dim", [256, 2048, 2880, 4096, 6144, 7168])
def test_oracle_accumulate_equals_torch_on_the_device_at_task_row_lengths(name, hidden_dim):
    """Random arrivals, K = 8 addends per token, at every hidden_dim of all2all/task.yml:48-65
    and of the five workloads."""
    rng = np.random.default_rng(hidden_dim)
    T, K = 6, 8
    rows = orc.f32_to_b16(rng.standard_normal((T * K, hidden_dim)).astype(np.float32), name)
    tk = rng.permutation(T * K)
    meta = np.zeros((T * K, 5), np.int32)
    meta[:, 2], meta[:, 3] = tk // K, tk % K
    w = rng.random((T, K), dtype=np.float32)
    want = orc.combine_recv(rows, meta, w, T, name)
    assert np.array_equal(torch_accumulate_on_device(rows, meta, w, T, DTYPES[name]), want)


@pytest.mark.parametrize("name_in,name_out", [("bf16", "bf16"), ("fp16", "fp16"), ("fp16", "bf16"), ("bf16", "fp16")])
def test_oracle_expert_scale_equals_torch_on_the_device(name_in, name_out):
    """all2all/reference.py:262, `expert_x.to(out_dtype) * (1 + rank)`, as torch executes it on
    the GPU, for every 16-bit pattern and every rank of an 8-rank job."""
    allbits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = from_bits(allbits, DTYPES[name_in]).to(DEV)
    for rank in range(8):
        got = bits(x.to(DTYPES[name_out]) * (1 + rank))
        want = orc.expert_scale(allbits, rank, name_in, name_out)
        nan = np.isnan(orc.b16_to_f32(want, name_out))
        assert np.array_equal(got[~nan], want[~nan]), rank
        assert np.isnan(orc.b16_to_f32(got[nan], name_out)).all(), rank


# ----------------------------------------------------------------------------- gathering exchange

@pytest.mark.parametrize("H,dt", [(72, torch.bfloat16), (2048, torch.float16), (67, torch.bfloat16)])
def test_gathering_exchange_equals_its_legs(H, dt):
    """`moe_a2a_exchange_gather_local` for one destination against one `moe_a2a_exchange_local` per
    source: the same rows, meta rows and counts, including a source that holds nothing for the
    destination, counts above the stated capacity, and rows that are not 16 bytes long."""
    print(f"gathering exchange H={H} {dt}", flush=True)
    from amd_distributed_2025_amd import _binding
    import ctypes as C
    from amd_distributed_2025_amd import _lib

    W, CAP, SENT = 5, 40, -777
    rng = np.random.default_rng(H)
    b = _binding.get("ctypes")
    st = torch.cuda.current_stream().cuda_stream
    counts = rng.integers(0, 9, (W, W)).astype(np.int32)      # [src][dst]
    counts[2, :] = 0                                           # a source with nothing to send
    counts[3, 1] = 1000                                        # a count beyond what its buffer holds
    bufs = [torch.from_numpy(rng.integers(0, 0x4400, (CAP, H), dtype=np.int16)).view(dt).to(DEV) for _ in range(W)]
    metas = [torch.from_numpy(rng.integers(0, 99, (CAP, 5)).astype(np.int32)).to(DEV) for _ in range(W)]
    cnts = [torch.from_numpy(counts[s]).to(DEV) for s in range(W)]
    for dst in range(W):
        for binding in ("ctypes", "ext"):
            bb = _binding.get(binding)
            got_buf = torch.zeros(CAP, H, dtype=dt, device=DEV)
            got_meta = torch.full((CAP, 5), SENT, dtype=torch.int32, device=DEV)
            got_cnt = torch.full((W,), SENT, dtype=torch.int32, device=DEV)
            src = bb.gather_sources(H, bufs, metas, cnts)
            for hint in (0, 3, CAP):
                got_meta.fill_(SENT)
                bb.exchange_gather(W, H, src, dst, got_buf, got_meta, got_cnt, hint, st)
                want_buf = torch.zeros(CAP, H, dtype=dt, device=DEV)
                want_meta = torch.full((CAP, 5), SENT, dtype=torch.int32, device=DEV)
                want_cnt = torch.from_numpy(np.minimum(counts[:, dst], CAP)).to(DEV)
                for s in range(W):
                    b.exchange_local(W, H, bufs[s], metas[s], cnts[s], dst, want_buf, want_meta, want_cnt, s, CAP, st)
                torch.cuda.synchronize()
                assert torch.equal(got_cnt, want_cnt), (dst, binding, hint)
                assert torch.equal(got_meta, want_meta), (dst, binding, hint)
                n = int((got_meta[:, 0] != SENT).sum())
                assert torch.equal(got_buf[:n].view(torch.int16), want_buf[:n].view(torch.int16)), (dst, binding, hint)
    # more ranks than one launch serves, null tables
    one = C.c_void_p(16)
    table = (C.c_void_p * 65)(*([16] * 65))
    lib = _lib.load()
    assert lib.moe_a2a_exchange_gather_local(65, H, table, table, table, 0, one, one, one, 1, 4, 4, None) == -1
    assert lib.moe_a2a_exchange_gather_local(4, H, None, table, table, 0, one, one, one, 1, 4, 4, None) == -1
    assert lib.moe_a2a_exchange_gather_local(4, H, table, table, table, 4, one, one, one, 1, 4, 4, None) == -1


def test_class_surface_without_counts_takes_the_short_stream_entry_points():
    """`dispatch()` through `LocalExchange` with loose launch sizes gets no row count from the
    exchange. The entry point is then chosen for the rows balanced routing delivers, not for the
    capacity of the receive buffers: at C4 (2048 rows expected, 16384 rows of capacity) no planning
    launch runs and no `row_position` workspace is made."""
    world = generate_world(WORKLOADS["C4"], 5)
    cfg, W = world[0][0], len(world)
    dev = [d.to(DEV) for _, d, _, _ in world]
    objs = {}

    def rank_main(rank, exchange):
        a = objs[rank] = HIPAllToAll(cfg, rank, W, exchange=exchange, device=DEV)
        num, ex, em = a.dispatch(dev[rank].x, dev[rank].indices)
        ey = a.expert_scale(ex, num)
        y = torch.zeros(cfg.max_num_tokens, cfg.hidden_dim, dtype=cfg.out_dtype, device=DEV)
        a.combine(y, dev[rank].weights, em, ey, num)
        torch.cuda.synchronize()
        return y[: dev[rank].num_tokens].clone()

    ys = run_lockstep(W, rank_main, exact_hints=False, device=DEV)
    want = run_oracle(world)
    for r in range(W):
        assert "row_position" not in objs[r]._ws and "entry_row" not in objs[r]._ws, r
        assert np.array_equal(bits(ys[r]), want[r].y), r


# ----------------------------------------------------------------------------- the entry point, call after call

def test_custom_kernel_call_after_call_with_changing_inputs():
    """The first call of a job runs launch by launch, the second captures the job, later ones replay
    it: every call must give the oracle's bits for the inputs of THAT call, also when the inputs
    (and with them every count the launches were sized by) change between calls, and when a job of
    other token counts comes in between."""
    from amd_distributed_2025_amd import custom_kernel, custom_kernel_job, set_peer_inputs

    wl = dict(WORKLOADS["C3"], num_tokens="full")
    try:
        for call, seed in enumerate([1, 2, 3, 4]):
            world = generate_world(wl, seed)
            on_dev = [(c, d.to(DEV), r, w) for c, d, r, w in world]
            want = run_oracle(world)
            set_peer_inputs(on_dev)
            y3 = custom_kernel(on_dev[3])
            ys = custom_kernel_job(on_dev)
            torch.cuda.synchronize()
            assert np.array_equal(bits(y3), want[3].y), f"call {call}"
            for r in range(len(world)):
                assert np.array_equal(bits(ys[r]), want[r].y), f"call {call} rank {r}"
            if call == 2:  # a job with other token counts in between (its own first call)
                other = generate_world(WORKLOADS["C3"], 9)
                other_dev = [(c, d.to(DEV), r, w) for c, d, r, w in other]
                set_peer_inputs(other_dev)
                yo = custom_kernel_job(other_dev)
                torch.cuda.synchronize()
                wo = run_oracle(other)
                for r in range(len(other)):
                    assert np.array_equal(bits(yo[r]), wo[r].y), f"other job rank {r}"
        # skewed routing after uniform on the same captured job: launches sized for other counts
        world = generate_world(dict(wl, routing="zipf"), 6)
        on_dev = [(c, d.to(DEV), r, w) for c, d, r, w in world]
        set_peer_inputs(on_dev)
        ys = custom_kernel_job(on_dev)
        torch.cuda.synchronize()
        want = run_oracle(world)
        for r in range(len(world)):
            assert np.array_equal(bits(ys[r]), want[r].y), f"zipf rank {r}"
        # every rank in turn asks for its own rows (a captured job per rank asked for), twice over
        for _ in range(2):
            for r in range(len(world)):
                y = custom_kernel(on_dev[r])
                assert np.array_equal(bits(y), want[r].y), f"rank {r} alone"
    finally:
        set_peer_inputs(None)
