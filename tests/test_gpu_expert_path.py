"""dispatch -> grouped GEMM -> combine: the expert of a model (`moe_a2a_expert_gemm`) in the place
where all2all/reference.py:262 has its stand-in, fed with what `dispatch_recv` really left in the
padded buffers and followed by the real `combine`.

Weights that only move and negate columns (one nonzero entry of +-1 per output) make every
summation order give the same bits, so `y` is compared bit for bit with the oracle stepping the
same job with the closed form of that expert. With random weights the matrix unit's summation
order is its own: there the expert's output is held to `oracle.linear_bound`, `y` is compared bit
for bit with the oracle's combine fed with the rows the GPU's expert produced (which pins the
hand-off of expert_meta / counts / plan around a real expert), and `y` is also held to that bound
carried through the combine (`oracle.combine_bound`)."""
import numpy as np
import pytest
import torch

from amd_distributed_2025_amd import LocalWorld, WORKLOADS, generate_world
from amd_distributed_2025_amd.task import dtype_name
from oracle import moe_a2a_oracle as orc
from tests.helpers import bits, run_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def selection_layer(rng, nle, out_dim, in_dim, dt):
    """Weights [nle, out_dim, in_dim] with one entry of +-1 per output row: output n of expert le is
    +-input src[le, n]. Returns (weights on the GPU, src, negate)."""
    src = np.stack([rng.permutation(max(out_dim, in_dim))[:out_dim] % in_dim for _ in range(nle)])
    neg = rng.random((nle, out_dim)) < 0.5
    w = torch.zeros(nle, out_dim, in_dim, dtype=dt, device=DEV)
    le = torch.arange(nle, device=DEV)[:, None].expand(nle, out_dim)
    n = torch.arange(out_dim, device=DEV)[None, :].expand(nle, out_dim)
    w[le, n, torch.from_numpy(src).to(DEV)] = torch.from_numpy(np.where(neg, -1.0, 1.0)).to(dt).to(DEV)
    return w, src, neg


def select_columns(rows, counts, src, neg):
    """The closed form of a selection layer on compact expert-major rows (bit patterns)."""
    out = np.empty((rows.shape[0], src.shape[1]), np.uint16)
    g = 0
    for le, c in enumerate(int(c) for c in counts):
        out[g:g + c] = rows[g:g + c][:, src[le]] ^ np.where(neg[le], 0x8000, 0).astype(np.uint16)
        g += c
    # a zero of either sign summed with the zeros of the other products (and the accumulator's +0) is +0
    out[(out & 0x7FFF) == 0] = 0
    return out


def compact(padded, counts):
    """Valid rows of a padded [nle, max_recv, H] tensor, expert 0 first."""
    return torch.cat([padded[le, :c] for le, c in enumerate(counts)], dim=0)


def world_on_gpu(name, seed):
    world = generate_world(WORKLOADS[name], seed)
    cfg = world[0][0]
    return world, cfg, [d.to(DEV) for _, d, _, _ in world]


@pytest.mark.parametrize("binding", ["ctypes", "ext"])
@pytest.mark.parametrize("name,inter", [("C2", 1024), ("C3", 4096), ("C3", 2048), ("C4", None)])
def test_selection_experts_give_the_oracle_bits(name, inter, binding):
    """One layer H -> H at C4; two layers H -> inter -> H (inter above, below and equal to H)
    elsewhere: every buffer and `y` bit for bit."""
    if name == "C4" and binding == "ext":
        pytest.skip("the large case runs once; the bindings are compared on the small ones")
    print(f"selection expert {name} inter={inter} {binding}", flush=True)
    world, cfg, dev = world_on_gpu(name, 11)
    W, H, dt = len(world), cfg.hidden_dim, cfg.in_dtype
    nle = cfg.num_experts // W
    rng = np.random.default_rng(5)
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

    lw = LocalWorld(cfg, W, device=DEV, binding=binding)
    ys = lw.run(dev, expert=gpu_expert)
    torch.cuda.synchronize()
    want = run_oracle(world, expert=oracle_expert)
    for r in range(W):
        g = lw.trace[r]
        counts = g["expert_num_tokens"].cpu().tolist()
        assert np.array_equal(np.array(counts), want[r].expert_num_tokens), f"rank {r}: counts"
        assert np.array_equal(bits(compact(g["expert_x"], counts)), want[r].expert_rows), f"rank {r}: expert_x"
        assert np.array_equal(bits(compact(g["expert_y"], counts)), want[r].expert_y_rows), f"rank {r}: expert_y"
        n_back = int(want[r].back_counts.sum())
        assert np.array_equal(g["back_counts"].cpu().numpy(), want[r].back_counts), f"rank {r}: back_counts"
        assert np.array_equal(bits(g["back_buf"][:n_back]), want[r].back_buf), f"rank {r}: back_buf"
        assert np.array_equal(bits(ys[r]), want[r].y), f"rank {r}: y"
    del lw, layers


def bound_on_gpu(x16, w16, b16, name):
    """`oracle.linear_bound` evaluated with float64 tensors on the GPU (the numpy statement takes
    minutes at 2048 x 7168 x 7168); the test below checks it against the numpy one first."""
    x, w = x16.double(), w16.double()
    exact = x @ w.T
    mass = x.abs() @ w.abs().T
    u16, floor = (2.0 ** -8, 2.0 ** -133) if name == "bf16" else (2.0 ** -11, 2.0 ** -24)
    sum_err = x.shape[1] * 2.0 ** -24 * mass
    tol = u16 * (exact.abs() + sum_err) + sum_err + floor
    if b16 is None:
        return exact, tol
    total = exact + b16.double()[None, :]
    return total, tol + (u16 + 2.0 ** -23) * (total.abs() + tol)


@pytest.mark.parametrize("name,with_bias", [("C3", True), ("C3", False), ("C4", True)])
def test_random_experts_stay_inside_the_bounds(name, with_bias):
    print(f"random expert {name} bias={with_bias}", flush=True)
    world, cfg, dev = world_on_gpu(name, 12)
    W, H, dt = len(world), cfg.hidden_dim, cfg.in_dtype
    nle, tname = cfg.num_experts // W, dtype_name(cfg.in_dtype)
    gen = torch.Generator(device=DEV).manual_seed(3)
    wts = torch.empty(nle, H, H, dtype=dt, device=DEV)  # (the same experts on every rank: 3.3 GB at C4)
    for le in range(nle):
        wts[le] = (torch.randn(H, H, generator=gen, device=DEV) / H ** 0.5).to(dt)
    bias = (torch.randn(nle, H, generator=gen, device=DEV) * 0.1).to(dt) if with_bias else None

    # the GPU statement of the bound against the numpy one, on a corner of the operands
    xs, ws = dev[0].x[:5], wts[0, :7]
    e_t, t_t = bound_on_gpu(xs, ws, None if bias is None else bias[0, :7], tname)
    e_n, t_n = orc.linear_bound(bits(xs), bits(ws), None if bias is None else bits(bias[0, :7]), tname)
    assert np.allclose(e_t.cpu().numpy(), e_n, rtol=1e-12, atol=1e-300)
    assert np.allclose(t_t.cpu().numpy(), t_n, rtol=1e-9, atol=1e-300)

    lw = LocalWorld(cfg, W, device=DEV)
    ys = lw.run(dev, expert=lambda a, ex, num, hint: a.expert_gemm(ex, num, wts, bias, hint))
    torch.cuda.synchronize()

    gpu_rows, exacts, tols = [], [], []
    for r in range(W):
        g = lw.trace[r]
        counts = g["expert_num_tokens"].cpu().tolist()
        got = compact(g["expert_y"], counts)
        ex_parts, tol_parts = [], []
        for le, c in enumerate(counts):
            e, t = bound_on_gpu(g["expert_x"][le, :c], wts[le], None if bias is None else bias[le], tname)
            ex_parts.append(e)
            tol_parts.append(t)
        exact, tol = torch.cat(ex_parts), torch.cat(tol_parts)
        err = (got.double() - exact).abs()
        assert bool((err <= tol).all()), f"rank {r}: expert_y outside the bound by {float((err - tol).max())}"
        gpu_rows.append(bits(got))
        exacts.append(exact.cpu().numpy())
        tols.append(tol.cpu().numpy())

    # the combine on exactly the rows the GPU's expert produced: y bit for bit
    want = run_oracle(world, expert=lambda rank, rows, counts: gpu_rows[rank])
    for r in range(W):
        assert np.array_equal(bits(ys[r]), want[r].y), f"rank {r}: y differs from the oracle's combine of the same rows"

    # and y against the exact value with the expert's bound carried through the combine
    for r in range(W):
        # rows come back to rank r in the order of want[r].ret_meta; find each one's owner-side row
        meta = want[r].ret_meta
        ret_exact = np.empty((meta.shape[0], H))
        ret_tol = np.empty((meta.shape[0], H))
        for owner in range(W):
            om = want[owner].expert_meta_rows  # compact expert-major meta rows on the owner
            key = {(int(m[1]), int(m[2]), int(m[3])): i for i, m in enumerate(om)}
            mine = np.nonzero(meta[:, 0] // nle == owner)[0]
            src = np.array([key[(r, int(meta[i, 2]), int(meta[i, 3]))] for i in mine], dtype=np.int64)
            ret_exact[mine] = exacts[owner][src]
            ret_tol[mine] = tols[owner][src]
        exact_y, tol_y = orc.combine_bound(ret_exact, ret_tol, meta, world[r][1].weights.numpy(),
                                           cfg.max_num_tokens, dtype_name(cfg.out_dtype))
        T = world[r][1].num_tokens
        got_y = orc.b16_to_f32(bits(ys[r]), dtype_name(cfg.out_dtype)).astype(np.float64)
        err = np.abs(got_y - exact_y[:T])
        assert (err <= tol_y[:T]).all(), f"rank {r}: y outside the carried bound by {(err - tol_y[:T]).max()}"
        if name == "C4" and r == 1:
            break  # (two ranks of the large case are enough; each takes a few seconds of host loops)
    del lw, wts
