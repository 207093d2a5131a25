"""Pins for the numpy oracle: each function is checked against something whose
meaning does not come from the oracle itself — brute-force loops on small
inputs, closed forms, invariants, and torch's own arithmetic."""
import numpy as np
import pytest
import torch

from oracle import moe_a2a_oracle as orc

RNG = np.random.default_rng(20251125)


# ----------------------------------------------------------------------------- 16-bit conversions

@pytest.mark.parametrize("name,tdt", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_widening_matches_torch_for_every_bit_pattern(name, tdt):
    allbits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    ours = orc.b16_to_f32(allbits, name)
    theirs = torch.from_numpy(allbits.view(np.int16)).view(tdt).to(torch.float32).numpy()
    nan = np.isnan(theirs)
    assert np.array_equal(np.isnan(ours), nan)  # NaN payloads are not compared
    assert np.array_equal(ours.view(np.uint32)[~nan], theirs.view(np.uint32)[~nan])


@pytest.mark.parametrize("name,tdt", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_rounding_matches_torch(name, tdt):
    # random bit patterns cover all exponents, subnormals, infinities; ties are added explicitly
    u = RNG.integers(0, 2**32, size=400_000, dtype=np.uint64).astype(np.uint32)
    ties_bf16 = (RNG.integers(0, 2**16, size=70_000, dtype=np.uint64).astype(np.uint32) << 16) | 0x8000
    h = RNG.integers(0, 2**16, size=70_000, dtype=np.uint64).astype(np.uint16)
    near_fp16 = orc.b16_to_f32(h, "fp16")
    with np.errstate(all="ignore"):
        ties_fp16 = (near_fp16 + np.spacing(near_fp16.astype(np.float16)).astype(np.float32) / 2).view(np.uint32)
    vals = np.concatenate([u, ties_bf16, ties_bf16 + 1, ties_bf16 - 1, ties_fp16]).view(np.float32)
    finite_or_inf = ~np.isnan(vals)
    ours = orc.f32_to_b16(vals, name)
    theirs = torch.from_numpy(vals.copy()).to(tdt).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours[finite_or_inf], theirs[finite_or_inf])
    # NaN stays NaN (payloads are not compared)
    back = orc.b16_to_f32(ours[~finite_or_inf], name)
    assert np.isnan(back).all()


def test_rounding_is_nearest_even_on_hand_cases():
    # bf16 keeps 8 significant bits: 1 + 2^-8 is a tie -> 1.0 (even); 1 + 3*2^-8 is a tie -> 1 + 2^-6
    f = np.array([1 + 2.0**-8, 1 + 3 * 2.0**-8, 1 + 2.0**-8 + 2.0**-20, 3.4e38], np.float32)
    got = orc.b16_to_f32(orc.f32_to_b16(f, "bf16"), "bf16")
    assert got.tolist() == [1.0, 1 + 2.0**-6, 1 + 2.0**-7, float("inf")]
    # fp16 keeps 11: 2048 + 1 is a tie -> 2048; 2048 + 3 -> 2052
    f = np.array([2049.0, 2051.0, 65520.0, 65519.0], np.float32)
    got = orc.b16_to_f32(orc.f32_to_b16(f, "fp16"), "fp16")
    assert got.tolist() == [2048.0, 2052.0, float("inf"), 65504.0]


# ----------------------------------------------------------------------------- orders

def brute_send(indices, nle, W):
    T, K = indices.shape
    groups = [[] for _ in range(W)]
    for t in range(T):
        for k in range(K):
            groups[int(indices[t, k]) // nle].append(t * K + k)
    return [len(g) for g in groups], [p for g in groups for p in g]


@pytest.mark.parametrize("W,E,K,T", [(1, 8, 2, 5), (2, 8, 3, 7), (4, 8, 2, 16), (8, 64, 6, 9), (8, 8, 1, 3), (3, 12, 4, 11)])
def test_send_order_matches_brute_force(W, E, K, T):
    nle = E // W
    for _ in range(20):
        idx = np.stack([RNG.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
        counts, order = orc.send_order(idx, nle, W)
        bc, bo = brute_send(idx, nle, W)
        assert counts.tolist() == bc
        assert order.tolist() == bo


def test_send_order_closed_forms():
    W, nle, K = 4, 2, 2
    # every entry to rank 2 -> identity order, all rows counted there
    idx = np.array([[4, 5]] * 6, np.int32)
    counts, order = orc.send_order(idx, nle, W)
    assert counts.tolist() == [0, 0, 12, 0] and order.tolist() == list(range(12))
    # destinations already non-decreasing along the (t,k) stream -> identity
    idx = np.array([[0, 1], [1, 2], [3, 4], [6, 7]], np.int32)
    counts, order = orc.send_order(idx, nle, W)
    assert order.tolist() == list(range(8)) and counts.tolist() == [3, 2, 1, 2]
    # strictly decreasing destinations -> reversed
    idx = np.array([[7, 5], [3, 1]], np.int32)
    counts, order = orc.send_order(idx, nle, W)
    assert order.tolist() == [3, 2, 1, 0]
    # k-minor tie-break: same destination inside one token keeps k order, across tokens t order
    idx = np.array([[1, 0], [0, 1]], np.int32)
    _, order = orc.send_order(idx, 2, 1)
    assert order.tolist() == [0, 1, 2, 3]


def test_dispatch_send_meta_is_closed_form():
    W, E, K, T, H = 4, 16, 3, 9, 8
    idx = np.stack([RNG.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    x = RNG.integers(0, 2**16, size=(T, H), dtype=np.uint64).astype(np.uint16)
    inp = orc.RankInput(x=x, indices=idx, weights=np.ones((T, K), np.float32))
    counts, order, buf, meta = orc.dispatch_send(inp, rank=2, world_size=W, num_local_experts=E // W)
    for p, flat in enumerate(order.tolist()):
        t, k = divmod(flat, K)
        assert meta[p].tolist() == [int(idx[t, k]), 2, t, k, 0]
        assert np.array_equal(buf[p], x[t])
    assert sorted(order.tolist()) == list(range(T * K))
    assert counts.sum() == T * K


def brute_place(meta, nle):
    cnt = [0] * nle
    where = []
    for i in range(meta.shape[0]):
        le = int(meta[i, 0]) % nle
        where.append((le, cnt[le]))
        cnt[le] += 1
    return cnt, where


def test_expert_placement_matches_brute_force():
    for nle, R in [(1, 5), (2, 9), (4, 33), (32, 200), (8, 0)]:
        meta = np.zeros((R, 5), np.int32)
        meta[:, 0] = RNG.integers(0, nle * 3, size=R)
        cnt, local, pos, order = orc.expert_placement(meta, nle)
        bc, where = brute_place(meta, nle)
        assert cnt.tolist() == bc
        assert list(zip(local.tolist(), pos.tolist())) == where
        # order lists rows expert-major, inside an expert in arrival order
        exp = sorted(range(R), key=lambda i: (where[i][0], i))
        assert order.tolist() == exp


def brute_return(meta_rows, W):
    groups = [[] for _ in range(W)]
    for g in range(meta_rows.shape[0]):
        groups[int(meta_rows[g, 1])].append(g)
    return [len(g) for g in groups], [p for g in groups for p in g]


def test_return_order_matches_brute_force():
    for W, R in [(1, 4), (2, 11), (8, 100), (8, 0)]:
        meta = np.zeros((R, 5), np.int32)
        meta[:, 1] = RNG.integers(0, W, size=R)
        counts, order = orc.return_order(meta, W)
        bc, bo = brute_return(meta, W)
        assert counts.tolist() == bc and order.tolist() == bo


def test_exchange_is_slicing_by_counts():
    W = 3
    counts = [np.array(c, np.int64) for c in ([1, 0, 2], [2, 2, 0], [0, 1, 1])]
    bufs, metas = [], []
    for s in range(W):
        n = int(counts[s].sum())
        bufs.append((np.arange(n)[:, None] + 100 * s).astype(np.uint16))
        m = np.zeros((n, 5), np.int32); m[:, 1] = s; m[:, 2] = np.arange(n)
        metas.append(m)
    got = orc.exchange(counts, bufs, metas)
    # rank 0 gets s0[0:1], s1[0:2]; rank 1 gets s1[2:4], s2[0:1]; rank 2 gets s0[1:3], s2[1:2]
    assert got[0][1].ravel().tolist() == [0, 100, 101] and got[0][0].tolist() == [1, 2, 0]
    assert got[1][1].ravel().tolist() == [102, 103, 200] and got[1][0].tolist() == [0, 2, 1]
    assert got[2][1].ravel().tolist() == [1, 2, 201] and got[2][0].tolist() == [2, 0, 1]
    assert got[2][2][:, 1].tolist() == [0, 0, 2]


# ----------------------------------------------------------------------------- simulated expert

@pytest.mark.parametrize("name,tdt", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_expert_scale_matches_torch_expression(name, tdt):
    rows = RNG.integers(0, 2**16, size=(64, 33), dtype=np.uint64).astype(np.uint16)
    t = torch.from_numpy(rows.view(np.int16)).view(tdt)
    for rank in (0, 1, 2, 6, 7):
        want = (t.to(tdt) * (1 + rank)).view(torch.int16).numpy().view(np.uint16)
        got = orc.expert_scale(rows, rank, name, name)
        ok = ~np.isnan(orc.b16_to_f32(want, name))
        assert np.array_equal(got[ok], want[ok])


def test_expert_scale_mixed_dtypes_matches_torch():
    rows = orc.f32_to_b16(RNG.standard_normal((16, 40)).astype(np.float32) * 50, "fp16")
    t = torch.from_numpy(rows.view(np.int16)).view(torch.float16)
    want = (t.to(torch.bfloat16) * 3).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.expert_scale(rows, 2, "fp16", "bf16"), want)


# ----------------------------------------------------------------------------- combine

def torch_accumulate(ret_bits, ret_meta, weights, rows_out, tdt):
    """The reference's own statement of the step, executed by torch."""
    rb = torch.from_numpy(ret_bits.view(np.int16)).view(tdt)
    w = torch.from_numpy(weights)
    y = torch.zeros(rows_out, ret_bits.shape[1], dtype=tdt)
    for i in range(ret_bits.shape[0]):
        t, k = int(ret_meta[i, 2]), int(ret_meta[i, 3])
        y[t] += rb[i].to(torch.float32) * w[t, k].to(torch.float32)
    return y.view(torch.int16).numpy().view(np.uint16)


def random_arrivals(T, K, H, name):
    x = orc.f32_to_b16(RNG.standard_normal((T * K, H)).astype(np.float32), name)
    meta = np.zeros((T * K, 5), np.int32)
    tk = RNG.permutation(T * K)
    meta[:, 2], meta[:, 3] = tk // K, tk % K
    w = RNG.random((T, K), dtype=np.float32)
    return x, meta, w


@pytest.mark.parametrize("name,tdt", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_combine_matches_torch_inplace_add(name, tdt):
    for T, K, H in [(1, 1, 4), (5, 2, 16), (16, 8, 64), (7, 3, 33)]:
        x, meta, w = random_arrivals(T, K, H, name)
        got = orc.combine_recv(x, meta, w, T + 2, name)
        want = torch_accumulate(x, meta, w, T + 2, tdt)
        assert np.array_equal(got, want)


def test_combine_detects_wrong_rounding_and_wrong_order():
    """The check above has teeth: plausible wrong versions give different bits."""
    T, K, H = 32, 8, 128
    x, meta, w = random_arrivals(T, K, H, "bf16")
    right = orc.combine_recv(x, meta, w, T, "bf16")
    # (1) accumulate in float32 and round once
    acc = np.zeros((T, H), np.float32)
    for i in range(x.shape[0]):
        acc[meta[i, 2]] += orc.b16_to_f32(x[i], "bf16") * w[meta[i, 2], meta[i, 3]]
    assert not np.array_equal(orc.f32_to_b16(acc, "bf16"), right)
    # (2) fused multiply-add (single rounding of v*w + y)
    y = np.zeros((T, H), np.uint16)
    for i in range(x.shape[0]):
        t = meta[i, 2]
        f = orc.b16_to_f32(x[i], "bf16").astype(np.float64) * np.float64(w[t, meta[i, 3]]) \
            + orc.b16_to_f32(y[t], "bf16").astype(np.float64)
        y[t] = orc.f32_to_b16(f.astype(np.float32), "bf16")
    assert not np.array_equal(y, right)
    # (3) reversed arrival order
    assert not np.array_equal(orc.combine_recv(x[::-1], meta[::-1], w, T, "bf16"), right)
    # (4) weights transposed in k (wrong operand)
    assert not np.array_equal(orc.combine_recv(x, meta, w[:, ::-1], T, "bf16"), right)


def test_combine_closed_forms():
    H = 64
    v = orc.f32_to_b16(RNG.standard_normal((6, H)).astype(np.float32), "bf16")
    meta = np.zeros((6, 5), np.int32); meta[:, 2] = [3, 0, 5, 1, 4, 2]
    # K = 1, weight 1: y[t] is exactly the arriving row
    y = orc.combine_recv(v, meta, np.ones((6, 1), np.float32), 6, "bf16")
    assert np.array_equal(y[meta[:, 2]], v)
    # K = 1, weight w: y = round(f32(v) * w), one rounding
    w = RNG.random((6, 1), dtype=np.float32)
    y = orc.combine_recv(v, meta, w, 6, "bf16")
    want = orc.f32_to_b16(orc.b16_to_f32(v, "bf16") * w[meta[:, 2]], "bf16")
    assert np.array_equal(y[meta[:, 2]], want)
    # small integers with power-of-two weights: every step is exact, so the sum is the integer sum
    ints = RNG.integers(-8, 9, size=(8, H)).astype(np.float32)
    vb = orc.f32_to_b16(ints, "fp16")
    meta = np.zeros((8, 5), np.int32); meta[:, 3] = np.arange(8)
    w = np.array([[0.5, 1, 2, 0.25, 1, 4, 0.5, 2]], np.float32)
    y = orc.combine_recv(vb, meta, w, 1, "fp16")
    assert np.array_equal(orc.b16_to_f32(y[0], "fp16"), (ints * w[0][:, None]).sum(0))
    # a tie that only per-step rounding resolves this way: 256 + 1 + 1 in bf16 stays 256
    vb = orc.f32_to_b16(np.array([[256.0], [1.0], [1.0]], np.float32), "bf16")
    meta = np.zeros((3, 5), np.int32); meta[:, 3] = [0, 1, 2]
    y = orc.combine_recv(vb, meta, np.ones((1, 3), np.float32), 1, "bf16")
    assert orc.b16_to_f32(y, "bf16")[0, 0] == 256.0
    # ... and in the other order the two ones add first: 1 + 1 + 256 = 258
    y = orc.combine_recv(vb[::-1], meta, np.ones((1, 3), np.float32), 1, "bf16")
    assert orc.b16_to_f32(y, "bf16")[0, 0] == 258.0


def test_combine_accumulates_onto_given_rows():
    x, meta, w = random_arrivals(4, 2, 8, "bf16")
    init = orc.f32_to_b16(RNG.standard_normal((4, 8)).astype(np.float32), "bf16")
    got = orc.combine_recv(x, meta, w, 4, "bf16", y_init=init)
    y = torch.from_numpy(init.view(np.int16).copy()).view(torch.bfloat16)
    rb = torch.from_numpy(x.view(np.int16)).view(torch.bfloat16)
    for i in range(8):
        t, k = int(meta[i, 2]), int(meta[i, 3])
        y[t] += rb[i].float() * torch.tensor(w[t, k])
    assert np.array_equal(got, y.view(torch.int16).numpy().view(np.uint16))


# ----------------------------------------------------------------------------- matrix products

def _b(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("name,tdt", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_gemm_oracle_on_inputs_where_every_summation_order_agrees(name, tdt):
    # small integers: a brute-force integer loop is the answer, whatever the order of the sum
    x = RNG.integers(-2, 3, (7, 24))
    w = RNG.integers(-2, 3, (5, 24))
    want = np.array([[sum(int(x[i, k]) * int(w[j, k]) for k in range(24)) for j in range(5)] for i in range(7)])
    got = orc.expert_gemm(_b(torch.from_numpy(x).to(tdt)), _b(torch.from_numpy(w).to(tdt)), name)
    assert np.array_equal(orc.b16_to_f32(got, name), want.astype(np.float32))
    # a signed permutation as weights moves columns: out[:, j] = sign[j] * x[:, perm[j]] (not its transpose)
    perm, sign = RNG.permutation(24), RNG.choice([-1.0, 1.0], 24)
    pw = np.zeros((24, 24), np.float32)
    pw[np.arange(24), perm] = sign
    rows = RNG.integers(0, 1 << 15, (9, 24), dtype=np.uint16)  # positive finite-or-not patterns
    rows[~np.isfinite(orc.b16_to_f32(rows, name))] = 0x3C00
    got = orc.expert_gemm(rows, _b(torch.from_numpy(pw).to(tdt)), name)
    want = np.where(sign[None, :] < 0, rows[:, perm] ^ 0x8000, rows[:, perm])
    zero = (want & 0x7FFF) == 0
    assert np.array_equal(got[~zero], want[~zero])


@pytest.mark.parametrize("name,tdt", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_linear_oracle_is_the_torch_expression(name, tdt):
    # gemm-rs/reference.py:54-57 on the CPU, on integers (exact in any order) ...
    x = torch.from_numpy(RNG.integers(-3, 4, (11, 40))).to(tdt)
    w = torch.from_numpy(RNG.integers(-3, 4, (6, 40))).to(tdt)
    b = torch.from_numpy(RNG.integers(-9, 10, 6)).to(tdt)
    assert np.array_equal(orc.linear(_b(x), _b(w), _b(b), name), _b(torch.matmul(x, w.T) + b))
    assert np.array_equal(orc.linear(_b(x), _b(w), None, name), _b(torch.matmul(x, w.T)))
    # ... and where the two roundings show: the product is rounded before the bias is added
    u = 2.0 ** -8 if name == "bf16" else 2.0 ** -11
    x = torch.tensor([[1.0, u]], dtype=tdt)
    w = torch.ones(3, 2, dtype=tdt)
    b = torch.full((3,), 2 * u, dtype=tdt)
    want = torch.matmul(x, w.T) + b
    assert float(want[0, 0]) == 1.0 + 2 * u  # (1 + u rounds to 1 first; added unrounded it would reach 1 + 4u)
    assert np.array_equal(orc.linear(_b(x), _b(w), _b(b), name), _b(want))


def test_gemm_bound_holds_for_torch_and_catches_a_dropped_term():
    x = torch.randn(33, 512, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    w = (torch.randn(48, 512, generator=torch.Generator().manual_seed(2)) / 512 ** 0.5).to(torch.bfloat16)
    exact, tol = orc.expert_gemm_bound(_b(x), _b(w), "bf16")
    for got in (orc.expert_gemm(_b(x), _b(w), "bf16"), _b(torch.matmul(x, w.T)),
                _b((x.float() @ w.float().T).to(torch.bfloat16))):
        assert (np.abs(orc.b16_to_f32(got, "bf16").astype(np.float64) - exact) <= tol).all()
    # one input left out of every sum: most results leave the bound
    short = _b((x[:, :-1].float() @ w[:, :-1].float().T).to(torch.bfloat16))
    assert (np.abs(orc.b16_to_f32(short, "bf16").astype(np.float64) - exact) > tol).mean() > 0.5
    # operands swapped (w @ x.T, transposed back) is the same product; a transposed weight is not
    sq = (torch.randn(512, 512, generator=torch.Generator().manual_seed(3)) / 512 ** 0.5).to(torch.bfloat16)
    exact, tol = orc.expert_gemm_bound(_b(x), _b(sq), "bf16")
    wrong = _b((x.float() @ sq.float()).to(torch.bfloat16))
    assert (np.abs(orc.b16_to_f32(wrong, "bf16").astype(np.float64) - exact) > tol).mean() > 0.5


@pytest.mark.parametrize("name,tdt", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_linear_bound_with_a_bias_holds_for_torch_and_catches_a_wrong_bias(name, tdt):
    g = torch.Generator().manual_seed(7)
    x = torch.randn(29, 384, generator=g).to(tdt)
    w = (torch.randn(40, 384, generator=g) / 384 ** 0.5).to(tdt)
    b = torch.randn(40, generator=g).to(tdt)
    exact, tol = orc.linear_bound(_b(x), _b(w), _b(b), name)
    assert np.allclose(exact, x.double().numpy() @ w.double().numpy().T + b.double().numpy()[None, :], rtol=1e-13)
    off = lambda t16: np.abs(orc.b16_to_f32(_b(t16), name).astype(np.float64) - exact)
    # torch's two statements (two roundings), the oracle's restatement of them, and the same sum
    # rounded once (a fused epilogue) all lie inside
    twice = torch.matmul(x, w.T) + b
    once = (x.float() @ w.float().T + b.float()).to(tdt)
    assert (off(twice) <= tol).all() and (off(once) <= tol).all()
    assert (np.abs(orc.b16_to_f32(orc.linear(_b(x), _b(w), _b(b), name), name).astype(np.float64) - exact) <= tol).all()
    # no bias, the bias twice, the bias of the neighbouring column: most results leave the bound
    plain = torch.matmul(x, w.T)
    for wrong in (plain, plain + b + b, plain + torch.roll(b, 1)):
        assert (off(wrong) > tol).mean() > 0.5
    # and the bound without a bias is the product's own
    e0, t0 = orc.linear_bound(_b(x), _b(w), None, name)
    e1, t1 = orc.expert_gemm_bound(_b(x), _b(w), name)
    assert np.array_equal(e0, e1) and np.array_equal(t0, t1)


def test_grouped_linear_is_a_linear_layer_per_expert():
    g = torch.Generator().manual_seed(8)
    counts = np.array([3, 0, 5, 1])
    rows = torch.from_numpy(RNG.integers(-3, 4, (int(counts.sum()), 16))).to(torch.bfloat16)
    w = torch.from_numpy(RNG.integers(-2, 3, (4, 24, 16))).to(torch.bfloat16)
    b = torch.from_numpy(RNG.integers(-5, 6, (4, 24))).to(torch.bfloat16)
    got = orc.grouped_linear(_b(rows), counts, _b(w), _b(b), "bf16")
    start = 0
    for le, c in enumerate(counts):  # small integers: exact in every order, so torch's result is THE result
        want = torch.matmul(rows[start:start + c], w[le].T) + b[le]
        assert np.array_equal(got[start:start + c], _b(want)), le
        start += c
    assert got.shape == (int(counts.sum()), 24)
    assert np.array_equal(orc.grouped_linear(_b(rows), counts, _b(w), None, "bf16")[:3], _b(torch.matmul(rows[:3], w[0].T)))


@pytest.mark.parametrize("name", ["bf16", "fp16"])
def test_combine_bound_holds_and_catches_a_dropped_addend(name):
    tdt = torch.bfloat16 if name == "bf16" else torch.float16
    T, K, H = 6, 8, 96
    g = torch.Generator().manual_seed(9)
    rows16 = torch.randn(T * K, H, generator=g).to(tdt)
    weights = torch.softmax(torch.randn(T, K, generator=g), dim=1).numpy()
    order = RNG.permutation(T * K)  # arrival order of the (token, k) pairs
    meta = np.zeros((T * K, 5), np.int32)
    meta[:, 2], meta[:, 3] = order // K, order % K
    exact_rows = rows16.double().numpy()
    got = orc.combine_recv(_b(rows16), meta, weights, T, name)
    exact, tol = orc.combine_bound(exact_rows, np.zeros_like(exact_rows), meta, weights, T, name)
    want = np.zeros((T, H))
    for i in range(T * K):
        want[meta[i, 2]] += float(weights[meta[i, 2], meta[i, 3]]) * exact_rows[i]
    assert np.allclose(exact, want, rtol=1e-12, atol=1e-300)
    err = np.abs(orc.b16_to_f32(got, name).astype(np.float64) - exact)
    assert (err <= tol).all()
    assert (tol <= 0.05 * np.abs(exact).max()).all()  # (a bound that allowed everything would pin nothing)
    # rows that are only known to within a tolerance: the result of any rows inside it stays inside
    wiggle = 2.0 ** -7 * np.abs(exact_rows)
    moved = torch.from_numpy(exact_rows * (1 + 2.0 ** -7 * RNG.choice([-1.0, 1.0], exact_rows.shape))).to(tdt)
    _, tol_w = orc.combine_bound(exact_rows, wiggle * 1.02 + 2.0 ** -8 * np.abs(exact_rows), meta, weights, T, name)
    err_w = np.abs(orc.b16_to_f32(orc.combine_recv(_b(moved), meta, weights, T, name), name).astype(np.float64) - exact)
    assert (err_w <= tol_w).all()
    # one addend of every token left out, and the weights of two k swapped: outside the bound
    keep = np.ones(T * K, bool)
    keep[[int(np.nonzero(meta[:, 2] == t)[0][3]) for t in range(T)]] = False
    short = orc.combine_recv(_b(rows16)[keep], meta[keep], weights, T, name)
    assert (np.abs(orc.b16_to_f32(short, name).astype(np.float64) - exact) > tol).mean() > 0.5
    swapped = orc.combine_recv(_b(rows16), meta, weights[:, ::-1].copy(), T, name)
    assert (np.abs(orc.b16_to_f32(swapped, name).astype(np.float64) - exact) > tol).mean() > 0.5
