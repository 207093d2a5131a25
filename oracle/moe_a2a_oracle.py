"""CPU oracle for the MoE dispatch/combine path — TEST INFRASTRUCTURE ONLY.

This file is the checker, never the product: only `tests/`, the smoke check in
`__graft_entry__.py` and the `cpu_baseline` leg of `bench.py` may import it.
The shipped path (`amd_distributed_2025_amd`) must not, and does not.

It restates, in numpy, what `all2all/reference.py` of the reference computes
for all `world_size` ranks of one job at once, with the three
`all_to_all_single` exchanges replaced by slicing and concatenation inside one
process. Integer work (orders, counts, meta rows, placements) uses library
routines whose meaning is fixed — `np.argsort(kind="stable")`, `np.bincount`,
`np.cumsum` — and 16-bit floating point is handled on raw bit patterns with
explicit round-to-nearest-even, so nothing here depends on torch.

What pins each function (see tests/test_oracle_pins.py):
  * `send_order` / `expert_placement` / `return_order` — brute-force Python
    loops on small inputs, closed forms for sorted and single-destination
    inputs, and the permutation / count invariants;
  * `f32_to_b16` / `b16_to_f32` — exhaustive comparison with torch's own
    conversions for all 65536 bit patterns and for random float32 values;
  * `combine_recv` — torch's in-place `y16[t] += f32` on the same addends
    (the library routine the reference calls), K=1 and unit-weight closed
    forms, and integer-valued inputs whose sums are exact;
  * `run_world` — the row-by-row torch implementation in
    `oracle/rowwise_torch.py`, written separately, on every committed case.
Parity of these functions with the reference is pinned by those checks and not
by an execution of the reference itself (it ships no vectors of its own).

Rows are 2-byte elements handled as `uint16` bit patterns; `dtype` is "bf16"
or "fp16".
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Sequence

import numpy as np

META_DIM = 5  # all2all/reference.py:56  {global_exp, src_rank, src_token, src_k, pad}

# ----------------------------------------------------------------------------- 16-bit floats


def b16_to_f32(bits: np.ndarray, dtype: str) -> np.ndarray:
    """Widen fp16/bf16 bit patterns to float32 (exact)."""
    bits = np.asarray(bits, dtype=np.uint16)
    if dtype == "bf16":
        return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)
    if dtype == "fp16":
        return bits.view(np.float16).astype(np.float32)
    raise ValueError(dtype)


def f32_to_b16(values: np.ndarray, dtype: str) -> np.ndarray:
    """Round float32 to fp16/bf16 bit patterns, nearest-even — the rounding torch
    applies when a float32 result is stored into a 16-bit tensor
    (the `+=` at all2all/reference.py:232, the product at :262)."""
    values = np.ascontiguousarray(values, dtype=np.float32)
    if dtype == "bf16":
        u = values.view(np.uint32)
        lsb = (u >> np.uint32(16)) & np.uint32(1)
        # uint32 wrap-around can only happen for NaN patterns, which are overwritten below
        rounded = ((u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)).astype(np.uint16)
        nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
        if nan.any():
            rounded[nan] = 0x7FC0
        return rounded
    if dtype == "fp16":
        with np.errstate(over="ignore"):
            return values.astype(np.float16).view(np.uint16)
    raise ValueError(dtype)


# ----------------------------------------------------------------------------- data holders


@dataclass
class RankInput:
    """Inputs of one rank (reference: RankTestData, all2all/reference.py:21-51)."""

    x: np.ndarray        # uint16 [T, H] bit patterns of the in_dtype rows
    indices: np.ndarray  # int32  [T, K] global expert ids
    weights: np.ndarray  # float32 [T, K]

    @property
    def num_tokens(self) -> int:
        return int(self.indices.shape[0])


@dataclass
class RankTrace:
    """Everything one rank produces along the path, for parity checks."""

    send_counts: np.ndarray = None      # int64 [W]
    send_order: np.ndarray = None       # flat (t*K+k) index of each sent row
    send_buf: np.ndarray = None         # uint16 [S, H]
    send_meta: np.ndarray = None        # int32 [S, 5]
    recv_counts: np.ndarray = None      # int64 [W]
    recv_buf: np.ndarray = None         # uint16 [R, H]
    recv_meta: np.ndarray = None        # int32 [R, 5]
    expert_num_tokens: np.ndarray = None  # int32 [nle]
    expert_rows: np.ndarray = None      # uint16 [R, H]: valid rows, expert-major (le, j)
    expert_meta_rows: np.ndarray = None  # int32 [R, 5], same order
    expert_y_rows: np.ndarray = None    # uint16 [R, H] after the simulated expert
    back_counts: np.ndarray = None      # int64 [W] rows returned to each origin rank
    back_buf: np.ndarray = None         # uint16 [R, H]
    back_meta: np.ndarray = None        # int32 [R, 5]
    ret_counts: np.ndarray = None       # int64 [W] rows arriving back from each owner
    ret_buf: np.ndarray = None          # uint16 [S, H]
    ret_meta: np.ndarray = None         # int32 [S, 5]
    y: np.ndarray = None                # uint16 [T, H] result rows (out_dtype bits)
    extra: dict = field(default_factory=dict)


# ----------------------------------------------------------------------------- dispatch


def send_order(indices: np.ndarray, num_local_experts: int, world_size: int):
    """Order in which one rank's (token, k) entries are sent.

    all2all/reference.py:79-86 appends entry (t, k) to the list of its
    destination `e // num_local_experts` while walking t then k; line 93
    concatenates the lists in rank order. That is a stable sort of the t-major,
    k-minor stream by destination.

    Returns (send_counts int64[W], order int64[S]) with order[p] = t*K + k.
    """
    flat = np.asarray(indices, dtype=np.int64).reshape(-1)
    dst = flat // num_local_experts
    order = np.argsort(dst, kind="stable")
    counts = np.bincount(dst, minlength=world_size).astype(np.int64)
    return counts, order


def dispatch_send(inp: RankInput, rank: int, world_size: int, num_local_experts: int):
    """send_counts, send_buf, send_meta of one rank (all2all/reference.py:74-102)."""
    T, K = inp.indices.shape
    counts, order = send_order(inp.indices, num_local_experts, world_size)
    t = order // K
    k = order % K
    e = inp.indices.reshape(-1)[order]
    meta = np.stack(
        [e, np.full_like(e, rank), t, k, np.zeros_like(e)], axis=1
    ).astype(np.int32).reshape(-1, META_DIM)
    buf = inp.x[t] if order.size else np.zeros((0, inp.x.shape[1]), np.uint16)
    return counts, order, buf, meta


def exchange(counts: Sequence[np.ndarray], bufs: Sequence[np.ndarray], metas: Sequence[np.ndarray]):
    """What the three all_to_all_single calls deliver (all2all/reference.py:91,107-119
    and :185,210-222): rank r receives, from s = 0..W-1 in that order, the
    segment of s's send buffer that s addressed to r."""
    W = len(counts)
    offs = [np.concatenate([[0], np.cumsum(c)]) for c in counts]
    out = []
    for r in range(W):
        rc = np.array([counts[s][r] for s in range(W)], dtype=np.int64)
        rb = np.concatenate([bufs[s][offs[s][r]:offs[s][r + 1]] for s in range(W)], axis=0)
        rm = np.concatenate([metas[s][offs[s][r]:offs[s][r + 1]] for s in range(W)], axis=0)
        out.append((rc, rb, rm))
    return out


def expert_placement(recv_meta: np.ndarray, num_local_experts: int):
    """Where each received row lands in the expert-major buffers.

    all2all/reference.py:140-146 walks the received rows in order, computes
    `local = meta[0] % num_local_experts` and appends to that expert. That is a
    stable partition of the received stream by local expert.

    Returns (expert_num_tokens int32[nle], local int64[R], pos int64[R],
    order int64[R]) where row i goes to (local[i], pos[i]) and `order` lists
    received-row indices in expert-major (le, j) order.
    """
    local = np.asarray(recv_meta[:, 0], dtype=np.int64) % num_local_experts
    order = np.argsort(local, kind="stable")
    counts = np.bincount(local, minlength=num_local_experts).astype(np.int32)
    starts = np.concatenate([[0], np.cumsum(counts)])[:-1]
    pos = np.empty(local.shape[0], dtype=np.int64)
    pos[order] = np.arange(local.shape[0]) - starts[local[order]]
    return counts, local, pos, order


def expert_scale(rows: np.ndarray, rank: int, in_dtype: str, out_dtype: str) -> np.ndarray:
    """`expert_x.to(out_dtype) * (1 + rank)` (all2all/reference.py:262): a 16-bit
    tensor times a Python int is evaluated in float32 and rounded once."""
    as_out = b16_to_f32(f32_to_b16(b16_to_f32(rows, in_dtype), out_dtype), out_dtype)
    return f32_to_b16(as_out * np.float32(1 + rank), out_dtype)


def expert_gemm(rows: np.ndarray, weights: np.ndarray, dtype: str) -> np.ndarray:
    """One expert's rows through a linear layer, `rows @ weights.T`, where a model
    has its expert and all2all/reference.py:262 has the stand-in: 16-bit operands
    (`rows` [n, H], `weights` [H_out, H_in] as bit patterns), products and sums in
    float32, one rounding to the 16-bit type. The order of a float32 sum is not
    fixed by this statement; `expert_gemm_bound` gives what every order satisfies."""
    acc = b16_to_f32(rows, dtype) @ b16_to_f32(weights, dtype).T
    return f32_to_b16(acc.astype(np.float32), dtype)


def expert_gemm_bound(rows: np.ndarray, weights: np.ndarray, dtype: str):
    """(exact, tol): the float64 value of `rows @ weights.T` and the distance from it
    that a float32-accumulated, once-rounded 16-bit result can have in any summation
    order: K terms summed in float32 are off by at most K * 2^-24 * sum|x||w|
    (products of two 16-bit values are exact in float32), and the final rounding
    by half a unit in the last place (2^-8 relative for bf16, 2^-11 for fp16; the
    2^-24 / 2^-133 floor covers subnormal results)."""
    x = b16_to_f32(rows, dtype).astype(np.float64)
    w = b16_to_f32(weights, dtype).astype(np.float64)
    exact = x @ w.T
    mass = np.abs(x) @ np.abs(w).T
    u16, floor = (2.0 ** -8, 2.0 ** -133) if dtype == "bf16" else (2.0 ** -11, 2.0 ** -24)
    sum_err = x.shape[1] * 2.0 ** -24 * mass
    return exact, u16 * (np.abs(exact) + sum_err) + sum_err + floor


def linear(inp: np.ndarray, weight: np.ndarray, bias, dtype: str) -> np.ndarray:
    """`torch.matmul(input, weight.T)` then `output + bias` on 16-bit tensors
    (gemm-rs/reference.py:54-57): the product is rounded to the 16-bit type, the
    bias is added to the rounded value in float32 and the sum rounded again."""
    out = expert_gemm(inp, weight, dtype)
    if bias is None:
        return out
    return f32_to_b16(b16_to_f32(out, dtype) + b16_to_f32(bias, dtype)[None, :], dtype)


def linear_bound(inp: np.ndarray, weight: np.ndarray, bias, dtype: str):
    """(exact, tol) for `linear`: the float64 value of input @ weight.T + bias and how far
    from it the twice-rounded result can lie for any float32 summation order."""
    exact, tol = expert_gemm_bound(inp, weight, dtype)
    if bias is None:
        return exact, tol
    u16 = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    total = exact + b16_to_f32(bias, dtype).astype(np.float64)[None, :]
    return total, tol + (u16 + 2.0 ** -23) * (np.abs(total) + tol)


# ----------------------------------------------------------------------------- combine


def return_order(expert_meta_rows: np.ndarray, world_size: int):
    """Order in which an owner rank returns its expert-major rows.

    all2all/reference.py:170-179 walks local experts ascending and rows j
    ascending, bucketing by `meta[1]` (the origin rank); the buckets are
    concatenated in rank order (:187-199). A stable partition by origin rank of
    the (le, j) stream, which is the order `expert_meta_rows` is given in.
    """
    dst = np.asarray(expert_meta_rows[:, 1], dtype=np.int64)
    order = np.argsort(dst, kind="stable")
    counts = np.bincount(dst, minlength=world_size).astype(np.int64)
    return counts, order


def combine_recv(
    ret_buf: np.ndarray,
    ret_meta: np.ndarray,
    weights: np.ndarray,
    num_rows_out: int,
    dtype: str,
    y_init: np.ndarray | None = None,
) -> np.ndarray:
    """Weighted accumulation into token order (all2all/reference.py:227-232).

    For i in arrival order: `y[t] += row_i.float() * w[t, k]` with y a 16-bit
    tensor, i.e. per element p = f32(v)*w, a = f32(y)+p, y = round16(a) after
    every addend. Tokens are independent, so the a-th arrival of every token is
    applied in one vector step; per token the arrival order is kept.
    """
    H = ret_buf.shape[1]
    y = np.zeros((num_rows_out, H), np.uint16) if y_init is None else y_init.copy()
    if ret_meta.shape[0] == 0:
        return y
    tok = ret_meta[:, 2].astype(np.int64)
    kk = ret_meta[:, 3].astype(np.int64)
    by_tok = np.argsort(tok, kind="stable")  # arrival order kept inside a token
    tok_sorted = tok[by_tok]
    first = np.concatenate([[True], tok_sorted[1:] != tok_sorted[:-1]])
    start_of = np.maximum.accumulate(np.where(first, np.arange(tok.size), 0))
    nth = np.arange(tok.size) - start_of  # 0 for a token's first arrival, 1 for the next...
    w_all = np.asarray(weights, dtype=np.float32)
    for a in range(int(nth.max()) + 1):
        rows = by_tok[nth == a]
        t = tok[rows]
        w = w_all[t, kk[rows]].astype(np.float32)[:, None]
        p = b16_to_f32(ret_buf[rows], dtype) * w           # float32 multiply, rounded
        acc = b16_to_f32(y[t], dtype) + p                  # float32 add, rounded
        y[t] = f32_to_b16(acc, dtype)
    return y


# ----------------------------------------------------------------------------- whole job


def grouped_linear(rows: np.ndarray, counts: np.ndarray, weights: np.ndarray, bias, dtype: str) -> np.ndarray:
    """A linear layer per local expert over the compact expert-major rows: the rows of expert le
    (`counts[le]` of them, experts back to back) go through `linear(rows, weights[le], bias[le])`.
    `weights` is [nle, out_dim, in_dim], `bias` [nle, out_dim] or None, as bit patterns."""
    out = np.empty((rows.shape[0], weights.shape[1]), np.uint16)
    g = 0
    for le, n in enumerate(int(c) for c in counts):
        out[g:g + n] = linear(rows[g:g + n], weights[le], None if bias is None else bias[le], dtype)
        g += n
    return out


def combine_bound(ret_exact: np.ndarray, ret_tol: np.ndarray, ret_meta: np.ndarray, weights: np.ndarray,
                  num_rows_out: int, dtype: str):
    """(exact, tol) for `combine_recv` when the arriving rows are only known to lie within
    `ret_tol` of `ret_exact` (float64, e.g. from `linear_bound`): the float64 value of
    sum_k w[t, k] * row and how far from it the 16-bit result of the per-addend-rounded
    accumulation can lie. Per addend: the row's own distance times |w|, a half unit of the 16-bit
    type on the value the row was rounded to before it was sent, the float32 product and sum
    (2^-23 of the running magnitude) and the rounding of the accumulator (a half unit of the
    running magnitude). The running magnitude is bounded by the sum of |w||row| so far plus the
    error so far."""
    u16, floor = (2.0 ** -8, 2.0 ** -133) if dtype == "bf16" else (2.0 ** -11, 2.0 ** -24)
    H = ret_exact.shape[1]
    exact = np.zeros((num_rows_out, H))
    mass = np.zeros((num_rows_out, H))
    tol = np.zeros((num_rows_out, H))
    w_all = np.asarray(weights, dtype=np.float64)
    for i in range(ret_meta.shape[0]):  # arrival order
        t, k = int(ret_meta[i, 2]), int(ret_meta[i, 3])
        w = abs(w_all[t, k])
        exact[t] += w_all[t, k] * ret_exact[i]
        mass[t] += w * np.abs(ret_exact[i])
        tol[t] += w * ret_tol[i]
        tol[t] += (u16 + 2.0 ** -22) * (mass[t] + tol[t]) + floor
    return exact, tol


def run_world(
    inputs: List[RankInput],
    num_experts: int,
    max_num_tokens: int,
    in_dtype: str = "bf16",
    out_dtype: str = "bf16",
    expert=None,
) -> List[RankTrace]:
    """`ref_kernel` (all2all/reference.py:256-272) for every rank of one job.

    Returns one RankTrace per rank. `y` has `num_tokens` rows (the reference
    returns `y[:num_tokens]`).

    `expert(rank, rows, counts)` stands where the reference has its simulated expert
    (reference.py:262): it gets the rank's compact expert-major rows ([R, H] bit patterns of
    `in_dtype`, the rows of local expert 0 first) and the rows per local expert, and returns
    [R, H] bit patterns of `out_dtype`. None is the reference's `x.to(out_dtype) * (1 + rank)`."""
    W = len(inputs)
    nle = num_experts // W
    max_recv = max_num_tokens * W
    tr = [RankTrace() for _ in range(W)]

    for r, inp in enumerate(inputs):
        c, o, b, m = dispatch_send(inp, r, W, nle)
        tr[r].send_counts, tr[r].send_order, tr[r].send_buf, tr[r].send_meta = c, o, b, m

    got = exchange([t.send_counts for t in tr], [t.send_buf for t in tr], [t.send_meta for t in tr])
    for r in range(W):
        tr[r].recv_counts, tr[r].recv_buf, tr[r].recv_meta = got[r]
        cnt, local, pos, order = expert_placement(tr[r].recv_meta, nle)
        if cnt.size and int(cnt.max(initial=0)) > max_recv:
            raise OverflowError("expert capacity exceeded (reference would index out of range)")
        tr[r].expert_num_tokens = cnt
        tr[r].expert_rows = tr[r].recv_buf[order]
        tr[r].expert_meta_rows = tr[r].recv_meta[order]
        tr[r].extra["local"], tr[r].extra["pos"] = local, pos
        if expert is None:
            tr[r].expert_y_rows = expert_scale(tr[r].expert_rows, r, in_dtype, out_dtype)
        else:
            tr[r].expert_y_rows = np.ascontiguousarray(expert(r, tr[r].expert_rows, cnt), dtype=np.uint16)
            if tr[r].expert_y_rows.shape != tr[r].expert_rows.shape:
                raise ValueError("the expert must return one row of hidden_dim per row it was given")
        bc, border = return_order(tr[r].expert_meta_rows, W)
        tr[r].back_counts = bc
        tr[r].back_buf = tr[r].expert_y_rows[border]
        tr[r].back_meta = tr[r].expert_meta_rows[border]

    got = exchange([t.back_counts for t in tr], [t.back_buf for t in tr], [t.back_meta for t in tr])
    for r, inp in enumerate(inputs):
        tr[r].ret_counts, tr[r].ret_buf, tr[r].ret_meta = got[r]
        y = combine_recv(tr[r].ret_buf, tr[r].ret_meta, inp.weights, max_num_tokens, out_dtype)
        tr[r].y = y[: inp.num_tokens]
    return tr


def padded_expert_buffers(trace: RankTrace, num_local_experts: int, max_recv: int):
    """Expand the compact expert-major rows to the reference's padded layout
    `[nle, max_recv, H]` / `[nle, max_recv, 5]` (all2all/reference.py:127-136),
    zero-filled where the reference leaves memory uninitialised."""
    H = trace.expert_rows.shape[1]
    ex = np.zeros((num_local_experts, max_recv, H), np.uint16)
    em = np.zeros((num_local_experts, max_recv, META_DIM), np.int32)
    g = 0
    for le in range(num_local_experts):
        n = int(trace.expert_num_tokens[le])
        ex[le, :n] = trace.expert_rows[g:g + n]
        em[le, :n] = trace.expert_meta_rows[g:g + n]
        g += n
    return ex, em
