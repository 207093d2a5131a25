"""Row-by-row torch-CPU statement of the path — TEST INFRASTRUCTURE ONLY.

Second, independent statement of what `all2all/reference.py` computes, used
(a) to cross-check the vectorised numpy oracle and (b) as the timed CPU
baseline of `bench.py`: it keeps the reference's granularity of work — one
Python-level step per (token, k) entry or per row, one `.item()` per scalar
read, one tensor row copy or in-place `+=` per row — so its run time stands
for the reference's CPU path. The arithmetic is torch's own (`y16[t] += f32`,
`x16 * int`), which is what the reference calls.

Only `tests/`, the smoke check and the `cpu_baseline` leg of `bench.py` import
this file; the shipped package never does.

All W ranks of a job are stepped inside one process; the exchanges
(all2all/reference.py:91,107-119,185,210-222) are slices of the senders'
buffers concatenated in sender order.
"""
from __future__ import annotations

from typing import List, Tuple

import torch

META_DIM = 5  # all2all/reference.py:56


def send_side(x: torch.Tensor, indices: torch.Tensor, rank: int, world_size: int, nle: int):
    """Per-destination grouping of one rank's entries (all2all/reference.py:74-102)."""
    rows_for = [[] for _ in range(world_size)]
    meta_for = [[] for _ in range(world_size)]
    t = 0
    for experts in indices.tolist():
        k = 0
        for e in experts:
            owner = e // nle
            rows_for[owner].append(t)
            meta_for[owner] += [e, rank, t, k, 0]
            k += 1
        t += 1
    counts = torch.tensor([len(r) for r in rows_for], dtype=torch.long)
    buf = torch.cat([x[r] for r in rows_for], dim=0)
    flat_meta = [v for m in meta_for for v in m]
    meta = torch.tensor(flat_meta, dtype=torch.int32).view(-1, META_DIM)
    return counts, buf, meta


def deliver(counts: List[torch.Tensor], bufs: List[torch.Tensor], metas: List[torch.Tensor], dst: int):
    """Rows and meta that rank `dst` receives: sender 0's segment first."""
    W = len(counts)
    rc, rb, rm = [], [], []
    for s in range(W):
        c = counts[s].tolist()
        lo = sum(c[:dst])
        hi = lo + c[dst]
        rc.append(c[dst])
        rb.append(bufs[s][lo:hi])
        rm.append(metas[s][lo:hi])
    return torch.tensor(rc, dtype=torch.long), torch.cat(rb, dim=0), torch.cat(rm, dim=0)


def place_rows(recv_buf: torch.Tensor, recv_meta: torch.Tensor, nle: int, max_recv: int):
    """Received stream -> padded expert-major buffers (all2all/reference.py:123-146)."""
    H = recv_buf.shape[1]
    n_per = torch.zeros(nle, dtype=torch.int32)
    ex = torch.empty((nle, max_recv, H), dtype=recv_buf.dtype)
    em = torch.empty((nle, max_recv, META_DIM), dtype=torch.int32)
    for i in range(recv_buf.shape[0]):
        le = int(recv_meta[i, 0].item()) % nle
        ex[le, n_per[le]] = recv_buf[i]
        em[le, n_per[le]] = recv_meta[i]
        n_per[le] += 1
    return n_per, ex, em


def simulated_expert(expert_x: torch.Tensor, rank: int, out_dtype: torch.dtype) -> torch.Tensor:
    """all2all/reference.py:262, over the whole padded buffer as the reference does."""
    return expert_x.to(out_dtype) * (1 + rank)


def return_side(expert_y: torch.Tensor, expert_meta: torch.Tensor, n_per: torch.Tensor, world_size: int):
    """Expert-major rows -> per-origin-rank groups (all2all/reference.py:163-199)."""
    H = expert_y.shape[2]
    rows_for = [[] for _ in range(world_size)]
    meta_for = [[] for _ in range(world_size)]
    for le in range(expert_y.shape[0]):
        for j in range(int(n_per[le].item())):
            m = expert_meta[le, j]
            origin = int(m[1].item())
            rows_for[origin].append(expert_y[le, j].unsqueeze(0))
            meta_for[origin] += m.tolist()
    counts = torch.tensor([len(r) for r in rows_for], dtype=torch.long)
    parts = [torch.cat(r, dim=0) if r else torch.empty((0, H), dtype=expert_y.dtype) for r in rows_for]
    buf = torch.cat(parts, dim=0)
    meta = torch.tensor([v for m in meta_for for v in m], dtype=torch.int32).view(-1, META_DIM)
    return counts, buf, meta


def accumulate(out_tokens: torch.Tensor, weights: torch.Tensor, recv_buf: torch.Tensor, recv_meta: torch.Tensor):
    """`out[t] += row.float() * w[t, k]` per arriving row (all2all/reference.py:227-232)."""
    for i in range(recv_buf.shape[0]):
        t = int(recv_meta[i, 2].item())
        k = int(recv_meta[i, 3].item())
        _origin = int(recv_meta[i, 1].item())
        w = weights[t, k].to(torch.float32)
        out_tokens[t] += recv_buf[i].to(torch.float32) * w
    return out_tokens


def run_world_rowwise(
    xs: List[torch.Tensor],
    indices: List[torch.Tensor],
    weights: List[torch.Tensor],
    num_experts: int,
    max_num_tokens: int,
    out_dtype: torch.dtype,
    keep: bool = True,
) -> List[dict]:
    """All ranks of one job, phase by phase. Returns one dict per rank with the
    same intermediate names as the numpy oracle's RankTrace (torch tensors;
    expert buffers in the padded layout)."""
    W = len(xs)
    nle = num_experts // W
    max_recv = max_num_tokens * W
    H = xs[0].shape[1]
    out = [dict() for _ in range(W)]

    sent = [send_side(xs[r], indices[r], r, W, nle) for r in range(W)]
    for r in range(W):
        out[r]["send_counts"], out[r]["send_buf"], out[r]["send_meta"] = sent[r]

    back = []
    for r in range(W):
        rc, rb, rm = deliver([s[0] for s in sent], [s[1] for s in sent], [s[2] for s in sent], r)
        n_per, ex, em = place_rows(rb, rm, nle, max_recv)
        ey = simulated_expert(ex, r, out_dtype)
        bc, bb, bm = return_side(ey, em, n_per, W)
        back.append((bc, bb, bm))
        out[r].update(recv_counts=rc, recv_buf=rb, recv_meta=rm, expert_num_tokens=n_per,
                      back_counts=bc, back_buf=bb, back_meta=bm)
        if keep:
            out[r].update(expert_x=ex, expert_meta=em, expert_y=ey)

    for r in range(W):
        rc, rb, rm = deliver([b[0] for b in back], [b[1] for b in back], [b[2] for b in back], r)
        y = torch.zeros(max_num_tokens, H, dtype=out_dtype)
        accumulate(y, weights[r], rb, rm)
        out[r].update(ret_counts=rc, ret_buf=rb, ret_meta=rm, y=y[: xs[r].shape[0]])
    return out
