"""Host side of the MoE dispatch/combine path.

`HIPAllToAll` keeps the surface of the reference's `PyTorchAllToAll`
(all2all/reference.py:55-234): `dispatch(dp_x, indices)` returns
`(expert_num_tokens, expert_x, expert_meta)` in the reference's layouts and
`combine(out_tokens, weights, expert_meta, expert_y, expert_num_tokens)`
accumulates into `out_tokens`. Each of the two is split into its send half and
its receive half (`dispatch_send`/`dispatch_recv`, `combine_send`/
`combine_recv`), because the exchange between the halves is not part of this
library: an `exchange` object supplies it. `LocalWorld` is the one-GPU
stand-in — it steps all ranks of a job in lockstep on one device and moves the
segments with device copies.

All device work goes through the C ABI in `libmoe_a2a.so`; torch only owns
memory and streams. Buffers live in a per-object workspace allocated once, so
the tensors returned by `dispatch` are views that stay valid until the next
`dispatch` on the same object.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib
from .task import MoEConfig, RankTestData, dtype_name

META_DIM = 5
_DT = {"fp16": _lib.F16, "bf16": _lib.BF16}


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream(device) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _need(t: torch.Tensor, dtype: torch.dtype, device, what: str) -> torch.Tensor:
    if t.dtype != dtype:
        raise TypeError(f"{what}: expected {dtype}, got {t.dtype}")
    if t.device != device:
        raise ValueError(f"{what}: expected device {device}, got {t.device}")
    if not t.is_contiguous():
        raise ValueError(f"{what}: must be contiguous")
    return t


class HIPAllToAll:
    META_DIM = META_DIM  # global_exp, src_rank, src_token, src_k, pad

    def __init__(self, cfg: MoEConfig, rank: int, world_size: int, exchange=None, device=None,
                 reuse_placement: bool = True):
        if cfg.num_experts % world_size:
            raise ValueError("num_experts must be a multiple of world_size")
        self.cfg = cfg
        self.rank = rank
        self.world_size = world_size
        self.num_local_experts = cfg.num_experts // world_size
        self.max_recv = cfg.max_num_tokens * world_size
        self.exchange = exchange
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        if self.device.type != "cuda":
            raise _lib.MoeA2AError("HIPAllToAll needs a GPU device; this path has no CPU fallback")
        _lib.load()
        self.shape = _lib.Shape(world_size, rank, cfg.num_experts, cfg.experts_per_token,
                                cfg.hidden_dim, cfg.max_num_tokens)
        self._shape_ref = C.byref(self.shape)
        # rows this rank can receive: every peer may route min(K, nle) entries of each token here
        self.max_rows_in = self.max_recv * min(cfg.experts_per_token, self.num_local_experts)
        self.max_rows_out = cfg.max_num_tokens * cfg.experts_per_token
        self._ws = {}
        # dispatch_recv leaves a plan of where combine_send will put every row; combine_send uses
        # it when it is handed the very tensors that dispatch_recv returned
        self.reuse_placement = reuse_placement
        self._planned_for = None

    # ------------------------------------------------------------------ workspace

    def _buf(self, name: str, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        t = self._ws.get(name)
        if t is None or tuple(t.shape) != tuple(shape) or t.dtype != dtype:
            t = torch.empty(tuple(shape), dtype=dtype, device=self.device)
            self._ws[name] = t
        return t

    def inbound_buffers(self, phase: str):
        """Where an exchange should deliver this rank's incoming rows.
        phase "dispatch": (recv_counts[W], recv_buf[max_rows_in,H], recv_meta[max_rows_in,5]);
        phase "combine": the same with max_rows_out rows of out_dtype."""
        H, W = self.cfg.hidden_dim, self.world_size
        if phase == "dispatch":
            return (self._buf("recv_counts", (W,), torch.int32),
                    self._buf("recv_buf", (self.max_rows_in, H), self.cfg.in_dtype),
                    self._buf("recv_meta", (self.max_rows_in, META_DIM), torch.int32))
        return (self._buf("ret_counts", (W,), torch.int32),
                self._buf("ret_buf", (self.max_rows_out, H), self.cfg.out_dtype),
                self._buf("ret_meta", (self.max_rows_out, META_DIM), torch.int32))

    # ------------------------------------------------------------------ halves

    def dispatch_send(self, dp_x: torch.Tensor, indices: torch.Tensor, want_slots: bool = False):
        """Group this rank's (token, k) entries by destination rank.
        Returns (send_counts int32[W], send_buf [T*K,H], send_meta [T*K,5])
        (+ send_slot int32[T*K] when `want_slots`)."""
        cfg = self.cfg
        T, K = indices.shape
        if K != cfg.experts_per_token or dp_x.shape != (T, cfg.hidden_dim):
            raise ValueError("dispatch: shapes of dp_x / indices do not match the config")
        _need(dp_x, cfg.in_dtype, self.device, "dp_x")
        _need(indices, torch.int32, self.device, "indices")
        S = T * K
        counts = self._buf("send_counts", (self.world_size,), torch.int32)
        buf = self._buf("send_buf", (self.max_rows_out, cfg.hidden_dim), cfg.in_dtype)
        meta = self._buf("send_meta", (self.max_rows_out, META_DIM), torch.int32)
        slots = self._buf("send_slot", (self.max_rows_out,), torch.int32) if want_slots else None
        _lib.call("moe_a2a_dispatch_send", self._shape_ref, _ptr(dp_x), _ptr(indices), T,
                  _ptr(buf), _ptr(meta), _ptr(counts), _ptr(slots), _stream(self.device))
        out = (counts, buf[:S], meta[:S])
        return out + (slots[:S],) if want_slots else out

    def plan_send(self, indices: torch.Tensor):
        """Counts, offsets and index maps of the send order, without moving rows.
        Returns (rank_counts[W], rank_offsets[W+1], expert_counts[E], dst_slot[T*K], src_entry[T*K])."""
        cfg = self.cfg
        T, K = indices.shape
        if K != cfg.experts_per_token:
            raise ValueError("plan_send: indices do not match the config")
        _need(indices, torch.int32, self.device, "indices")
        S = T * K
        rc = self._buf("plan_rank_counts", (self.world_size,), torch.int32)
        ro = self._buf("plan_rank_offsets", (self.world_size + 1,), torch.int32)
        ec = self._buf("plan_expert_counts", (cfg.num_experts,), torch.int32)
        ds = self._buf("plan_dst_slot", (self.max_rows_out,), torch.int32)
        se = self._buf("plan_src_entry", (self.max_rows_out,), torch.int32)
        _lib.call("moe_a2a_plan_send", self._shape_ref, _ptr(indices), T, _ptr(rc), _ptr(ro), _ptr(ec),
                  _ptr(ds), _ptr(se), _stream(self.device))
        return rc, ro, ec, ds[:S], se[:S]

    def dispatch_recv(self, recv_counts, recv_buf, recv_meta, rows_hint: Optional[int] = None):
        """Received stream -> (expert_num_tokens[nle], expert_x[nle,max_recv,H],
        expert_meta[nle,max_recv,5]); rows past expert_num_tokens[le] are not written."""
        cfg = self.cfg
        _need(recv_counts, torch.int32, self.device, "recv_counts")
        _need(recv_buf, cfg.in_dtype, self.device, "recv_buf")
        _need(recv_meta, torch.int32, self.device, "recv_meta")
        capacity = min(recv_buf.shape[0], recv_meta.shape[0])
        hint = min(capacity, self.max_rows_in if rows_hint is None else int(rows_hint))
        nle = self.num_local_experts
        num = self._buf("expert_num_tokens", (nle,), torch.int32)
        ex = self._buf("expert_x", (nle, self.max_recv, cfg.hidden_dim), cfg.in_dtype)
        em = self._buf("expert_meta", (nle, self.max_recv, META_DIM), torch.int32)
        plan = self._buf("send_back_plan", (2 * cfg.num_experts,), torch.int32) if self.reuse_placement else None
        _lib.call("moe_a2a_dispatch_recv", self._shape_ref, _ptr(recv_buf), _ptr(recv_meta),
                  _ptr(recv_counts), hint, capacity, _ptr(num), _ptr(ex), _ptr(em), _ptr(plan),
                  _stream(self.device))
        self._planned_for = None if plan is None else (em.data_ptr(), num.data_ptr())
        self._rows_in_hint = hint
        return num, ex, em

    def expert_scale(self, expert_x, expert_num_tokens, rows_hint: Optional[int] = None):
        """Stand-in expert: `expert_x.to(out_dtype) * (1 + rank)` on the valid rows."""
        cfg = self.cfg
        _need(expert_x, cfg.in_dtype, self.device, "expert_x")
        _need(expert_num_tokens, torch.int32, self.device, "expert_num_tokens")
        hint = self._default_rows_in(rows_hint)
        ey = self._buf("expert_y", tuple(expert_x.shape), cfg.out_dtype)
        _lib.call("moe_a2a_expert_scale", self._shape_ref, _ptr(expert_x), _ptr(expert_num_tokens),
                  hint, _DT[dtype_name(cfg.in_dtype)], _DT[dtype_name(cfg.out_dtype)], _ptr(ey),
                  _stream(self.device))
        return ey

    def combine_send(self, expert_meta, expert_y, expert_num_tokens, rows_hint: Optional[int] = None):
        """Expert-major results -> rows grouped by origin rank.
        Returns (back_counts int32[W], back_buf [max_rows_in,H], back_meta [max_rows_in,5]);
        the first sum(back_counts) rows are valid."""
        cfg = self.cfg
        _need(expert_meta, torch.int32, self.device, "expert_meta")
        _need(expert_y, cfg.out_dtype, self.device, "expert_y")
        _need(expert_num_tokens, torch.int32, self.device, "expert_num_tokens")
        if tuple(expert_y.shape) != (self.num_local_experts, self.max_recv, cfg.hidden_dim):
            raise ValueError("combine: expert_y must be [num_local_experts, max_recv, hidden_dim]")
        hint = self._default_rows_in(rows_hint)
        counts = self._buf("back_counts", (self.world_size,), torch.int32)
        buf = self._buf("back_buf", (self.max_rows_in, cfg.hidden_dim), cfg.out_dtype)
        meta = self._buf("back_meta", (self.max_rows_in, META_DIM), torch.int32)
        # the plan describes expert_meta / expert_num_tokens as dispatch_recv wrote them: a caller
        # that edits them in place between the two calls must build the object with
        # reuse_placement=False
        plan = None
        if self._planned_for == (expert_meta.data_ptr(), expert_num_tokens.data_ptr()):
            plan = self._ws["send_back_plan"]
        _lib.call("moe_a2a_combine_send", self._shape_ref, _ptr(expert_y), _ptr(expert_meta),
                  _ptr(expert_num_tokens), min(hint, self.max_rows_in), self.max_rows_in, _ptr(buf),
                  _ptr(meta), _ptr(counts), _ptr(plan), _stream(self.device))
        return counts, buf, meta

    def combine_recv(self, out_tokens, weights, ret_counts, ret_buf, ret_meta, accumulate: bool = True):
        """`out_tokens[t] += row.float() * weights[t, k]` for the arriving rows, in
        arrival order, rounding to out_dtype after every addend. With
        `accumulate=False` the sum starts from zero and `out_tokens` is only written."""
        cfg = self.cfg
        _need(out_tokens, cfg.out_dtype, self.device, "out_tokens")
        _need(weights, torch.float32, self.device, "weights")
        _need(ret_counts, torch.int32, self.device, "ret_counts")
        _need(ret_buf, cfg.out_dtype, self.device, "ret_buf")
        _need(ret_meta, torch.int32, self.device, "ret_meta")
        T = weights.shape[0]
        if out_tokens.shape[0] < T or out_tokens.shape[1] != cfg.hidden_dim:
            raise ValueError("combine: out_tokens must hold num_tokens rows of hidden_dim")
        capacity = min(ret_buf.shape[0], ret_meta.shape[0])
        hint = min(capacity, T * cfg.experts_per_token)
        _lib.call("moe_a2a_combine_recv", self._shape_ref, _ptr(ret_buf), _ptr(ret_meta),
                  _ptr(ret_counts), hint, capacity, _ptr(weights), T, _ptr(out_tokens), int(bool(accumulate)),
                  _DT[dtype_name(cfg.out_dtype)], _stream(self.device))
        return out_tokens

    def _default_rows_in(self, rows_hint):
        if rows_hint is not None:
            return int(rows_hint)
        return int(getattr(self, "_rows_in_hint", self.max_rows_in))

    # ------------------------------------------------------------------ reference surface

    def dispatch(self, dp_x: torch.Tensor, indices: torch.Tensor):
        """all2all/reference.py:68-148 with the exchange delegated to `self.exchange`."""
        if self.exchange is None:
            raise RuntimeError("dispatch() needs an exchange; use the halves or LocalWorld")
        counts, buf, meta = self.dispatch_send(dp_x, indices)
        rc, rb, rm, hint = self.exchange.deliver(self, "dispatch", counts, buf, meta)
        return self.dispatch_recv(rc, rb, rm, hint)

    def combine(self, out_tokens, weights, expert_meta, expert_y, expert_num_tokens):
        """all2all/reference.py:151-234 with the exchange delegated to `self.exchange`."""
        if self.exchange is None:
            raise RuntimeError("combine() needs an exchange; use the halves or LocalWorld")
        counts, buf, meta = self.combine_send(expert_meta, expert_y, expert_num_tokens)
        rc, rb, rm, _ = self.exchange.deliver(self, "combine", counts, buf, meta)
        return self.combine_recv(out_tokens, weights, rc, rb, rm, accumulate=True)


def exchange_leg(src: HIPAllToAll, dst: HIPAllToAll, send_counts, send_buf, send_meta,
                 recv_counts, recv_buf, recv_meta, rows_hint: int) -> None:
    """One source->destination leg of an exchange as a device copy. The copy stays inside the
    rows the four buffers were allocated with, whatever the counts say."""
    send_capacity = min(send_buf.shape[0], send_meta.shape[0])
    recv_capacity = min(recv_buf.shape[0], recv_meta.shape[0])
    _lib.call("moe_a2a_exchange_local", src.world_size, src.cfg.hidden_dim, _ptr(send_buf),
              _ptr(send_meta), _ptr(send_counts), dst.rank, _ptr(recv_buf), _ptr(recv_meta),
              _ptr(recv_counts), src.rank, int(rows_hint), send_capacity, recv_capacity,
              _stream(src.device))


class LocalWorld:
    """All ranks of one job on one GPU, stepped in lockstep; the exchanges are
    device copies (stand-in for all2all/reference.py:91,107-119,185,210-222)."""

    def __init__(self, cfg: MoEConfig, world_size: int, device=None, exact_hints: bool = True,
                 reuse_placement: bool = True):
        self.cfg, self.world_size = cfg, world_size
        self.ranks = [HIPAllToAll(cfg, r, world_size, device=device, reuse_placement=reuse_placement)
                      for r in range(world_size)]
        self.device = self.ranks[0].device
        # True: read the counts back to size every launch exactly (synchronises the host);
        # False: size for the worst case; "last": reuse what the previous run read back, for
        # replaying the same job without touching the host (graph capture)
        self.exact_hints = exact_hints
        self._last_counts = {}
        self.trace: List[dict] = [dict() for _ in range(world_size)]

    def _exchange(self, phase: str, sent: List[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]]):
        W = self.world_size
        all_counts = torch.stack([s[0] for s in sent])      # [src, dst]
        per_dst = all_counts.t().contiguous()                # [dst, src]
        bound = sent[0][1].shape[0]
        if self.exact_hints == "last":  # the counts read back by the previous run of the same job
            host = self._last_counts[phase]
        else:
            host = all_counts.cpu().tolist() if self.exact_hints else None
            self._last_counts[phase] = host
        got = []
        for r, dst in enumerate(self.ranks):
            rc, rb, rm = dst.inbound_buffers(phase)
            rc.copy_(per_dst[r])
            for s, src in enumerate(self.ranks):
                hint = host[s][r] if host is not None else min(bound, sent[s][1].shape[0])
                if host is not None and hint == 0:
                    continue  # the counts were read back: this leg is known to be empty
                exchange_leg(src, dst, sent[s][0], sent[s][1], sent[s][2], rc, rb, rm, hint)
            total = sum(host[s][r] for s in range(W)) if host is not None else None
            got.append((rc, rb, rm, total))
        return got

    def run(self, rank_data: Sequence[RankTestData], accumulate: bool = False) -> List[torch.Tensor]:
        """`ref_kernel` (all2all/reference.py:256-272) for every rank; returns each
        rank's `y[:num_tokens]`. Intermediates are kept in `self.trace[r]`."""
        cfg = self.cfg
        sent = []
        for r, a in enumerate(self.ranks):
            d = rank_data[r]
            c, b, m, sl = a.dispatch_send(d.x, d.indices, want_slots=True)
            sent.append((c, b, m))
            self.trace[r].update(send_counts=c, send_buf=b, send_meta=m, send_slot=sl)
        got = self._exchange("dispatch", sent)
        back = []
        for r, a in enumerate(self.ranks):
            rc, rb, rm, total = got[r]
            num, ex, em = a.dispatch_recv(rc, rb, rm, total)
            ey = a.expert_scale(ex, num, total)
            bc, bb, bm = a.combine_send(em, ey, num, total)
            back.append((bc, bb, bm))
            self.trace[r].update(recv_counts=rc, recv_buf=rb, recv_meta=rm, expert_num_tokens=num,
                                 expert_x=ex, expert_meta=em, expert_y=ey,
                                 back_counts=bc, back_buf=bb, back_meta=bm)
        got = self._exchange("combine", back)
        ys = []
        for r, a in enumerate(self.ranks):
            rc, rb, rm, _ = got[r]
            d = rank_data[r]
            if accumulate:
                y = torch.zeros(cfg.max_num_tokens, cfg.hidden_dim, dtype=cfg.out_dtype, device=self.device)
            else:
                y = a._buf("y", (cfg.max_num_tokens, cfg.hidden_dim), cfg.out_dtype)
            a.combine_recv(y, d.weights, rc, rb, rm, accumulate=accumulate)
            self.trace[r].update(ret_counts=rc, ret_buf=rb, ret_meta=rm, y=y)
            ys.append(y[: d.num_tokens])
        return ys
