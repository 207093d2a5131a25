"""Host side of the MoE dispatch/combine path.

`HIPAllToAll` keeps the surface of the reference's `PyTorchAllToAll`
(all2all/reference.py:55-234): `dispatch(dp_x, indices)` returns
`(expert_num_tokens, expert_x, expert_meta)` in the reference's layouts and
`combine(out_tokens, weights, expert_meta, expert_y, expert_num_tokens)`
accumulates into `out_tokens`. Each of the two is split into its send half and
its receive half (`dispatch_send`/`dispatch_recv`, `combine_send`/
`combine_recv`), because the exchange between the halves is not part of this
library: an `exchange` object supplies it through one method,
`deliver(rank_object, phase, counts, buf, meta) -> (recv_counts, recv_buf,
recv_meta, rows_hint)`. `LocalExchange` is the one-GPU stand-in for the
reference's `all_to_all_single` calls: the ranks of a job run as threads of one
process, meet in `deliver` as processes meet in a collective, and the segments
move by device copies. `run_lockstep` starts such a job. `LocalWorld` steps all
ranks of a job from one thread, half by half, with the same copies.

All device work goes through the C ABI in `libmoe_a2a.so`, bound either with
ctypes or through the torch extension (`binding="ext"`); torch only owns
memory and streams. Buffers live in a per-object workspace allocated once, so
the tensors returned by `dispatch` are views that stay valid until the next
`dispatch` on the same object.
"""
from __future__ import annotations

import threading
from typing import Callable, List, Optional, Sequence, Tuple

import torch

from . import _binding, _lib
from .task import MoEConfig, RankTestData

META_DIM = 5
# Streams of more rows than this take the entry points that rank in a planning launch of their
# own (moe_a2a_dispatch_recv_long, moe_a2a_combine_recv_long); shorter ones the one-launch
# entry points, whose movers rank by scanning. Results are the same; the second launch costs
# about 5 us, which the combine has earned back at 4096 rows and the dispatch, whose scans hide
# behind its payload for longer, at 8192 (measured at hidden_dim 7168; at 12288 rows the two
# together are 17 % ahead, at 32768 rows 40 %).
LONG_STREAM_ROWS = {"dispatch": 8192, "combine": 4096}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device) -> int:
    """The current HIP stream of `device` as an integer handle. The raw accessor costs a fraction of
    a microsecond; `torch.cuda.current_stream()` builds a Stream object (about 5 us, a third of what
    the host spends on a launch here)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


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
                 reuse_placement: bool = True, binding: str = "ctypes", layout: str = "padded",
                 compact_rows: Optional[int] = None):
        if cfg.num_experts % world_size:
            raise ValueError("num_experts must be a multiple of world_size")
        self.cfg = cfg
        self.rank = rank
        self.world_size = world_size
        self.num_local_experts = cfg.num_experts // world_size
        self.max_recv = cfg.max_num_tokens * world_size
        # a job of one rank exchanges with itself; larger jobs need the object their ranks share
        self.exchange = LocalExchange(1) if exchange is None and world_size == 1 else exchange
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        if self.device.type != "cuda":
            raise _lib.MoeA2AError("HIPAllToAll needs a GPU device; this path has no CPU fallback")
        self.binding = _binding.get(binding)  # raises if the native code has not been built
        self.shape = _lib.Shape(world_size, rank, cfg.num_experts, cfg.experts_per_token,
                                cfg.hidden_dim, cfg.max_num_tokens)
        # rows this rank can receive: every peer may route min(K, nle) entries of each token here
        self.max_rows_in = self.max_recv * min(cfg.experts_per_token, self.num_local_experts)
        self.max_rows_out = cfg.max_num_tokens * cfg.experts_per_token
        # "padded": the reference's expert buffers [nle, max_recv, H] (all2all/reference.py:123-136).
        # "compact": the experts' rows back to back in buffers of `compact_rows` rows (default: every
        # row the rank can receive), row pos of expert le at expert_offsets[le] + pos; dispatch()
        # then returns 2-D expert_x / expert_meta, which expert_scale, expert_gemm and combine accept.
        if layout not in ("padded", "compact"):
            raise ValueError(f"layout must be 'padded' or 'compact', got {layout!r}")
        self.layout = layout
        self.compact_rows = self.max_rows_in if compact_rows is None else int(compact_rows)
        if layout == "compact":
            if self.compact_rows < 1:
                raise ValueError("compact_rows must be at least 1")
            # a rank that keeps at most compact_rows rows needs no room to receive or return more
            self.max_rows_in = min(self.max_rows_in, self.compact_rows)
        self.expert_offsets = None  # compact layout: int32[nle + 1], written by dispatch_recv
        self._ws = {}
        # dispatch_recv leaves a plan of where combine_send will put every row; combine_send uses
        # it when it is handed the very tensors that dispatch_recv returned
        self.reuse_placement = reuse_placement
        self._planned_for = None
        self.long_stream_rows = None  # an int overrides both thresholds of LONG_STREAM_ROWS

    # ------------------------------------------------------------------ workspace

    def _buf(self, name: str, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        t = self._ws.get(name)
        if t is None or tuple(t.shape) != tuple(shape) or t.dtype != dtype:
            t = torch.empty(tuple(shape), dtype=dtype, device=self.device)
            self._ws[name] = t
        return t

    def workspace_bytes(self) -> int:
        """Device memory of the buffers this object has made so far."""
        return sum(t.numel() * t.element_size() for t in self._ws.values())

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

    def outbound_buffers(self, phase: str):
        """What this rank's send half of `phase` wrote, as the whole workspace tensors (the send
        halves return views cut to the rows in use): (counts[W], buf, meta)."""
        names = ("send_counts", "send_buf", "send_meta") if phase == "dispatch" else ("back_counts", "back_buf", "back_meta")
        return tuple(self._ws[n] for n in names)

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
        self.binding.dispatch_send(self.shape, dp_x, indices, T, buf, meta, counts, slots, _stream(self.device))
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
        self.binding.plan_send(self.shape, indices, T, rc, ro, ec, ds, se, _stream(self.device))
        return rc, ro, ec, ds[:S], se[:S]

    def dispatch_recv(self, recv_counts, recv_buf, recv_meta, rows_hint: Optional[int] = None):
        """Received stream -> (expert_num_tokens[nle], expert_x[nle,max_recv,H],
        expert_meta[nle,max_recv,5]); rows past expert_num_tokens[le] are not written."""
        cfg = self.cfg
        _need(recv_counts, torch.int32, self.device, "recv_counts")
        _need(recv_buf, cfg.in_dtype, self.device, "recv_buf")
        _need(recv_meta, torch.int32, self.device, "recv_meta")
        capacity = min(recv_buf.shape[0], recv_meta.shape[0])
        # without a count from the caller: what balanced routing delivers (every rank sends its
        # max_num_tokens * K rows and receives as many). A hint only sizes launches and picks the
        # entry point; the kernels move whatever the device-side counts say.
        hint = min(capacity, self.max_rows_out if rows_hint is None else int(rows_hint))
        nle = self.num_local_experts
        num = self._buf("expert_num_tokens", (nle,), torch.int32)
        plan = self._buf("send_back_plan", (2 * cfg.num_experts,), torch.int32) if self.reuse_placement else None
        if self.layout == "compact":
            ex = self._buf("expert_x", (self.compact_rows, cfg.hidden_dim), cfg.in_dtype)
            em = self._buf("expert_meta", (self.compact_rows, META_DIM), torch.int32)
            self.expert_offsets = self._buf("expert_offsets", (nle + 1,), torch.int32)
            self.binding.dispatch_recv_compact(self.shape, recv_buf, recv_meta, recv_counts, hint, num,
                                               self.expert_offsets, ex, em, plan, _stream(self.device))
        else:
            ex = self._buf("expert_x", (nle, self.max_recv, cfg.hidden_dim), cfg.in_dtype)
            em = self._buf("expert_meta", (nle, self.max_recv, META_DIM), torch.int32)
            pos = self._buf("row_position", (capacity,), torch.int32) if hint > self._long_from("dispatch") else None
            self.binding.dispatch_recv(self.shape, recv_buf, recv_meta, recv_counts, hint, num, ex, em, plan,
                                       _stream(self.device), pos)
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
        if expert_x.dim() == 2:  # the compact layout
            self.binding.expert_scale_compact(self.shape, expert_x, expert_num_tokens, hint, ey, _stream(self.device))
        else:
            self.binding.expert_scale(self.shape, expert_x, expert_num_tokens, hint, ey, _stream(self.device))
        return ey

    def expert_gemm(self, expert_x, expert_num_tokens, weights, bias=None, rows_hint: Optional[int] = None,
                    out: Optional[torch.Tensor] = None):
        """One linear layer of the expert as a grouped GEMM over the expert-major layout:
        `expert_x[le, j] @ weights[le].T (+ bias[le])` on the valid rows, float32 accumulation, one
        rounding (two with a bias, as `x @ w.T + b` on 16-bit tensors). Takes the place of
        all2all/reference.py:262 in a model.

        `expert_x` is [nle, max_recv, in_dim] (what `dispatch` returned, or the result of an earlier
        layer), `weights` [nle, out_dim, in_dim] with the input index contiguous, `bias` [nle,
        out_dim] or None, all of one 16-bit type; returns [nle, max_recv, out_dim] (a workspace
        buffer per out_dim unless `out` is given; never the input's memory). Limits of the
        kernels: out_dim % 32 == 0 and in_dim % 8 == 0."""
        nle = self.num_local_experts
        dt = expert_x.dtype
        if dt not in _binding._DT:
            raise TypeError(f"expert_x: expected a 16-bit float type, got {dt}")
        _need(expert_x, dt, self.device, "expert_x")
        _need(expert_num_tokens, torch.int32, self.device, "expert_num_tokens")
        _need(weights, dt, self.device, "weights")
        compact = expert_x.dim() == 2  # [rows, in_dim]: the experts' rows back to back
        if not compact and (expert_x.dim() != 3 or tuple(expert_x.shape[:2]) != (nle, self.max_recv)):
            raise ValueError(f"expert_x must be [{nle}, {self.max_recv}, in_dim] or [rows, in_dim], "
                             f"got {tuple(expert_x.shape)}")
        in_dim = expert_x.shape[-1]
        rows_shape = tuple(expert_x.shape[:-1])
        if weights.dim() != 3 or weights.shape[0] != nle or weights.shape[2] != in_dim:
            raise ValueError(f"weights must be [{nle}, out_dim, {in_dim}], got {tuple(weights.shape)}")
        out_dim = weights.shape[1]
        if bias is not None:
            _need(bias, dt, self.device, "bias")
            if tuple(bias.shape) != (nle, out_dim):
                raise ValueError(f"bias must be [{nle}, {out_dim}], got {tuple(bias.shape)}")
        hint = self._default_rows_in(rows_hint)
        if out is None:
            name = f"expert_out_{out_dim}"
            if name in self._ws and self._ws[name].data_ptr() == expert_x.data_ptr():
                name += "_b"  # a layer of equal width reading the buffer the one before it wrote
            out = self._buf(name, rows_shape + (out_dim,), dt)
        else:
            _need(out, dt, self.device, "out")
            if tuple(out.shape) != rows_shape + (out_dim,) or out.data_ptr() == expert_x.data_ptr():
                raise ValueError(f"out must be {list(rows_shape) + [out_dim]} and not the input")
        gemm = self.binding.expert_gemm_compact if compact else self.binding.expert_gemm
        gemm(self.shape, expert_x, expert_num_tokens, hint, weights, bias, out, _stream(self.device))
        return out

    def combine_send(self, expert_meta, expert_y, expert_num_tokens, rows_hint: Optional[int] = None):
        """Expert-major results -> rows grouped by origin rank.
        Returns (back_counts int32[W], back_buf [max_rows_in,H], back_meta [max_rows_in,5]);
        the first sum(back_counts) rows are valid."""
        cfg = self.cfg
        _need(expert_meta, torch.int32, self.device, "expert_meta")
        _need(expert_y, cfg.out_dtype, self.device, "expert_y")
        _need(expert_num_tokens, torch.int32, self.device, "expert_num_tokens")
        compact = expert_y.dim() == 2
        if compact:
            if expert_y.shape[1] != cfg.hidden_dim or expert_meta.dim() != 2:
                raise ValueError("combine: compact expert_y / expert_meta must be [rows, hidden_dim] / [rows, 5]")
        elif tuple(expert_y.shape) != (self.num_local_experts, self.max_recv, cfg.hidden_dim):
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
        send = self.binding.combine_send_compact if compact else self.binding.combine_send
        send(self.shape, expert_y, expert_meta, expert_num_tokens, min(hint, self.max_rows_in), buf, meta, counts,
             plan, _stream(self.device))
        return counts, buf, meta

    def combine_recv(self, out_tokens, weights, ret_counts, ret_buf, ret_meta, accumulate: bool = True,
                     unique_pairs: bool = True):
        """`out_tokens[t] += row.float() * weights[t, k]` for the arriving rows, in
        arrival order, rounding to out_dtype after every addend. With
        `accumulate=False` the sum starts from zero and `out_tokens` is only written.

        Streams of more than `LONG_STREAM_ROWS["combine"]` rows go through a (token, k) -> row
        table, which holds ONE row per pair: every stream a dispatch produced has each pair once,
        and for those the result is the same. A caller that feeds a stream in which a (src_token,
        src_k) pair may arrive more than once (the reference, all2all/reference.py:227-232, adds
        every arriving row) says so with `unique_pairs=False`; the rows are then found by scanning
        whatever the length, and every one of them is added."""
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
        table = None
        if unique_pairs and hint > self._long_from("combine"):
            table = self._buf("entry_row", (cfg.max_num_tokens * cfg.experts_per_token,), torch.int32)
        self.binding.combine_recv(self.shape, ret_buf, ret_meta, ret_counts, hint, weights, T, out_tokens,
                                  accumulate, _stream(self.device), table)
        return out_tokens

    def _long_from(self, phase: str) -> int:
        return LONG_STREAM_ROWS[phase] if self.long_stream_rows is None else self.long_stream_rows

    def _default_rows_in(self, rows_hint):
        if rows_hint is not None:
            return int(rows_hint)
        return int(getattr(self, "_rows_in_hint", min(self.max_rows_in, self.max_rows_out)))

    # ------------------------------------------------------------------ reference surface

    def dispatch(self, dp_x: torch.Tensor, indices: torch.Tensor):
        """all2all/reference.py:68-148 with the exchange delegated to `self.exchange`."""
        if self.exchange is None:
            raise RuntimeError("dispatch() of a job with several ranks needs the exchange its ranks share "
                               "(LocalExchange on one GPU); or use the halves, or LocalWorld")
        counts, buf, meta = self.dispatch_send(dp_x, indices)
        rc, rb, rm, hint = self.exchange.deliver(self, "dispatch", counts, buf, meta)
        return self.dispatch_recv(rc, rb, rm, hint)

    def combine(self, out_tokens, weights, expert_meta, expert_y, expert_num_tokens):
        """all2all/reference.py:151-234 with the exchange delegated to `self.exchange`."""
        if self.exchange is None:
            raise RuntimeError("combine() of a job with several ranks needs the exchange its ranks share "
                               "(LocalExchange on one GPU); or use the halves, or LocalWorld")
        counts, buf, meta = self.combine_send(expert_meta, expert_y, expert_num_tokens)
        rc, rb, rm, _ = self.exchange.deliver(self, "combine", counts, buf, meta)
        return self.combine_recv(out_tokens, weights, rc, rb, rm, accumulate=True)


def exchange_leg(src: HIPAllToAll, dst: HIPAllToAll, send_counts, send_buf, send_meta,
                 recv_counts, recv_buf, recv_meta, rows_hint: int) -> None:
    """One source->destination leg of an exchange as a device copy. The copy stays inside the
    rows the four buffers were allocated with, whatever the counts say."""
    src.binding.exchange_local(src.world_size, src.cfg.hidden_dim, send_buf, send_meta, send_counts, dst.rank,
                               recv_buf, recv_meta, recv_counts, src.rank, int(rows_hint), _stream(src.device))


GATHER_MAX_RANKS = 64  # source ranks one launch of moe_a2a_exchange_gather_local serves


def gather_sources(ranks: Sequence[HIPAllToAll], phase: str):
    """The source side of `exchange_gather` for all ranks of a job (whose send halves of `phase`
    have run at least once, so that their workspaces exist); stays valid while those do."""
    out = [a.outbound_buffers(phase) for a in ranks]
    a0 = ranks[0]
    return a0.binding.gather_sources(a0.cfg.hidden_dim, [o[1] for o in out], [o[2] for o in out], [o[0] for o in out])


def exchange_gather(dst: HIPAllToAll, sources, recv_counts, recv_buf, recv_meta, rows_hint: int) -> None:
    """Everything the ranks of a job hold for `dst`, counts included, in one launch."""
    dst.binding.exchange_gather(dst.world_size, dst.cfg.hidden_dim, sources, dst.rank, recv_buf, recv_meta,
                                recv_counts, int(rows_hint), _stream(dst.device))


class LocalExchange:
    """The exchange of a job whose ranks share one GPU and one process: stand-in for the
    `all_to_all_single` calls of all2all/reference.py:91,107-119 (dispatch) and :185,210-222
    (combine).

    Every rank runs in a thread of its own and calls `dispatch()` / `combine()` as a process
    of the reference would; `deliver` is where they meet. Each rank posts what it sends and
    waits for the others (as in a collective), then copies the segments addressed to it out of
    its peers' send buffers with `moe_a2a_exchange_local`, and waits again so that no peer
    reuses a send buffer before every copy out of it has been launched. All launches go to the
    callers' current stream, which the ranks must share (the default stream does), so launch
    order is execution order.

    `exact_hints=True` reads the counts back (one host synchronisation per call, as the
    reference's `.tolist()` at reference.py:110-111) and sizes every launch exactly; otherwise
    launches are sized for the largest segment the buffers can hold and nothing waits for the
    device.
    """

    def __init__(self, world_size: int, exact_hints: bool = False, timeout: float = 120.0):
        self.world_size = world_size
        self.exact_hints = exact_hints
        self._posted: List[Optional[tuple]] = [None] * world_size
        # a rank that fails leaves the others waiting: the time-out turns that into an error
        self._barrier = threading.Barrier(world_size, timeout=timeout)

    def deliver(self, a: "HIPAllToAll", phase: str, counts, buf, meta):
        W = self.world_size
        if a.world_size != W:
            raise ValueError("this exchange serves a job of another size")
        self._posted[a.rank] = (a, counts, buf, meta)
        self._barrier.wait()  # every rank has launched its send half
        posted = list(self._posted)
        rc, rb, rm = a.inbound_buffers(phase)
        bound = min(rb.shape[0], rm.shape[0])
        if W <= GATHER_MAX_RANKS:
            # one launch copies every source's segment and delivers the counts
            host = None
            if self.exact_hints:
                host = torch.stack([p[1] for p in posted])[:, a.rank].cpu().tolist()
            per_source = max(host) if host is not None else min(bound, max(1, 2 * a.max_rows_out // W))
            exchange_gather(a, gather_sources([p[0] for p in posted], phase), rc, rb, rm, per_source)
        else:
            sent_here = torch.stack([p[1] for p in posted])[:, a.rank]  # rows each source holds for this rank
            rc.copy_(sent_here)
            host = sent_here.cpu().tolist() if self.exact_hints else None
            for s, (src, sc, sb, sm) in enumerate(posted):
                hint = host[s] if host is not None else min(bound, sb.shape[0])
                if hint > 0:
                    exchange_leg(src, a, sc, sb, sm, rc, rb, rm, hint)
        self._barrier.wait()  # every copy out of every send buffer has been launched
        return rc, rb, rm, (sum(host) if host is not None else None)


def run_lockstep(world_size: int, rank_main: Callable[[int, LocalExchange], object],
                 exact_hints: bool = False, device=None) -> list:
    """Run `rank_main(rank, exchange)` for every rank of a job, one thread per rank on one
    GPU, and return the results in rank order: what a launcher with one process per GPU does
    for the reference. The first exception of any rank is raised again here."""
    exchange = LocalExchange(world_size, exact_hints=exact_hints)
    results: list = [None] * world_size
    errors: list = [None] * world_size
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)

    def body(r: int):
        try:
            with torch.cuda.device(dev):
                results[r] = rank_main(r, exchange)
        except BaseException as e:  # noqa: BLE001 - handed to the caller below
            errors[r] = e
            exchange._barrier.abort()  # release the ranks waiting for this one

    threads = [threading.Thread(target=body, args=(r,), name=f"rank{r}") for r in range(world_size)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    real = [e for e in errors if e is not None and not isinstance(e, threading.BrokenBarrierError)]
    if real or any(errors):
        raise (real or [e for e in errors if e is not None])[0]
    return results


class LocalWorld:
    """All ranks of one job on one GPU, stepped in lockstep; the exchanges are
    device copies (stand-in for all2all/reference.py:91,107-119,185,210-222)."""

    def __init__(self, cfg: MoEConfig, world_size: int, device=None, exact_hints: bool = True,
                 reuse_placement: bool = True, binding: str = "ctypes",
                 long_stream_rows: Optional[int] = None, layout: str = "padded",
                 compact_rows: Optional[int] = None):
        self.cfg, self.world_size = cfg, world_size
        self.ranks = [HIPAllToAll(cfg, r, world_size, device=device, reuse_placement=reuse_placement,
                                  binding=binding, layout=layout, compact_rows=compact_rows)
                      for r in range(world_size)]
        if long_stream_rows is not None:  # (0: every receive half takes the long-stream entry points)
            for a in self.ranks:
                a.long_stream_rows = long_stream_rows
        self.device = self.ranks[0].device
        # True: read the counts back to size every launch exactly (synchronises the host);
        # False: size for the worst case; "last": reuse what the previous run read back, for
        # replaying the same job without touching the host (graph capture)
        self.exact_hints = exact_hints
        self._last_counts = {}
        self._sources = {}  # phase -> the source tables of the gathering exchange
        self.trace: List[dict] = [dict() for _ in range(world_size)]

    def _exchange_hints(self, phase: str, sent):
        """Host-side row counts [src][dst] that size the launches of one exchange, or None."""
        if self.exact_hints == "last":  # the counts read back by the previous run of the same job
            return self._last_counts[phase]
        host = torch.stack([s[0] for s in sent]).cpu().tolist() if self.exact_hints else None
        self._last_counts[phase] = host
        return host

    def _deliver(self, phase: str, r: int, sent, host):
        """The inbound half of one exchange for rank r: (counts, buf, meta, rows or None)."""
        W, dst = self.world_size, self.ranks[r]
        rc, rb, rm = dst.inbound_buffers(phase)
        # (with "last" the host counts are an earlier run's: they size launches and are no
        # statement about this run)
        total = sum(host[s][r] for s in range(W)) if host is not None else None
        if W <= GATHER_MAX_RANKS:
            # one launch per destination copies every source's segment and delivers the counts
            sources = self._sources.get(phase)
            if sources is None:  # (the workspaces the tables point into live as long as the ranks)
                sources = self._sources[phase] = gather_sources(self.ranks, phase)
            loose = max(1, 2 * self.ranks[0].max_rows_out // W)
            per_source = max(host[s][r] for s in range(W)) if host is not None else loose
            exchange_gather(dst, sources, rc, rb, rm, min(per_source, rb.shape[0]))
            return rc, rb, rm, total
        rc.copy_(torch.stack([s[0][r] for s in sent]))
        bound = sent[0][1].shape[0]
        for s, src in enumerate(self.ranks):
            hint = host[s][r] if host is not None else min(bound, sent[s][1].shape[0])
            if host is not None and hint == 0 and self.exact_hints != "last":
                continue  # the counts were read back: this leg is known to be empty
            exchange_leg(src, dst, sent[s][0], sent[s][1], sent[s][2], rc, rb, rm, max(hint, 1))
        return rc, rb, rm, total

    def _exchange(self, phase: str, sent: List[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]]):
        host = self._exchange_hints(phase, sent)
        return [self._deliver(phase, r, sent, host) for r in range(self.world_size)]

    def run(self, rank_data: Sequence[RankTestData], accumulate: bool = False,
            expert: Optional[Callable] = None, only: Optional[int] = None) -> List[torch.Tensor]:
        """`ref_kernel` (all2all/reference.py:256-272) for every rank; returns each
        rank's `y[:num_tokens]`. Intermediates are kept in `self.trace[r]`.

        `expert(rank_object, expert_x, expert_num_tokens, rows_hint)` returns the rank's
        `expert_y [nle, max_recv, hidden_dim]` of `out_dtype`: what a model runs where the
        reference has `expert_x.to(out_dtype) * (1 + rank)` (reference.py:262), for example layers
        of `HIPAllToAll.expert_gemm`. None is the reference's stand-in.

        `only=r`: the caller wants rank r's result alone. Every rank still dispatches, runs its
        experts and sends back (rank r's rows come from all of them), but the return exchange and
        the weighted sum run for rank r only; the other entries of the result are None."""
        cfg = self.cfg
        sent = []
        for r, a in enumerate(self.ranks):
            d = rank_data[r]
            c, b, m, sl = a.dispatch_send(d.x, d.indices, want_slots=True)
            sent.append((c, b, m))
            self.trace[r].update(send_counts=c, send_buf=b, send_meta=m, send_slot=sl)
        host = self._exchange_hints("dispatch", sent)
        back = []
        for r, a in enumerate(self.ranks):
            rc, rb, rm, total = self._deliver("dispatch", r, sent, host)
            num, ex, em = a.dispatch_recv(rc, rb, rm, total)
            ey = a.expert_scale(ex, num, total) if expert is None else expert(a, ex, num, total)
            bc, bb, bm = a.combine_send(em, ey, num, total)
            back.append((bc, bb, bm))
            self.trace[r].update(recv_counts=rc, recv_buf=rb, recv_meta=rm, expert_num_tokens=num,
                                 expert_x=ex, expert_meta=em, expert_y=ey,
                                 back_counts=bc, back_buf=bb, back_meta=bm)
        host = self._exchange_hints("combine", back)
        ys = []
        for r, a in enumerate(self.ranks):
            if only is not None and r != only:
                ys.append(None)
                continue
            d = rank_data[r]
            rc, rb, rm, _ = self._deliver("combine", r, back, host)
            if accumulate:
                y = torch.zeros(cfg.max_num_tokens, cfg.hidden_dim, dtype=cfg.out_dtype, device=self.device)
            else:
                y = a._buf("y", (cfg.max_num_tokens, cfg.hidden_dim), cfg.out_dtype)
            a.combine_recv(y, d.weights, rc, rb, rm, accumulate=accumulate)
            self.trace[r].update(ret_counts=rc, ret_buf=rb, ret_meta=rm, y=y)
            ys.append(y[: d.num_tokens])
        return ys
