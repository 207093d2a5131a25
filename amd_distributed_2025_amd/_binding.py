"""The two ways the host layer reaches the C ABI of libmoe_a2a.so.

`CtypesBinding` calls the exported functions directly (include/moe_a2a.h);
`ExtBinding` goes through the torch extension of `csrc/moe_a2a_torch.cpp`, the
binding idiom of the reference's submissions (all2all/hipv8.py:230-252). Both
offer the same methods with the same arguments — tensors, sizes and the stream
handle — and both end in the same kernels, so results are identical. Neither has
a fallback: a missing library or a nonzero status raises.

Capacities (`capacity_rows` of the C ABI) are taken from the tensors: the rows a
row buffer and its meta buffer were allocated with.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib

META_DIM = 5
_DT = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _rows(buf: torch.Tensor, meta: torch.Tensor, hidden_dim: int) -> int:
    return min(buf.numel() // max(hidden_dim, 1), meta.numel() // META_DIM)


class CtypesBinding:
    name = "ctypes"

    def __init__(self):
        _lib.load()

    def version(self) -> str:
        return _lib.load().moe_a2a_version().decode()

    def dispatch_send(self, shape, x, indices, num_tokens, send_buf, send_meta, send_counts, send_slot, stream):
        _lib.call("moe_a2a_dispatch_send", C.byref(shape), _ptr(x), _ptr(indices), num_tokens, _ptr(send_buf),
                  _ptr(send_meta), _ptr(send_counts), _ptr(send_slot), C.c_void_p(stream))

    def plan_send(self, shape, indices, num_tokens, rank_counts, rank_offsets, expert_counts, dst_slot,
                  src_entry, stream):
        _lib.call("moe_a2a_plan_send", C.byref(shape), _ptr(indices), num_tokens, _ptr(rank_counts),
                  _ptr(rank_offsets), _ptr(expert_counts), _ptr(dst_slot), _ptr(src_entry), C.c_void_p(stream))

    def dispatch_recv(self, shape, recv_buf, recv_meta, recv_counts, rows_hint, expert_num_tokens, expert_x,
                      expert_meta, send_back_plan, stream, row_position=None):
        capacity = _rows(recv_buf, recv_meta, shape.hidden_dim)
        args = (C.byref(shape), _ptr(recv_buf), _ptr(recv_meta), _ptr(recv_counts),
                min(rows_hint, capacity), capacity, _ptr(expert_num_tokens), _ptr(expert_x), _ptr(expert_meta),
                _ptr(send_back_plan))
        if row_position is None:
            _lib.call("moe_a2a_dispatch_recv", *args, C.c_void_p(stream))
        else:  # long streams: positions from a planning launch
            if row_position.numel() < capacity:
                raise ValueError("row_position must hold one int per row of the receive buffers")
            _lib.call("moe_a2a_dispatch_recv_long", *args, _ptr(row_position), C.c_void_p(stream))

    def combine_send(self, shape, expert_y, expert_meta, expert_num_tokens, rows_hint, send_buf, send_meta,
                     send_counts, send_back_plan, stream):
        capacity = _rows(send_buf, send_meta, shape.hidden_dim)
        _lib.call("moe_a2a_combine_send", C.byref(shape), _ptr(expert_y), _ptr(expert_meta),
                  _ptr(expert_num_tokens), min(rows_hint, capacity), capacity, _ptr(send_buf), _ptr(send_meta),
                  _ptr(send_counts), _ptr(send_back_plan), C.c_void_p(stream))

    def combine_recv(self, shape, recv_buf, recv_meta, recv_counts, rows_hint, weights, num_tokens, out_tokens,
                     accumulate, stream, entry_row=None):
        capacity = _rows(recv_buf, recv_meta, shape.hidden_dim)
        args = (C.byref(shape), _ptr(recv_buf), _ptr(recv_meta), _ptr(recv_counts),
                min(rows_hint, capacity), capacity, _ptr(weights), num_tokens, _ptr(out_tokens),
                int(bool(accumulate)), _DT[out_tokens.dtype])
        if entry_row is None:
            _lib.call("moe_a2a_combine_recv", *args, C.c_void_p(stream))
        else:  # long streams: rows looked up in a (token, k) -> row table
            if entry_row.numel() < num_tokens * shape.experts_per_token:
                raise ValueError("entry_row must hold num_tokens * experts_per_token ints")
            _lib.call("moe_a2a_combine_recv_long", *args, _ptr(entry_row), C.c_void_p(stream))

    def expert_scale(self, shape, expert_x, expert_num_tokens, rows_hint, expert_y, stream):
        _lib.call("moe_a2a_expert_scale", C.byref(shape), _ptr(expert_x), _ptr(expert_num_tokens), rows_hint,
                  _DT[expert_x.dtype], _DT[expert_y.dtype], _ptr(expert_y), C.c_void_p(stream))

    def expert_gemm(self, shape, expert_x, expert_num_tokens, rows_hint, weights, bias, expert_y, stream):
        _lib.call("moe_a2a_expert_gemm", C.byref(shape), _ptr(expert_x), _ptr(expert_num_tokens), rows_hint,
                  _ptr(weights), _ptr(bias), weights.shape[2], weights.shape[1], _DT[expert_x.dtype],
                  _ptr(expert_y), C.c_void_p(stream))

    def linear(self, input, weight, bias, output, stream):
        m, k = input.shape
        _lib.call("moe_a2a_linear", _ptr(input), _ptr(weight), _ptr(bias), m, weight.shape[0], k, _DT[input.dtype],
                  _ptr(output), C.c_void_p(stream))

    def exchange_local(self, world_size, hidden_dim, send_buf, send_meta, send_counts, dst_rank, recv_buf,
                       recv_meta, recv_counts, src_rank, rows_hint, stream):
        _lib.call("moe_a2a_exchange_local", world_size, hidden_dim, _ptr(send_buf), _ptr(send_meta),
                  _ptr(send_counts), dst_rank, _ptr(recv_buf), _ptr(recv_meta), _ptr(recv_counts), src_rank,
                  rows_hint, _rows(send_buf, send_meta, hidden_dim), _rows(recv_buf, recv_meta, hidden_dim),
                  C.c_void_p(stream))

    # ---- the compact expert-major layout (rows of the experts back to back)

    def dispatch_recv_compact(self, shape, recv_buf, recv_meta, recv_counts, rows_hint, expert_num_tokens,
                              expert_offsets, expert_x, expert_meta, send_back_plan, stream):
        capacity = _rows(recv_buf, recv_meta, shape.hidden_dim)
        _lib.call("moe_a2a_dispatch_recv_compact", C.byref(shape), _ptr(recv_buf), _ptr(recv_meta),
                  _ptr(recv_counts), min(rows_hint, capacity), capacity, _ptr(expert_num_tokens),
                  _ptr(expert_offsets), _ptr(expert_x), _ptr(expert_meta),
                  _rows(expert_x, expert_meta, shape.hidden_dim), _ptr(send_back_plan), C.c_void_p(stream))

    def expert_scale_compact(self, shape, expert_x, expert_num_tokens, rows_hint, expert_y, stream):
        _lib.call("moe_a2a_expert_scale_compact", C.byref(shape), _ptr(expert_x), _ptr(expert_num_tokens),
                  rows_hint, min(expert_x.shape[0], expert_y.shape[0]), _DT[expert_x.dtype], _DT[expert_y.dtype],
                  _ptr(expert_y), C.c_void_p(stream))

    def expert_gemm_compact(self, shape, expert_x, expert_num_tokens, rows_hint, weights, bias, expert_y, stream):
        _lib.call("moe_a2a_expert_gemm_compact", C.byref(shape), _ptr(expert_x), _ptr(expert_num_tokens),
                  rows_hint, min(expert_x.shape[0], expert_y.shape[0]), _ptr(weights), _ptr(bias),
                  weights.shape[2], weights.shape[1], _DT[expert_x.dtype], _ptr(expert_y), C.c_void_p(stream))

    def combine_send_compact(self, shape, expert_y, expert_meta, expert_num_tokens, rows_hint, send_buf,
                             send_meta, send_counts, send_back_plan, stream):
        capacity = _rows(send_buf, send_meta, shape.hidden_dim)
        _lib.call("moe_a2a_combine_send_compact", C.byref(shape), _ptr(expert_y), _ptr(expert_meta),
                  _ptr(expert_num_tokens), min(rows_hint, capacity),
                  _rows(expert_y, expert_meta, shape.hidden_dim), capacity, _ptr(send_buf), _ptr(send_meta),
                  _ptr(send_counts), _ptr(send_back_plan), C.c_void_p(stream))

    def gather_sources(self, hidden_dim, send_bufs, send_metas, send_counts):
        """The per-source pointer tables of `exchange_gather`, built once for buffers that stay where
        they are (a workspace): (tables, rows every send buffer holds, the tensors kept alive)."""
        table = C.c_void_p * len(send_bufs)
        return ((table(*[t.data_ptr() for t in send_bufs]), table(*[t.data_ptr() for t in send_metas]),
                 table(*[t.data_ptr() for t in send_counts])),
                min(_rows(b, m, hidden_dim) for b, m in zip(send_bufs, send_metas)),
                (list(send_bufs), list(send_metas), list(send_counts)))

    def exchange_gather(self, world_size, hidden_dim, sources, dst_rank, recv_buf, recv_meta, recv_counts,
                        rows_hint, stream):
        (bufs, metas, counts), send_capacity, _ = sources
        _lib.call("moe_a2a_exchange_gather_local", world_size, hidden_dim, bufs, metas, counts, dst_rank,
                  _ptr(recv_buf), _ptr(recv_meta), _ptr(recv_counts), rows_hint, send_capacity,
                  _rows(recv_buf, recv_meta, hidden_dim), C.c_void_p(stream))


class ExtBinding:
    name = "ext"

    def __init__(self):
        from . import _ext

        self._m = _ext.load()

    @staticmethod
    def _shape(shape) -> list:
        return [getattr(shape, f) for f, _ in _lib.Shape._fields_]

    def version(self) -> str:
        return self._m.a2a_version()

    def dispatch_send(self, shape, x, indices, num_tokens, send_buf, send_meta, send_counts, send_slot, stream):
        self._m.a2a_dispatch_send(self._shape(shape), x, indices, num_tokens, send_buf, send_meta, send_counts,
                                  send_slot, stream)

    def plan_send(self, shape, indices, num_tokens, rank_counts, rank_offsets, expert_counts, dst_slot,
                  src_entry, stream):
        self._m.a2a_plan_send(self._shape(shape), indices, num_tokens, rank_counts, rank_offsets, expert_counts,
                              dst_slot, src_entry, stream)

    def dispatch_recv(self, shape, recv_buf, recv_meta, recv_counts, rows_hint, expert_num_tokens, expert_x,
                      expert_meta, send_back_plan, stream, row_position=None):
        self._m.a2a_dispatch_recv(self._shape(shape), recv_buf, recv_meta, recv_counts, rows_hint,
                                  expert_num_tokens, expert_x, expert_meta, send_back_plan, row_position, stream)

    def combine_send(self, shape, expert_y, expert_meta, expert_num_tokens, rows_hint, send_buf, send_meta,
                     send_counts, send_back_plan, stream):
        self._m.a2a_combine_send(self._shape(shape), expert_y, expert_meta, expert_num_tokens, rows_hint,
                                 send_buf, send_meta, send_counts, send_back_plan, stream)

    def combine_recv(self, shape, recv_buf, recv_meta, recv_counts, rows_hint, weights, num_tokens, out_tokens,
                     accumulate, stream, entry_row=None):
        self._m.a2a_combine_recv(self._shape(shape), recv_buf, recv_meta, recv_counts, rows_hint, weights,
                                 num_tokens, out_tokens, bool(accumulate), entry_row, stream)

    def expert_scale(self, shape, expert_x, expert_num_tokens, rows_hint, expert_y, stream):
        self._m.a2a_expert_scale(self._shape(shape), expert_x, expert_num_tokens, rows_hint, expert_y, stream)

    def expert_gemm(self, shape, expert_x, expert_num_tokens, rows_hint, weights, bias, expert_y, stream):
        self._m.a2a_expert_gemm(self._shape(shape), expert_x, expert_num_tokens, rows_hint, weights, bias,
                                expert_y, stream)

    def linear(self, input, weight, bias, output, stream):
        self._m.a2a_linear(input, weight, bias, output, stream)

    def exchange_local(self, world_size, hidden_dim, send_buf, send_meta, send_counts, dst_rank, recv_buf,
                       recv_meta, recv_counts, src_rank, rows_hint, stream):
        self._m.a2a_exchange_local(world_size, hidden_dim, send_buf, send_meta, send_counts, dst_rank, recv_buf,
                                   recv_meta, recv_counts, src_rank, rows_hint, stream)

    def dispatch_recv_compact(self, shape, recv_buf, recv_meta, recv_counts, rows_hint, expert_num_tokens,
                              expert_offsets, expert_x, expert_meta, send_back_plan, stream):
        self._m.a2a_dispatch_recv_compact(self._shape(shape), recv_buf, recv_meta, recv_counts, rows_hint,
                                          expert_num_tokens, expert_offsets, expert_x, expert_meta,
                                          send_back_plan, stream)

    def expert_scale_compact(self, shape, expert_x, expert_num_tokens, rows_hint, expert_y, stream):
        self._m.a2a_expert_scale_compact(self._shape(shape), expert_x, expert_num_tokens, rows_hint, expert_y,
                                         stream)

    def expert_gemm_compact(self, shape, expert_x, expert_num_tokens, rows_hint, weights, bias, expert_y, stream):
        self._m.a2a_expert_gemm_compact(self._shape(shape), expert_x, expert_num_tokens, rows_hint, weights, bias,
                                        expert_y, stream)

    def combine_send_compact(self, shape, expert_y, expert_meta, expert_num_tokens, rows_hint, send_buf,
                             send_meta, send_counts, send_back_plan, stream):
        self._m.a2a_combine_send_compact(self._shape(shape), expert_y, expert_meta, expert_num_tokens, rows_hint,
                                         send_buf, send_meta, send_counts, send_back_plan, stream)

    def gather_sources(self, hidden_dim, send_bufs, send_metas, send_counts):
        return (list(send_bufs), list(send_metas), list(send_counts))

    def exchange_gather(self, world_size, hidden_dim, sources, dst_rank, recv_buf, recv_meta, recv_counts,
                        rows_hint, stream):
        bufs, metas, counts = sources
        self._m.a2a_exchange_gather_local(world_size, hidden_dim, bufs, metas, counts, dst_rank, recv_buf,
                                          recv_meta, recv_counts, rows_hint, stream)


_BINDINGS = {}


def get(name: str):
    """`"ctypes"` or `"ext"`; bindings are created once."""
    b = _BINDINGS.get(name)
    if b is None:
        if name == "ctypes":
            b = CtypesBinding()
        elif name == "ext":
            b = ExtBinding()
        else:
            raise ValueError(f"unknown binding {name!r} (ctypes or ext)")
        _BINDINGS[name] = b
    return b
