"""Device buffers and C-ABI calls of the low-latency path for one rank.

``LowLatencyState`` plays the part of the reference's ``_ll_get_cache``
(deep_ep/buffer.py:1623-1813): every tensor the path needs is allocated once
per shape and reused by later calls, so a dispatch/combine pair launches
kernels and nothing else.  Nothing is ever zero-filled per call (the
reference clears ~240 MB per dispatch, deep_ep/buffer.py:2370-2378); rows at
or beyond ``packed_recv_count`` are simply not defined.
"""
from dataclasses import dataclass

import torch

from . import _capi

ROW_BF16, ROW_FP8, ROW_FP8_POW2, ROW_FP8_UE8M0 = 0, 1, 2, 3


def row_format(use_fp8: bool, round_scale: bool, use_ue8m0: bool) -> int:
    if not use_fp8:
        return ROW_BF16
    if use_ue8m0:
        assert round_scale, "use_ue8m0 requires round_scale"
        return ROW_FP8_UE8M0
    return ROW_FP8_POW2 if round_scale else ROW_FP8


def current_stream_ptr():
    return torch.cuda.current_stream().cuda_stream


@dataclass(frozen=True)
class LLShape:
    num_ranks: int
    rank: int
    num_experts: int
    max_tokens: int  # num_max_dispatch_tokens_per_rank
    hidden: int
    num_topk: int
    fmt: int

    @property
    def num_local_experts(self) -> int:
        return self.num_experts // self.num_ranks

    @property
    def slots_per_expert(self) -> int:
        return self.max_tokens * self.num_ranks


class LowLatencyState:
    """All device memory of one rank's low-latency dispatch + combine for one shape."""

    def __init__(self, shape: LLShape, device="cuda", keep_remote_rows: bool = True):
        lib = _capi.load()
        self.lib = lib
        self.shape = s = shape
        assert s.num_experts % s.num_ranks == 0 and 0 <= s.rank < s.num_ranks
        assert s.hidden % 128 == 0
        self.stride = lib.deepep_ll_row_stride(s.hidden, s.fmt)
        self.payload_bytes = lib.deepep_ll_row_payload_bytes(s.hidden, s.fmt)  # what a staged row carries
        self.data_bytes = lib.deepep_ll_row_data_bytes(s.hidden, s.fmt)
        self.scale_bytes = lib.deepep_ll_row_scale_bytes(s.hidden, s.fmt)
        el, r, m, e, h = s.num_local_experts, s.num_ranks, s.max_tokens, s.num_experts, s.hidden
        u8 = dict(dtype=torch.uint8, device=device)
        i32 = dict(dtype=torch.int32, device=device)
        # dispatch
        self.recv_staging = torch.empty(el * r * m * self.stride, **u8)
        self.recv_count = torch.zeros(el * r, **i32)
        self.send_slots = torch.empty(e * m * self.stride, **u8) if keep_remote_rows else None
        self.send_count = torch.zeros(e, **i32)
        self.pair_slot = torch.full((m, s.num_topk), -1, **i32)
        self.workspace = torch.empty(max(256, lib.deepep_ll_dispatch_workspace_bytes(m, s.num_topk, e)), **u8)
        # index + flat-copy scratch of the receive / combine-send kernels, only needed for large batches
        self.expected_rows = m * s.num_topk
        self.segment_workspace = (torch.empty(lib.deepep_ll_segment_workspace_bytes(e, m), **u8)
                                  if self.expected_rows > 8192 else None)
        if s.fmt == ROW_BF16:
            self.packed_recv_x = torch.empty((el, r * m, h), dtype=torch.bfloat16, device=device)
            self.packed_recv_scales = None
        else:
            self.packed_recv_x = torch.empty((el, r * m, h), dtype=torch.float8_e4m3fn, device=device)
            if s.fmt == ROW_FP8_UE8M0:
                self.packed_recv_scales = torch.empty((el, r * m, h // 512), **i32)
            else:
                self.packed_recv_scales = torch.empty((el, r * m, h // 128), dtype=torch.float32, device=device)
        self.packed_recv_count = torch.zeros(el, **i32)
        self.packed_recv_src_info = torch.empty((el, r * m), **i32)
        self.packed_recv_layout_range = torch.zeros((el, r), dtype=torch.int64, device=device)
        # combine
        self.combine_staging = torch.empty((e, m, h), dtype=torch.bfloat16, device=device)
        self.combine_send_slots = (torch.empty((el, r, m, h), dtype=torch.bfloat16, device=device)
                                   if keep_remote_rows else None)
        self.combined_x = torch.empty((m, h), dtype=torch.bfloat16, device=device)

    # -- dispatch ---------------------------------------------------------
    def dispatch_send(self, x: torch.Tensor, topk_idx: torch.Tensor) -> None:
        s = self.shape
        t = x.shape[0]
        _capi.check(self.lib.deepep_ll_dispatch_send(
            _capi.ptr(x), _capi.ptr(topk_idx), t, s.hidden, s.num_topk, s.num_experts, s.num_ranks, s.rank,
            s.max_tokens, s.fmt, _capi.ptr(self.recv_staging), _capi.ptr(self.recv_count),
            _capi.ptr(self.send_slots), _capi.ptr(self.send_count), _capi.ptr(self.pair_slot),
            _capi.ptr(self.workspace), self.workspace.numel(), current_stream_ptr()))

    def dispatch_recv(self, stats: torch.Tensor = None) -> None:
        s = self.shape
        _capi.check(self.lib.deepep_ll_dispatch_recv(
            _capi.ptr(self.recv_staging), _capi.ptr(self.recv_count), s.hidden, s.num_experts, s.num_ranks,
            s.max_tokens, s.fmt, _capi.ptr(self.packed_recv_x), _capi.ptr(self.packed_recv_scales),
            _capi.ptr(self.packed_recv_src_info), _capi.ptr(self.packed_recv_layout_range),
            _capi.ptr(self.packed_recv_count), _capi.ptr(stats), self.expected_rows,
            _capi.ptr(self.segment_workspace),
            0 if self.segment_workspace is None else self.segment_workspace.numel(), current_stream_ptr()))

    def dispatch(self, x: torch.Tensor, topk_idx: torch.Tensor, stats: torch.Tensor = None) -> None:
        """Send + receive in one call; the peers' rows must already be staged."""
        s = self.shape
        t = x.shape[0]
        sw = self.segment_workspace
        _capi.check(self.lib.deepep_ll_dispatch(
            _capi.ptr(x), _capi.ptr(topk_idx), t, s.hidden, s.num_topk, s.num_experts, s.num_ranks, s.rank,
            s.max_tokens, s.fmt, _capi.ptr(self.recv_staging), _capi.ptr(self.recv_count),
            _capi.ptr(self.send_slots), _capi.ptr(self.send_count), _capi.ptr(self.pair_slot),
            _capi.ptr(self.packed_recv_x), _capi.ptr(self.packed_recv_scales),
            _capi.ptr(self.packed_recv_src_info), _capi.ptr(self.packed_recv_layout_range),
            _capi.ptr(self.packed_recv_count), _capi.ptr(stats), self.expected_rows,
            _capi.ptr(self.workspace), self.workspace.numel(), _capi.ptr(sw), 0 if sw is None else sw.numel(),
            current_stream_ptr()))

    # -- combine ----------------------------------------------------------
    def combine_send(self, x: torch.Tensor, layout_range: torch.Tensor = None) -> None:
        s = self.shape
        lr = self.packed_recv_layout_range if layout_range is None else layout_range
        _capi.check(self.lib.deepep_ll_combine_send(
            _capi.ptr(x), _capi.ptr(lr), s.hidden, s.num_experts, s.num_ranks, s.rank, s.max_tokens,
            _capi.ptr(self.combine_staging), _capi.ptr(self.combine_send_slots), self.expected_rows,
            _capi.ptr(self.segment_workspace),
            0 if self.segment_workspace is None else self.segment_workspace.numel(), current_stream_ptr()))

    def combine_recv(self, topk_idx: torch.Tensor, topk_weights: torch.Tensor, out: torch.Tensor,
                     accumulate: bool = False) -> None:
        s = self.shape
        t = topk_idx.shape[0]
        _capi.check(self.lib.deepep_ll_combine_recv(
            _capi.ptr(self.combine_staging), _capi.ptr(topk_idx), _capi.ptr(topk_weights), _capi.ptr(self.pair_slot),
            t, s.hidden, s.num_topk, s.num_experts, s.max_tokens, int(accumulate), _capi.ptr(out),
            current_stream_ptr()))

    def combine(self, x: torch.Tensor, topk_idx: torch.Tensor, topk_weights: torch.Tensor, out: torch.Tensor,
                layout_range: torch.Tensor = None, accumulate: bool = False, zero_copy: bool = False) -> None:
        """Row return + weighted reduce in one call; the remote experts' answers must already be staged.
        zero_copy: no row return, the transport sends the ranges of layout_range straight from x."""
        s = self.shape
        t = topk_idx.shape[0]
        lr = self.packed_recv_layout_range if layout_range is None else layout_range
        sw = self.segment_workspace
        _capi.check(self.lib.deepep_ll_combine(
            _capi.ptr(x), _capi.ptr(lr), _capi.ptr(topk_idx), _capi.ptr(topk_weights), _capi.ptr(self.pair_slot),
            t, s.hidden, s.num_topk, s.num_experts, s.num_ranks, s.rank, s.max_tokens, int(accumulate),
            _capi.ptr(self.combine_staging), None if zero_copy else _capi.ptr(self.combine_send_slots),
            _capi.ptr(out), self.expected_rows, _capi.ptr(sw), 0 if sw is None else sw.numel(),
            current_stream_ptr()))


def exchange_metadata(all_num_routed: torch.Tensor, rank: int, max_tokens: int, row_capacity: int) -> dict:
    """Send / receive counts, combine offsets and one record per expected row from the gathered
    per-expert route counts [R, E] int32 (csrc/transport/ll_pipeline.cpp:1204-1361), on the current stream."""
    lib = _capi.load()
    r, e = all_num_routed.shape
    dev = all_num_routed.device
    i32 = dict(dtype=torch.int32, device=dev)
    out = dict(send_counts=torch.empty(r, **i32), recv_counts=torch.empty(r, **i32), totals=torch.empty(3, **i32),
               combine_remote_recv_offset=torch.empty(r, dtype=torch.int64, device=dev),
               source_rank=torch.empty(row_capacity, **i32), source_offset=torch.empty(row_capacity, **i32),
               padded_index=torch.empty(row_capacity, **i32), combine_send_offset=torch.empty(row_capacity, **i32),
               num_recv_tokens=torch.empty(2, **i32), tokens_per_expert=torch.empty(e // r, **i32))
    _capi.check(lib.deepep_ll_exchange_metadata(
        _capi.ptr(all_num_routed), e, r, rank, max_tokens, row_capacity, _capi.ptr(out["send_counts"]),
        _capi.ptr(out["recv_counts"]), _capi.ptr(out["totals"]), _capi.ptr(out["combine_remote_recv_offset"]),
        _capi.ptr(out["source_rank"]), _capi.ptr(out["source_offset"]), _capi.ptr(out["padded_index"]),
        _capi.ptr(out["combine_send_offset"]), _capi.ptr(out["num_recv_tokens"]), _capi.ptr(out["tokens_per_expert"]),
        current_stream_ptr()))
    return out


class AllToAllState:
    """Device buffers and C-ABI calls of one rank's low-latency step over a transport that ships one
    contiguous message per peer in each direction (the reference's dist.all_to_all_single branch,
    deep_ep/buffer.py:2266-2301 and :2735).  The transport itself is the caller's: it moves
    ``send_rows[send_cumsum[d]:send_cumsum[d + 1]]`` to row ``rank * slot_rows`` of rank d's
    ``recv_by_source``, and on the way back ``send_flat[first(s):first(s) + recv_counts[s]]`` (first = the
    prefix of ``recv_counts``) to row ``send_cumsum_of_s[rank]`` of rank s's ``recv_flat``.
    """

    def __init__(self, shape: LLShape, slot_rows: int = None, device="cuda"):
        lib = _capi.load()
        self.lib = lib
        self.shape = s = shape
        el, r, m, e, h, k = s.num_local_experts, s.num_ranks, s.max_tokens, s.num_experts, s.hidden, s.num_topk
        self.stride = lib.deepep_ll_row_stride(h, s.fmt)
        u8 = dict(dtype=torch.uint8, device=device)
        i32 = dict(dtype=torch.int32, device=device)
        # dispatch, send side
        self.send_capacity = max(1, min(m * k, e * m))
        self.send_rows = torch.empty((self.send_capacity, self.stride), **u8)
        self.send_count = torch.zeros(e, **i32)
        self.send_expert_prefix = torch.zeros(e + 1, **i32)
        self.send_counts = torch.zeros(r, **i32)
        self.send_cumsum = torch.zeros(r + 1, dtype=torch.int64, device=device)
        self.pair_slot = torch.full((m, k), -1, **i32)
        self.workspace = torch.empty(max(256, lib.deepep_ll_dispatch_workspace_bytes(m, k, e)), **u8)
        # dispatch, receive side: one slot of slot_rows rows per source rank
        self.slot_rows = m * min(k, el) if slot_rows is None else slot_rows
        self.row_capacity = r * self.slot_rows
        self.recv_by_source = torch.empty((self.row_capacity, self.stride), **u8)
        self.by_source_workspace = torch.empty(lib.deepep_ll_by_source_workspace_bytes(e, self.row_capacity), **u8)
        self.record_packed_row = torch.full((self.row_capacity,), -1, **i32)
        self.tokens_per_expert = torch.zeros(el, **i32)
        if s.fmt == ROW_BF16:
            self.packed_recv_x = torch.empty((el, r * m, h), dtype=torch.bfloat16, device=device)
            self.packed_recv_scales = None
        else:
            self.packed_recv_x = torch.empty((el, r * m, h), dtype=torch.float8_e4m3fn, device=device)
            if s.fmt == ROW_FP8_UE8M0:
                self.packed_recv_scales = torch.empty((el, r * m, h // 512), **i32)
            else:
                self.packed_recv_scales = torch.empty((el, r * m, h // 128), dtype=torch.float32, device=device)
        self.packed_recv_count = torch.zeros(el, **i32)
        self.packed_recv_src_info = torch.empty((el, r * m), **i32)
        self.packed_recv_layout_range = torch.zeros((el, r), dtype=torch.int64, device=device)
        # combine: the rows owed to the other ranks in arrival order; the answers in send order
        self.send_flat = torch.empty((self.row_capacity, h), dtype=torch.bfloat16, device=device)
        self.recv_flat = torch.empty((self.send_capacity, h), dtype=torch.bfloat16, device=device)
        self.meta = None
        self.expected_rows = m * k  # what a balanced world delivers; sizes grids, never the result

    def dispatch_send(self, x: torch.Tensor, topk_idx: torch.Tensor) -> None:
        s = self.shape
        _capi.check(self.lib.deepep_ll_dispatch_send_by_dest(
            _capi.ptr(x), _capi.ptr(topk_idx), x.shape[0], s.hidden, s.num_topk, s.num_experts, s.num_ranks, s.rank,
            s.max_tokens, s.fmt, _capi.ptr(self.send_rows), self.send_capacity, _capi.ptr(self.send_count),
            _capi.ptr(self.send_expert_prefix), _capi.ptr(self.send_counts), _capi.ptr(self.send_cumsum),
            _capi.ptr(self.pair_slot), _capi.ptr(self.workspace), self.workspace.numel(), current_stream_ptr()))

    def exchange_metadata(self, all_num_routed: torch.Tensor) -> dict:
        """all_num_routed [R, E] int32: the ranks' send_count, as an all-gather leaves them everywhere."""
        self.meta = exchange_metadata(all_num_routed, self.shape.rank, self.slot_rows, self.row_capacity)
        return self.meta

    def dispatch_recv_ordered(self, all_num_routed: torch.Tensor, stats: torch.Tensor = None) -> None:
        """The receive for messages in this build's own order (what dispatch_send emits): places every row by
        arithmetic on the gathered counts, without the record list and without reading the rows' tails."""
        s = self.shape
        _capi.check(self.lib.deepep_ll_dispatch_recv_by_source_ordered(
            _capi.ptr(self.recv_by_source), self.slot_rows, _capi.ptr(all_num_routed), s.hidden, s.num_experts,
            s.num_ranks, s.rank, s.max_tokens, s.fmt, _capi.ptr(self.packed_recv_x),
            _capi.ptr(self.packed_recv_scales), _capi.ptr(self.packed_recv_src_info),
            _capi.ptr(self.packed_recv_layout_range), _capi.ptr(self.packed_recv_count), _capi.ptr(stats),
            _capi.ptr(self.tokens_per_expert), _capi.ptr(self.record_packed_row), self.row_capacity,
            self.expected_rows, _capi.ptr(self.by_source_workspace), self.by_source_workspace.numel(),
            current_stream_ptr()))

    def dispatch_recv(self, stats: torch.Tensor = None) -> None:
        s, m = self.shape, self.meta
        _capi.check(self.lib.deepep_ll_dispatch_recv_by_source(
            _capi.ptr(self.recv_by_source), self.slot_rows, _capi.ptr(m["recv_counts"]), _capi.ptr(m["source_offset"]),
            _capi.ptr(m["num_recv_tokens"]), self.row_capacity, s.hidden, s.num_experts, s.num_ranks, s.max_tokens,
            s.fmt, _capi.ptr(self.packed_recv_x), _capi.ptr(self.packed_recv_scales),
            _capi.ptr(self.packed_recv_src_info), _capi.ptr(self.packed_recv_layout_range),
            _capi.ptr(self.packed_recv_count), _capi.ptr(stats), _capi.ptr(self.tokens_per_expert),
            _capi.ptr(self.record_packed_row), self.expected_rows, _capi.ptr(self.by_source_workspace),
            self.by_source_workspace.numel(), current_stream_ptr()))

    def combine_send(self, y: torch.Tensor, peer_recv_flat: torch.Tensor = None,
                     peer_recv_rows: torch.Tensor = None) -> None:
        """Rows owed to the other ranks into send_flat, or, with a table of the ranks' recv_flat addresses
        (int64 [R]) and their row counts, straight to their place in those buffers."""
        s, m = self.shape, self.meta
        _capi.check(self.lib.deepep_ll_combine_send_by_dest(
            _capi.ptr(y), _capi.ptr(self.record_packed_row), _capi.ptr(m["source_rank"]), _capi.ptr(m["padded_index"]),
            _capi.ptr(m["combine_send_offset"]), _capi.ptr(m["num_recv_tokens"]), self.row_capacity, s.hidden,
            s.num_experts, s.num_ranks, s.max_tokens, _capi.ptr(self.send_flat), _capi.ptr(m["recv_counts"]),
            _capi.ptr(m["combine_remote_recv_offset"]), _capi.ptr(peer_recv_flat), _capi.ptr(peer_recv_rows),
            self.expected_rows, current_stream_ptr()))

    def combine_recv(self, topk_idx: torch.Tensor, topk_weights: torch.Tensor, out: torch.Tensor,
                     recv: torch.Tensor = None, slot_rows: int = 0, accumulate: bool = False) -> None:
        s = self.shape
        buf = self.recv_flat if recv is None else recv
        _capi.check(self.lib.deepep_ll_combine_recv_flat(
            _capi.ptr(buf), buf.shape[0], slot_rows, _capi.ptr(self.send_expert_prefix), _capi.ptr(topk_idx),
            _capi.ptr(topk_weights), _capi.ptr(self.pair_slot), topk_idx.shape[0], s.hidden, s.num_topk,
            s.num_experts, s.num_ranks, s.max_tokens, int(accumulate), _capi.ptr(out), current_stream_ptr()))
