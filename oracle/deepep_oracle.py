"""CPU oracle of the MoE token dispatch/combine hot path.

TEST INFRASTRUCTURE ONLY.  This module restates, on the CPU with torch and
numpy, what the reference computes on this path; it is the checker for the
HIP kernels and the timed CPU baseline of ``bench.py``.  Nothing in the
product package imports it, and the product never falls back to it.

Every function names the reference lines it follows.  What pins each one
(the reference stores no golden vectors for this path; its tests are
generative on CUDA RNG streams that cannot be replayed here):

* layout counts, ``is_token_in_rank``  — brute force over tiny inputs written as
  literal Python loops, and the closed forms of ``tests/test_intranode.py:35-66``.
* FP8 cast — follows the live CUDA kernel (``csrc/kernels/efa_kernels.cu:156-169``:
  ``scale = amax / 448.0f``, ``inv = 448.0f / amax``, IEEE float32 division; nvcc
  flags in ``setup.py:12-13`` carry no fast-math).  The reference's torch helpers
  (``deep_ep/buffer.py:1602``, ``tests/utils.py:57``) write ``448.0 / amax``, which
  torch evaluates as ``amax.reciprocal() * 448.0`` — one ulp off for ~27 % of amax
  values, and therefore a different FP8 byte for the rare element that lands on
  a rounding tie.  ``per_token_cast_to_fp8_torch_helper`` keeps that form so the
  difference stays measured (``tests/test_oracle.py``).  Pinned by torch's own
  ``float8_e4m3fn`` CPU cast (a library routine), an
  independent bit-level encoder in ``oracle_kernels.c`` run over every float32
  that a bf16 x scale product can produce in the tests, and special cases
  (all-zero group, exact powers of two, ±448 saturation, -0).
* dispatch outputs — the invariants ``tests/test_low_latency.py:119-147``
  checks, plus a literal serial restatement of the reference's deterministic
  kernels (``_serial_dispatch``) compared against the vectorised form.
* combine — the closed form ``x * sum(w)`` of ``tests/test_low_latency.py:181``
  and a float64 sum.
* layout, route slots, dispatch outputs and the combine — also a
  two-rank world worked out on paper, ``tests/golden/ll_tiny_world.json``.
* ``topk_remap``, ``build_recv_src_meta`` — the torch expressions the reference's kernels
  replaced (named in their headers, ``csrc/kernels/efa_kernels.cu:321-337,438-446``), pinned
  by literal Python loops over the kernels' own per-element rule.
* ``combine_reduce`` — ``zero_() + index_add_`` (``deep_ep/buffer.py:1542-1557``) in float64,
  the identity "one rank per token returns the row itself", and a float32 chain in rank order.
* ``ll_exchange_metadata`` — the reference's host loops restated loop for loop; pinned by the
  hand-derived two-rank world (``tests/golden/ll_tiny_world.json``) and by the identities that tie it to
  the dispatch (recv_counts = row sums of the receiver's ``recv_count``; records = a running index).
* ``ll_send_by_dest``, ``ll_record_packed_rows``, ``ll_combine_send_by_dest``, ``ll_combine_recv_flat_rows`` — the
  hand-derived two-rank world (``tests/golden/ll_tiny_world.json``: message order, per-record packed rows,
  the flat buffers of both directions) and, on hypothesis-drawn tiny worlds, the round trip through literal
  message copies: with identity experts every pair must get back exactly the row its token sent, and the
  per-record rows must point at what ``ll_dispatch`` put there.
* ``get_low_latency_rdma_size_hint`` — hand-computed values.
* ``round_scale`` scales — the reference computes ``exp2(ceil(log2(s)))`` in float32
  (``deep_ep/buffer.py:1601``, ``csrc/kernels/efa_kernels.cu:158``); this oracle (and the kernel)
  take the smallest power of two >= s from the bit pattern.  The two could differ only for s
  within a few ulps above a power of two, where log2f's rounding decides the ceiling; on this
  path s = amax / 448 with amax a bf16 value or the 1e-4 clamp, and over every such amax log2(s) is
  an integer exactly or at least 0.006 away from one, so every libm gives the same answer.
  Pinned by that enumeration and by torch's float32 log2 / ceil / exp2 on the CPU agreeing on all of
  them (``tests/test_oracle.py::test_round_scale_has_one_answer_for_every_bf16_amax``).
"""
from __future__ import annotations

import numpy as np
import torch

FP8_MAX = 448.0
GROUP = 128

ROW_BF16, ROW_FP8, ROW_FP8_POW2, ROW_FP8_UE8M0 = 0, 1, 2, 3


# ----------------------------------------------------------------------------
# Sizes
# ----------------------------------------------------------------------------
def align_up(a: int, b: int) -> int:
    return (a + b - 1) // b * b


def get_low_latency_rdma_size_hint(num_max_dispatch_tokens_per_rank: int, hidden: int, num_ranks: int,
                                   num_experts: int) -> int:
    """csrc/config.hpp:127-193 (LowLatencyLayout + get_low_latency_rdma_size_hint)."""
    num_scales = hidden // 128
    dispatch_msg = 16 + max(hidden * 2, hidden + num_scales * 4)
    combine_msg = num_scales * 4 + hidden * 2
    m, e = num_max_dispatch_tokens_per_rank, num_experts
    send = max(m * dispatch_msg, e * m * combine_msg)
    recv = max(e * m * dispatch_msg, e * m * combine_msg)
    sig = align_up(e * 4, 128)
    total = send * 2 + recv * 2 + sig * 2
    return (total + 128) // 128 * 128


def row_data_bytes(hidden: int, fmt: int) -> int:
    return hidden * 2 if fmt == ROW_BF16 else hidden


def row_scale_bytes(hidden: int, fmt: int) -> int:
    if fmt == ROW_BF16:
        return 0
    g = hidden // GROUP
    return g if fmt == ROW_FP8_UE8M0 else 4 * g


def row_payload(hidden: int, fmt: int) -> int:
    """data and scales padded to 16 B + 16 B tail (csrc/kernels/coop_dispatch_send.cu:73-75)."""
    return align_up(row_data_bytes(hidden, fmt), 16) + align_up(row_scale_bytes(hidden, fmt), 16) + 16


def row_stride(hidden: int, fmt: int) -> int:
    """Distance between staged rows: the payload rounded up to whole 128-byte cache lines (this build's
    choice; the bytes behind the tail are never written)."""
    return align_up(row_payload(hidden, fmt), 128)


# ----------------------------------------------------------------------------
# Layout
# ----------------------------------------------------------------------------
def get_dispatch_layout(topk_idx: torch.Tensor, num_experts: int, num_ranks: int):
    """csrc/kernels/layout.cu:9-121; recipe of tests/test_intranode.py:35-66.

    Returns (num_tokens_per_rank i32 [R], num_tokens_per_rdma_rank i32 [R/8] or None,
    num_tokens_per_expert i32 [E], is_token_in_rank bool [T, R]).
    """
    t = topk_idx.shape[0]
    epr = num_experts // num_ranks
    valid = (topk_idx >= 0) & (topk_idx < num_experts)
    flat = topk_idx[valid]
    per_expert = torch.bincount(flat, minlength=num_experts).to(torch.int32)
    is_in = torch.zeros((t, num_ranks), dtype=torch.bool)
    tok = torch.arange(t).view(-1, 1).expand_as(topk_idx)[valid]
    is_in[tok, flat // epr] = True
    per_rank = is_in.sum(0).to(torch.int32)
    per_rdma = None
    if num_ranks > 8 and num_ranks % 8 == 0:
        per_rdma = is_in.view(t, num_ranks // 8, 8).any(-1).sum(0).to(torch.int32)
    return per_rank, per_rdma, per_expert, is_in


def moe_routing_sort(is_token_in_rank: torch.Tensor):
    """csrc/kernels/efa_kernels.cu:220-318,1591-1651: ids ascending inside each rank."""
    t, r = is_token_in_rank.shape
    rank_of, tok_of = torch.nonzero(is_token_in_rank.t().contiguous(), as_tuple=True)
    counts = is_token_in_rank.sum(0).to(torch.int32)
    cumsum = torch.zeros(r + 1, dtype=torch.int64)
    cumsum[1:] = torch.cumsum(counts.to(torch.int64), 0)
    return tok_of.to(torch.int64), counts, cumsum, int(cumsum[-1])


def channel_prefix_matrix(is_token_in_rank: torch.Tensor, num_channels: int) -> torch.Tensor:
    """csrc/kernels/intranode.cu:90-112 with the ranges of csrc/kernels/utils.cuh:434-438."""
    t, r = is_token_in_rank.shape
    per = (t + num_channels - 1) // num_channels
    out = torch.zeros((r, num_channels), dtype=torch.int32)
    for c in range(num_channels):
        b = min(per * c, t)
        e = min(b + per, t)
        out[:, c] = is_token_in_rank[b:e].sum(0).to(torch.int32)
    return torch.cumsum(out, 1).to(torch.int32)


# ----------------------------------------------------------------------------
# Normal mode: the steps either side of the per-rank pack
# ----------------------------------------------------------------------------
def topk_remap(topk_idx: torch.Tensor, topk_weights: torch.Tensor, sorted_token_ids: torch.Tensor,
               send_cumsum: torch.Tensor, num_local_experts: int):
    """csrc/kernels/efa_kernels.cu:339-387, written as the torch expression that kernel replaced
    (repeat_interleave + broadcast compare + where, :323): per send row, the token's top-k in the
    destination rank's expert numbering; entries naming other ranks' experts become (-1, 0.0)."""
    r = send_cumsum.numel() - 1
    counts = (send_cumsum[1:] - send_cumsum[:-1]).to(torch.int64)
    total = int(send_cumsum[r])
    dst = torch.repeat_interleave(torch.arange(r, dtype=torch.int64), counts)
    ids = sorted_token_ids[:total].to(torch.int64)
    e = topk_idx[ids]
    w = topk_weights[ids]
    first = (dst * num_local_experts).view(-1, 1)
    ok = (e >= first) & (e < first + num_local_experts)
    return torch.where(ok, e - first, torch.full_like(e, -1)), torch.where(ok, w, torch.zeros_like(w))


def build_recv_src_meta(recv_cumsum: torch.Tensor, num_local_ranks: int) -> torch.Tensor:
    """csrc/kernels/efa_kernels.cu:448-482 as the expression it replaced (repeat_interleave +
    division + shift, :440): [N, 8] uint8 holding the int32 pair (src // L, 1 << (src % L))."""
    r = recv_cumsum.numel() - 1
    counts = (recv_cumsum[1:] - recv_cumsum[:-1]).to(torch.int64)
    src = torch.repeat_interleave(torch.arange(r, dtype=torch.int64), counts)
    meta = torch.stack([src // num_local_ranks, torch.ones_like(src) << (src % num_local_ranks)], dim=1)
    return meta.to(torch.int32).contiguous().view(torch.uint8).view(-1, 8)


def combine_reduce(recv_x: torch.Tensor, recv_w, sorted_token_ids: torch.Tensor, num_tokens: int,
                   bias_0=None, bias_1=None):
    """deep_ep/buffer.py:1542-1557 in float64: zeros, index_add_ of the returned rows at their token
    ids, then the biases.  Returns (x float64 [T, H], w float64 [T, K] or None)."""
    total = sorted_token_ids.numel()
    out = torch.zeros((num_tokens, recv_x.shape[1]), dtype=torch.float64)
    out.index_add_(0, sorted_token_ids.to(torch.int64), recv_x[:total].double())
    for b in (bias_0, bias_1):
        if b is not None:
            out += b.double()
    w = None
    if recv_w is not None:
        w = torch.zeros((num_tokens, recv_w.shape[1]), dtype=torch.float64)
        w.index_add_(0, sorted_token_ids.to(torch.int64), recv_w[:total].double())
    return out, w


def combine_reduce_f32_chain(recv_x: torch.Tensor, recv_w, sorted_token_ids: torch.Tensor,
                             send_cumsum: torch.Tensor, num_tokens: int, bias_0=None, bias_1=None):
    """The bit-level definition the kernel implements: float32 adds in ascending rank order (a token
    occurs at most once per rank segment, so a per-segment indexed add is that order exactly), the
    biases last, one rounding to bf16; weights the same way without the rounding."""
    r = send_cumsum.numel() - 1
    acc = torch.zeros((num_tokens, recv_x.shape[1]), dtype=torch.float32)
    wacc = None if recv_w is None else torch.zeros((num_tokens, recv_w.shape[1]), dtype=torch.float32)
    for rank in range(r):
        lo, hi = int(send_cumsum[rank]), int(send_cumsum[rank + 1])
        ids = sorted_token_ids[lo:hi].to(torch.int64)
        acc[ids] = acc[ids] + recv_x[lo:hi].float()
        if wacc is not None:
            wacc[ids] = wacc[ids] + recv_w[lo:hi]
    for b in (bias_0, bias_1):
        if b is not None:
            acc = acc + b.float()
    return acc.to(torch.bfloat16), wacc


# ----------------------------------------------------------------------------
# FP8
# ----------------------------------------------------------------------------
def pow2_ceil(s: torch.Tensor) -> torch.Tensor:
    """Smallest power of two >= s for positive normal float32 (bit arithmetic)."""
    bits = s.contiguous().view(torch.int32)
    ex = (bits >> 23) & 0xFF
    ex = ex + ((bits & 0x7FFFFF) != 0).to(torch.int32)
    return (ex << 23).view(torch.float32)


def per_token_cast_to_fp8(x: torch.Tensor, round_scale: bool = False, use_ue8m0: bool = False):
    """deep_ep/buffer.py:1590-1621 and csrc/kernels/efa_kernels.cu:143-185.

    x [M, N] bf16 -> (x_fp8 [M, N] float8_e4m3fn, scales [M, N/128] f32 | [M, N/512] i32).
    """
    assert x.dim() == 2 and x.shape[1] % GROUP == 0
    m, n = x.shape
    xg = x.view(m, n // GROUP, GROUP).float()
    amax = xg.abs().amax(dim=2).clamp(min=1e-4)
    scales = amax / FP8_MAX
    if round_scale:
        scales = pow2_ceil(scales)
        inv = torch.ones_like(scales) / scales  # exact: scales are powers of two
    else:
        inv = torch.full_like(amax, FP8_MAX) / amax  # tensor / tensor: IEEE division, as 448.0f / amax
    q = (xg * inv.unsqueeze(2)).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn).view(m, n)
    if use_ue8m0:
        assert round_scale and (n // GROUP) % 4 == 0
        ex = ((scales.contiguous().view(torch.int32) >> 23) & 0xFF).to(torch.uint8)
        return q, ex.view(m, n // GROUP // 4, 4).contiguous().view(torch.int32).view(m, n // GROUP // 4)
    return q, scales


def per_token_cast_to_fp8_torch_helper(x: torch.Tensor):
    """tests/utils.py:50-58 verbatim in meaning: ``448.0 / amax`` is reciprocal-then-multiply in torch."""
    m, n = x.shape
    xv = x.view(m, -1, GROUP)
    amax = xv.abs().float().amax(dim=2).view(m, -1).clamp(1e-4)
    return (xv * (448.0 / amax.unsqueeze(2))).to(torch.float8_e4m3fn).view(m, n), (amax / 448.0).view(m, -1)


def per_token_cast_back(x_fp8: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """tests/utils.py:61-74."""
    if x_fp8.numel() == 0:
        return x_fp8.to(torch.bfloat16)
    m, n = x_fp8.shape
    if scales.dtype == torch.int32:
        scales = (scales.contiguous().view(torch.uint8).to(torch.int32) << 23).view(torch.float32)
    xf = x_fp8.to(torch.float32).view(m, -1, GROUP)
    return (xf * scales.reshape(m, -1, 1)).view(m, n).to(torch.bfloat16)


def quantise_rows(x: torch.Tensor, fmt: int):
    """Payload bytes [T, data_bytes] u8 and scale bytes [T, scale_bytes] u8 of each token row."""
    t = x.shape[0]
    if t == 0:
        return (torch.zeros((0, row_data_bytes(x.shape[1], fmt)), dtype=torch.uint8),
                torch.zeros((0, row_scale_bytes(x.shape[1], fmt)), dtype=torch.uint8))
    if fmt == ROW_BF16:
        return x.contiguous().view(torch.uint8).view(t, x.shape[1] * 2), torch.zeros((t, 0), dtype=torch.uint8)
    q, s = per_token_cast_to_fp8(x, round_scale=fmt != ROW_FP8, use_ue8m0=fmt == ROW_FP8_UE8M0)
    return q.view(torch.uint8).view(t, x.shape[1]), s.contiguous().view(torch.uint8).view(t, row_scale_bytes(x.shape[1], fmt))


# ----------------------------------------------------------------------------
# Low-latency dispatch
# ----------------------------------------------------------------------------
def route(topk_idx: torch.Tensor, num_experts: int, max_tokens: int):
    """Send-side routing of one rank.

    send_count[e] = pairs (t,k) naming expert e (csrc/kernels/coop_dispatch_send.cuh:360-395
    num_routed); pair_slot[t,k] = rank of the pair among this rank's pairs for
    that expert in ascending (t,k) order — the order of the reference's serial
    scan (csrc/kernels/efa_kernels.cu:617-637).  Pairs beyond max_tokens are dropped.
    """
    t, k = topk_idx.shape
    flat = topk_idx.reshape(-1)
    valid = (flat >= 0) & (flat < num_experts)
    idx = torch.nonzero(valid).view(-1)
    e = flat[idx]
    order = torch.sort(e, stable=True).indices
    e_sorted = e[order]
    counts = torch.bincount(e_sorted, minlength=num_experts)
    starts = torch.cumsum(counts, 0) - counts
    slot_sorted = torch.arange(e_sorted.numel()) - starts[e_sorted]
    pair_slot = torch.full((t * k,), -1, dtype=torch.int32)
    pair_slot[idx[order]] = slot_sorted.to(torch.int32)
    pair_slot[pair_slot >= max_tokens] = -1
    send_count = counts.clamp(max=max_tokens).to(torch.int32)
    return send_count, pair_slot.view(t, k)


def ll_dispatch(all_x, all_topk_idx, rank: int, num_experts: int, max_tokens: int, fmt: int = ROW_FP8):
    """What rank `rank` receives when every rank of the world dispatches.

    Inside each expert's packed range the source ranks come in ascending order:
    begin(e, s) = sum of cnt(e, s') over s' < s, the serial prefix of the reference's range
    builders (csrc/kernels/efa_kernels.cu:991-1010 and :1031-1050).  Its atomics only decide
    the order of the rows inside one (expert, source) segment (:1227-1389); here that order is
    the sender's ascending (token, k) order, as in its deterministic scatter.

    all_x: list of R tensors [T_s, H] bf16; all_topk_idx: list of R tensors [T_s, K] int64.
    Follows deep_ep/buffer.py:1816-1887,2266-2457 (nccl-fallback branch) with
    ll_recv_build_positions (csrc/kernels/efa_kernels.cu:1017-1052) for the
    ranges and the deterministic scatter (:1059-1213) for the slot order.

    Returns dict with packed_recv_x u8 [E_l, N, data_bytes], packed_recv_scales u8
    [E_l, N, scale_bytes], packed_recv_count i32 [E_l], packed_recv_src_info i32
    [E_l, N], packed_recv_layout_range i64 [E_l, R]; rows past the count are zero.
    """
    r = len(all_x)
    epr = num_experts // r
    n = max_tokens * r
    hidden = all_x[0].shape[1]
    db, sb = row_data_bytes(hidden, fmt), row_scale_bytes(hidden, fmt)
    px = torch.zeros((epr, n, db), dtype=torch.uint8)
    ps = torch.zeros((epr, n, sb), dtype=torch.uint8)
    src_info = torch.zeros((epr, n), dtype=torch.int32)
    layout = torch.zeros((epr, r), dtype=torch.int64)
    count = torch.zeros(epr, dtype=torch.int32)
    cursor = [0] * epr
    per_src = []
    for s in range(r):
        _, pair_slot = route(all_topk_idx[s], num_experts, max_tokens)
        data, scales = quantise_rows(all_x[s], fmt)
        per_src.append((pair_slot, data, scales))
    for le in range(epr):
        e = rank * epr + le
        for s in range(r):
            pair_slot, data, scales = per_src[s]
            sel = (all_topk_idx[s] == e) & (pair_slot >= 0)
            tok, kk = torch.nonzero(sel, as_tuple=True)
            slots = pair_slot[tok, kk].to(torch.int64)
            c = int(tok.numel())
            if c:
                b = cursor[le]
                px[le, b + slots] = data[tok]
                if sb:
                    ps[le, b + slots] = scales[tok]
                src_info[le, b + slots] = tok.to(torch.int32)
                layout[le, s] = (b << 32) | c
                cursor[le] += c
        count[le] = cursor[le]
    return dict(packed_recv_x=px, packed_recv_scales=ps, packed_recv_count=count,
                packed_recv_src_info=src_info, packed_recv_layout_range=layout)


def _serial_dispatch(all_x, all_topk_idx, rank: int, num_experts: int, max_tokens: int, fmt: int = ROW_FP8):
    """Literal restatement, in Python loops, of the reference's deterministic kernels:
    sender scan csrc/kernels/efa_kernels.cu:617-637 (per destination rank, (t,k) order),
    receiver count/build :877-923,1017-1052 and scatter :1112-1141 (arrival order per
    source, position = pair_cumsum + running pair counter).  Small inputs only."""
    r = len(all_x)
    epr = num_experts // r
    n = max_tokens * r
    hidden = all_x[0].shape[1]
    db, sb = row_data_bytes(hidden, fmt), row_scale_bytes(hidden, fmt)
    arrivals = []  # per source: list of (token, local_eid) in send order
    for s in range(r):
        rows = []
        tk = all_topk_idx[s].tolist()
        for t, row in enumerate(tk):
            for e in row:
                if e >= 0 and e // epr == rank:
                    rows.append((t, e % epr))
        arrivals.append(rows)
    pair_counts = [[0] * r for _ in range(epr)]
    for s in range(r):
        for _, le in arrivals[s]:
            pair_counts[le][s] += 1
    px = torch.zeros((epr, n, db), dtype=torch.uint8)
    ps = torch.zeros((epr, n, sb), dtype=torch.uint8)
    src_info = torch.zeros((epr, n), dtype=torch.int32)
    layout = torch.zeros((epr, r), dtype=torch.int64)
    count = torch.zeros(epr, dtype=torch.int32)
    pair_cumsum = [[0] * r for _ in range(epr)]
    for le in range(epr):
        pos = 0
        for s in range(r):
            c = pair_counts[le][s]
            pair_cumsum[le][s] = pos
            layout[le, s] = ((pos << 32) | c) if c > 0 else 0
            pos += c
        count[le] = pos
    for s in range(r):
        data, scales = quantise_rows(all_x[s], fmt)
        written = [0] * epr
        for t, le in arrivals[s]:
            p = pair_cumsum[le][s] + written[le]
            written[le] += 1
            px[le, p] = data[t]
            if sb:
                ps[le, p] = scales[t]
            src_info[le, p] = t
    return dict(packed_recv_x=px, packed_recv_scales=ps, packed_recv_count=count,
                packed_recv_src_info=src_info, packed_recv_layout_range=layout)


def staged_rows(x: torch.Tensor, topk_idx: torch.Tensor, src_rank: int, num_experts: int, max_tokens: int,
                fmt: int, num_ranks: int):
    """Rows one rank emits, keyed (expert, slot) -> stride-sized row bytes, as the
    send side stages them: [data|pad][scales|pad][token, k, src_rank, local expert] (the reference's
    packed rows end in [token, local_eid], csrc/kernels/efa_kernels.cu:797-800)."""
    hidden = x.shape[1]
    db, sb = row_data_bytes(hidden, fmt), row_scale_bytes(hidden, fmt)
    dp, sp = align_up(db, 16), align_up(sb, 16)
    stride = row_stride(hidden, fmt)
    send_count, pair_slot = route(topk_idx, num_experts, max_tokens)
    data, scales = quantise_rows(x, fmt)
    tok, kk = torch.nonzero(pair_slot >= 0, as_tuple=True)
    rows = torch.zeros((tok.numel(), stride), dtype=torch.uint8)
    rows[:, :db] = data[tok]
    if sb:
        rows[:, dp:dp + sb] = scales[tok]
    experts_per_rank = num_experts // num_ranks
    local = (topk_idx[tok, kk] % experts_per_rank).to(torch.int32)
    tail = torch.stack([tok.to(torch.int32), kk.to(torch.int32), torch.full_like(tok, src_rank, dtype=torch.int32),
                        local], 1).contiguous()
    rows[:, dp + sp:dp + sp + 16] = tail.view(torch.uint8).view(-1, 16)
    experts = topk_idx[tok, kk]
    slots = pair_slot[tok, kk].to(torch.int64)
    return send_count, pair_slot, experts, slots, rows


# ----------------------------------------------------------------------------
# Low-latency path over an all-to-all shaped transport: one contiguous message per peer in both
# directions (deep_ep/buffer.py:2266-2301 dispatch, :2601-2608 and :2735 combine)
# ----------------------------------------------------------------------------
def ll_send_by_dest(x: torch.Tensor, topk_idx: torch.Tensor, src_rank: int, num_experts: int, max_tokens: int,
                    fmt: int, num_ranks: int):
    """The rows one rank sends, as ONE buffer that is contiguous per destination rank.

    csrc/kernels/efa_kernels.cu:2332-2400 (ll_dispatch_route_and_pack_v3): send_counts[r] = pairs whose
    expert lives on rank r, send_cumsum = their exclusive prefix (int64, [R] = total), rows grouped by
    destination rank in send_cumsum order, every row ending in its [token, local expert] (:797-800).
    Inside one destination's message the reference's live kernel leaves the order to an atomic
    (rank_write_pos, :2378-2380); this build's order is by expert, then by the pair's slot (ascending
    (token, k) inside an expert), i.e. the per-expert send slots laid end to end.  A row's place is then
    send_expert_prefix[expert] + pair_slot, with send_expert_prefix the exclusive prefix of send_count.
    Returns dict(send_count i32 [E], send_expert_prefix i32 [E+1], send_counts i32 [R], send_cumsum i64 [R+1],
    pair_slot i32 [T, K], pair_send_row i32 [T, K] (-1 = not sent), rows u8 [P, stride]).
    """
    epr = num_experts // num_ranks
    send_count, pair_slot, experts, slots, rows = staged_rows(x, topk_idx, src_rank, num_experts, max_tokens, fmt,
                                                              num_ranks)
    prefix = torch.zeros(num_experts + 1, dtype=torch.int64)
    prefix[1:] = torch.cumsum(send_count.to(torch.int64), 0)
    place = prefix[experts] + slots
    out = torch.zeros_like(rows)
    out[place] = rows
    pair_send_row = torch.full(topk_idx.shape, -1, dtype=torch.int32)
    tok, kk = torch.nonzero(pair_slot >= 0, as_tuple=True)
    pair_send_row[tok, kk] = place.to(torch.int32)
    send_counts = send_count.view(num_ranks, epr).sum(1).to(torch.int32)
    return dict(send_count=send_count, send_expert_prefix=prefix.to(torch.int32), send_counts=send_counts,
                send_cumsum=prefix[::epr].clone(), pair_slot=pair_slot, pair_send_row=pair_send_row, rows=out)


def ll_record_packed_rows(all_topk_idx, rank: int, num_experts: int, max_tokens: int):
    """For every row rank `rank` receives, in arrival order (source ranks ascending, inside a source the
    order of that source's message, ll_send_by_dest): the packed row the receive side gives it,
    local_expert * N + begin(expert, source) + its place among that pair's rows, N = R * max_tokens.

    This is the per-row bookkeeping the reference's receive kernel leaves for the combine:
    recv_expert_ids / recv_expert_pos of ll_recv_unpack_v2 (csrc/kernels/efa_kernels.cu:2121-2231,
    scatter :1227-1389), which deep_ep/buffer.py:2601 uses as x[recv_expert_ids, recv_expert_pos].
    Literal loops; returns int64 [rows received].
    """
    r = len(all_topk_idx)
    epr = num_experts // r
    n = max_tokens * r
    cnt = [[0] * r for _ in range(epr)]
    per_source = []
    for s in range(r):
        send_count, pair_slot = route(all_topk_idx[s], num_experts, max_tokens)
        msg = []  # (local expert, slot) in message order: expert by expert, slots ascending
        for le in range(epr):
            c = int(send_count[rank * epr + le])
            cnt[le][s] = c
            msg += [(le, j) for j in range(c)]
        per_source.append(msg)
    out = []
    for s in range(r):
        for le, j in per_source[s]:
            begin = sum(cnt[le][:s])
            out.append(le * n + begin + j)
    return torch.tensor(out, dtype=torch.int64)


def ll_combine_send_by_dest(y: torch.Tensor, record_packed_row: torch.Tensor, padded_index: torch.Tensor,
                            combine_send_offset: torch.Tensor) -> torch.Tensor:
    """The expert outputs owed to the other ranks as one flat [Rv, H] buffer in arrival order, which is
    contiguous per destination rank: flat[combine_send_offset[i]] = y_rows[record_packed_row[padded_index[i]]].

    deep_ep/buffer.py:2601-2608 (x[recv_expert_ids, recv_expert_pos] un-sorted to arrival order) and
    csrc/kernels/coop_combine_send.cuh:37-170 (send_buffer[combine_send_offset[i]] = expert_x[padded_index[i]]).
    y [E_l, N, H] bf16.  Records whose row is -1 leave their flat row zero.
    """
    h = y.shape[-1]
    rows = y.reshape(-1, h)
    n = combine_send_offset.numel()
    flat = torch.zeros((n, h), dtype=y.dtype)
    for i in range(n):
        src = int(record_packed_row[int(padded_index[i])])
        if src >= 0:
            flat[int(combine_send_offset[i])] = rows[src]
    return flat


def ll_combine_recv_flat_rows(recv_flat: torch.Tensor, slot_rows: int, send_expert_prefix: torch.Tensor,
                              topk_idx: torch.Tensor, pair_slot: torch.Tensor, experts_per_rank: int):
    """pair_rows[t, k] = the row of the returned buffer that answers pair (t, k), and which pairs are live.

    The buffer holds one row per row sent, in send order (ll_send_by_dest), either flat (slot_rows == 0) or
    with the rows from rank r starting at row r * slot_rows: csrc/kernels/efa_kernels.cu:1449-1466 (src_rank
    from send_cumsum, within_rank = send_idx - send_cumsum[src_rank], byte offset src_rank * slot_size +
    within_rank * hidden * 2, or send_idx * hidden when flat).
    """
    t, k = topk_idx.shape
    h = recv_flat.shape[-1]
    live = pair_slot >= 0
    pair_rows = torch.zeros((t, k, h), dtype=recv_flat.dtype)
    for ti in range(t):
        for ki in range(k):
            if not live[ti, ki]:
                continue
            e = int(topk_idx[ti, ki])
            send_idx = int(send_expert_prefix[e]) + int(pair_slot[ti, ki])
            if slot_rows > 0:
                src_rank = e // experts_per_rank
                within = send_idx - int(send_expert_prefix[src_rank * experts_per_rank])
                send_idx = src_rank * slot_rows + within
            pair_rows[ti, ki] = recv_flat[send_idx]
    return pair_rows, live


# ----------------------------------------------------------------------------
# Low-latency combine
# ----------------------------------------------------------------------------
def ll_exchange_metadata(all_num_routed: torch.Tensor, rank: int, max_tokens: int):
    """The host-side bookkeeping between the route-count gather and the exchange, loop for loop.

    all_num_routed [R, E] int: row s = pairs rank s routed to each expert.
    compute_send_recv_counts (csrc/transport/ll_pipeline.cpp:1204-1269): any count above the
    per-expert bound (max_tokens, 4096 if that is not positive) zeroes every send and receive count;
    otherwise send[r] = sum of this rank's row over rank r's experts, recv[r] = sum of rank r's row
    over this rank's experts.
    upload_recv_metadata (:1277-1361): combine_remote_recv_offset[j] = what peer j routed to the
    ranks below this one; per expected row, grouped by source rank: (source_rank, source_offset =
    r * max_tokens + t, padded_index = running index, combine_send_offset = rows of lower sources + t);
    a total outside [0, R * max_tokens * 8] receives nothing.
    Returns a dict of int64 tensors / ints under the reference's names.
    """
    num_ranks, num_experts = all_num_routed.shape
    epr = num_experts // num_ranks
    routed = all_num_routed.to(torch.int64) & 0xFFFFFFFF  # the reference reads them as uint32
    bound = max_tokens if max_tokens > 0 else 4096
    send = [0] * num_ranks
    recv = [0] * num_ranks
    corrupt = bool((routed > bound).any())
    if not corrupt:
        for e in range(num_experts):
            send[e // epr] += int(routed[rank, e])
        for r in range(num_ranks):
            for e in range(rank * epr, (rank + 1) * epr):
                recv[r] += int(routed[r, e])
    total_send, total_recv = sum(send), sum(recv)
    remote = []
    for j in range(num_ranks):
        off = 0
        for r in range(rank):
            for e in range(r * epr, (r + 1) * epr):
                off += int(routed[j, e])
        remote.append(off)
    if total_recv < 0 or total_recv > num_ranks * max_tokens * 8:
        total_recv = 0
    src_rank, src_off, padded, comb = [], [], [], []
    group = [0] * num_ranks
    acc = 0
    for r in range(num_ranks):
        group[r] = acc
        acc += recv[r]
    idx = 0
    if total_recv:
        for r in range(num_ranks):
            for t in range(recv[r]):
                src_rank.append(r)
                src_off.append(r * max_tokens + t)
                padded.append(idx)
                comb.append(group[r] + t)
                idx += 1
    as_t = lambda v: torch.tensor(v, dtype=torch.int64)
    return dict(send_counts=as_t(send), recv_counts=as_t(recv), total_send=total_send, total_recv=total_recv,
                corrupt=corrupt, combine_remote_recv_offset=as_t(remote), source_rank=as_t(src_rank),
                source_offset=as_t(src_off), padded_index=as_t(padded), combine_send_offset=as_t(comb))


def ll_combine(pair_rows: torch.Tensor, topk_idx: torch.Tensor, topk_weights: torch.Tensor,
               pair_live: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = sum_k [live] w[t,k] * f32(pair_rows[t,k]) in float64, rounded to bf16 by the caller's check.

    pair_rows [T, K, H] bf16 — the expert output returned for each pair.
    csrc/kernels/efa_kernels.cu:1413-1474 (weight lookup + accumulate) and
    csrc/kernels/coop_combine_recv.cuh:222-260 (per-pair, k order).  Returns float64 [T, H].
    """
    live = (topk_idx >= 0) if pair_live is None else pair_live
    w = topk_weights.double() * live.double()
    return (pair_rows.double() * w.unsqueeze(-1)).sum(1)


def ll_combine_f32_chain(pair_rows: torch.Tensor, topk_weights: torch.Tensor, pair_live: torch.Tensor,
                         initial: torch.Tensor = None):
    """Bit-level definition: acc = 0; for k: acc = fma(f32(row_k), w_k, acc); bf16_rne(acc).
    `initial` [T, H] bf16: the accumulate variant (csrc/kernels/coop_combine_recv.cuh:174-179),
    acc starts as f32(initial) instead of zero.

    float32 FMA emulated exactly: the product of two float32 is exact in float64;
    the float64 sum with a float32 addend is rounded once to float64 and once more
    to float32 — double rounding can differ from a true FMA only when the float64
    result sits exactly on a float32 rounding boundary, which the C checker
    (oracle_kernels.c, fmaf) covers; this torch form is used for speed.
    """
    t, k, h = pair_rows.shape
    acc = torch.zeros((t, h), dtype=torch.float32) if initial is None else initial.float().clone()
    for j in range(k):
        prod = pair_rows[:, j].double() * topk_weights[:, j].double().unsqueeze(1)
        nxt = (prod + acc.double()).float()
        acc = torch.where(pair_live[:, j].unsqueeze(1), nxt, acc)
    return acc.to(torch.bfloat16)


def calc_diff(x: torch.Tensor, y: torch.Tensor) -> float:
    """tests/utils.py:39-43."""
    x, y = x.double() + 1, y.double() + 1
    den = (x * x + y * y).sum()
    return float(1 - 2 * (x * y).sum() / den)


# ----------------------------------------------------------------------------
# Seeded world (mirrors the synthesiser kernels; integer hashing + exact float32 steps)
# ----------------------------------------------------------------------------
_M32 = np.uint64(0xFFFFFFFF)


def mix32(x):
    x = np.asarray(x, dtype=np.uint64) & _M32
    x ^= x >> np.uint64(16)
    x = (x * np.uint64(0x7FEB352D)) & _M32
    x ^= x >> np.uint64(15)
    x = (x * np.uint64(0x846CA68B)) & _M32
    x ^= x >> np.uint64(16)
    return x


def row_hash(seed: int, key):
    key = np.asarray(key, dtype=np.uint64)
    return mix32(np.uint64(seed & 0xFFFFFFFF) ^ mix32((key + np.uint64(0x9E3779B9)) & _M32))


def synth_bf16_rows(keys, hidden: int, seed: int, outlier_period: int = 0) -> torch.Tensor:
    """bf16 rows [len(keys), hidden]; value(seed, key, col) as the synthesiser defines it."""
    keys = np.asarray(keys, dtype=np.uint64)
    rh = row_hash(seed, keys)[:, None]
    col = np.arange(hidden, dtype=np.uint64)[None, :]
    h = mix32(rh ^ ((col * np.uint64(0x9E3779B1) + np.uint64(0x85EBCA6B)) & _M32))
    s = (h & np.uint64(255)) + ((h >> np.uint64(8)) & np.uint64(255)) + ((h >> np.uint64(16)) & np.uint64(255)) + (
        h >> np.uint64(24))
    f = (s.astype(np.int64) - 510).astype(np.float32) * np.array([0x3BDDB47B], dtype=np.uint32).view(np.float32)[0]
    if outlier_period > 0:
        hot = (mix32(rh ^ np.uint64(0x5BD1E995)) % np.uint64(outlier_period)) == 0
        f = np.where(hot, f * np.float32(100.0), f).astype(np.float32)
    return torch.from_numpy(f).to(torch.bfloat16)


def uniform_cdf(num_experts: int) -> np.ndarray:
    """Inclusive 32-bit upper bounds of E equal cells."""
    return (((np.arange(1, num_experts + 1, dtype=np.uint64) << np.uint64(32)) // np.uint64(num_experts)) -
            np.uint64(1)).astype(np.uint32)


def zipf_cdf(num_experts: int, s: float = 1.2) -> np.ndarray:
    """p(e) proportional to (e+1)^-s, as inclusive 32-bit upper bounds; last cell closes at 2^32-1."""
    p = (np.arange(1, num_experts + 1, dtype=np.float64)) ** (-s)
    c = np.cumsum(p / p.sum())
    out = np.minimum(np.floor(c * 4294967296.0), 4294967295.0).astype(np.uint64)
    out[-1] = 0xFFFFFFFF
    return out.astype(np.uint32)


def synth_topk_idx(cdf: np.ndarray, ranks, num_tokens: int, num_topk: int, seed: int) -> torch.Tensor:
    """int64 [len(ranks), T, K]: K distinct experts per token by repeated inverse-CDF draws."""
    num_experts = len(cdf)
    ranks = np.asarray(ranks, dtype=np.uint64)
    keys = (ranks[:, None] * np.uint64(num_tokens) + np.arange(num_tokens, dtype=np.uint64)[None, :]) & _M32
    th = row_hash((seed ^ 0x7F4A7C15) & 0xFFFFFFFF, keys).reshape(-1)
    n = th.shape[0]
    chosen = np.full((n, num_topk), -1, dtype=np.int64)
    have = np.zeros(n, dtype=np.int64)
    cdf64 = cdf.astype(np.uint64)
    for c in range(64 * num_topk):
        todo = have < num_topk
        if not todo.any():
            break
        u = mix32((th + np.uint64((c * 0x9E3779B9) & 0xFFFFFFFF)) & _M32)
        e = np.searchsorted(cdf64, u, side='left').astype(np.int64)
        seen = (chosen == e[:, None]).any(1)
        take = todo & ~seen
        rows = np.nonzero(take)[0]
        chosen[rows, have[rows]] = e[rows]
        have[rows] += 1
    for row in np.nonzero(have < num_topk)[0]:
        for e in range(num_experts):
            if have[row] >= num_topk:
                break
            if e not in chosen[row, :have[row]]:
                chosen[row, have[row]] = e
                have[row] += 1
    return torch.from_numpy(chosen.reshape(len(ranks), num_tokens, num_topk))
