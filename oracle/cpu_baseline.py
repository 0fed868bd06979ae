"""Timed CPU baseline: one rank's share of a low-latency dispatch + combine in torch on the host cores.

TEST/BENCH INFRASTRUCTURE ONLY (the ``cpu_baseline`` leg of bench.py).  Does
the same work the GPU step does for rank `rank`, on the same kind of inputs:
  send     quantise own tokens (per_token_cast_to_fp8), route, copy each row into its expert slot
  recv     compact the staged segments into [E_l, N, H] + scales + src_info + ranges
  csend    gather the live expert-output rows back into per-pair slots
  crecv    top-k weighted float32 reduction to bf16
following deep_ep/buffer.py:1863-2457 (dispatch) and :2564-2803 (combine).
"""
import os
import time

import torch

from . import deepep_oracle as O


class CpuRankStep:
    def __init__(self, x, topk_idx, topk_weights, staged, staged_count, num_experts, num_ranks, rank, max_tokens):
        """staged: u8 [E_l, R, M, stride] rows already delivered by the peers; staged_count i32 [E_l, R]."""
        self.x, self.topk, self.w = x, topk_idx, topk_weights
        self.staged, self.staged_count = staged, staged_count
        self.e, self.r, self.rank, self.m = num_experts, num_ranks, rank, max_tokens
        self.h = x.shape[1]
        self.epr = num_experts // num_ranks
        self.n = max_tokens * num_ranks
        self.stride = O.row_stride(self.h, O.ROW_FP8)
        self.send_slots = torch.empty((num_experts, max_tokens, self.stride), dtype=torch.uint8)
        self.px = torch.empty((self.epr, self.n, self.h), dtype=torch.uint8)
        self.ps = torch.empty((self.epr, self.n, self.h // 128 * 4), dtype=torch.uint8)
        self.src_info = torch.empty((self.epr, self.n), dtype=torch.int32)
        self.y = torch.randn((self.epr, self.n, self.h), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
        self.combine_staging = torch.zeros((num_experts, max_tokens, self.h), dtype=torch.bfloat16)

    def step(self):
        h, epr, r, m = self.h, self.epr, self.r, self.m
        # ---- send
        q, s = O.per_token_cast_to_fp8(self.x)
        send_count, pair_slot = O.route(self.topk, self.e, m)
        tok, kk = torch.nonzero(pair_slot >= 0, as_tuple=True)
        ex = self.topk[tok, kk]
        sl = pair_slot[tok, kk].long()
        self.send_slots[ex, sl, :h] = q.view(torch.uint8)[tok]
        self.send_slots[ex, sl, h:h + h // 32] = s.view(torch.uint8).view(-1, h // 32)[tok]
        mine = (ex // epr) == self.rank
        self.staged[ex[mine] % epr, self.rank, sl[mine]] = self.send_slots[ex[mine], sl[mine]]
        self.staged_count[:, self.rank] = send_count[self.rank * epr:(self.rank + 1) * epr]
        # ---- recv
        cnt = self.staged_count.long()
        begin = torch.cumsum(cnt, 1) - cnt
        layout = torch.where(cnt > 0, (begin << 32) | cnt, torch.zeros_like(cnt))
        seg_e, seg_s = torch.nonzero(cnt > 0, as_tuple=True)
        for le, sr in zip(seg_e.tolist(), seg_s.tolist()):
            c, b = int(cnt[le, sr]), int(begin[le, sr])
            rows = self.staged[le, sr, :c]
            self.px[le, b:b + c] = rows[:, :h]
            self.ps[le, b:b + c] = rows[:, h:h + h // 32]
            tail = O.row_payload(h, O.ROW_FP8) - 16
            self.src_info[le, b:b + c] = rows[:, tail:tail + 4].contiguous().view(torch.int32).view(-1)
        # ---- combine send (own pairs only come back locally; peers' rows are already staged)
        for le in range(epr):
            c, b = int(cnt[le, self.rank]), int(begin[le, self.rank])
            self.combine_staging[self.rank * epr + le, :c] = self.y[le, b:b + c]
        # rows owed to other ranks are gathered as well (they would be sent)
        owed = [self.y[le, int(begin[le, sr]):int(begin[le, sr]) + int(cnt[le, sr])].clone()
                for le, sr in zip(seg_e.tolist(), seg_s.tolist()) if sr != self.rank]
        # ---- combine recv
        live = pair_slot >= 0
        rows = self.combine_staging[self.topk.clamp(min=0), pair_slot.clamp(min=0).long()]
        out = (rows.float() * (self.w * live).unsqueeze(-1)).sum(1).to(torch.bfloat16)
        return out, layout, len(owed)


def host_threads() -> int:
    """Threads the CPU legs run on: every core the host reports, or the share of them the job was
    given when the launcher says so through OMP_NUM_THREADS (a GPU box hands one GPU's job 16 cores of a
    host that reports many more)."""
    n = os.cpu_count() or 1
    share = os.environ.get("OMP_NUM_THREADS", "")
    return min(n, int(share)) if share.isdigit() and int(share) > 0 else n


def time_cpu_step(step: CpuRankStep, budget_s: float = 15.0, min_runs: int = 5):
    threads = host_threads()
    torch.set_num_threads(threads)
    for _ in range(2):
        step.step()
    times = []
    t0 = time.perf_counter()
    while len(times) < min_runs or (time.perf_counter() - t0 < budget_s and len(times) < 200):
        a = time.perf_counter()
        step.step()
        times.append(time.perf_counter() - a)
    times.sort()
    return times[len(times) // 2], threads, len(times)


class CpuReferenceCase:
    """The reference's own CPU-runnable case: 128 tokens x 7168 bf16 ~N(0,1), 256 experts, top-8 uniform without
    replacement, weights = softmax of N(0,1) logits, simulated EP=16 (16 local experts per rank).  One pass =
    get_dispatch_layout counts (csrc/kernels/layout.cu:9-121), the per-token per-128-channel FP8 cast
    (deep_ep/buffer.py:1590-1621) and the top-k weighted combine sum with float32 accumulation
    (csrc/kernels/coop_combine_recv.cuh:222-260) over the dequantised rows."""

    def __init__(self, num_tokens=128, hidden=7168, num_experts=256, num_topk=8, num_ranks=16, seed=0):
        g = torch.Generator().manual_seed(seed)
        self.x = torch.randn((num_tokens, hidden), generator=g).to(torch.bfloat16)
        self.topk = torch.stack([torch.randperm(num_experts, generator=g)[:num_topk] for _ in range(num_tokens)])
        self.w = torch.softmax(torch.randn((num_tokens, num_topk), generator=g), dim=-1)
        self.e, self.r, self.k = num_experts, num_ranks, num_topk

    def step(self):
        per_rank, _, per_expert, is_in = O.get_dispatch_layout(self.topk, self.e, self.r)
        q, s = O.per_token_cast_to_fp8(self.x)
        y = O.per_token_cast_back(q, s)  # every expert returns the row it was sent
        pair_rows = y.unsqueeze(1).expand(-1, self.k, -1)
        out = O.ll_combine_f32_chain(pair_rows, self.w, self.topk >= 0)
        return per_rank, per_expert, is_in, q, s, out


def time_reference_case(budget_s: float = 5.0, min_runs: int = 5):
    case = CpuReferenceCase()
    threads = host_threads()
    torch.set_num_threads(threads)
    for _ in range(2):
        case.step()
    times = []
    t0 = time.perf_counter()
    while len(times) < min_runs or (time.perf_counter() - t0 < budget_s and len(times) < 200):
        a = time.perf_counter()
        case.step()
        times.append(time.perf_counter() - a)
    times.sort()
    return times[len(times) // 2], threads, len(times)
