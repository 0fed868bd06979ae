"""deep_ep.Buffer for one MI355X: layout, low-latency dispatch and low-latency combine.

Signatures, argument meaning, return tuples and the handle layout follow the
reference (deep_ep/buffer.py:80-110, 422-448, 1816-1823, 2460-2464,
2805-2852).  The process owns one GPU and plays rank `sim_rank` of a
`sim_num_ranks`-rank expert-parallel world; what the other ranks would send is
produced in HBM by the loopback world (`loopback_set_world` /
`loopback_synthesise`).  Everything that needs a second GPU or a network
(normal-mode dispatch/combine, EFA set-up) raises NotImplementedError.
"""
import os
import sys
from collections import defaultdict
from typing import Callable, Optional, Tuple

import numpy as np
import torch

from . import deep_ep_cpp
from .deep_ep_cpp import Config, EventHandle
from .loopback import uniform_cdf, zipf_cdf
from .utils import EventOverlap

_PROFILE_ENABLED = os.environ.get("DEEPEP_PROFILE", "0") == "1"
_PROFILE_PRINT_EVERY = int(os.environ.get("DEEPEP_PROFILE_INTERVAL", "20"))
_PROFILE_WARMUP = int(os.environ.get("DEEPEP_PROFILE_WARMUP", "5"))


class _LLProfiler:
    """Per-phase timing of the low-latency calls, enabled by DEEPEP_PROFILE=1 (the reference's switch and
    report line, deep_ep/buffer.py:20-77).  A mark is a HIP event recorded on the current stream, so marking
    costs no device synchronisation; the events of DEEPEP_PROFILE_INTERVAL calls are resolved together, after
    one synchronisation, when the report is due.  The first DEEPEP_PROFILE_WARMUP calls are not counted."""

    def __init__(self, name: str, rank: int):
        self.name, self.rank = name, rank
        self.skip = _PROFILE_WARMUP
        self.current = []   # (label, event) of the call in progress
        self.finished = []  # one such list per counted call

    def mark(self, label: str) -> None:
        event = torch.cuda.Event(enable_timing=True)
        event.record()
        self.current.append((label, event))

    def finish_iter(self, extra_info: str = "") -> None:
        marks, self.current = self.current, []
        if self.skip > 0:
            self.skip -= 1
            return
        self.finished.append(marks)
        if len(self.finished) < _PROFILE_PRINT_EVERY:
            return
        torch.cuda.synchronize()
        sums = defaultdict(float)
        for marks in self.finished:
            for (a, ea), (b, eb) in zip(marks, marks[1:]):
                sums[f"{a}->{b}"] += ea.elapsed_time(eb) * 1e3
            if len(marks) >= 2:
                sums["TOTAL"] += marks[0][1].elapsed_time(marks[-1][1]) * 1e3
        n = len(self.finished)
        self.finished = []
        line = " | ".join(f"{phase}={total / n:.1f}us" for phase, total in sums.items())
        tail = f" | {extra_info}" if extra_info else ""
        print(f"[LL_PROFILE rank={self.rank}] {self.name} (avg of {n}): {line}{tail}", file=sys.stderr, flush=True)


class Buffer:
    """Expert-parallel communication buffer, low-latency mode, one GPU's share.

    Attributes mirror the reference: num_sms, rank, group_size, group,
    num_nvl_bytes, num_rdma_bytes, runtime.
    """

    num_sms: int = 20

    def __init__(self, group=None, num_nvl_bytes: int = 0, num_rdma_bytes: int = 0, low_latency_mode: bool = False,
                 num_qps_per_rank: int = 24, allow_nvlink_for_low_latency_mode: bool = True, allow_mnnvl: bool = False,
                 use_fabric: bool = False, explicitly_destroy: bool = False, enable_shrink: bool = False, comm=None, *,
                 sim_num_ranks: Optional[int] = None, sim_rank: int = 0, sim_seed: int = 0) -> None:
        if group is not None:
            real_rank, real_size = group.rank(), group.size()
        elif comm is not None:
            real_rank, real_size = comm.Get_rank(), comm.Get_size()
        elif sim_num_ranks is not None:
            real_rank, real_size = 0, 1
        else:
            raise ValueError("Either 'group' or 'comm' must be provided.")
        if real_size != 1:
            raise NotImplementedError(
                "this build runs one GPU's share of the expert-parallel world: use a 1-rank group (or group=None) "
                "and give the simulated world with sim_num_ranks / sim_rank")
        self.group = group if group is not None else comm
        self.rank = sim_rank if sim_num_ranks is not None else real_rank
        self.group_size = sim_num_ranks if sim_num_ranks is not None else real_size
        self.sim_seed = sim_seed
        self.num_nvl_bytes, self.num_rdma_bytes = num_nvl_bytes, num_rdma_bytes
        self.low_latency_mode = low_latency_mode
        self.explicitly_destroy = explicitly_destroy
        self.enable_shrink = enable_shrink
        self.runtime = deep_ep_cpp.Buffer(self.rank, self.group_size, num_nvl_bytes, num_rdma_bytes, low_latency_mode,
                                          explicitly_destroy, enable_shrink, use_fabric)
        self.runtime.sync([self.runtime.get_local_device_id()], [None], None)
        assert self.runtime.is_available()
        self._ll_handle_shape = None

    # -- lifetime / static helpers (reference: deep_ep/buffer.py:267-349) --------
    def destroy(self) -> None:
        assert self.explicitly_destroy, "`explicitly_destroy` flag must be set"
        self.runtime.destroy()
        self.runtime = None

    @staticmethod
    def is_sm90_compiled() -> bool:
        return deep_ep_cpp.is_sm90_compiled()

    @staticmethod
    def set_num_sms(new_num_sms: int) -> None:
        assert new_num_sms % 2 == 0, "The SM count must be even"
        Buffer.num_sms = new_num_sms

    @staticmethod
    def capture() -> EventOverlap:
        return EventOverlap(EventHandle())

    @staticmethod
    def get_low_latency_rdma_size_hint(num_max_dispatch_tokens_per_rank: int, hidden: int, num_ranks: int,
                                       num_experts: int) -> int:
        return deep_ep_cpp.get_low_latency_rdma_size_hint(num_max_dispatch_tokens_per_rank, hidden, num_ranks,
                                                          num_experts)

    def get_comm_stream(self) -> torch.Stream:
        ts = self.runtime.get_comm_stream()
        return torch.cuda.Stream(stream_id=ts.stream_id, device_index=ts.device_index, device_type=ts.device_type)

    def get_local_buffer_tensor(self, dtype: torch.dtype, size: Optional[torch.Size] = None, offset: int = 0,
                                use_rdma_buffer: bool = False) -> torch.Tensor:
        tensor = self.runtime.get_local_buffer_tensor(dtype, offset, use_rdma_buffer)
        if size is None:
            return tensor
        assert tensor.numel() >= size.numel()
        return tensor[:size.numel()].view(size)

    # Recommended chunk settings per world size (reference: deep_ep/buffer.py:361-419); values only.
    _DISPATCH_CONFIGS = {2: (24, 256, 6, 128), 4: (6, 256, 6, 128), 8: (6, 256, 6, 128), 16: (36, 288, 20, 128),
                         24: (32, 288, 8, 128), 32: (32, 288, 8, 128), 48: (32, 288, 8, 128), 64: (32, 288, 8, 128),
                         96: (20, 480, 12, 128), 128: (20, 560, 12, 128), 144: (32, 720, 12, 128),
                         160: (28, 720, 12, 128)}
    _COMBINE_CONFIGS = {2: (10, 256, 6, 128), 4: (9, 256, 6, 128), 8: (4, 256, 6, 128), 16: (4, 288, 12, 128),
                        24: (1, 288, 8, 128), 32: (1, 288, 8, 128), 48: (1, 288, 8, 128), 64: (1, 288, 8, 128),
                        96: (1, 480, 8, 128), 128: (1, 560, 8, 128), 144: (2, 720, 8, 128), 160: (2, 720, 8, 128)}

    @staticmethod
    def get_dispatch_config(num_ranks: int) -> Config:
        assert num_ranks in Buffer._DISPATCH_CONFIGS, f"Unsupported number of EP ranks: {num_ranks}"
        return Config(Buffer.num_sms, *Buffer._DISPATCH_CONFIGS[num_ranks])

    @staticmethod
    def get_combine_config(num_ranks: int) -> Config:
        assert num_ranks in Buffer._COMBINE_CONFIGS, f"Unsupported number of EP ranks: {num_ranks}"
        return Config(Buffer.num_sms, *Buffer._COMBINE_CONFIGS[num_ranks])

    # -- layout (reference: deep_ep/buffer.py:422-448) -----------------------------
    def get_dispatch_layout(self, topk_idx: torch.Tensor, num_experts: int,
                            previous_event: Optional[EventOverlap] = None, async_finish: bool = False,
                            allocate_on_comm_stream: bool = False):
        """Returns (num_tokens_per_rank [R] int32, num_tokens_per_rdma_rank [R/8] int32 or None,
        num_tokens_per_expert [E] int32, is_token_in_rank [T, R] bool, EventOverlap)."""
        per_rank, per_rdma, per_expert, is_in, event = self.runtime.get_dispatch_layout(
            topk_idx, num_experts, getattr(previous_event, "event", None), async_finish, allocate_on_comm_stream)
        return per_rank, per_rdma, per_expert, is_in, EventOverlap(event)

    # -- loopback world -------------------------------------------------------------
    def loopback_set_world(self, x_all: torch.Tensor, topk_idx_all: torch.Tensor) -> None:
        """Every rank's inputs: x_all [R, T, H] bf16 and topk_idx_all [R, T, K] int64 on the device.
        Entry `self.rank` is this rank's own batch; the others drive the synthesised exchange."""
        self.runtime.loopback_set_world(x_all.contiguous(), topk_idx_all.contiguous())

    def loopback_synthesise(self, num_tokens: int, hidden: int, num_topk: int, num_experts: int,
                            popularity: str = "uniform", outlier_period: int = 0, seed: Optional[int] = None):
        """Seeded inputs for all ranks, generated on the device; returns this rank's (x, topk_idx)."""
        cdf = uniform_cdf(num_experts) if popularity == "uniform" else zipf_cdf(num_experts)
        cdf_dev = torch.from_numpy(cdf.view(np.int32)).cuda()
        self.runtime.loopback_synthesise(num_tokens, hidden, num_topk, num_experts, cdf_dev, outlier_period,
                                         self.sim_seed if seed is None else seed)
        return self.runtime.loopback_own_inputs()

    def loopback_clear_world(self) -> None:
        self.runtime.loopback_clear_world()

    def loopback_set_combine_mode(self, mode: int, seed: int = 0) -> None:
        """What remote experts return for this rank's pairs: 0 = the dequantised row they were
        sent (an identity expert), 1 = seeded rows keyed expert * M + slot."""
        self.runtime.loopback_set_combine_mode(mode, seed)

    # -- low latency (reference: deep_ep/buffer.py:1562-1584, 1816-2457, 2460-2852) ----
    def clean_low_latency_buffer(self, num_max_dispatch_tokens_per_rank: int, hidden: int, num_experts: int) -> None:
        self.runtime.clean_low_latency_buffer(num_max_dispatch_tokens_per_rank, hidden, num_experts)

    def low_latency_dispatch(self, x: torch.Tensor, topk_idx: torch.Tensor, num_max_dispatch_tokens_per_rank: int,
                             num_experts: int, cumulative_local_expert_recv_stats: Optional[torch.Tensor] = None,
                             dispatch_wait_recv_cost_stats: Optional[torch.Tensor] = None, use_fp8: bool = True,
                             round_scale: bool = False, use_ue8m0: bool = False, async_finish: bool = False,
                             return_recv_hook: bool = False, topk_weights: Optional[torch.Tensor] = None):
        """x [T, H] bf16, topk_idx [T, K] int64 (-1 = no selection).

        Returns (recv_x, recv_count, handle, event, hook):
          recv_x   (packed_recv_x [E_l, N, H] float8_e4m3fn, packed_recv_scales [E_l, N, H/128] float32
                   or [E_l, N, H/512] int32 with use_ue8m0) if use_fp8 else packed_recv_x [E_l, N, H] bf16;
          recv_count [E_l] int32 rows valid per local expert; rows beyond it are undefined (never cleared);
          handle   (src_info [E_l, N] int32, layout_range [E_l, R] int64 = (begin << 32) | count,
                   num_max_dispatch_tokens_per_rank, hidden, num_experts);
          the returned tensors are reused by the next call with the same shape.
        async_finish is accepted and an event is returned either way, as in the reference
        (deep_ep/buffer.py:2449 returns EventOverlap(EventHandle()) whatever the flag says).
        """
        prof = None
        if _PROFILE_ENABLED:
            if not hasattr(self, "_ll_dispatch_profiler"):
                self._ll_dispatch_profiler = _LLProfiler("DISPATCH", self.rank)
            prof = self._ll_dispatch_profiler
            prof.mark("start")
        recv_x, recv_scales, recv_count, src_info, layout_range, event, hook = self.runtime.low_latency_dispatch(
            x, topk_idx, cumulative_local_expert_recv_stats, dispatch_wait_recv_cost_stats,
            num_max_dispatch_tokens_per_rank, num_experts, use_fp8, round_scale, use_ue8m0, True, return_recv_hook)
        handle = (src_info, layout_range, num_max_dispatch_tokens_per_rank, x.size(1), num_experts)
        if prof:
            prof.mark("end")
            prof.finish_iter()
        out = (recv_x, recv_scales) if use_fp8 else recv_x
        return out, recv_count, handle, EventOverlap(event), hook

    def low_latency_combine(self, x: torch.Tensor, topk_idx: torch.Tensor, topk_weights: torch.Tensor, handle: tuple,
                            use_logfmt: bool = False, zero_copy: bool = False, async_finish: bool = False,
                            return_recv_hook: bool = False, out: Optional[torch.Tensor] = None,
                            combine_wait_recv_cost_stats: Optional[torch.Tensor] = None, *,
                            accumulate: bool = False):
        """x [E_l, N, H] bf16 expert outputs laid out like the dispatch result.

        Returns (combined_x [T, H] bf16, event, hook) with
        combined_x[t] = bf16(sum_k [topk_idx[t,k] >= 0] * topk_weights[t,k] * x_returned[t,k]), float32 accumulate.
        accumulate (needs `out`): the sum starts from float32(out[t]) instead of zero — the flag the
        reference's reduce takes (csrc/kernels/coop_combine_recv.cuh:174-179) and its Python fixes to False
        (deep_ep/buffer.py:2541).
        async_finish is accepted and an event is returned either way, as in the reference
        (deep_ep/buffer.py:2801-2803 returns EventOverlap(EventHandle()) whatever the flag says).
        """
        assert not accumulate or out is not None, "accumulate adds to `out`"
        src_info, layout_range, num_max_dispatch_tokens_per_rank, hidden, num_experts = handle
        prof = None
        if _PROFILE_ENABLED:
            if not hasattr(self, "_ll_combine_profiler"):
                self._ll_combine_profiler = _LLProfiler("COMBINE", self.rank)
            prof = self._ll_combine_profiler
            prof.mark("start")
        combined_x, event, hook = self.runtime.low_latency_combine(
            x, topk_idx, topk_weights, src_info, layout_range, combine_wait_recv_cost_stats,
            num_max_dispatch_tokens_per_rank, num_experts, use_logfmt, zero_copy, True, return_recv_hook, out,
            accumulate)
        if prof:
            prof.mark("end")
            prof.finish_iter()
        return combined_x, EventOverlap(event), hook

    def low_latency_update_mask_buffer(self, rank_to_mask: int, mask: bool = False) -> None:
        self.runtime.low_latency_update_mask_buffer(rank_to_mask, mask)

    def low_latency_query_mask_buffer(self, mask_status: torch.Tensor) -> None:
        self.runtime.low_latency_query_mask_buffer(mask_status)

    def low_latency_clean_mask_buffer(self) -> None:
        self.runtime.low_latency_clean_mask_buffer()

    def get_next_low_latency_combine_buffer(self, handle: tuple) -> torch.Tensor:
        """The [E_l, N, H] bf16 buffer the next `low_latency_combine(..., zero_copy=True)` reads and the transport
        sends from (the rows of a source rank are one contiguous range of it, `layout_range`): that combine skips
        the row return, as deep_ep/buffer.py:2831-2852 promises."""
        _, _, num_max_dispatch_tokens_per_rank, hidden, num_experts = handle
        return self.runtime.get_next_low_latency_combine_buffer(num_max_dispatch_tokens_per_rank, hidden, num_experts)

    # -- not part of this build ------------------------------------------------------
    def dispatch(self, *args, **kwargs):
        raise NotImplementedError("normal-mode dispatch moves tokens between GPUs; this build covers the "
                                  "single-GPU share of the low-latency path (see get_dispatch_layout, "
                                  "low_latency_dispatch, low_latency_combine)")

    def combine(self, *args, **kwargs):
        raise NotImplementedError("normal-mode combine moves tokens between GPUs; not part of this build")

    def internode_dispatch(self, *args, **kwargs):
        raise NotImplementedError("internode dispatch moves tokens between nodes; not part of this build (its "
                                  "GPU-side steps are deep_ep_cpp.moe_routing_sort, pack_rows, topk_remap and "
                                  "build_recv_src_meta)")

    def internode_combine(self, *args, **kwargs):
        raise NotImplementedError("internode combine moves tokens between nodes; not part of this build (its "
                                  "GPU-side reduction is deep_ep_cpp.combine_reduce)")
