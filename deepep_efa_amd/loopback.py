"""Single-GPU loopback world: the other ranks of an expert-parallel group, kept in HBM.

Stands where the reference has its transport (csrc/transport/*, the
``dist.all_to_all_single`` calls at deep_ep/buffer.py:2268,2297,2735).  The
peers' inputs are either given explicitly (``set_inputs``) or generated on
the device from a seed (``synthesise``); their rows for this rank's experts
are produced by running the same send kernels in their name, so the receive
side sees exactly what a real exchange would deliver.
"""
import numpy as np
import torch

from . import _capi
from .ll_runtime import LowLatencyState, current_stream_ptr


def uniform_cdf(num_experts: int) -> np.ndarray:
    """Inclusive 32-bit upper bounds of E equal probability cells."""
    e = np.arange(1, num_experts + 1, dtype=np.uint64)
    return (((e << np.uint64(32)) // np.uint64(num_experts)) - np.uint64(1)).astype(np.uint32)


def zipf_cdf(num_experts: int, s: float = 1.2) -> np.ndarray:
    """Expert popularity proportional to (e + 1) ** -s, as inclusive 32-bit upper bounds."""
    p = np.arange(1, num_experts + 1, dtype=np.float64) ** (-s)
    c = np.cumsum(p / p.sum())
    out = np.minimum(np.floor(c * 4294967296.0), 4294967295.0).astype(np.uint64)
    out[-1] = 0xFFFFFFFF
    return out.astype(np.uint32)


class LoopbackWorld:
    """All R ranks' token batches and routing, resident on one GPU."""

    def __init__(self, num_ranks: int, rank: int, seed: int = 0, device="cuda"):
        assert 0 <= rank < num_ranks
        self.num_ranks, self.rank, self.seed, self.device = num_ranks, rank, seed & 0xFFFFFFFF, device
        self.lib = _capi.load()
        self.x_all = None         # [R, T, H] bf16
        self.topk_idx_all = None  # [R, T, K] int64
        self._peer_ws = None
        lo = torch.arange(0, rank, dtype=torch.int32)
        hi = torch.arange(rank + 1, num_ranks, dtype=torch.int32)
        self._ranks_below = lo.to(device)
        self._ranks_above = hi.to(device)

    # -- inputs -----------------------------------------------------------
    def set_inputs(self, x_all: torch.Tensor, topk_idx_all: torch.Tensor) -> None:
        """x_all [R, T, H] bf16 and topk_idx_all [R, T, K] int64, both on the device."""
        assert x_all.dim() == 3 and topk_idx_all.dim() == 3
        assert x_all.shape[0] == self.num_ranks and topk_idx_all.shape[0] == self.num_ranks
        assert x_all.dtype == torch.bfloat16 and topk_idx_all.dtype == torch.int64
        self.x_all, self.topk_idx_all = x_all.contiguous(), topk_idx_all.contiguous()

    def synthesise(self, num_tokens: int, hidden: int, num_topk: int, num_experts: int,
                   popularity: str = "uniform", outlier_period: int = 0) -> None:
        """Seeded inputs for every rank: x ~ approximately N(0,1), K distinct experts per token."""
        cdf = uniform_cdf(num_experts) if popularity == "uniform" else zipf_cdf(num_experts)
        cdf_dev = torch.from_numpy(cdf.view(np.int32)).to(self.device)
        ranks = torch.arange(self.num_ranks, dtype=torch.int32, device=self.device)
        topk = torch.empty((self.num_ranks, num_tokens, num_topk), dtype=torch.int64, device=self.device)
        _capi.check(self.lib.deepep_synth_topk_idx(_capi.ptr(cdf_dev), _capi.ptr(ranks), self.num_ranks, num_tokens,
                                                   num_topk, num_experts, self.seed, _capi.ptr(topk),
                                                   current_stream_ptr()))
        x = torch.empty((self.num_ranks, num_tokens, hidden), dtype=torch.bfloat16, device=self.device)
        _capi.check(self.lib.deepep_synth_bf16_rows(_capi.ptr(x), self.num_ranks * num_tokens, hidden, hidden * 2,
                                                    None, 0, self.seed, outlier_period, current_stream_ptr()))
        self.x_all, self.topk_idx_all = x, topk

    def own_inputs(self):
        return self.x_all[self.rank], self.topk_idx_all[self.rank]

    # -- what the exchange would deliver ------------------------------------
    def dispatch_from_peers(self, state: LowLatencyState) -> None:
        """Stages every peer's rows for this rank's experts, with their counts."""
        s = state.shape
        assert s.num_ranks == self.num_ranks and s.rank == self.rank
        r, t, h = self.x_all.shape
        k = self.topk_idx_all.shape[2]
        assert h == s.hidden and k == s.num_topk and t <= s.max_tokens
        per = self.lib.deepep_ll_dispatch_workspace_bytes(t, k, s.num_experts)
        need = max(256, per * max(self.rank, self.num_ranks - 1 - self.rank, 1))
        if self._peer_ws is None or self._peer_ws.numel() < need:
            self._peer_ws = torch.empty(need, dtype=torch.uint8, device=self.device)
        for ranks, first in ((self._ranks_below, 0), (self._ranks_above, self.rank + 1)):
            n = ranks.numel()
            if n == 0:
                continue
            _capi.check(self.lib.deepep_loopback_dispatch_from_peers(
                _capi.ptr(self.x_all[first]), _capi.ptr(self.topk_idx_all[first]), _capi.ptr(ranks), n, t, h, k,
                s.num_experts, s.num_ranks, s.rank, s.max_tokens, s.fmt, _capi.ptr(state.recv_staging),
                _capi.ptr(state.recv_count), _capi.ptr(self._peer_ws), self._peer_ws.numel(), current_stream_ptr()))

    def combine_from_peers(self, state: LowLatencyState, mode: int = 0, seed: int = 0) -> None:
        """Fills the combine staging rows owed by remote experts (mode 0: identity expert
        on the dequantised row; mode 1: seeded rows keyed expert * M + slot)."""
        s = state.shape
        assert mode == 1 or state.send_slots is not None
        _capi.check(self.lib.deepep_loopback_combine_from_peers(
            _capi.ptr(state.send_slots), _capi.ptr(state.send_count), s.hidden, s.num_experts, s.num_ranks, s.rank,
            s.max_tokens, s.fmt, mode, seed & 0xFFFFFFFF, _capi.ptr(state.combine_staging), current_stream_ptr()))
