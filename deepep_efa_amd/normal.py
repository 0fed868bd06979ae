"""Normal-mode layout helpers on the device: per-rank token sort, channel prefix matrix, row pack.

Thin Python names over the host module; shapes follow the reference
(moe_routing_sort: csrc/kernels/efa_kernels.cu:1591-1651; channel_prefix_matrix:
csrc/kernels/intranode.cu:90-112; pack: deep_ep/buffer.py:877,917).
"""
from typing import Optional

import torch

from . import deep_ep_cpp


def moe_routing_sort(is_token_in_rank: torch.Tensor):
    """[T, R] bool -> (sorted_token_ids [S] int64, send_counts [R] int32, send_cumsum [R+1] int64, S)."""
    return deep_ep_cpp.moe_routing_sort(is_token_in_rank)


def channel_prefix_matrix(is_token_in_rank: torch.Tensor, num_channels: int) -> torch.Tensor:
    """[T, R] bool -> [R, C] int32 inclusive prefix over channels of tokens bound for each rank."""
    return deep_ep_cpp.channel_prefix_matrix(is_token_in_rank, num_channels)


def pack_rows(x: torch.Tensor, x_scales: Optional[torch.Tensor], sorted_token_ids: torch.Tensor,
              send_cumsum: torch.Tensor):
    """send_x = x[sorted_token_ids] (and scales likewise), contiguous per destination rank."""
    return deep_ep_cpp.pack_rows(x, x_scales, sorted_token_ids, send_cumsum)
