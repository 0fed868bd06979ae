"""Normal-mode layout helpers on the device: per-rank token sort, channel prefix matrix, row pack,
and the steps either side of the exchange (top-k remap, source metadata, per-token reduce).

Thin Python names over the host module; shapes follow the reference
(moe_routing_sort: csrc/kernels/efa_kernels.cu:1591-1651; channel_prefix_matrix:
csrc/kernels/intranode.cu:90-112; pack: deep_ep/buffer.py:877,917; topk_remap:
csrc/kernels/efa_kernels.cu:1653-1691; build_recv_src_meta: :1726-1749; the combine
reduce: deep_ep/buffer.py:1542-1557).
"""
from typing import Optional

import torch

from . import deep_ep_cpp


def moe_routing_sort(is_token_in_rank: torch.Tensor):
    """[T, R] bool -> (sorted_token_ids [S] int64, send_counts [R] int32, send_cumsum [R+1] int64, S)."""
    return deep_ep_cpp.moe_routing_sort(is_token_in_rank)


def moe_routing_sort_with_positions(is_token_in_rank: torch.Tensor):
    """moe_routing_sort plus the inverse of the list, row_of_pair [T, R] int32 (-1 = token not sent to the rank):
    handed to combine_reduce it saves that call a launch."""
    return deep_ep_cpp.moe_routing_sort_with_positions(is_token_in_rank)


def channel_prefix_matrix(is_token_in_rank: torch.Tensor, num_channels: int) -> torch.Tensor:
    """[T, R] bool -> [R, C] int32 inclusive prefix over channels of tokens bound for each rank."""
    return deep_ep_cpp.channel_prefix_matrix(is_token_in_rank, num_channels)


def pack_rows(x: torch.Tensor, x_scales: Optional[torch.Tensor], sorted_token_ids: torch.Tensor,
              send_cumsum: torch.Tensor):
    """send_x = x[sorted_token_ids] (and scales likewise), contiguous per destination rank."""
    return deep_ep_cpp.pack_rows(x, x_scales, sorted_token_ids, send_cumsum)


def topk_remap(topk_idx: torch.Tensor, topk_weights: torch.Tensor, sorted_token_ids: torch.Tensor,
               send_cumsum: torch.Tensor, total_send: int, num_ranks: int, num_local_experts: int):
    """Per send row, the token's top-k in the destination rank's expert numbering; (-1, 0.0) for other ranks' experts."""
    return deep_ep_cpp.topk_remap(topk_idx, topk_weights, sorted_token_ids, send_cumsum, total_send, num_ranks,
                                  num_local_experts)


def build_recv_src_meta(recv_counts: torch.Tensor, recv_cumsum: torch.Tensor, num_recv_tokens: int, num_ranks: int,
                        num_local_ranks: int) -> torch.Tensor:
    """[num_recv_tokens, 8] uint8: the int32 pair (source rank // num_local_ranks, 1 << source rank % num_local_ranks)."""
    return deep_ep_cpp.build_recv_src_meta(recv_counts, recv_cumsum, num_recv_tokens, num_ranks, num_local_ranks)


def combine_reduce(recv_x: torch.Tensor, recv_topk_weights: Optional[torch.Tensor], sorted_token_ids: torch.Tensor,
                   send_cumsum: torch.Tensor, is_token_in_rank: torch.Tensor, bias_0: Optional[torch.Tensor] = None,
                   bias_1: Optional[torch.Tensor] = None, row_of_pair: Optional[torch.Tensor] = None):
    """combined_x[t] = sum over the ranks holding t of the row that came back (+ biases), float32 accumulate.
    row_of_pair: the table of moe_routing_sort_with_positions (one launch instead of two)."""
    return deep_ep_cpp.combine_reduce(recv_x, recv_topk_weights, sorted_token_ids, send_cumsum, is_token_in_rank,
                                      bias_0, bias_1, row_of_pair)
