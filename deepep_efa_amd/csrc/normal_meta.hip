// Normal-mode steps either side of the per-rank pack: the top-k remap of the
// rows being sent, the source metadata of the rows received, and the reduce
// that adds the rows coming back for each token.
#include "common.hpp"
#include "../../include/deepep_hip.h"

namespace deepep {

constexpr int kMetaThreads = 256;

// Largest r with cumsum[r] <= i, for cumsum[0] = 0 non-decreasing, cumsum[num_ranks] > i.
__device__ __forceinline__ int rank_of_row(const int64_t* cumsum, int num_ranks, int64_t i) {
    int lo = 0, hi = num_ranks;  // invariant: cumsum[lo] <= i < cumsum[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cumsum[mid] <= i) lo = mid; else hi = mid;
    }
    return lo;
}

// ---------------------------------------------------------------------
// topk_remap: for every row of the per-rank send list, the token's top-k
// entries in the expert numbering of the destination rank; entries for
// other ranks' experts become (-1, 0.0).  One thread per (row, k); the
// R + 1 prefix lives in LDS.
// Reference: csrc/kernels/efa_kernels.cu:339-387.
// ---------------------------------------------------------------------
__global__ __launch_bounds__(kMetaThreads) void topk_remap_kernel(
    const int64_t* __restrict__ topk_idx, const float* __restrict__ topk_weights,
    const int64_t* __restrict__ sorted_token_ids, const int64_t* __restrict__ send_cumsum, int num_tokens,
    int num_topk, int num_ranks, int num_local_experts, int64_t max_send, int64_t* __restrict__ remapped_topk,
    float* __restrict__ remapped_weights) {
    extern __shared__ int64_t cumsum[];  // [R + 1]
    for (int r = threadIdx.x; r <= num_ranks; r += kMetaThreads) cumsum[r] = send_cumsum[r];
    __syncthreads();
    int64_t total = cumsum[num_ranks];
    if (total > max_send) total = max_send;
    const int64_t work = total * num_topk;
    for (int64_t idx = int64_t(blockIdx.x) * kMetaThreads + threadIdx.x; idx < work;
         idx += int64_t(gridDim.x) * kMetaThreads) {
        const int64_t row = idx / num_topk;
        const int k = int(idx - row * num_topk);
        const int dst_rank = rank_of_row(cumsum, num_ranks, row);
        const int64_t token = sorted_token_ids[row];
        int64_t out_e = -1;
        float out_w = 0.0f;
        if (token >= 0 && token < num_tokens) {
            const int64_t e = topk_idx[token * num_topk + k];
            const int64_t first = int64_t(dst_rank) * num_local_experts;
            if (e >= first && e < first + num_local_experts) {
                out_e = e - first;
                out_w = topk_weights[token * num_topk + k];
            }
        }
        remapped_topk[idx] = out_e;
        remapped_weights[idx] = out_w;
    }
}

// ---------------------------------------------------------------------
// build_recv_src_meta: row i of the receive list came from rank s with
// recv_cumsum[s] <= i < recv_cumsum[s + 1]; its 8 metadata bytes are the two
// int32 {s / num_local_ranks, 1 << (s % num_local_ranks)}.
// Reference: csrc/kernels/efa_kernels.cu:448-482.
// ---------------------------------------------------------------------
__global__ __launch_bounds__(kMetaThreads) void recv_src_meta_kernel(const int64_t* __restrict__ recv_cumsum,
                                                                     int num_ranks, int num_local_ranks,
                                                                     int64_t max_recv, u32x2* __restrict__ meta) {
    extern __shared__ int64_t cumsum[];  // [R + 1]
    for (int r = threadIdx.x; r <= num_ranks; r += kMetaThreads) cumsum[r] = recv_cumsum[r];
    __syncthreads();
    int64_t total = cumsum[num_ranks];
    if (total > max_recv) total = max_recv;
    for (int64_t i = int64_t(blockIdx.x) * kMetaThreads + threadIdx.x; i < total;
         i += int64_t(gridDim.x) * kMetaThreads) {
        const int s = rank_of_row(cumsum, num_ranks, i);
        u32x2 m = {uint32_t(s / num_local_ranks), uint32_t(1) << (s % num_local_ranks)};
        meta[i] = m;
    }
}

// ---------------------------------------------------------------------
// Combine reduce, step 1: where in the returned list is the row of
// (token, rank)?  Row j of rank r's segment belongs to token
// sorted_token_ids[j]; the table is only read where is_token_in_rank says
// the pair exists, so nothing has to be cleared first.
// ---------------------------------------------------------------------
__global__ __launch_bounds__(kMetaThreads) void combine_positions_kernel(
    const int64_t* __restrict__ sorted_token_ids, const int64_t* __restrict__ send_cumsum, int num_tokens,
    int num_ranks, int64_t max_rows, int32_t* __restrict__ row_of_pair) {
    extern __shared__ int64_t cumsum[];  // [R + 1]
    for (int r = threadIdx.x; r <= num_ranks; r += kMetaThreads) cumsum[r] = send_cumsum[r];
    __syncthreads();
    int64_t total = cumsum[num_ranks];
    if (total > max_rows) total = max_rows;
    for (int64_t j = int64_t(blockIdx.x) * kMetaThreads + threadIdx.x; j < total;
         j += int64_t(gridDim.x) * kMetaThreads) {
        const int r = rank_of_row(cumsum, num_ranks, j);
        const int64_t token = sorted_token_ids[j];
        if (token >= 0 && token < num_tokens) row_of_pair[token * num_ranks + r] = int32_t(j);
    }
}

// ---------------------------------------------------------------------
// Combine reduce, step 2: out[t, :] = bf16( sum over the ranks r holding
// token t, ascending, of f32(recv_x[row_of_pair[t, r], :]) + bias_0 + bias_1 ),
// accumulated in float32 in that fixed order and rounded once; the top-k
// weights are added the same way.  One wave = one (token, 1 KiB piece):
// lane r fetches rank r's membership byte and row index (one round of loads
// for all ranks), the rows are then loaded eight at a time.
// Reference: the zero_() + index_add_ of deep_ep/buffer.py:1542-1557, which
// accumulates in bf16 through atomics in arrival order.
// ---------------------------------------------------------------------
template <bool kStream>  // the returned rows exceed what the caches hold: read them with the non-temporal hint
__global__ __launch_bounds__(kMetaThreads) void combine_reduce_kernel(
    const uint8_t* __restrict__ recv_x, const float* __restrict__ recv_w,
    const uint8_t* __restrict__ is_token_in_rank, const int32_t* __restrict__ row_of_pair,
    const uint8_t* __restrict__ bias_0, const uint8_t* __restrict__ bias_1, int num_tokens, int hidden,
    int num_topk, int num_ranks, int64_t max_rows, int pieces_per_row, uint8_t* __restrict__ out_x,
    float* __restrict__ out_w) {
    const int lane = lane_id();
    const int64_t item = int64_t(blockIdx.x) * (kMetaThreads / kWave) + wave_in_block();
    if (item >= int64_t(num_tokens) * pieces_per_row) return;
    const int t = int(item / pieces_per_row);
    const int piece = int(item - int64_t(t) * pieces_per_row);
    const int64_t row_bytes = int64_t(hidden) * 2;
    const int64_t off = int64_t(piece) * 1024 + lane * 16;
    const bool lane_live = off < row_bytes;

    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    float w_acc = 0.0f;  // lane k of piece 0: the token's combined weight k
    const bool weights_here = piece == 0 && recv_w != nullptr && out_w != nullptr;

    for (int r0 = 0; r0 < num_ranks; r0 += kWave) {
        const int r = r0 + lane;
        int64_t my_row = -1;
        if (r < num_ranks && is_token_in_rank[int64_t(t) * num_ranks + r] != 0) {
            my_row = row_of_pair[int64_t(t) * num_ranks + r];
            if (my_row < 0 || my_row >= max_rows) my_row = -1;
        }
        uint64_t present = __ballot(my_row >= 0);
        while (present != 0) {
            u32x4 v[8];
            int rows[8];
            int n = 0;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                rows[u] = -1;
                if (present != 0) {
                    const int src_lane = __builtin_ctzll(present);
                    present &= present - 1;
                    rows[u] = __builtin_amdgcn_readlane(int(my_row), src_lane);
                    if (lane_live) v[u] = load_u32x4<kStream>(recv_x + int64_t(rows[u]) * row_bytes + off);
                    n = u + 1;
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (u >= n) continue;
                if (lane_live) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        acc[2 * i] += bf16_lo(v[u][i]);
                        acc[2 * i + 1] += bf16_hi(v[u][i]);
                    }
                }
                if (weights_here && lane < num_topk) w_acc += recv_w[int64_t(rows[u]) * num_topk + lane];
            }
        }
    }
    if (lane_live) {
        if (bias_0 != nullptr) {
            const u32x4 b = load_global_u32x4(bias_0 + int64_t(t) * row_bytes + off);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[2 * i] += bf16_lo(b[i]), acc[2 * i + 1] += bf16_hi(b[i]);
        }
        if (bias_1 != nullptr) {
            const u32x4 b = load_global_u32x4(bias_1 + int64_t(t) * row_bytes + off);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[2 * i] += bf16_lo(b[i]), acc[2 * i + 1] += bf16_hi(b[i]);
        }
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = pack_bf16x2(acc[2 * i], acc[2 * i + 1]);
        store_u32x4<kStream>(out_x + int64_t(t) * row_bytes + off, o);
    }
    if (weights_here && lane < num_topk) out_w[int64_t(t) * num_topk + lane] = w_acc;
}

static unsigned meta_grid(int64_t work) {
    int64_t blocks = (work + kMetaThreads - 1) / kMetaThreads;
    if (blocks < 1) blocks = 1;
    if (blocks > 65536) blocks = 65536;  // grid-stride beyond that
    return unsigned(blocks);
}

}  // namespace deepep

using namespace deepep;

extern "C" {

int deepep_topk_remap(const int64_t* topk_idx, const float* topk_weights, const int64_t* sorted_token_ids,
                      const int64_t* send_cumsum, int num_tokens, int num_topk, int num_ranks,
                      int num_local_experts, int64_t max_send, int64_t* remapped_topk, float* remapped_weights,
                      void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_tokens >= 0 && num_topk > 0 && num_ranks > 0 && num_ranks <= 4096);
    EP_HOST_ASSERT(num_local_experts > 0 && max_send >= 0);
    EP_HOST_ASSERT(max_send * num_topk < (int64_t(1) << 40));
    if (max_send == 0) return 0;
    EP_HOST_ASSERT(topk_idx != nullptr && topk_weights != nullptr && sorted_token_ids != nullptr &&
                   send_cumsum != nullptr && remapped_topk != nullptr && remapped_weights != nullptr);
    topk_remap_kernel<<<meta_grid(max_send * num_topk), kMetaThreads, size_t(num_ranks + 1) * sizeof(int64_t),
                        reinterpret_cast<hipStream_t>(stream)>>>(
        topk_idx, topk_weights, sorted_token_ids, send_cumsum, num_tokens, num_topk, num_ranks, num_local_experts,
        max_send, remapped_topk, remapped_weights);
    EP_LAUNCH_CHECK();
    return 0;
}

int deepep_build_recv_src_meta(const int64_t* recv_cumsum, int num_ranks, int num_local_ranks,
                               int64_t max_recv_tokens, uint8_t* recv_src_meta, void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_ranks > 0 && num_ranks <= 4096 && max_recv_tokens >= 0);
    EP_HOST_ASSERT(num_local_ranks > 0 && num_local_ranks <= 32);
    if (max_recv_tokens == 0) return 0;
    EP_HOST_ASSERT(recv_cumsum != nullptr && recv_src_meta != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(recv_src_meta) & 7) == 0);
    recv_src_meta_kernel<<<meta_grid(max_recv_tokens), kMetaThreads, size_t(num_ranks + 1) * sizeof(int64_t),
                           reinterpret_cast<hipStream_t>(stream)>>>(recv_cumsum, num_ranks, num_local_ranks,
                                                                    max_recv_tokens,
                                                                    reinterpret_cast<u32x2*>(recv_src_meta));
    EP_LAUNCH_CHECK();
    return 0;
}

size_t deepep_combine_reduce_workspace_bytes(int num_tokens, int num_ranks) {
    return (size_t(num_tokens) * size_t(num_ranks) * sizeof(int32_t) + 255) & ~size_t(255);
}

int deepep_combine_reduce(const void* recv_x, const float* recv_topk_weights, const int64_t* sorted_token_ids,
                          const int64_t* send_cumsum, const uint8_t* is_token_in_rank, const void* bias_0,
                          const void* bias_1, int num_tokens, int hidden, int num_topk, int num_ranks,
                          int64_t max_rows, const int32_t* row_of_pair_in, void* combined_x,
                          float* combined_topk_weights, void* workspace, size_t workspace_bytes, void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_tokens >= 0 && hidden > 0 && hidden % 8 == 0 && num_ranks > 0 && num_ranks <= 4096);
    EP_HOST_ASSERT(max_rows >= 0 && max_rows < (int64_t(1) << 31));
    EP_HOST_ASSERT(num_topk >= 0 && num_topk <= kWave);
    if (num_tokens == 0) return 0;
    EP_HOST_ASSERT(sorted_token_ids != nullptr && send_cumsum != nullptr && is_token_in_rank != nullptr &&
                   combined_x != nullptr);
    EP_HOST_ASSERT(max_rows == 0 || recv_x != nullptr);
    EP_HOST_ASSERT(row_of_pair_in != nullptr ||
                   (workspace != nullptr &&
                    workspace_bytes >= deepep_combine_reduce_workspace_bytes(num_tokens, num_ranks)));
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(recv_x) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(combined_x) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(bias_0) & 15) == 0 && (reinterpret_cast<uintptr_t>(bias_1) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(workspace) & 3) == 0);
    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
    // with the table the routing sort left (where it wrote every list entry it also wrote the entry's
    // place) the reduce is the only launch; otherwise the table is rebuilt from the list first
    const int32_t* row_of_pair = row_of_pair_in;
    if (row_of_pair_in == nullptr) row_of_pair = reinterpret_cast<int32_t*>(workspace);
    if (max_rows > 0 && row_of_pair_in == nullptr) {
        combine_positions_kernel<<<meta_grid(max_rows), kMetaThreads, size_t(num_ranks + 1) * sizeof(int64_t), hs>>>(
            sorted_token_ids, send_cumsum, num_tokens, num_ranks, max_rows, reinterpret_cast<int32_t*>(workspace));
        EP_LAUNCH_CHECK();
    }
    const int pieces = (hidden * 2 + 1023) / 1024;
    const int64_t blocks = (int64_t(num_tokens) * pieces + (kMetaThreads / kWave) - 1) / (kMetaThreads / kWave);
    EP_HOST_ASSERT(blocks < (int64_t(1) << 31));
#define DEEPEP_LAUNCH_REDUCE(STREAM)                                                                          \
    combine_reduce_kernel<STREAM><<<dim3(unsigned(blocks)), kMetaThreads, 0, hs>>>(                             \
        reinterpret_cast<const uint8_t*>(recv_x), recv_topk_weights, is_token_in_rank, row_of_pair,               \
        reinterpret_cast<const uint8_t*>(bias_0), reinterpret_cast<const uint8_t*>(bias_1), num_tokens, hidden,  \
        num_topk, num_ranks, max_rows, pieces, reinterpret_cast<uint8_t*>(combined_x), combined_topk_weights)
    if (max_rows * hidden * 2 > stream_bytes()) DEEPEP_LAUNCH_REDUCE(true);
    else DEEPEP_LAUNCH_REDUCE(false);
#undef DEEPEP_LAUNCH_REDUCE
    EP_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
