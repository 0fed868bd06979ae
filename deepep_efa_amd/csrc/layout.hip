// Route counting and layout for the normal-mode path: per-expert / per-rank
// counts with the token x rank membership matrix, the per-rank token sort,
// the channel prefix matrix, and the row gather that packs per-rank send
// buffers.
#include "common.hpp"
#include "../../include/deepep_hip.h"

namespace deepep {

constexpr int kLayoutThreads = 256;
constexpr int kMaxRankWords = 4;  // membership bitmask: up to 256 ranks

// Spreads the 8 bits of b into 8 bytes (byte i = bit i, value 0 or 1).
__device__ __forceinline__ uint64_t bits_to_bool_bytes(uint32_t b) {
    uint64_t x = (uint64_t(b & 0xffu) * 0x0101010101010101ull) & 0x8040201008040201ull;
    return ((x + 0x7f7f7f7f7f7f7f7full) >> 7) & 0x0101010101010101ull;
}

// ---------------------------------------------------------------------
// get_dispatch_layout: one pass over topk_idx, one token per lane.
//   * per-expert pair counts: LDS histogram (integer adds — the result does
//     not depend on their order);
//   * per-rank and per-node distinct-token counts: each lane folds its K
//     selections into a rank bitmask, then one 64-lane ballot + popcount per
//     rank gives the wave's count;
//   * is_token_in_rank: the bitmask expanded to bool bytes, 8 per store.
// Each workgroup writes a partial row [E | R | R/8]; with one workgroup the
// partial row is the result, otherwise a second small kernel adds the rows.
// Reference: csrc/kernels/layout.cu:9-121 (which re-reads topk_idx once per
// 4 experts / 8 ranks).
// ---------------------------------------------------------------------
__global__ __launch_bounds__(kLayoutThreads) void layout_count_kernel(
    const int64_t* __restrict__ topk_idx, int num_tokens, int num_topk, int num_ranks, int num_experts,
    uint32_t rank_magic, int num_nodes, uint8_t* __restrict__ is_token_in_rank, int32_t* __restrict__ partial,
    int32_t* __restrict__ per_rank, int32_t* __restrict__ per_node, int32_t* __restrict__ per_expert) {
    extern __shared__ int32_t hist[];  // [E + R + nodes]
    const int tid = threadIdx.x, lane = lane_id();
    const int width = num_experts + num_ranks + num_nodes;
    for (int j = tid; j < width; j += kLayoutThreads) hist[j] = 0;
    __syncthreads();

    const int t = blockIdx.x * kLayoutThreads + tid;
    uint64_t member[kMaxRankWords] = {0, 0, 0, 0};
    if (t < num_tokens) {
        const int64_t* row = topk_idx + int64_t(t) * num_topk;
        for (int k0 = 0; k0 < num_topk; k0 += 8) {
            int64_t e[8];  // the eight loads of a round in flight before the first is used
#pragma unroll
            for (int u = 0; u < 8; ++u) e[u] = k0 + u < num_topk ? row[k0 + u] : -1;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (e[u] < 0 || e[u] >= num_experts) continue;
                atomicAdd(&hist[int(e[u])], 1);
                // e / E_l by multiply-high (exact below 2^16 experts); magic 0 stands for E_l == 1
                const int r = rank_magic != 0 ? int(__umulhi(uint32_t(e[u]), rank_magic)) : int(e[u]);
#pragma unroll
                for (int q = 0; q < kMaxRankWords; ++q)
                    if ((r >> 6) == q) member[q] |= uint64_t(1) << (r & 63);
            }
        }
        uint8_t* out = is_token_in_rank + int64_t(t) * num_ranks;
        if ((num_ranks & 7) == 0) {
            for (int r8 = 0; r8 < num_ranks; r8 += 8)
                *reinterpret_cast<uint64_t*>(out + r8) = bits_to_bool_bytes(uint32_t(member[r8 >> 6] >> (r8 & 63)));
        } else {
            for (int r = 0; r < num_ranks; ++r) out[r] = uint8_t((member[r >> 6] >> (r & 63)) & 1);
        }
    }
    for (int r = 0; r < num_ranks; ++r) {
        const uint64_t votes = __ballot((member[r >> 6] >> (r & 63)) & 1);
        if (lane == 0 && votes != 0) atomicAdd(&hist[num_experts + r], __popcll(votes));
    }
    for (int nd = 0; nd < num_nodes; ++nd) {
        const int r0 = nd * 8;  // 8 ranks per node (reference: NUM_MAX_NVL_PEERS, csrc/kernels/configs.cuh:3)
        const uint64_t votes = __ballot((member[r0 >> 6] >> (r0 & 63)) & 0xffull);
        if (lane == 0 && votes != 0) atomicAdd(&hist[num_experts + num_ranks + nd], __popcll(votes));
    }
    __syncthreads();
    if (gridDim.x == 1) {  // the partial row is the result
        for (int j = tid; j < width; j += kLayoutThreads) {
            if (j < num_experts)
                per_expert[j] = hist[j];
            else if (j < num_experts + num_ranks)
                per_rank[j - num_experts] = hist[j];
            else
                per_node[j - num_experts - num_ranks] = hist[j];
        }
        return;
    }
    int32_t* dst = partial + int64_t(blockIdx.x) * width;
    for (int j = tid; j < width; j += kLayoutThreads) dst[j] = hist[j];
}

__global__ __launch_bounds__(kLayoutThreads) void layout_reduce_kernel(const int32_t* __restrict__ partial,
                                                                       int num_partials, int num_experts,
                                                                       int num_ranks, int num_nodes,
                                                                       int32_t* __restrict__ per_rank,
                                                                       int32_t* __restrict__ per_node,
                                                                       int32_t* __restrict__ per_expert) {
    const int width = num_experts + num_ranks + num_nodes;
    const int j = blockIdx.x * kLayoutThreads + threadIdx.x;
    if (j >= width) return;
    int sum = 0;
    for (int p0 = 0; p0 < num_partials; p0 += 8) {  // eight loads in flight
        int v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = p0 + u < num_partials ? partial[int64_t(p0 + u) * width + j] : 0;
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += v[u];
    }
    if (j < num_experts)
        per_expert[j] = sum;
    else if (j < num_experts + num_ranks)
        per_rank[j - num_experts] = sum;
    else
        per_node[j - num_experts - num_ranks] = sum;
}

// ---------------------------------------------------------------------
// moe_routing_sort: stable partition of token ids by destination rank.
//   count:   per 1024-token chunk and rank, tokens bound for that rank
//            (ballot + popcount per wave, summed over the chunk's 16 waves);
//   scan:    one workgroup turns the [chunk][rank] table into write offsets
//            (rank-major, chunk-minor) and emits send_counts / send_cumsum;
//   scatter: the count pass again, this time writing the ids.
// Ascending token order inside a rank follows from the chunk/wave/lane order.
// Reference: csrc/kernels/efa_kernels.cu:220-318 (one thread per rank there).
// Small batches take the one-launch variant further down.
// ---------------------------------------------------------------------
constexpr int kSortChunk = 1024;

template <bool kScatter>
__global__ __launch_bounds__(kSortChunk) void routing_sort_pass_kernel(
    const uint8_t* __restrict__ is_token_in_rank, int num_tokens, int num_ranks, int32_t* __restrict__ chunk_table,
    int64_t* __restrict__ sorted_token_ids, int32_t* __restrict__ row_of_pair) {
    extern __shared__ int32_t wave_cnt[];  // [16][R]
    const int tid = threadIdx.x, lane = lane_id(), w = wave_in_block();
    const int c = blockIdx.x;
    const int t = c * kSortChunk + tid;
    const uint8_t* row = is_token_in_rank + int64_t(t) * num_ranks;
    for (int r = 0; r < num_ranks; ++r) {
        const bool in = t < num_tokens && row[r] != 0;
        const uint64_t votes = __ballot(in);
        if (lane == 0) wave_cnt[w * num_ranks + r] = __popcll(votes);
    }
    __syncthreads();
    if constexpr (!kScatter) {
        for (int r = tid; r < num_ranks; r += kSortChunk) {
            int sum = 0;
            for (int w2 = 0; w2 < kSortChunk / kWave; ++w2) sum += wave_cnt[w2 * num_ranks + r];
            chunk_table[int64_t(c) * num_ranks + r] = sum;
        }
    } else {
        // one thread per rank turns the 16 per-wave counts into the waves' first positions
        for (int r = tid; r < num_ranks; r += kSortChunk) {
            int run = chunk_table[int64_t(c) * num_ranks + r];
#pragma unroll
            for (int w2 = 0; w2 < kSortChunk / kWave; ++w2) {
                const int cnt = wave_cnt[w2 * num_ranks + r];
                wave_cnt[w2 * num_ranks + r] = run;
                run += cnt;
            }
        }
        __syncthreads();
        for (int r = 0; r < num_ranks; ++r) {
            const bool in = t < num_tokens && row[r] != 0;
            const uint64_t votes = __ballot(in);
            const int pos = wave_cnt[w * num_ranks + r] + __popcll(votes & lanes_below(lane));
            if (in) sorted_token_ids[pos] = t;
            if (row_of_pair != nullptr && t < num_tokens) row_of_pair[int64_t(t) * num_ranks + r] = in ? pos : -1;
        }
    }
}

__global__ __launch_bounds__(256) void routing_sort_scan_kernel(int32_t* __restrict__ chunk_table, int num_chunks,
                                                                int num_ranks, int32_t* __restrict__ send_counts,
                                                                int64_t* __restrict__ send_cumsum) {
    extern __shared__ int64_t rank_base[];  // [R + 1]
    const int tid = threadIdx.x;
    for (int r = tid; r < num_ranks; r += 256) {
        int sum = 0;
        for (int c = 0; c < num_chunks; ++c) sum += chunk_table[int64_t(c) * num_ranks + r];
        send_counts[r] = sum;
        rank_base[r + 1] = sum;
    }
    __syncthreads();
    if (tid == 0) {
        rank_base[0] = 0;
        for (int r = 0; r < num_ranks; ++r) rank_base[r + 1] += rank_base[r];
    }
    __syncthreads();
    for (int r = tid; r <= num_ranks; r += 256) send_cumsum[r] = rank_base[r];
    for (int r = tid; r < num_ranks; r += 256) {
        int run = int(rank_base[r]);
        for (int c = 0; c < num_chunks; ++c) {
            const int cnt = chunk_table[int64_t(c) * num_ranks + r];
            chunk_table[int64_t(c) * num_ranks + r] = run;
            run += cnt;
        }
    }
}

// ---------------------------------------------------------------------
// The same sort in one launch, for up to 8192 tokens and 64 ranks: one workgroup per destination
// rank, each thread a run of consecutive tokens.  The workgroup reads the whole membership matrix
// (a few tens of KiB, from L2), so besides the positions of its own rank's tokens (a scan of one
// count per thread) it gets the number of memberships of all lower ranks — where its ids start —
// from the same data, without waiting for anybody.  One barrier; 10 us of three launches become 4.
// ---------------------------------------------------------------------
constexpr int kSingleSortTokensPerThread = 8;

// Bit r of the result = is_token_in_rank[t][r] != 0, for up to 64 ranks.
__device__ __forceinline__ uint64_t membership_mask(const uint8_t* row, int num_ranks) {
    uint64_t mask = 0;
    if ((num_ranks & 7) == 0 && (reinterpret_cast<uintptr_t>(row) & 7) == 0) {
        for (int r8 = 0; r8 < num_ranks; r8 += 8) {
            uint64_t v = *reinterpret_cast<const uint64_t*>(row + r8);
            v |= v >> 4, v |= v >> 2, v |= v >> 1;  // any bit of a byte -> its bit 0
            v &= 0x0101010101010101ull;
            mask |= ((v * 0x0102040810204080ull) >> 56) << r8;  // gather the eight bit-0s into one byte
        }
    } else {
        for (int r = 0; r < num_ranks; ++r) mask |= uint64_t(row[r] != 0) << r;
    }
    return mask;
}

__global__ __launch_bounds__(kSortChunk) void routing_sort_single_kernel(
    const uint8_t* __restrict__ is_token_in_rank, int num_tokens, int num_ranks, int tokens_per_thread,
    int32_t* __restrict__ send_counts, int64_t* __restrict__ send_cumsum, int64_t* __restrict__ sorted_token_ids,
    int32_t* __restrict__ row_of_pair) {
    constexpr int kWaves = kSortChunk / kWave;
    __shared__ int32_t wave_own[kWaves];    // tokens of this rank in each wave
    __shared__ int32_t wave_lower[kWaves];  // memberships of lower ranks in each wave
    const int tid = threadIdx.x, lane = lane_id(), w = wave_in_block();
    const int r = blockIdx.x;
    const uint64_t lower_mask = (uint64_t(1) << r) - 1;
    const int first = tid * tokens_per_thread;
    uint32_t own_bits = 0;  // bit i: token first + i goes to rank r
    int lower = 0;
#pragma unroll
    for (int i = 0; i < kSingleSortTokensPerThread; ++i) {
        const int t = first + i;
        if (i < tokens_per_thread && t < num_tokens) {
            const uint64_t m = membership_mask(is_token_in_rank + int64_t(t) * num_ranks, num_ranks);
            own_bits |= uint32_t((m >> r) & 1) << i;
            lower += __popcll(m & lower_mask);
        }
    }
    const int own = __popc(own_bits);
    const int incl = wave_inclusive_sum(own);
    const int lower_wave = wave_inclusive_sum(lower);
    if (lane == kWave - 1) wave_own[w] = incl, wave_lower[w] = lower_wave;
    lds_barrier();
    int before = 0, total = 0, base = 0;
#pragma unroll
    for (int w2 = 0; w2 < kWaves; ++w2) {
        const int c = wave_own[w2];
        if (w2 < w) before += c;
        total += c;
        base += wave_lower[w2];
    }
    int64_t pos = int64_t(base) + before + incl - own;
#pragma unroll
    for (int i = 0; i < kSingleSortTokensPerThread; ++i) {
        const bool mine = (own_bits >> i) & 1;
        // the inverse of the list, for the reduce that adds up the rows coming back: where is (token, rank)?
        if (row_of_pair != nullptr && i < tokens_per_thread && first + i < num_tokens)
            row_of_pair[int64_t(first + i) * num_ranks + r] = mine ? int32_t(pos) : -1;
        if (mine) sorted_token_ids[pos++] = first + i;
    }
    if (tid == 0) {
        send_counts[r] = total;
        send_cumsum[r] = base;
        if (r == num_ranks - 1) send_cumsum[num_ranks] = int64_t(base) + total;
    }
}

// ---------------------------------------------------------------------
// channel_prefix_matrix: one workgroup per destination rank, one wave per
// channel (up to sixteen at a time), then an in-place prefix over channels.
// Reference: csrc/kernels/intranode.cu:90-112.
// ---------------------------------------------------------------------
__global__ __launch_bounds__(1024) void channel_prefix_kernel(const uint8_t* __restrict__ is_token_in_rank,
                                                              int num_tokens, int num_ranks, int num_channels,
                                                              int32_t* __restrict__ cpm) {
    extern __shared__ int32_t per_channel[];  // [C]
    const int dst = blockIdx.x, lane = lane_id(), w = wave_in_block();
    const int waves = int(blockDim.x) >> 6;
    const int per = (num_tokens + num_channels - 1) / num_channels;
    for (int ch = w; ch < num_channels; ch += waves) {
        const int begin = min(per * ch, num_tokens), end = min(begin + per, num_tokens);
        int count = 0;
        for (int t0 = begin + lane; t0 < end; t0 += kWave * 8) {  // eight loads in flight per lane
            uint8_t v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int t = t0 + u * kWave;
                v[u] = t < end ? is_token_in_rank[int64_t(t) * num_ranks + dst] : uint8_t(0);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) count += v[u] != 0;
        }
        count = wave_sum(count);
        if (lane == 0) per_channel[ch] = count;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int ch = 0; ch < num_channels; ++ch) {
            run += per_channel[ch];
            cpm[int64_t(dst) * num_channels + ch] = run;
        }
    }
}

// ---------------------------------------------------------------------
// pack_rows: dst[i] = src[ids[i]].  One workgroup per output row, one 16-byte
// vector per thread (rows wider than 1024 vectors loop): the same shape as a
// flat copy, which is what reaches the highest HBM rate on this GPU.  The row
// count is read from device memory so no host sync is needed; workgroups past
// it exit.  Plain loads: a source row is gathered about five times, so it
// should stay in L2 / Infinity Cache.
// Reference: deep_ep/buffer.py:877,917 (torch advanced-index gathers).
// ---------------------------------------------------------------------
// kStream: the packed rows exceed what the caches hold, so they are written with the non-temporal
// hint; the source rows are read the ordinary way because several destinations re-read them.
template <bool kStream>
__global__ __launch_bounds__(1024) void pack_rows_kernel(const uint8_t* __restrict__ src,
                                                         const uint8_t* __restrict__ scale_src,
                                                         const int64_t* __restrict__ ids,
                                                         const int64_t* __restrict__ num_rows_dev, int64_t max_rows,
                                                         int num_src_rows, int row_bytes, int scale_row_bytes,
                                                         uint8_t* __restrict__ dst, uint8_t* __restrict__ scale_dst) {
    int64_t num_rows = *num_rows_dev;
    if (num_rows > max_rows) num_rows = max_rows;
    const int num_vec = row_bytes / 16;
    for (int64_t i = blockIdx.x; i < num_rows; i += gridDim.x) {
        const int64_t id = ids[i];
        if (id < 0 || id >= num_src_rows) continue;
        const uint8_t* s = src + id * row_bytes;
        uint8_t* d = dst + i * row_bytes;
        for (int v = threadIdx.x; v < num_vec; v += blockDim.x)
            store_u32x4<kStream>(d + int64_t(v) * 16, load_u32x4<false>(s + int64_t(v) * 16));
        if (scale_src != nullptr) {
            const uint32_t* ss = reinterpret_cast<const uint32_t*>(scale_src + id * scale_row_bytes);
            uint32_t* sd = reinterpret_cast<uint32_t*>(scale_dst + i * scale_row_bytes);
            for (int v = threadIdx.x; v < scale_row_bytes / 4; v += blockDim.x) sd[v] = ss[v];
        }
    }
}

}  // namespace deepep

using namespace deepep;

extern "C" {

size_t deepep_layout_workspace_bytes(int num_tokens, int num_ranks, int num_experts) {
    const int64_t blocks = (int64_t(num_tokens) + kLayoutThreads - 1) / kLayoutThreads;
    const int64_t width = int64_t(num_experts) + num_ranks + num_ranks / 8 + 1;
    return size_t((blocks < 1 ? 1 : blocks) * width * 4);
}

int deepep_get_dispatch_layout(const int64_t* topk_idx, int num_tokens, int num_topk, int num_ranks,
                               int num_experts, int32_t* num_tokens_per_rank, int32_t* num_tokens_per_rdma_rank,
                               int32_t* num_tokens_per_expert, uint8_t* is_token_in_rank, void* workspace,
                               size_t workspace_bytes, void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_tokens >= 0 && num_topk > 0);
    EP_HOST_ASSERT(num_experts > 0);
    EP_HOST_ASSERT(num_ranks > 0 && num_experts % num_ranks == 0);
    EP_HOST_ASSERT(num_ranks <= 64 * kMaxRankWords);
    EP_HOST_ASSERT(num_tokens_per_rdma_rank == nullptr || (num_ranks % 8 == 0 && num_ranks > 8));
    EP_HOST_ASSERT(num_tokens_per_rank != nullptr && num_tokens_per_expert != nullptr);
    EP_HOST_ASSERT(num_tokens == 0 || (topk_idx != nullptr && is_token_in_rank != nullptr));
    EP_HOST_ASSERT((num_ranks & 7) != 0 || (reinterpret_cast<uintptr_t>(is_token_in_rank) & 7) == 0);
    const int num_nodes = num_tokens_per_rdma_rank != nullptr ? num_ranks / 8 : 0;
    const int width = num_experts + num_ranks + num_nodes;
    EP_HOST_ASSERT(size_t(width) * 4 <= 64 * 1024);
    const int blocks = num_tokens == 0 ? 1 : (num_tokens + kLayoutThreads - 1) / kLayoutThreads;
    EP_HOST_ASSERT(workspace != nullptr && workspace_bytes >= size_t(blocks) * width * 4);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    int32_t* partial = reinterpret_cast<int32_t*>(workspace);
    const uint32_t experts_per_rank = uint32_t(num_experts / num_ranks);
    EP_HOST_ASSERT(num_experts < 65536);
    const uint32_t rank_magic =
        experts_per_rank == 1 ? 0u : uint32_t(((uint64_t(1) << 32) + experts_per_rank - 1) / experts_per_rank);
    layout_count_kernel<<<blocks, kLayoutThreads, size_t(width) * 4, s>>>(
        topk_idx, num_tokens, num_topk, num_ranks, num_experts, rank_magic, num_nodes, is_token_in_rank, partial,
        num_tokens_per_rank, num_tokens_per_rdma_rank, num_tokens_per_expert);
    EP_LAUNCH_CHECK();
    if (blocks == 1) return 0;
    layout_reduce_kernel<<<(width + kLayoutThreads - 1) / kLayoutThreads, kLayoutThreads, 0, s>>>(
        partial, blocks, num_experts, num_ranks, num_nodes, num_tokens_per_rank, num_tokens_per_rdma_rank,
        num_tokens_per_expert);
    EP_LAUNCH_CHECK();
    return 0;
}

size_t deepep_routing_sort_workspace_bytes(int num_tokens, int num_ranks) {
    const int64_t chunks = (int64_t(num_tokens) + kSortChunk - 1) / kSortChunk;
    return size_t((chunks < 1 ? 1 : chunks) * num_ranks * 4);
}

int deepep_moe_routing_sort(const uint8_t* is_token_in_rank, int num_tokens, int num_ranks,
                            int64_t* sorted_token_ids, int32_t* send_counts, int64_t* send_cumsum,
                            int32_t* row_of_pair, void* workspace, size_t workspace_bytes, void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_tokens >= 0 && num_ranks > 0 && num_ranks <= 1024);
    EP_HOST_ASSERT(send_counts != nullptr && send_cumsum != nullptr);
    EP_HOST_ASSERT(num_tokens == 0 || (is_token_in_rank != nullptr && sorted_token_ids != nullptr));
    const int chunks = num_tokens == 0 ? 1 : (num_tokens + kSortChunk - 1) / kSortChunk;
    EP_HOST_ASSERT(workspace != nullptr && workspace_bytes >= size_t(chunks) * num_ranks * 4);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (num_tokens <= kSortChunk * kSingleSortTokensPerThread && num_ranks <= 64) {
        const int per_thread = num_tokens == 0 ? 1 : (num_tokens + kSortChunk - 1) / kSortChunk;
        routing_sort_single_kernel<<<num_ranks, kSortChunk, 0, s>>>(is_token_in_rank, num_tokens, num_ranks, per_thread,
                                                                   send_counts, send_cumsum, sorted_token_ids,
                                                                   row_of_pair);
        EP_LAUNCH_CHECK();
        return 0;
    }
    int32_t* table = reinterpret_cast<int32_t*>(workspace);
    const size_t lds = size_t(kSortChunk / kWave) * num_ranks * 4;
    routing_sort_pass_kernel<false><<<chunks, kSortChunk, lds, s>>>(is_token_in_rank, num_tokens, num_ranks, table,
                                                                    sorted_token_ids, nullptr);
    EP_LAUNCH_CHECK();
    routing_sort_scan_kernel<<<1, 256, size_t(num_ranks + 1) * 8, s>>>(table, chunks, num_ranks, send_counts,
                                                                       send_cumsum);
    EP_LAUNCH_CHECK();
    if (num_tokens > 0) {
        routing_sort_pass_kernel<true><<<chunks, kSortChunk, lds, s>>>(is_token_in_rank, num_tokens, num_ranks,
                                                                       table, sorted_token_ids, row_of_pair);
        EP_LAUNCH_CHECK();
    }
    return 0;
}

int deepep_channel_prefix_matrix(const uint8_t* is_token_in_rank, int num_tokens, int num_ranks, int num_channels,
                                 int32_t* channel_prefix_matrix, void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_tokens >= 0 && num_ranks > 0 && num_channels > 0 && num_channels <= 4096);
    EP_HOST_ASSERT(channel_prefix_matrix != nullptr);
    EP_HOST_ASSERT(num_tokens == 0 || is_token_in_rank != nullptr);
    // one wave per channel, up to sixteen at a time
    const int threads = num_channels >= 16 ? 1024 : ((num_channels + 3) / 4) * 256;
    channel_prefix_kernel<<<num_ranks, threads, size_t(num_channels) * 4, reinterpret_cast<hipStream_t>(stream)>>>(
        is_token_in_rank, num_tokens, num_ranks, num_channels, channel_prefix_matrix);
    EP_LAUNCH_CHECK();
    return 0;
}

int deepep_pack_rows(const void* src, const void* scale_src, const int64_t* sorted_token_ids,
                     const int64_t* num_rows_dev, int64_t max_rows, int num_src_rows, int row_bytes,
                     int scale_row_bytes, void* dst, void* scale_dst, void* stream) {
    clear_error();
    EP_HOST_ASSERT(max_rows >= 0 && num_src_rows >= 0);
    EP_HOST_ASSERT(row_bytes > 0 && row_bytes % 16 == 0);
    EP_HOST_ASSERT(scale_src == nullptr || (scale_dst != nullptr && scale_row_bytes > 0 && scale_row_bytes % 4 == 0));
    if (max_rows == 0) return 0;
    EP_HOST_ASSERT(src != nullptr && dst != nullptr && sorted_token_ids != nullptr && num_rows_dev != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(src) & 15) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(scale_src) & 3) == 0 && (reinterpret_cast<uintptr_t>(scale_dst) & 3) == 0);
    const int num_vec = row_bytes / 16;
    int threads = ((num_vec + 63) / 64) * 64;
    if (threads > 1024) threads = 1024;
    int64_t blocks = max_rows;
    if (blocks > (int64_t(1) << 22)) blocks = int64_t(1) << 22;
#define DEEPEP_LAUNCH_PACK(STREAM)                                                                              \
    pack_rows_kernel<STREAM><<<dim3(unsigned(blocks)), threads, 0, reinterpret_cast<hipStream_t>(stream)>>>(      \
        reinterpret_cast<const uint8_t*>(src), reinterpret_cast<const uint8_t*>(scale_src), sorted_token_ids,      \
        num_rows_dev, max_rows, num_src_rows, row_bytes, scale_row_bytes, reinterpret_cast<uint8_t*>(dst),         \
        reinterpret_cast<uint8_t*>(scale_dst))
    if (max_rows * row_bytes > stream_bytes()) DEEPEP_LAUNCH_PACK(true);
    else DEEPEP_LAUNCH_PACK(false);
#undef DEEPEP_LAUNCH_PACK
    EP_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
