// What a rank derives from the gathered route counts before the exchange of a
// low-latency dispatch: rows to send to and to expect from every rank, where its
// returned rows start inside every peer's combine buffer, and one metadata
// record per row it will receive.  The reference computes all of it on the host
// from three device-to-host copies (csrc/transport/ll_pipeline.cpp:1204-1269 and
// :1277-1361); here it is one launch on the stream the counts arrive on.
#include "common.hpp"
#include "../../include/deepep_hip.h"

namespace deepep {

constexpr int kExchangeThreads = 1024;
constexpr int kExchangeMaxRanks = 1024;

__device__ __forceinline__ int64_t wave_sum_i64(int64_t v) {
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) v += __shfl_xor(v, d, kWave);
    return v;
}

// Every workgroup derives the per-rank tables itself (the R x E counts once, from L2: one wave per
// source rank, every load of a row in flight together) and then fills its share of the row
// records; workgroup 0 also writes the per-rank outputs.
__global__ __launch_bounds__(kExchangeThreads) void ll_exchange_meta_kernel(
    const int32_t* __restrict__ all_num_routed, int num_experts, int num_ranks, int rank, int max_tokens,
    int64_t row_capacity, int32_t* __restrict__ send_counts, int32_t* __restrict__ recv_counts,
    int32_t* __restrict__ totals, int64_t* __restrict__ combine_remote_recv_offset,
    uint32_t* __restrict__ source_rank, uint32_t* __restrict__ source_offset, uint32_t* __restrict__ padded_index,
    uint32_t* __restrict__ combine_send_offset, uint32_t* __restrict__ num_recv_tokens,
    uint32_t* __restrict__ tokens_per_expert) {
    __shared__ int32_t recv_prefix[kExchangeMaxRanks + 1];
    __shared__ int32_t recv_of[kExchangeMaxRanks];
    __shared__ int32_t send_to[kExchangeMaxRanks];
    __shared__ int64_t below_of[kExchangeMaxRanks];
    __shared__ int32_t wave_bad[kExchangeThreads / kWave];
    const int tid = threadIdx.x, lane = lane_id(), w = wave_in_block();
    constexpr int kWaves = kExchangeThreads / kWave;
    const int experts_per_rank = num_experts / num_ranks;
    const int first_expert = rank * experts_per_rank;
    // a count above the per-expert bound marks the whole gather as corrupt: nobody sends or
    // receives this time (csrc/transport/ll_pipeline.cpp:1216-1248)
    const uint32_t max_per_expert = max_tokens > 0 ? uint32_t(max_tokens) : 4096u;
    bool bad = false;
    for (int r = w; r < num_ranks; r += kWaves) {
        const int32_t* row = all_num_routed + int64_t(r) * num_experts;
        int64_t below = 0;  // what rank r routed to the ranks below this one
        int to_me = 0;      // ... and to this rank's experts
        for (int e0 = 0; e0 < num_experts; e0 += 4 * kWave) {
            uint32_t v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int e = e0 + u * kWave + lane;
                v[u] = e < num_experts ? uint32_t(row[e]) : 0u;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int e = e0 + u * kWave + lane;
                bad |= v[u] > max_per_expert;
                if (e < first_expert) below += int64_t(v[u]);
                else if (e < first_expert + experts_per_rank) to_me += int(v[u]);
            }
        }
        below = wave_sum_i64(below);
        to_me = __builtin_amdgcn_readlane(wave_inclusive_sum(to_me), kWave - 1);
        if (lane == 0) below_of[r] = below, recv_of[r] = to_me;
    }
    {
        const bool any = __ballot(bad) != 0;
        if (lane == 0) wave_bad[w] = any ? 1 : 0;
    }
    // this rank's own row, summed per destination rank
    const int32_t* mine = all_num_routed + int64_t(rank) * num_experts;
    for (int r = w; r < num_ranks; r += kWaves) {
        int part = 0;
        for (int e = lane; e < experts_per_rank; e += kWave) part += mine[r * experts_per_rank + e];
        part = __builtin_amdgcn_readlane(wave_inclusive_sum(part), kWave - 1);
        if (lane == 0) send_to[r] = part;
    }
    lds_barrier();
    bool is_corrupt = false;
#pragma unroll
    for (int i = 0; i < kWaves; ++i) is_corrupt |= wave_bad[i] != 0;

    if (tid < kWave) {  // exclusive prefix over the ranks, one wave
        int carry = 0;
        for (int r0 = 0; r0 < num_ranks; r0 += kWave) {
            const int r = r0 + tid;
            const int v = r < num_ranks && !is_corrupt ? recv_of[r] : 0;
            const int inc = wave_inclusive_sum(v);
            if (r < num_ranks) recv_prefix[r] = carry + inc - v;
            carry += __builtin_amdgcn_readlane(inc, kWave - 1);
        }
        if (tid == 0) recv_prefix[num_ranks] = carry;
    }
    lds_barrier();
    int total_recv = recv_prefix[num_ranks];

    if (blockIdx.x == 0) {
        for (int r = tid; r < num_ranks; r += kExchangeThreads) {
            send_counts[r] = is_corrupt ? 0 : send_to[r];
            recv_counts[r] = is_corrupt ? 0 : recv_of[r];
            // where this rank's returned rows start in peer r's combine buffer: behind what peer r
            // sent to the ranks below this one (csrc/transport/ll_pipeline.cpp:1283-1295, computed
            // from the raw counts whatever their state)
            combine_remote_recv_offset[r] = below_of[r];
        }
        for (int e = tid; e < experts_per_rank; e += kExchangeThreads) tokens_per_expert[e] = 0;
        if (tid >= kWave && tid < 2 * kWave) {  // wave 1: total sent
            int part = 0;
            if (!is_corrupt)
                for (int r = lane; r < num_ranks; r += kWave) part += send_to[r];
            const int total_send = __builtin_amdgcn_readlane(wave_inclusive_sum(part), kWave - 1);
            if (lane == 0) totals[0] = total_send, totals[1] = total_recv, totals[2] = is_corrupt ? 1 : 0;
        }
    }
    // csrc/transport/ll_pipeline.cpp:1306-1312: an impossible total receives nothing
    const int64_t max_possible = int64_t(num_ranks) * max_tokens * 8;
    int64_t rows = total_recv;
    if (rows < 0 || rows > max_possible) rows = 0, total_recv = 0;
    if (rows > row_capacity) rows = row_capacity;
    if (blockIdx.x == 0 && tid == 0) num_recv_tokens[0] = uint32_t(total_recv), num_recv_tokens[1] = uint32_t(rows);

    // one record per expected row, grouped by source rank (csrc/transport/ll_pipeline.cpp:1319-1343)
    for (int64_t i = int64_t(blockIdx.x) * kExchangeThreads + tid; i < rows; i += int64_t(gridDim.x) * kExchangeThreads) {
        int lo = 0, hi = num_ranks;  // recv_prefix[lo] <= i < recv_prefix[hi]
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (recv_prefix[mid] <= i) lo = mid; else hi = mid;
        }
        const uint32_t t = uint32_t(i - recv_prefix[lo]);
        source_rank[i] = uint32_t(lo);
        source_offset[i] = uint32_t(lo) * uint32_t(max_tokens) + t;
        padded_index[i] = uint32_t(i);
        combine_send_offset[i] = uint32_t(recv_prefix[lo]) + t;
    }
}

}  // namespace deepep

using namespace deepep;

extern "C" int deepep_ll_exchange_metadata(const int32_t* all_num_routed, int num_experts, int num_ranks, int rank,
                                           int num_max_dispatch_tokens_per_rank, int64_t row_capacity,
                                           int32_t* send_counts, int32_t* recv_counts, int32_t* totals,
                                           int64_t* combine_remote_recv_offset, uint32_t* source_rank,
                                           uint32_t* source_offset, uint32_t* padded_index,
                                           uint32_t* combine_send_offset, uint32_t* num_recv_tokens,
                                           uint32_t* tokens_per_expert, void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_ranks > 0 && num_ranks <= kExchangeMaxRanks);
    EP_HOST_ASSERT(num_experts > 0 && num_experts % num_ranks == 0);
    EP_HOST_ASSERT(rank >= 0 && rank < num_ranks);
    EP_HOST_ASSERT(int64_t(num_ranks) * num_experts < (int64_t(1) << 30));
    EP_HOST_ASSERT(row_capacity >= 0 && row_capacity < (int64_t(1) << 32));
    EP_HOST_ASSERT(all_num_routed != nullptr && send_counts != nullptr && recv_counts != nullptr && totals != nullptr);
    EP_HOST_ASSERT(combine_remote_recv_offset != nullptr && num_recv_tokens != nullptr && tokens_per_expert != nullptr);
    EP_HOST_ASSERT(row_capacity == 0 || (source_rank != nullptr && source_offset != nullptr &&
                                         padded_index != nullptr && combine_send_offset != nullptr));
    int64_t blocks = (row_capacity + 4 * kExchangeThreads - 1) / (4 * kExchangeThreads);
    blocks = blocks < 1 ? 1 : (blocks > 64 ? 64 : blocks);
    ll_exchange_meta_kernel<<<unsigned(blocks), kExchangeThreads, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        all_num_routed, num_experts, num_ranks, rank, num_max_dispatch_tokens_per_rank, row_capacity, send_counts,
        recv_counts, totals, combine_remote_recv_offset, source_rank, source_offset, padded_index,
        combine_send_offset, num_recv_tokens, tokens_per_expert);
    EP_LAUNCH_CHECK();
    return 0;
}
