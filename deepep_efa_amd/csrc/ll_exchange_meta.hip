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

// Every workgroup derives the per-rank tables itself (R * E_l reads each, from L2) and then fills
// its share of the row records; workgroup 0 also writes the per-rank outputs.
__global__ __launch_bounds__(kExchangeThreads) void ll_exchange_meta_kernel(
    const int32_t* __restrict__ all_num_routed, int num_experts, int num_ranks, int rank, int max_tokens,
    int64_t row_capacity, int32_t* __restrict__ send_counts, int32_t* __restrict__ recv_counts,
    int32_t* __restrict__ totals, int64_t* __restrict__ combine_remote_recv_offset,
    uint32_t* __restrict__ source_rank, uint32_t* __restrict__ source_offset, uint32_t* __restrict__ padded_index,
    uint32_t* __restrict__ combine_send_offset, uint32_t* __restrict__ num_recv_tokens,
    uint32_t* __restrict__ tokens_per_expert) {
    __shared__ int32_t recv_prefix[kExchangeMaxRanks + 1];
    __shared__ int32_t recv_of[kExchangeMaxRanks];
    __shared__ int corrupt;
    const int tid = threadIdx.x;
    const int experts_per_rank = num_experts / num_ranks;
    const int first_expert = rank * experts_per_rank;
    // a count above the per-expert bound marks the whole gather as corrupt: nobody sends or
    // receives this time (csrc/transport/ll_pipeline.cpp:1216-1248)
    const uint32_t max_per_expert = max_tokens > 0 ? uint32_t(max_tokens) : 4096u;
    if (tid == 0) corrupt = 0;
    lds_barrier();
    bool bad = false;
    for (int i = tid; i < num_ranks * num_experts; i += kExchangeThreads)
        bad |= uint32_t(all_num_routed[i]) > max_per_expert;
    if (bad) corrupt = 1;  // every writer stores the same value
    lds_barrier();
    const bool is_corrupt = corrupt != 0;

    for (int r = tid; r < num_ranks; r += kExchangeThreads) {
        int sum = 0;
        if (!is_corrupt)
            for (int e = 0; e < experts_per_rank; ++e) sum += all_num_routed[r * num_experts + first_expert + e];
        recv_of[r] = sum;
    }
    lds_barrier();
    if (tid < kWave) {  // exclusive prefix over the ranks, one wave
        int carry = 0;
        for (int r0 = 0; r0 < num_ranks; r0 += kWave) {
            const int r = r0 + tid;
            const int v = r < num_ranks ? recv_of[r] : 0;
            const int inc = wave_inclusive_sum(v);
            if (r < num_ranks) recv_prefix[r] = carry + inc - v;
            carry += __builtin_amdgcn_readlane(inc, kWave - 1);
        }
        if (tid == 0) recv_prefix[num_ranks] = carry;
    }
    lds_barrier();
    int total_recv = recv_prefix[num_ranks];

    if (blockIdx.x == 0) {
        const int32_t* mine = all_num_routed + int64_t(rank) * num_experts;
        for (int r = tid; r < num_ranks; r += kExchangeThreads) {
            int sum = 0;
            if (!is_corrupt)
                for (int e = 0; e < experts_per_rank; ++e) sum += mine[r * experts_per_rank + e];
            send_counts[r] = sum;
            recv_counts[r] = recv_of[r];
            // where this rank's returned rows start in peer r's combine buffer: behind what peer r
            // sent to the ranks below this one (csrc/transport/ll_pipeline.cpp:1283-1295; the reference
            // computes this one even for a corrupt gather)
            int64_t offset = 0;
            const int32_t* theirs = all_num_routed + int64_t(r) * num_experts;
            for (int e = 0; e < first_expert; ++e) offset += int64_t(uint32_t(theirs[e]));
            combine_remote_recv_offset[r] = offset;
        }
        for (int e = tid; e < experts_per_rank; e += kExchangeThreads) tokens_per_expert[e] = 0;
        if (tid < kWave) {
            int part = 0;
            if (!is_corrupt)
                for (int e = tid; e < num_experts; e += kWave) part += mine[e];
            const int total_send = __builtin_amdgcn_readlane(wave_inclusive_sum(part), kWave - 1);
            if (tid == 0) totals[0] = total_send, totals[1] = total_recv, totals[2] = is_corrupt ? 1 : 0;
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
