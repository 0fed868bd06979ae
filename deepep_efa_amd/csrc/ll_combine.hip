// Low-latency combine: return of the expert outputs (send side) and the
// top-k weighted reduction (receive side).
//
// Data layout in HBM:
//   x (expert outputs)  [E_l][N][H] bf16, live rows given by layout_range
//   combine_staging     [E][M][H] bf16 — slot j of expert e holds the output
//                       for this rank's pair whose dispatch slot was j
//   combine_send_slots  [E_l][R][M][H] bf16 — rows owed to other ranks
#include "common.hpp"
#include "segments.hpp"
#include "../../include/deepep_hip.h"

namespace deepep {

// ---------------------------------------------------------------------
// Send side: one wave per live row, rows enumerated segment by segment in
// arrival order (reference: deep_ep/buffer.py:2601-2608 gathers
// x[recv_expert_ids, recv_expert_pos] and un-sorts to arrival order).
// ---------------------------------------------------------------------
__global__ __launch_bounds__(256) void ll_combine_send_kernel(
    const uint8_t* __restrict__ x, const int64_t* __restrict__ layout_range, int hidden, int num_local_experts,
    int num_ranks, int rank, int max_tokens, int parts, uint8_t* __restrict__ combine_staging,
    uint8_t* __restrict__ combine_send_slots) {
    extern __shared__ int32_t flat[];  // [num_segments + 1] then begin[num_segments]
    __shared__ int32_t wave_totals[4];
    const int tid = threadIdx.x, lane = lane_id(), w = wave_in_block();
    const int num_segments = num_local_experts * num_ranks;
    int32_t* begin = flat + num_segments + 1;

    for (int s = tid; s < num_segments; s += 256) {
        const int64_t lr = layout_range[s];
        int c = int(lr & 0xffffffffll);
        c = c < 0 ? 0 : (c > max_tokens ? max_tokens : c);
        flat[s] = c;
        begin[s] = int(lr >> 32);
    }
    __syncthreads();
    block_exclusive_scan_256(flat, num_segments, wave_totals);
    const int total_rows = flat[num_segments];

    const int64_t row_bytes = int64_t(hidden) * 2;
    const int num_vec = int(row_bytes / 16);
    const int64_t slots_per_expert = int64_t(max_tokens) * num_ranks;
    const int64_t waves_total = int64_t(gridDim.x) * 4;

    for (int64_t item = blockIdx.x * 4 + w; item < int64_t(total_rows) * parts; item += waves_total) {
        const int row = int(item / parts), part = int(item - int64_t(row) * parts);
        const int seg = __builtin_amdgcn_readfirstlane(find_segment(flat, num_segments, row));
        const int j = row - __builtin_amdgcn_readfirstlane(flat[seg]);
        const int le = seg / num_ranks;
        const int s = seg - le * num_ranks;
        const int b = __builtin_amdgcn_readfirstlane(begin[seg]);
        if (b < 0 || int64_t(b) + j >= slots_per_expert) continue;  // malformed range: never read past the expert
        const uint8_t* src = x + (int64_t(le) * slots_per_expert + b + j) * row_bytes;
        uint8_t* dst;
        if (s == rank)
            dst = combine_staging + ((int64_t(rank) * num_local_experts + le) * max_tokens + j) * row_bytes;
        else if (combine_send_slots != nullptr)
            dst = combine_send_slots + (int64_t(seg) * max_tokens + j) * row_bytes;
        else
            continue;
        int v_begin, v_end;
        row_part_range(num_vec, parts, part, v_begin, v_end);
        wave_copy_vec16(src, dst, v_begin, v_end, lane);
    }
}

// ---------------------------------------------------------------------
// Receive side: one wave = one (token, 1 KiB piece of the output row).
// All K source vectors are loaded before the FMA chain so K 16-byte loads
// are in flight per lane; accumulation order is k = 0..K-1, float32 FMA,
// one rounding to bf16 at the end
// (reference: csrc/kernels/coop_combine_recv.cuh:222-260).
// ---------------------------------------------------------------------
__global__ __launch_bounds__(256) void ll_combine_recv_kernel(
    const uint8_t* __restrict__ combine_staging, const int64_t* __restrict__ topk_idx,
    const float* __restrict__ topk_weights, const int32_t* __restrict__ pair_slot, int num_tokens, int hidden,
    int num_topk, int num_experts, int max_tokens, int pieces_per_row, uint8_t* __restrict__ out) {
    const int lane = lane_id();
    const int64_t item = int64_t(blockIdx.x) * 4 + wave_in_block();
    if (item >= int64_t(num_tokens) * pieces_per_row) return;
    const int t = int(item / pieces_per_row);
    const int piece = int(item - int64_t(t) * pieces_per_row);
    const int64_t row_bytes = int64_t(hidden) * 2;
    const int64_t off = int64_t(piece) * 1024 + lane * 16;
    const bool lane_live = off < row_bytes;

    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;

    for (int k0 = 0; k0 < num_topk; k0 += 8) {
        u32x4 v[8];
        float wgt[8];
        bool live[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int k = k0 + u;
            live[u] = false;
            wgt[u] = 0.0f;
            if (k < num_topk) {
                const int slot = pair_slot[int64_t(t) * num_topk + k];
                const int64_t e = topk_idx[int64_t(t) * num_topk + k];
                if (slot >= 0 && slot < max_tokens && e >= 0 && e < num_experts) {
                    live[u] = true;
                    wgt[u] = topk_weights[int64_t(t) * num_topk + k];
                    if (lane_live)
                        v[u] = *reinterpret_cast<const u32x4*>(combine_staging +
                                                               (e * max_tokens + slot) * row_bytes + off);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (!live[u] || !lane_live) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i] = __builtin_fmaf(bf16_lo(v[u][i]), wgt[u], acc[2 * i]);
                acc[2 * i + 1] = __builtin_fmaf(bf16_hi(v[u][i]), wgt[u], acc[2 * i + 1]);
            }
        }
    }
    if (lane_live) {
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = pack_bf16x2(acc[2 * i], acc[2 * i + 1]);
        *reinterpret_cast<u32x4*>(out + int64_t(t) * row_bytes + off) = o;
    }
}

}  // namespace deepep

using namespace deepep;

extern "C" {

int deepep_ll_combine_send(const void* x, const int64_t* layout_range, int hidden, int num_experts, int num_ranks,
                           int rank, int num_max_dispatch_tokens_per_rank, void* combine_staging,
                           void* combine_send_slots, int64_t expected_rows, void* workspace, size_t workspace_bytes,
                           void* stream) {
    clear_error();
    EP_HOST_ASSERT(hidden > 0 && hidden % 128 == 0);
    EP_HOST_ASSERT(num_ranks > 0 && num_experts > 0 && num_experts % num_ranks == 0);
    EP_HOST_ASSERT(rank >= 0 && rank < num_ranks);
    EP_HOST_ASSERT(num_max_dispatch_tokens_per_rank > 0);
    EP_HOST_ASSERT(num_experts <= 1024);
    EP_HOST_ASSERT(x != nullptr && layout_range != nullptr && combine_staging != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(combine_staging) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(combine_send_slots) & 15) == 0);
    const int num_local_experts = num_experts / num_ranks;
    const int64_t max_rows = int64_t(num_experts) * num_max_dispatch_tokens_per_rank;
    EP_HOST_ASSERT(max_rows < (int64_t(1) << 31));
    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
    if (max_rows > kLargeBatchRows && workspace != nullptr) {
        EP_HOST_ASSERT(workspace_bytes >= size_t(segment_workspace_bytes(num_experts, num_max_dispatch_tokens_per_rank)));
        EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(workspace) & 15) == 0);
        int32_t* flat = reinterpret_cast<int32_t*>(workspace);
        RowDesc* desc = reinterpret_cast<RowDesc*>(reinterpret_cast<uint8_t*>(workspace) +
                                                   (((int64_t(num_experts) + 1) * 4 + 255) & ~int64_t(255)));
        ll_segment_index_kernel<<<num_experts, kIndexThreads, 0, hs>>>(
            1, nullptr, layout_range, num_local_experts, num_ranks, rank, num_max_dispatch_tokens_per_rank, nullptr,
            nullptr, nullptr, flat, desc);
        EP_LAUNCH_CHECK();
        const int num_vec = hidden * 2 / 16;
        int threads = ((num_vec + 63) / 64) * 64;
        if (threads > 1024) threads = 1024;
        ll_rows_flat_kernel<<<flat_grid_blocks(expected_rows, max_rows, num_max_dispatch_tokens_per_rank), threads, 0,
                              hs>>>(flat, num_experts, desc, reinterpret_cast<const uint8_t*>(x), int64_t(hidden) * 2,
                                    num_vec, reinterpret_cast<uint8_t*>(combine_send_slots),
                                    reinterpret_cast<uint8_t*>(combine_staging), int64_t(hidden) * 2, 0, 0, nullptr, 0,
                                    nullptr, 0);
        EP_LAUNCH_CHECK();
        return 0;
    }
    const int parts = choose_row_parts(max_rows, int64_t(hidden) * 2);
    int64_t blocks = (max_rows * parts + 3) / 4;
    const int64_t cap = max_rows > kLargeBatchRows ? 4096 : 1024;
    if (blocks > cap) blocks = cap;
    const size_t lds = size_t(2 * num_experts + 1) * sizeof(int32_t);
    ll_combine_send_kernel<<<dim3(unsigned(blocks)), 256, lds, hs>>>(
        reinterpret_cast<const uint8_t*>(x), layout_range, hidden, num_local_experts, num_ranks, rank,
        num_max_dispatch_tokens_per_rank, parts, reinterpret_cast<uint8_t*>(combine_staging),
        reinterpret_cast<uint8_t*>(combine_send_slots));
    EP_LAUNCH_CHECK();
    return 0;
}

int deepep_ll_combine_recv(const void* combine_staging, const int64_t* topk_idx, const float* topk_weights,
                           const int32_t* pair_slot, int num_tokens, int hidden, int num_topk, int num_experts,
                           int num_max_dispatch_tokens_per_rank, void* out, void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_tokens >= 0 && hidden > 0 && hidden % 128 == 0 && num_topk > 0);
    EP_HOST_ASSERT(num_experts > 0 && num_max_dispatch_tokens_per_rank > 0);
    if (num_tokens == 0) return 0;
    EP_HOST_ASSERT(combine_staging != nullptr && topk_idx != nullptr && topk_weights != nullptr &&
                   pair_slot != nullptr && out != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(combine_staging) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(out) & 15) == 0);
    const int pieces = (hidden * 2 + 1023) / 1024;
    const int64_t blocks = (int64_t(num_tokens) * pieces + 3) / 4;
    EP_HOST_ASSERT(blocks < (int64_t(1) << 31));
    ll_combine_recv_kernel<<<dim3(unsigned(blocks)), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        reinterpret_cast<const uint8_t*>(combine_staging), topk_idx, topk_weights, pair_slot, num_tokens, hidden,
        num_topk, num_experts, num_max_dispatch_tokens_per_rank, pieces, reinterpret_cast<uint8_t*>(out));
    EP_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
