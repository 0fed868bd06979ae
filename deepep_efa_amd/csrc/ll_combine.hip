// Low-latency combine: return of the expert outputs (send side) and the
// top-k weighted reduction (receive side).
//
// Data layout in HBM:
//   x (expert outputs)  [E_l][N][H] bf16, live rows given by layout_range
//   combine_staging     [E][M][H] bf16 — slot j of expert e holds the output
//                       for this rank's pair whose dispatch slot was j
//   combine_send_slots  [E_l][R][M][H] bf16 — rows owed to other ranks
#include <cstdlib>

#include "common.hpp"
#include "segments.hpp"
#include "../../include/deepep_hip.h"

namespace deepep {

// ---------------------------------------------------------------------
// Send side: one wave per live row part, rows enumerated segment by segment in
// arrival order (reference: deep_ep/buffer.py:2601-2608 gathers
// x[recv_expert_ids, recv_expert_pos] and un-sorts to arrival order).
// skip_own: the rows owed to this rank itself are left where they are (the
// single-launch combine reads them from x directly).
// ---------------------------------------------------------------------
struct CombineSendArgs {
    const uint8_t* x;
    const int64_t* layout_range;
    int hidden, num_local_experts, num_ranks, rank, max_tokens, parts_log2;
    uint8_t* combine_staging;
    uint8_t* combine_send_slots;
};

// No LDS and no barrier: each wave holds the segment counts and begins in registers.
template <int kPer, bool kStream>
__device__ __forceinline__ void combine_send_rows_impl(const CombineSendArgs& a, int block, int num_blocks,
                                                       bool skip_own) {
    const int lane = lane_id(), w = wave_in_block();
    const int waves = int(blockDim.x) >> 6;
    const int num_ranks = a.num_ranks, max_tokens = a.max_tokens;
    const int num_segments = a.num_local_experts * num_ranks;

    WaveSegments<kPer> seg_table;
    int64_t ranges[kPer];
    DEEPEP_PHASE(0);
    wave_load_int64<kPer>(a.layout_range, num_segments, lane, ranges);
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
        const int s = lane * kPer + u;
        int c = int(ranges[u] & 0xffffffffll);
        c = c < 0 ? 0 : (c > max_tokens ? max_tokens : c);
        if (skip_own && s % num_ranks == a.rank) c = 0;
        seg_table.cnt[u] = c;
        seg_table.aux[u] = int(ranges[u] >> 32);
    }
    wave_segments_finish(seg_table);
    DEEPEP_PHASE(1);

    const int64_t row_bytes = int64_t(a.hidden) * 2;
    const int num_vec = int(row_bytes / 16);
    const int64_t slots_per_expert = int64_t(max_tokens) * num_ranks;
    const int waves_total = num_blocks * waves;
    const int parts = 1 << a.parts_log2;
    const int num_items = seg_table.total << a.parts_log2;

    for (int item = block * waves + w; item < num_items; item += waves_total) {
        const int row = item >> a.parts_log2, part = item & (parts - 1);
        int seg_first, b;
        const int seg = wave_segments_find(seg_table, row, seg_first, b);
        const int j = row - seg_first;
        const int le = seg / num_ranks;
        const int s = seg - le * num_ranks;
        if (b < 0 || int64_t(b) + j >= slots_per_expert) continue;  // malformed range: never read past the expert
        const uint8_t* src = a.x + (int64_t(le) * slots_per_expert + b + j) * row_bytes;
        uint8_t* dst;
        if (s == a.rank)
            dst = a.combine_staging + ((int64_t(a.rank) * a.num_local_experts + le) * max_tokens + j) * row_bytes;
        else if (a.combine_send_slots != nullptr)
            dst = a.combine_send_slots + (int64_t(seg) * max_tokens + j) * row_bytes;
        else
            continue;
        int v_begin, v_end;
        row_part_range(num_vec, parts, part, v_begin, v_end);
        wave_copy_vec16<4, kStream>(src, dst, v_begin, v_end, lane);
    }
    DEEPEP_PHASE(2);
}

template <bool kStream>
__device__ __forceinline__ void combine_send_rows(const CombineSendArgs& a, int block, int num_blocks, bool skip_own) {
    if (a.num_local_experts * a.num_ranks <= 4 * kWave)
        combine_send_rows_impl<4, kStream>(a, block, num_blocks, skip_own);
    else
        combine_send_rows_impl<16, kStream>(a, block, num_blocks, skip_own);
}

// skip_own: the rows owed to this rank itself stay where they are (the reduce reads them from x).
__global__ __launch_bounds__(256) void ll_combine_send_kernel(CombineSendArgs a, bool skip_own) {
    combine_send_rows<false>(a, blockIdx.x, gridDim.x, skip_own);
}

// ---------------------------------------------------------------------
// Receive side: one wave = one (token, 1 KiB piece of the output row).
// All K source vectors are loaded before the FMA chain so K 16-byte loads
// are in flight per lane; accumulation order is k = 0..K-1, float32 FMA,
// one rounding to bf16 at the end
// (reference: csrc/kernels/coop_combine_recv.cuh:222-260).
// own_begin != null (single-launch combine): the answers of this rank's own
// experts are read from the expert-output tensor own_x at
// [e_l][own_begin[e_l] + slot] instead of the staging area.
// ---------------------------------------------------------------------
struct CombineRecvArgs {
    const uint8_t* combine_staging;
    const int64_t* topk_idx;
    const float* topk_weights;
    const int32_t* pair_slot;
    int num_tokens, hidden, num_topk, num_experts, max_tokens, pieces_per_row;
    int accumulate;  // non-zero: the sum starts from what `out` already holds
    uint8_t* out;
    // Flat form (rows returned through an all-to-all): combine_staging is one buffer with a row per row
    // sent, in send order; pair (t, k) is answered by row flat_prefix[expert] + slot, or, when the rows of
    // every answering rank start at a slot of flat_slot_rows rows, by row rank * flat_slot_rows + (that
    // minus the first row sent to the rank).  Null flat_prefix: the per-expert staging area.
    const int32_t* flat_prefix;  // [E + 1]
    int64_t flat_rows, flat_slot_rows;
    int experts_per_rank;
};

// What lane k of a wave knows about selection k of its token once the index loads are back.
struct CombineSelection {
    int slot;
    int64_t expert;
    float weight;
};

// Issues the loads of selection `lane`'s (slot, expert, weight): one round of loads for the whole token.
// Nothing here waits for them, so a caller can put other latency (the own-range lookup of the
// single-launch combine) behind the same round trip.
__device__ __forceinline__ CombineSelection combine_load_selection(const CombineRecvArgs& a, int64_t item) {
    CombineSelection s = {-1, -1, 0.0f};
    const int lane = lane_id();
    if (item < int64_t(a.num_tokens) * a.pieces_per_row && lane < a.num_topk) {
        const int64_t idx = (item / a.pieces_per_row) * a.num_topk + lane;
        s.slot = a.pair_slot[idx];
        s.expert = a.topk_idx[idx];
        s.weight = a.topk_weights[idx];
    }
    return s;
}

template <bool kStream>
__device__ __forceinline__ void combine_recv_piece(const CombineRecvArgs& a, int64_t item, const CombineSelection& sel,
                                                   const uint8_t* own_x, const int32_t* own_begin,
                                                   int own_first_expert, int num_local_experts,
                                                   int64_t slots_per_expert) {
    const int lane = lane_id();
    if (item >= int64_t(a.num_tokens) * a.pieces_per_row) return;
    const int t = int(item / a.pieces_per_row);
    const int piece = int(item - int64_t(t) * a.pieces_per_row);
    const int64_t row_bytes = int64_t(a.hidden) * 2;
    const int64_t off = int64_t(piece) * 1024 + lane * 16;
    const bool lane_live = off < row_bytes;
    const int num_topk = a.num_topk;

    DEEPEP_PHASE(0);
    // Lane k works out where selection k's row is; the loop below reads the results back lane by
    // lane, as wave-uniform values.
    uint64_t my_row = 0;
    const float my_weight = sel.weight;
    bool my_live = false;
    if (lane < num_topk) {
        const int slot = sel.slot;
        const int64_t e = sel.expert;
        if (a.flat_prefix != nullptr) {
            // csrc/kernels/efa_kernels.cu:1449-1466: the row's index in send order, flat or inside its rank's slot
            if (slot >= 0 && e >= 0 && e < a.num_experts) {
                const int first = a.flat_prefix[e], next = a.flat_prefix[e + 1];
                int64_t idx = int64_t(first) + slot;
                my_live = first >= 0 && slot < next - first;
                if (a.flat_slot_rows > 0) {
                    const int64_t r = e / a.experts_per_rank;
                    const int64_t within = idx - a.flat_prefix[r * a.experts_per_rank];
                    my_live = my_live && within >= 0 && within < a.flat_slot_rows;
                    idx = r * a.flat_slot_rows + within;
                }
                my_live = my_live && idx < a.flat_rows;
                my_row = reinterpret_cast<uint64_t>(a.combine_staging + idx * row_bytes);
            }
        } else if (slot >= 0 && slot < a.max_tokens && e >= 0 && e < a.num_experts) {
            const uint8_t* row = a.combine_staging + (e * a.max_tokens + slot) * row_bytes;
            my_live = true;
            const int64_t le = e - own_first_expert;
            if (own_begin != nullptr && le >= 0 && le < num_local_experts) {
                const int64_t pos = int64_t(own_begin[le]) + slot;
                my_live = own_begin[le] >= 0 && pos < slots_per_expert;
                row = own_x + (le * slots_per_expert + pos) * row_bytes;
            }
            my_row = reinterpret_cast<uint64_t>(row);
        }
    }
    const uint64_t live_mask = __ballot(my_live);

    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    if (a.accumulate != 0 && lane_live) {  // reference: csrc/kernels/coop_combine_recv.cuh:174-179
        const u32x4 prev = load_global_u32x4(a.out + int64_t(t) * row_bytes + off);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[2 * i] = bf16_lo(prev[i]), acc[2 * i + 1] = bf16_hi(prev[i]);
    }

    for (int k0 = 0; k0 < num_topk; k0 += 8) {
        u32x4 v[8];
        float wgt[8];
        bool live[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int k = k0 + u;
            live[u] = k < num_topk && ((live_mask >> k) & 1) != 0;
            wgt[u] = 0.0f;
            if (live[u]) {
                const uint32_t lo32 = __builtin_amdgcn_readlane(uint32_t(my_row), k);
                const uint32_t hi32 = __builtin_amdgcn_readlane(uint32_t(my_row >> 32), k);
                wgt[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_weight), k));
                const uint8_t* row = reinterpret_cast<const uint8_t*>((uint64_t(hi32) << 32) | lo32);
                if (lane_live) v[u] = load_u32x4<kStream>(row + off);
            }
        }
        DEEPEP_PHASE(1);
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
    DEEPEP_PHASE(2);
    if (lane_live) {
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = pack_bf16x2(acc[2 * i], acc[2 * i + 1]);
        store_u32x4<kStream>(a.out + int64_t(t) * row_bytes + off, o);
    }
    DEEPEP_PHASE(3);
}

// kStream: the gathered rows exceed what the caches hold, so they are read (and the result written)
// with the non-temporal hint.  own_x != null: the answers of this rank's own experts are read from
// the expert-output tensor directly (layout_range says where each own segment begins).
template <bool kStream>
__global__ __launch_bounds__(1024) void ll_combine_recv_kernel(CombineRecvArgs a, const uint8_t* own_x,
                                                               const int64_t* layout_range, int rank,
                                                               int num_local_experts, int num_ranks) {
    extern __shared__ int32_t own_begin[];  // [E_l], with own_x only
    const int64_t item = int64_t(blockIdx.x) * (blockDim.x >> 6) + wave_in_block();
    const CombineSelection sel = combine_load_selection(a, item);  // in flight while the own ranges are fetched
    if (own_x != nullptr) {
        for (int le = threadIdx.x; le < num_local_experts; le += blockDim.x) {
            const int64_t lr = layout_range[le * num_ranks + rank];
            own_begin[le] = (lr & 0xffffffffll) > 0 ? int(lr >> 32) : 0;
        }
        lds_barrier();
    }
    combine_recv_piece<kStream>(a, item, sel, own_x, own_x != nullptr ? own_begin : nullptr, rank * num_local_experts,
                                num_local_experts, int64_t(a.max_tokens) * num_ranks);
}

// ---------------------------------------------------------------------
// Single-launch combine for small batches (at most 8192 expected rows): the reduce workgroups
// and the row-return workgroups of the two kernels above in one grid.  No
// workgroup waits on another: the reduce reads the answers of this rank's own
// experts straight from x (layout_range says where each segment begins), so the
// row return only has to move the rows owed to other ranks.
// (The reference's combine is one kernel with a send and a receive phase as
// well: csrc/kernels/coop_combine_send.cuh:37, coop_combine_recv.cuh:72.)
// ---------------------------------------------------------------------
template <bool kStream>
__global__ __launch_bounds__(256) void ll_combine_fused_kernel(CombineSendArgs sa, CombineRecvArgs ra,
                                                               int num_recv_blocks) {
    extern __shared__ int32_t dyn_lds[];  // reduce workgroups: own_begin[E_l]
    const int block = blockIdx.x;
    if (block < num_recv_blocks) {
        // the token's index loads and the own-range loads go out together: one memory round trip
        // before the row loads instead of two
        const int64_t item = int64_t(block) * 4 + wave_in_block();
        const CombineSelection sel = combine_load_selection(ra, item);
        for (int le = threadIdx.x; le < sa.num_local_experts; le += blockDim.x) {
            const int64_t lr = sa.layout_range[le * sa.num_ranks + sa.rank];
            dyn_lds[le] = (lr & 0xffffffffll) > 0 ? int(lr >> 32) : 0;
        }
        lds_barrier();
        combine_recv_piece<kStream>(ra, item, sel, sa.x, dyn_lds, sa.rank * sa.num_local_experts,
                                    sa.num_local_experts, int64_t(sa.max_tokens) * sa.num_ranks);
    } else {
        combine_send_rows<kStream>(sa, block - num_recv_blocks, int(gridDim.x) - num_recv_blocks, true);
    }
}

// ---------------------------------------------------------------------
// Send side for an all-to-all shaped transport: the live expert-output rows in
// arrival order, which is contiguous per destination rank.  Record i of the
// exchange metadata names the row (padded_index[i] picks the record whose packed
// row is read, record_packed_row says where the receive side put it) and its place
// in the flat buffer (combine_send_offset[i]); reference:
// send_buffer[combine_send_offset[i]] = expert_x[padded_index[i]]
// (csrc/kernels/coop_combine_send.cuh:37-170; torch form deep_ep/buffer.py:2601-2608).
// With a table of peer buffers the row skips the send buffer and goes straight to
// its place in the destination's receive buffer, behind what that rank sent to the
// ranks below this one (combine_remote_recv_offset,
// csrc/transport/ll_pipeline.cpp:1283-1295; the reference's peer stores:
// coop_combine_send.cuh:205-246).  One workgroup per record, one 16-byte vector per thread.
// ---------------------------------------------------------------------
struct CombineByDestArgs {
    const uint8_t* x;
    const int32_t* record_packed_row;
    const uint32_t* source_rank;
    const uint32_t* padded_index;
    const uint32_t* combine_send_offset;
    const uint32_t* num_recv_tokens;
    int64_t row_capacity, x_rows;
    int num_ranks, num_vec;
    uint8_t* send_flat;
    // direct delivery
    uint8_t* const* peer_recv;  // [R] device pointers, or null
    const int64_t* peer_rows;   // [R] rows each peer buffer holds
    const int32_t* recv_counts;
    const int64_t* remote_offset;
};

template <bool kStream>
__global__ __launch_bounds__(1024) void ll_combine_send_by_dest_kernel(CombineByDestArgs a) {
    int64_t records = a.num_recv_tokens[1];
    if (records > a.row_capacity) records = a.row_capacity;
    const int lane = lane_id();
    const int64_t row_bytes = int64_t(a.num_vec) * 16;
    for (int64_t i = blockIdx.x; i < records; i += gridDim.x) {
        // padded_index[i] is i whenever the records come from deepep_ll_exchange_metadata, so the packed row
        // is fetched for that guess together with the record itself, and again only if the guess was wrong:
        // one round trip in front of the row loads instead of two
        const uint32_t p = a.padded_index[i];
        int64_t src_row = a.record_packed_row[i];
        const int64_t offset = a.combine_send_offset[i];
        if (int64_t(p) >= a.row_capacity) continue;
        if (int64_t(p) != i) src_row = a.record_packed_row[p];
        if (src_row < 0 || src_row >= a.x_rows) continue;  // the record has no row
        uint8_t* dst;
        if (a.peer_recv == nullptr) {
            if (offset >= a.row_capacity) continue;
            dst = a.send_flat + offset * row_bytes;
        } else {
            const uint32_t s = a.source_rank[i];
            if (s >= uint32_t(a.num_ranks)) continue;
            // the record's place among the rows of its source: offset minus the rows of the lower sources
            int part = 0;
            for (int r = lane; r < int(s); r += kWave) part += a.recv_counts[r] < 0 ? 0 : a.recv_counts[r];
            const int64_t j = offset - __builtin_amdgcn_readlane(wave_inclusive_sum(part), kWave - 1);
            const int64_t at = a.remote_offset[s] + j;
            if (j < 0 || j >= a.recv_counts[s] || at < 0 || at >= a.peer_rows[s]) continue;
            dst = a.peer_recv[s] + at * row_bytes;
        }
        const uint8_t* src = a.x + src_row * row_bytes;
        for (int v = threadIdx.x; v < a.num_vec; v += blockDim.x)
            store_u32x4<kStream>(dst + int64_t(v) * 16, load_u32x4<kStream>(src + int64_t(v) * 16));
    }
}

static CombineSendArgs make_combine_send_args(const void* x, const int64_t* layout_range, int hidden, int num_experts,
                                              int num_ranks, int rank, int max_tokens, void* combine_staging,
                                              void* combine_send_slots, int64_t expected_rows) {
    CombineSendArgs sa;
    sa.x = reinterpret_cast<const uint8_t*>(x);
    sa.layout_range = layout_range;
    sa.hidden = hidden, sa.num_local_experts = num_experts / num_ranks, sa.num_ranks = num_ranks, sa.rank = rank;
    sa.max_tokens = max_tokens;
    sa.parts_log2 = choose_row_parts_log2(estimated_rows(expected_rows, num_experts, max_tokens), int64_t(hidden) * 2);
    sa.combine_staging = reinterpret_cast<uint8_t*>(combine_staging);
    sa.combine_send_slots = reinterpret_cast<uint8_t*>(combine_send_slots);
    return sa;
}

static CombineRecvArgs make_combine_recv_args(const void* combine_staging, const int64_t* topk_idx,
                                              const float* topk_weights, const int32_t* pair_slot, int num_tokens,
                                              int hidden, int num_topk, int num_experts, int max_tokens, int accumulate,
                                              void* out) {
    CombineRecvArgs ra;
    ra.combine_staging = reinterpret_cast<const uint8_t*>(combine_staging);
    ra.topk_idx = topk_idx, ra.topk_weights = topk_weights, ra.pair_slot = pair_slot;
    ra.num_tokens = num_tokens, ra.hidden = hidden, ra.num_topk = num_topk, ra.num_experts = num_experts;
    ra.max_tokens = max_tokens, ra.pieces_per_row = (hidden * 2 + 1023) / 1024;
    ra.accumulate = accumulate;
    ra.out = reinterpret_cast<uint8_t*>(out);
    ra.flat_prefix = nullptr, ra.flat_rows = 0, ra.flat_slot_rows = 0, ra.experts_per_rank = 1;
    return ra;
}

static int check_combine_send_args(const void* x, const int64_t* layout_range, int hidden, int num_experts,
                                   int num_ranks, int rank, int max_tokens, const void* combine_staging,
                                   const void* combine_send_slots) {
    EP_HOST_ASSERT(hidden > 0 && hidden % 128 == 0);
    EP_HOST_ASSERT(num_ranks > 0 && num_experts > 0 && num_experts % num_ranks == 0);
    EP_HOST_ASSERT(rank >= 0 && rank < num_ranks);
    EP_HOST_ASSERT(max_tokens > 0);
    EP_HOST_ASSERT(num_experts <= 1024);
    EP_HOST_ASSERT(x != nullptr && layout_range != nullptr && combine_staging != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(layout_range) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(combine_staging) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(combine_send_slots) & 15) == 0);
    EP_HOST_ASSERT(int64_t(num_experts) * max_tokens < (int64_t(1) << 31));
    return 0;
}

static int check_combine_recv_args(const void* combine_staging, const int64_t* topk_idx, const float* topk_weights,
                                   const int32_t* pair_slot, int num_tokens, int hidden, int num_topk,
                                   int num_experts, int max_tokens, const void* out) {
    EP_HOST_ASSERT(num_tokens >= 0 && hidden > 0 && hidden % 128 == 0 && num_topk > 0);
    EP_HOST_ASSERT(num_experts > 0 && max_tokens > 0);
    if (num_tokens == 0) return 0;
    EP_HOST_ASSERT(combine_staging != nullptr && topk_idx != nullptr && topk_weights != nullptr &&
                   pair_slot != nullptr && out != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(combine_staging) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(out) & 15) == 0);
    EP_HOST_ASSERT((int64_t(num_tokens) * ((hidden * 2 + 1023) / 1024) + 3) / 4 < (int64_t(1) << 31));
    return 0;
}

}  // namespace deepep

using namespace deepep;

extern "C" {

// skip_own: the rows owed to this rank itself are not moved (the reduce will read them from x).
static int launch_combine_send(const void* x, const int64_t* layout_range, int hidden, int num_experts, int num_ranks,
                               int rank, int num_max_dispatch_tokens_per_rank, void* combine_staging,
                               void* combine_send_slots, int64_t expected_rows, void* workspace,
                               size_t workspace_bytes, bool skip_own, void* stream) {
    if (int rc = check_combine_send_args(x, layout_range, hidden, num_experts, num_ranks, rank,
                                         num_max_dispatch_tokens_per_rank, combine_staging, combine_send_slots))
        return rc;
    const int num_local_experts = num_experts / num_ranks;
    const int64_t max_rows = int64_t(num_experts) * num_max_dispatch_tokens_per_rank;
    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
    const bool large = estimated_rows(expected_rows, num_experts, num_max_dispatch_tokens_per_rank) > kLargeBatchRows;
    if (large && workspace != nullptr) {
        EP_HOST_ASSERT(workspace_bytes >= size_t(segment_workspace_bytes(num_experts, num_max_dispatch_tokens_per_rank)));
        EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(workspace) & 15) == 0);
        int32_t* flat = reinterpret_cast<int32_t*>(workspace);
        RowDesc* desc = reinterpret_cast<RowDesc*>(reinterpret_cast<uint8_t*>(workspace) +
                                                   (((int64_t(num_experts) + 1) * 4 + 255) & ~int64_t(255)));
        ll_segment_index_kernel<<<num_experts, kIndexThreads, 0, hs>>>(
            skip_own ? 2 : 1, nullptr, layout_range, num_local_experts, num_ranks, rank,
            num_max_dispatch_tokens_per_rank, nullptr,
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
    const CombineSendArgs sa = make_combine_send_args(x, layout_range, hidden, num_experts, num_ranks, rank,
                                                      num_max_dispatch_tokens_per_rank, combine_staging,
                                                      combine_send_slots, expected_rows);
    int64_t blocks = ((max_rows << sa.parts_log2) + 3) / 4;
    const int64_t cap = large ? 4096 : 1024;
    if (blocks > cap) blocks = cap;
    ll_combine_send_kernel<<<dim3(unsigned(blocks)), 256, 0, hs>>>(sa, skip_own);
    EP_LAUNCH_CHECK();
    return 0;
}

int deepep_ll_combine_send(const void* x, const int64_t* layout_range, int hidden, int num_experts, int num_ranks,
                           int rank, int num_max_dispatch_tokens_per_rank, void* combine_staging,
                           void* combine_send_slots, int64_t expected_rows, void* workspace, size_t workspace_bytes,
                           void* stream) {
    clear_error();
    return launch_combine_send(x, layout_range, hidden, num_experts, num_ranks, rank,
                               num_max_dispatch_tokens_per_rank, combine_staging, combine_send_slots, expected_rows,
                               workspace, workspace_bytes, false, stream);
}

// own_x != null: the answers of this rank's own experts are read from own_x at the positions
// layout_range gives, instead of from combine_staging.
static int launch_combine_recv(const void* combine_staging, const int64_t* topk_idx, const float* topk_weights,
                               const int32_t* pair_slot, int num_tokens, int hidden, int num_topk, int num_experts,
                               int num_max_dispatch_tokens_per_rank, int accumulate, void* out, const void* own_x,
                               const int64_t* layout_range, int rank, int num_ranks, void* stream) {
    if (int rc = check_combine_recv_args(combine_staging, topk_idx, topk_weights, pair_slot, num_tokens, hidden,
                                         num_topk, num_experts, num_max_dispatch_tokens_per_rank, out))
        return rc;
    if (num_tokens == 0) return 0;
    const CombineRecvArgs ra = make_combine_recv_args(combine_staging, topk_idx, topk_weights, pair_slot, num_tokens,
                                                      hidden, num_topk, num_experts,
                                                      num_max_dispatch_tokens_per_rank, accumulate, out);
    const int waves = 4;  // block shape makes no measurable difference (1..16 waves: within 5 %)
    const int64_t blocks = (int64_t(num_tokens) * ra.pieces_per_row + waves - 1) / waves;
    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
    const int num_local_experts = own_x != nullptr ? num_experts / num_ranks : 0;
    const size_t lds = size_t(num_local_experts) * sizeof(int32_t);
    const uint8_t* own = reinterpret_cast<const uint8_t*>(own_x);
    if (int64_t(num_tokens) * num_topk * hidden * 2 > stream_bytes())
        ll_combine_recv_kernel<true><<<dim3(unsigned(blocks)), waves * kWave, lds, hs>>>(ra, own, layout_range, rank,
                                                                                        num_local_experts, num_ranks);
    else
        ll_combine_recv_kernel<false><<<dim3(unsigned(blocks)), waves * kWave, lds, hs>>>(ra, own, layout_range, rank,
                                                                                         num_local_experts, num_ranks);
    EP_LAUNCH_CHECK();
    return 0;
}

int deepep_ll_combine_recv(const void* combine_staging, const int64_t* topk_idx, const float* topk_weights,
                           const int32_t* pair_slot, int num_tokens, int hidden, int num_topk, int num_experts,
                           int num_max_dispatch_tokens_per_rank, int accumulate, void* out, void* stream) {
    clear_error();
    return launch_combine_recv(combine_staging, topk_idx, topk_weights, pair_slot, num_tokens, hidden, num_topk,
                               num_experts, num_max_dispatch_tokens_per_rank, accumulate, out, nullptr, nullptr, 0, 1,
                               stream);
}

int deepep_ll_combine_send_by_dest(const void* x, const int32_t* record_packed_row, const uint32_t* source_rank,
                                   const uint32_t* padded_index, const uint32_t* combine_send_offset,
                                   const uint32_t* num_recv_tokens, int64_t row_capacity, int hidden, int num_experts,
                                   int num_ranks, int num_max_dispatch_tokens_per_rank, void* send_flat,
                                   const int32_t* recv_counts, const int64_t* combine_remote_recv_offset,
                                   void* const* peer_recv_flat, const int64_t* peer_recv_rows,
                                   int64_t expected_rows, void* stream) {
    clear_error();
    EP_HOST_ASSERT(hidden > 0 && hidden % 128 == 0);
    EP_HOST_ASSERT(num_ranks > 0 && num_experts > 0 && num_experts % num_ranks == 0);
    EP_HOST_ASSERT(num_max_dispatch_tokens_per_rank > 0);
    EP_HOST_ASSERT(row_capacity >= 0 && row_capacity < (int64_t(1) << 31));
    if (row_capacity == 0) return 0;
    EP_HOST_ASSERT(x != nullptr && record_packed_row != nullptr && padded_index != nullptr &&
                   combine_send_offset != nullptr && num_recv_tokens != nullptr);
    const bool direct = peer_recv_flat != nullptr;
    EP_HOST_ASSERT(direct || send_flat != nullptr);
    EP_HOST_ASSERT(!direct || (source_rank != nullptr && recv_counts != nullptr &&
                               combine_remote_recv_offset != nullptr && peer_recv_rows != nullptr));
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(send_flat) & 15) == 0);
    CombineByDestArgs a;
    a.x = reinterpret_cast<const uint8_t*>(x);
    a.record_packed_row = record_packed_row, a.source_rank = source_rank, a.padded_index = padded_index;
    a.combine_send_offset = combine_send_offset, a.num_recv_tokens = num_recv_tokens;
    a.row_capacity = row_capacity;
    a.x_rows = int64_t(num_experts) * num_max_dispatch_tokens_per_rank;  // E_l * R * M rows of expert outputs
    a.num_ranks = num_ranks, a.num_vec = hidden * 2 / 16;
    a.send_flat = reinterpret_cast<uint8_t*>(send_flat);
    a.peer_recv = reinterpret_cast<uint8_t* const*>(peer_recv_flat), a.peer_rows = peer_recv_rows;
    a.recv_counts = recv_counts, a.remote_offset = combine_remote_recv_offset;
    int threads = ((a.num_vec + 63) / 64) * 64;
    if (threads > 1024) threads = 1024;
    // grid from the rows expected, not from the capacity (an idle workgroup is not free)
    const int64_t rows = expected_rows > 0 && expected_rows < row_capacity ? expected_rows : row_capacity;
    const unsigned blocks = flat_grid_blocks(rows, row_capacity, num_max_dispatch_tokens_per_rank);
    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
    if (2 * rows * hidden * 2 > stream_bytes())
        ll_combine_send_by_dest_kernel<true><<<blocks, threads, 0, hs>>>(a);
    else
        ll_combine_send_by_dest_kernel<false><<<blocks, threads, 0, hs>>>(a);
    EP_LAUNCH_CHECK();
    return 0;
}

int deepep_ll_combine_recv_flat(const void* recv_flat, int64_t recv_flat_rows, int64_t slot_rows,
                                const int32_t* send_expert_prefix, const int64_t* topk_idx,
                                const float* topk_weights, const int32_t* pair_slot, int num_tokens, int hidden,
                                int num_topk, int num_experts, int num_ranks, int num_max_dispatch_tokens_per_rank,
                                int accumulate, void* out, void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_ranks > 0 && num_experts > 0 && num_experts % num_ranks == 0);
    EP_HOST_ASSERT(recv_flat_rows >= 0 && slot_rows >= 0);
    EP_HOST_ASSERT(slot_rows == 0 || slot_rows * num_ranks <= recv_flat_rows);
    if (int rc = check_combine_recv_args(recv_flat, topk_idx, topk_weights, pair_slot, num_tokens, hidden, num_topk,
                                         num_experts, num_max_dispatch_tokens_per_rank, out))
        return rc;
    if (num_tokens == 0) return 0;
    EP_HOST_ASSERT(send_expert_prefix != nullptr);
    CombineRecvArgs ra = make_combine_recv_args(recv_flat, topk_idx, topk_weights, pair_slot, num_tokens, hidden,
                                                num_topk, num_experts, num_max_dispatch_tokens_per_rank, accumulate,
                                                out);
    ra.flat_prefix = send_expert_prefix, ra.flat_rows = recv_flat_rows, ra.flat_slot_rows = slot_rows;
    ra.experts_per_rank = num_experts / num_ranks;
    const int waves = 4;
    const int64_t blocks = (int64_t(num_tokens) * ra.pieces_per_row + waves - 1) / waves;
    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
    if (int64_t(num_tokens) * num_topk * hidden * 2 > stream_bytes())
        ll_combine_recv_kernel<true><<<dim3(unsigned(blocks)), waves * kWave, 0, hs>>>(ra, nullptr, nullptr, 0, 0, 1);
    else
        ll_combine_recv_kernel<false><<<dim3(unsigned(blocks)), waves * kWave, 0, hs>>>(ra, nullptr, nullptr, 0, 0, 1);
    EP_LAUNCH_CHECK();
    return 0;
}

int deepep_ll_combine(const void* x, const int64_t* layout_range, const int64_t* topk_idx, const float* topk_weights,
                      const int32_t* pair_slot, int num_tokens, int hidden, int num_topk, int num_experts,
                      int num_ranks, int rank, int num_max_dispatch_tokens_per_rank, int accumulate,
                      void* combine_staging, void* combine_send_slots, void* out, int64_t expected_rows,
                      void* workspace, size_t workspace_bytes, void* stream) {
    clear_error();
    const int64_t max_rows = int64_t(num_experts) * num_max_dispatch_tokens_per_rank;
    // measured as whole calls the single launch wins up to this bound (512 tokens: 36 us against 40 for
    // the phases back to back), although each phase timed alone on cache-warm data suggests otherwise
    if (estimated_rows(expected_rows, num_experts, num_max_dispatch_tokens_per_rank) > kLargeBatchRows) {
        // the two phases back to back, with the single launch's shortcut: the rows owed to this rank
        // itself are not moved, the reduce reads them from x.  Without send slots (zero copy: the transport
        // sends layout_range's ranges straight from x) there is nothing to return.
        if (combine_send_slots == nullptr) {
            if (int rc = check_combine_send_args(x, layout_range, hidden, num_experts, num_ranks, rank,
                                                 num_max_dispatch_tokens_per_rank, combine_staging, nullptr))
                return rc;
        } else if (int rc = launch_combine_send(x, layout_range, hidden, num_experts, num_ranks, rank,
                                                num_max_dispatch_tokens_per_rank, combine_staging,
                                                combine_send_slots, expected_rows, workspace, workspace_bytes, true,
                                                stream)) {
            return rc;
        }
        return launch_combine_recv(combine_staging, topk_idx, topk_weights, pair_slot, num_tokens, hidden, num_topk,
                                   num_experts, num_max_dispatch_tokens_per_rank, accumulate, out, x, layout_range,
                                   rank, num_ranks, stream);
    }
    if (int rc = check_combine_send_args(x, layout_range, hidden, num_experts, num_ranks, rank,
                                         num_max_dispatch_tokens_per_rank, combine_staging, combine_send_slots))
        return rc;
    if (int rc = check_combine_recv_args(combine_staging, topk_idx, topk_weights, pair_slot, num_tokens, hidden,
                                         num_topk, num_experts, num_max_dispatch_tokens_per_rank, out))
        return rc;
    const CombineSendArgs sa = make_combine_send_args(x, layout_range, hidden, num_experts, num_ranks, rank,
                                                      num_max_dispatch_tokens_per_rank, combine_staging,
                                                      combine_send_slots, expected_rows);
    const CombineRecvArgs ra = make_combine_recv_args(combine_staging, topk_idx, topk_weights, pair_slot, num_tokens,
                                                      hidden, num_topk, num_experts,
                                                      num_max_dispatch_tokens_per_rank, accumulate, out);
    const int64_t recv_blocks = (int64_t(num_tokens) * ra.pieces_per_row + 3) / 4;
    int64_t rows = expected_rows > 0 ? expected_rows : int64_t(num_max_dispatch_tokens_per_rank) * num_topk;
    rows += rows / 8 + 16;
    if (rows > max_rows) rows = max_rows;
    int64_t send_blocks = combine_send_slots != nullptr ? ((rows << sa.parts_log2) + 3) / 4 : 0;
    if (send_blocks > 1024) send_blocks = 1024;
    if (recv_blocks + send_blocks == 0) return 0;
    const size_t lds = size_t(sa.num_local_experts) * sizeof(int32_t);
    // rows returned (read + written) plus rows gathered: past what the caches hold, stream
    const int64_t traffic = (2 * rows + int64_t(num_tokens) * num_topk) * hidden * 2;
    if (traffic > stream_bytes())
        ll_combine_fused_kernel<true><<<dim3(unsigned(recv_blocks + send_blocks)), 256, lds,
                                        reinterpret_cast<hipStream_t>(stream)>>>(sa, ra, int(recv_blocks));
    else
        ll_combine_fused_kernel<false><<<dim3(unsigned(recv_blocks + send_blocks)), 256, lds,
                                         reinterpret_cast<hipStream_t>(stream)>>>(sa, ra, int(recv_blocks));
    EP_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
