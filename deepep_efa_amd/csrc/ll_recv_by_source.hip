// Receive side of the low-latency dispatch for a transport that delivers rows grouped by source
// rank, the way an all-to-all does: the rows of source s sit in slot s of one buffer in the order
// they arrived, and the records of deepep_ll_exchange_metadata say where each expected row is
// (source_offset).  Every row carries its local expert in the last word of its tail, as the
// reference's packed rows carry [token, local_eid] (csrc/kernels/efa_kernels.cu:797-800).
//
// Same outputs as deepep_ll_dispatch_recv.  Reference: ll_recv_unpack_v2
// (csrc/kernels/efa_kernels.cu:2121-2231): count the (expert, source) pairs from the rows' metadata
// (:877-923, slot addressing :906-913), build the ranges as a prefix over ascending source rank
// (:991-1010), scatter every row to range begin + its rank inside the pair (:1227-1389).  The
// reference claims that rank with an atomic; here it is the row's arrival order inside its source,
// so the result does not depend on scheduling.
//
// Work is cut into chunks of 512 records that never straddle two sources (the records come grouped
// by source, ascending).  Large batches, three launches: per-chunk expert histograms (one workgroup
// per chunk); ranges + one {source row, packed row} descriptor per record (one workgroup per chunk:
// it adds up the histograms into the (expert, source) counts, scans them into the ranges, and ranks
// its own 512 rows on top of the histograms of its source's earlier chunks); and the flat row copy
// the other large-batch paths use.  Small batches, two launches: no histograms, one workgroup per
// source counts every record's expert itself and walks its source's chunks in order.
#include <algorithm>

#include "common.hpp"
#include "segments.hpp"
#include "../../include/deepep_hip.h"

namespace deepep {

constexpr int kBySourceThreads = 512;
constexpr int kBySourceWaves = kBySourceThreads / kWave;
constexpr int kBySourceMaxRanks = 1024;
constexpr int kBySourceMaxLocalExperts = 1024;

// Exclusive prefix of recv_counts (negative counts read as 0) over the ranks, by the whole workgroup:
// records [prefix[s], prefix[s + 1]) belong to source s.  prefix has num_ranks + 1 entries.
__device__ __forceinline__ void source_prefix(const int32_t* __restrict__ recv_counts, int num_ranks, int32_t* prefix,
                                              int32_t* scan_tmp) {
    for (int r = threadIdx.x; r < num_ranks; r += blockDim.x) {
        const int c = recv_counts[r];
        prefix[r] = c < 0 ? 0 : c;
    }
    lds_barrier();
    block_exclusive_scan(prefix, num_ranks, scan_tmp);
}

// The records of source s that are looked at: [begin, end) exist, those from `live_end` on lie past the
// source's slot of slot_rows rows (or past the records written) and are not copied.
__device__ __forceinline__ void source_records(const int32_t* prefix, int s, int num_ranks, int slot_rows,
                                               int64_t records, int64_t& begin, int64_t& end, int64_t& live_end) {
    begin = prefix[s];
    end = prefix[s + 1];
    if (end > records) end = records;
    if (begin > end) begin = end;
    live_end = begin + slot_rows < end ? begin + slot_rows : end;
}

// Local expert of the row a record points at, or -1 when the record or the row's tail is out of range.
__device__ __forceinline__ int record_expert(const uint8_t* __restrict__ recv_by_source, int64_t stride,
                                             int64_t tail_off, uint32_t offset, int64_t buffer_rows,
                                             int num_local_experts) {
    if (int64_t(offset) >= buffer_rows) return -1;
    const int e = *reinterpret_cast<const int32_t*>(recv_by_source + int64_t(offset) * stride + tail_off + 12);
    return e >= 0 && e < num_local_experts ? e : -1;
}

constexpr int kBySourceSmallRecords = 4096;  // up to here (record capacity) the two-launch form

// Exclusive prefix over the sources of their chunk counts, ceil(records of the source / 512); chunk g
// of the launch belongs to the source s with chunk_prefix[s] <= g < chunk_prefix[s + 1].
__device__ __forceinline__ void source_chunk_prefix(const int32_t* prefix, int num_ranks, int64_t records,
                                                    int32_t* chunk_prefix, int32_t* scan_tmp) {
    for (int r = threadIdx.x; r < num_ranks; r += blockDim.x) {
        int64_t begin = prefix[r], end = prefix[r + 1];
        if (end > records) end = records;
        if (begin > end) begin = end;
        chunk_prefix[r] = int32_t((end - begin + kBySourceThreads - 1) / kBySourceThreads);
    }
    lds_barrier();
    block_exclusive_scan(chunk_prefix, num_ranks, scan_tmp);
}

// Largest s with table[s] <= v, for an ascending table of n + 1 entries with table[0] <= v < table[n].
__device__ __forceinline__ int upper_source(const int32_t* table, int n, int64_t v) {
    int lo = 0, hi = n;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (table[mid] <= v) lo = mid;
        else hi = mid;
    }
    return lo;
}

// Sum of hist[c * E_l + e] over the chunks [c_begin, c_end), eight loads in flight at a time.
__device__ __forceinline__ int sum_chunk_counts(const int32_t* __restrict__ hist, int num_local_experts, int e,
                                                int c_begin, int c_end) {
    int sum = 0;
    for (int c0 = c_begin; c0 < c_end; c0 += 8) {
        int v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = c0 + u < c_end ? hist[int64_t(c0 + u) * num_local_experts + e] : 0;
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += v[u];
    }
    return sum;
}

// Large batches, first launch: hist[g * E_l + e] = records of chunk g, inside their source's slot,
// whose row names local expert e.
__global__ __launch_bounds__(kBySourceThreads) void ll_by_source_count_kernel(
    const uint8_t* __restrict__ recv_by_source, int64_t stride, int64_t tail_off, int64_t buffer_rows, int slot_rows,
    const int32_t* __restrict__ recv_counts, const uint32_t* __restrict__ source_offset,
    const uint32_t* __restrict__ num_recv_tokens, int64_t row_capacity, int num_local_experts, int num_ranks,
    int32_t* __restrict__ hist) {
    extern __shared__ int32_t lds[];  // prefix [R + 1] | chunk_prefix [R + 1] | counts [E_l]
    __shared__ int32_t scan_tmp[kMaxBlockWaves];
    int32_t* prefix = lds;
    int32_t* chunk_prefix = prefix + num_ranks + 1;
    int32_t* counts = chunk_prefix + num_ranks + 1;
    const int g = blockIdx.x, tid = threadIdx.x;
    source_prefix(recv_counts, num_ranks, prefix, scan_tmp);
    int64_t records = num_recv_tokens[1];
    if (records > row_capacity) records = row_capacity;
    source_chunk_prefix(prefix, num_ranks, records, chunk_prefix, scan_tmp);
    if (g >= chunk_prefix[num_ranks]) return;
    for (int e = tid; e < num_local_experts; e += kBySourceThreads) counts[e] = 0;
    lds_barrier();
    const int s = upper_source(chunk_prefix, num_ranks, g);
    int64_t begin, end, live_end;
    source_records(prefix, s, num_ranks, slot_rows, records, begin, end, live_end);
    const int64_t i = begin + int64_t(g - chunk_prefix[s]) * kBySourceThreads + tid;
    if (i < live_end) {
        const int e = record_expert(recv_by_source, stride, tail_off, source_offset[i], buffer_rows, num_local_experts);
        if (e >= 0) atomicAdd(&counts[e], 1);
    }
    lds_barrier();
    for (int e = tid; e < num_local_experts; e += kBySourceThreads) hist[int64_t(g) * num_local_experts + e] = counts[e];
}

// Ranges from the (expert, source) counts (every workgroup builds them, the first one writes them),
// then for this workgroup's records, in arrival order: packed row = range begin + rows of the same
// pair before it.  kChunked: the workgroup is chunk blockIdx.x and the counts come from the chunk
// histograms; otherwise it is source blockIdx.x, counts the experts of all records itself and walks
// the source's chunks one after the other.
template <bool kChunked>
__global__ __launch_bounds__(kBySourceThreads) void ll_by_source_index_kernel(
    const uint8_t* __restrict__ recv_by_source, int64_t stride, int64_t tail_off, int64_t buffer_rows, int slot_rows,
    const int32_t* __restrict__ recv_counts, const uint32_t* __restrict__ source_offset,
    const uint32_t* __restrict__ num_recv_tokens, int64_t row_capacity, int num_local_experts, int num_ranks,
    int max_tokens, const int32_t* __restrict__ hist, int64_t* __restrict__ layout_range,
    int32_t* __restrict__ packed_count, int32_t* __restrict__ stats, uint32_t* __restrict__ tokens_per_expert,
    int32_t* __restrict__ record_packed_row, int32_t* __restrict__ flat_total, RowDesc* __restrict__ desc) {
    // prefix [R + 1] | chunk_prefix [R + 1] | pair_prefix [E_l * R + 1] | running [E_l] | wave_cnt [waves][E_l]
    extern __shared__ int32_t lds[];
    __shared__ int32_t scan_tmp[kMaxBlockWaves];
    const int num_segments = num_local_experts * num_ranks;
    int32_t* prefix = lds;
    int32_t* chunk_prefix = prefix + num_ranks + 1;
    int32_t* pair_prefix = chunk_prefix + num_ranks + 1;
    int32_t* running = pair_prefix + num_segments + 1;
    int32_t* wave_cnt = running + num_local_experts;
    const int tid = threadIdx.x, lane = lane_id(), w = wave_in_block();
    const int64_t slots_per_expert = int64_t(max_tokens) * num_ranks;

    source_prefix(recv_counts, num_ranks, prefix, scan_tmp);
    int64_t records = num_recv_tokens[1];
    if (records > row_capacity) records = row_capacity;
    int s, first_chunk = 0, num_chunks;
    if constexpr (kChunked) {
        source_chunk_prefix(prefix, num_ranks, records, chunk_prefix, scan_tmp);
        const int g = blockIdx.x;
        if (g >= chunk_prefix[num_ranks] && g != 0) return;  // workgroup 0 writes the ranges even of an empty world
        // (expert, source) counts: the column sums of the source's chunk histograms
        for (int q = tid; q < num_segments; q += kBySourceThreads) {
            const int e = q / num_ranks, src = q - e * num_ranks;
            pair_prefix[q] = sum_chunk_counts(hist, num_local_experts, e, chunk_prefix[src], chunk_prefix[src + 1]);
        }
        const bool has_rows = g < chunk_prefix[num_ranks];
        s = has_rows ? upper_source(chunk_prefix, num_ranks, g) : 0;
        first_chunk = has_rows ? g - chunk_prefix[s] : 0;
        num_chunks = has_rows ? 1 : 0;
        // rows of the same (expert, source) pair in the source's earlier chunks
        for (int e = tid; e < num_local_experts; e += kBySourceThreads)
            running[e] = sum_chunk_counts(hist, num_local_experts, e, chunk_prefix[s], chunk_prefix[s] + first_chunk);
    } else {
        s = blockIdx.x;
        for (int q = tid; q < num_segments; q += kBySourceThreads) pair_prefix[q] = 0;
        for (int e = tid; e < num_local_experts; e += kBySourceThreads) running[e] = 0;
        lds_barrier();
        const int64_t expected = records < prefix[num_ranks] ? records : prefix[num_ranks];
        for (int64_t i = tid; i < expected; i += kBySourceThreads) {
            const int src = upper_source(prefix, num_ranks, i);
            if (i - prefix[src] >= slot_rows) continue;  // past the source's slot
            const int e = record_expert(recv_by_source, stride, tail_off, source_offset[i], buffer_rows, num_local_experts);
            if (e >= 0) atomicAdd(&pair_prefix[e * num_ranks + src], 1);
        }
        num_chunks = 1 << 30;  // until the source's records end
    }
    lds_barrier();
    // a pair holds at most max_tokens rows, like a segment of the staged form (whose counts the staged
    // receive clamps the same way): rows past that are dropped below, so that an expert's ranges never
    // exceed its num_ranks * max_tokens packed slots whatever the slots and tails hold
    for (int q = tid; q < num_segments; q += kBySourceThreads)
        if (pair_prefix[q] > max_tokens) pair_prefix[q] = max_tokens;
    lds_barrier();
    block_exclusive_scan(pair_prefix, num_segments, scan_tmp);
    if (blockIdx.x == 0) {
        // csrc/kernels/efa_kernels.cu:991-1010: begin = rows of the lower source ranks, 0 where the count is 0
        for (int q = tid; q < num_segments; q += kBySourceThreads) {
            const int le = q / num_ranks;
            const int64_t cnt = pair_prefix[q + 1] - pair_prefix[q];
            const int64_t begin = pair_prefix[q] - pair_prefix[le * num_ranks];
            layout_range[q] = cnt > 0 ? ((begin << 32) | cnt) : 0;
        }
        for (int le = tid; le < num_local_experts; le += kBySourceThreads) {
            const int c = pair_prefix[(le + 1) * num_ranks] - pair_prefix[le * num_ranks];
            packed_count[le] = c;
            if (stats != nullptr) stats[le] += c;
            if (tokens_per_expert != nullptr) tokens_per_expert[le] = uint32_t(c);
        }
        if (tid == 0) flat_total[0] = pair_prefix[num_segments];  // one descriptor per row that names an expert
    }

    int64_t begin, end, live_end;
    source_records(prefix, s, num_ranks, slot_rows, records, begin, end, live_end);
    int expert_bits = 0;
    while ((1 << expert_bits) < num_local_experts) ++expert_bits;
    int64_t base = begin + int64_t(first_chunk) * kBySourceThreads;
    for (int chunk = 0; chunk < num_chunks && base < end; ++chunk, base += kBySourceThreads) {  // in arrival order
        for (int q = tid; q < kBySourceWaves * num_local_experts; q += kBySourceThreads) wave_cnt[q] = 0;
        lds_barrier();
        const int64_t i = base + tid;
        uint32_t offset = 0;
        int e = -1;
        if (i < live_end) {
            offset = source_offset[i];
            e = record_expert(recv_by_source, stride, tail_off, offset, buffer_rows, num_local_experts);
        }
        // the lanes of this wave whose row names the same expert: one ballot per bit of the expert id
        uint64_t same = __ballot(e >= 0);
        for (int bit = 0; bit < expert_bits; ++bit) {
            const uint64_t set = __ballot(e >= 0 && ((e >> bit) & 1) != 0);
            same &= ((e >> bit) & 1) != 0 ? set : ~set;
        }
        const int before_in_wave = __popcll(same & lanes_below(lane));
        if (e >= 0 && (same >> lane) >> 1 == 0) wave_cnt[w * num_local_experts + e] = __popcll(same);  // the group's last lane
        lds_barrier();
        int32_t packed_row = -1;  // where this record's row lands; -1: nowhere
        if (e >= 0) {
            // The descriptors are laid out in the order of the packed rows (expert, source, arrival), not of
            // the records: the copy then writes consecutive rows from consecutive workgroups.
            int pos = running[e] + before_in_wave;
            for (int w2 = 0; w2 < w; ++w2) pos += wave_cnt[w2 * num_local_experts + e];
            const int64_t pair_begin = pair_prefix[e * num_ranks + s] - pair_prefix[e * num_ranks];
            if (pos < max_tokens) {  // a row past its pair's max_tokens rows has no place and no descriptor
                RowDesc d;
                d.src_row = int32_t(offset);
                d.dst_row = int32_t(int64_t(e) * slots_per_expert + pair_begin + pos);
                desc[pair_prefix[e * num_ranks + s] + pos] = d;
                packed_row = d.dst_row;
            }
        }
        // what the combine needs to return the rows in arrival order: the reference's recv_expert_ids /
        // recv_expert_pos (csrc/kernels/efa_kernels.cu:2121-2231), as one row index per record
        if (record_packed_row != nullptr && i < end) record_packed_row[i] = packed_row;
        if constexpr (kChunked) break;  // one chunk per workgroup
        lds_barrier();
        for (int e2 = tid; e2 < num_local_experts; e2 += kBySourceThreads) {
            int add = 0;
            for (int w2 = 0; w2 < kBySourceWaves; ++w2) add += wave_cnt[w2 * num_local_experts + e2];
            running[e2] += add;
        }
        lds_barrier();
    }
}

// ---------------------------------------------------------------------
// The same receive when every source's message is known to come ordered by local expert, the rows of
// an expert in the sender's slot order -- what deepep_ll_dispatch_send_by_dest emits -- and the
// gathered route counts are at hand.  Then nothing has to be read from the rows to place them: row j
// of source s belongs to the expert e whose run [first(e, s), first(e, s) + cnt(e, s)) holds j, with
// first(e, s) the count of the lower experts in that source's column of the counts, and it lands at
// begin(e, s) + (j - first(e, s)), begin being the prefix over the lower sources
// (csrc/kernels/efa_kernels.cu:991-1010).  One launch of arithmetic (a workgroup per (expert, source)
// pair, like ll_segment_index_kernel) in front of the flat row copy; both sides of every pair are
// contiguous runs of rows.  Rows of a message past the source's slot are lost: a pair keeps
// min(cnt, slot_rows - first) rows.
// ---------------------------------------------------------------------
__global__ __launch_bounds__(kIndexThreads) void ll_by_source_ordered_index_kernel(
    const int32_t* __restrict__ all_num_routed, int num_experts, int num_local_experts, int num_ranks, int rank,
    int max_tokens, int slot_rows, int64_t row_capacity, int64_t* __restrict__ layout_range,
    int32_t* __restrict__ packed_count, int32_t* __restrict__ stats, uint32_t* __restrict__ tokens_per_expert,
    int32_t* __restrict__ record_packed_row, int32_t* __restrict__ flat_total, RowDesc* __restrict__ desc) {
    __shared__ int32_t sent[kIndexThreads];       // cnt(e, s) as the sender counted it (clamped to max_tokens)
    __shared__ int32_t place[kIndexThreads + 1];  // prefix over the rows kept, pairs in (expert, source) order
    __shared__ int32_t source_total[kIndexThreads];
    __shared__ int32_t wave_totals[kIndexThreads / kWave];
    const int tid = threadIdx.x;
    const int num_segments = num_local_experts * num_ranks;
    const int le_of = tid / num_ranks, s_of = tid - le_of * num_ranks;
    int c = 0;
    if (tid < num_segments) {
        c = all_num_routed[int64_t(s_of) * num_experts + rank * num_local_experts + le_of];
        c = c < 0 ? 0 : (c > max_tokens ? max_tokens : c);
    }
    sent[tid] = c;
    __syncthreads();
    // first(e, s): this source's rows for the lower experts; the source's whole message
    int first = 0, kept = 0;
    if (tid < num_segments) {
        for (int e2 = 0; e2 < le_of; ++e2) first += sent[e2 * num_ranks + s_of];
        const int room = slot_rows - first;
        kept = room <= 0 ? 0 : (c < room ? c : room);
    }
    if (tid < num_ranks) {
        int total = 0;
        for (int e2 = 0; e2 < num_local_experts; ++e2) total += sent[e2 * num_ranks + tid];
        source_total[tid] = total;
    }
    int total;
    const int prefix = block_exclusive_scan_1024(kept, wave_totals, total);
    if (tid < num_segments) place[tid] = prefix;
    if (tid == 0) place[num_segments] = total;
    __syncthreads();
    const int64_t slots_per_expert = int64_t(max_tokens) * num_ranks;
    if (blockIdx.x == 0) {
        if (tid < num_segments) {
            const int64_t begin = place[tid] - place[le_of * num_ranks];
            layout_range[tid] = kept > 0 ? ((begin << 32) | int64_t(kept)) : 0;
        }
        if (tid < num_local_experts) {
            const int n = place[(tid + 1) * num_ranks] - place[tid * num_ranks];
            packed_count[tid] = n;
            if (stats != nullptr) stats[tid] += n;
            if (tokens_per_expert != nullptr) tokens_per_expert[tid] = uint32_t(n);
        }
        if (tid == 0) flat_total[0] = total;
    }
    // this workgroup's pair: one descriptor per row kept, and every record of the pair
    const int seg = blockIdx.x;
    const int le = seg / num_ranks, s = seg - le * num_ranks;
    // thread `seg` holds the pair's numbers; hand them to the workgroup
    __shared__ int32_t pair_first, pair_kept, pair_sent;
    if (tid == seg) pair_first = first, pair_kept = kept, pair_sent = c;
    __syncthreads();
    const int64_t begin = place[seg] - place[le * num_ranks];
    int64_t record_base = 0;  // records of the lower sources: their whole messages, kept or not
    for (int s2 = 0; s2 < s; ++s2) record_base += source_total[s2];
    record_base += pair_first;
    for (int j = tid; j < pair_sent; j += kIndexThreads) {
        int32_t packed_row = -1;
        if (j < pair_kept) {
            RowDesc d;
            d.src_row = int32_t(int64_t(s) * slot_rows + pair_first + j);
            d.dst_row = int32_t(int64_t(le) * slots_per_expert + begin + j);
            desc[place[seg] + j] = d;
            packed_row = d.dst_row;
        }
        if (record_packed_row != nullptr && record_base + j < row_capacity) record_packed_row[record_base + j] = packed_row;
    }
}

// ---------------------------------------------------------------------
// The ordered receive for small batches (at most kLargeBatchRows rows expected): index and copy in one
// launch, like the staged receive's ll_recv_kernel.  Every workgroup works out the (expert, source)
// pairs' numbers for itself in LDS -- sent(e, s) from the gathered counts, first(e, s) (where the pair
// starts in its source's message) and kept(e, s) -- one thread per pair; a copying wave then holds kept
// and first in its registers (WaveSegments) and walks the flat index space of the rows kept, one wave
// per row part; the first E_l * R waves of the grid then write the records' packed rows, a pair each.
// The last workgroup copies nothing: it writes layout_range, packed_count, stats and tokens_per_expert.
// lds: [4 * (E_l * R + 1)] ints.
// ---------------------------------------------------------------------
struct OrderedRecvArgs {
    const uint8_t* rows;            // [R * slot_rows] staged rows
    const int32_t* all_num_routed;  // [R, E]
    int num_experts, num_local_experts, num_ranks, rank, max_tokens;
    int hidden, fmt, parts_log2;
    int64_t slot_rows, row_capacity;
    uint8_t* packed_x;
    uint8_t* packed_scales;
    int32_t* src_info;
    int64_t* layout_range;
    int32_t* packed_count;
    int32_t* stats;
    uint32_t* tokens_per_expert;
    int32_t* record_packed_row;
};

constexpr int kOrderedDepth = 4;  // 16-byte loads in flight per lane

template <int kPer>
__device__ __forceinline__ void ordered_recv_impl(const OrderedRecvArgs& a, int block, int num_copy_blocks,
                                                  int32_t* lds, int32_t* wave_totals) {
    const int tid = threadIdx.x, lane = lane_id(), w = wave_in_block();
    const int threads = blockDim.x, waves = threads >> 6;
    const int num_ranks = a.num_ranks, max_tokens = a.max_tokens, num_local = a.num_local_experts;
    const int num_segments = num_local * num_ranks;
    int32_t* sent = lds;                       // [S]
    int32_t* first = sent + num_segments + 1;  // [S]
    int32_t* kept = first + num_segments + 1;  // [S + 1] (scanned in place by the last workgroup)
    int32_t* place = kept + num_segments + 1;  // [S + 1] (last workgroup only)

    // sent / first / kept of every pair, pairs in (expert, source) order: one global load per pair,
    // the sums over the lower experts from LDS
    for (int seg = tid; seg < num_segments; seg += threads) {
        const int le = seg / num_ranks, src = seg - le * num_ranks;
        const int c = a.all_num_routed[int64_t(src) * a.num_experts + a.rank * num_local + le];
        sent[seg] = c < 0 ? 0 : (c > max_tokens ? max_tokens : c);
    }
    lds_barrier();
    for (int seg = tid; seg < num_segments; seg += threads) {
        const int le = seg / num_ranks, src = seg - le * num_ranks;
        int before = 0;
        for (int e2 = 0; e2 < le; ++e2) before += sent[e2 * num_ranks + src];
        const int64_t room = a.slot_rows - before;
        const int mine = sent[seg];
        first[seg] = before;
        kept[seg] = room <= 0 ? 0 : (mine < room ? mine : int(room));
    }
    lds_barrier();

    const int64_t slots_per_expert = int64_t(max_tokens) * num_ranks;
    if (block == num_copy_blocks) {  // the metadata workgroup
        for (int seg = tid; seg < num_segments; seg += threads) place[seg] = kept[seg];
        lds_barrier();
        block_exclusive_scan(place, num_segments, wave_totals);
        for (int seg = tid; seg < num_segments; seg += threads) {
            const int le = seg / num_ranks;
            const int64_t begin = place[seg] - place[le * num_ranks];
            a.layout_range[seg] = kept[seg] > 0 ? ((begin << 32) | int64_t(kept[seg])) : 0;
        }
        for (int le = tid; le < num_local; le += threads) {
            const int n = place[(le + 1) * num_ranks] - place[le * num_ranks];
            a.packed_count[le] = n;
            if (a.stats != nullptr) a.stats[le] += n;
            if (a.tokens_per_expert != nullptr) a.tokens_per_expert[le] = uint32_t(n);
        }
        return;
    }

    WaveSegments<kPer> seg_table;
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
        const int seg = lane * kPer + u;
        seg_table.cnt[u] = seg < num_segments ? kept[seg] : 0;
        seg_table.aux[u] = seg < num_segments ? first[seg] : 0;
    }
    wave_segments_finish(seg_table);

    const int64_t data_bytes = row_data_bytes(a.hidden, a.fmt);
    const int64_t data_pad = align16(data_bytes);
    const int64_t scale_bytes = row_scale_bytes(a.hidden, a.fmt);
    const int64_t stride = row_stride_bytes(a.hidden, a.fmt);
    const int num_vec = int(data_bytes / 16);
    const int parts = 1 << a.parts_log2;
    const int num_items = seg_table.total << a.parts_log2;
    const int waves_total = num_copy_blocks * waves;
    const int scale_dwords = int(scale_bytes / 4);
    const bool has_scales = a.packed_scales != nullptr && scale_dwords > 0;

    for (int item = block * waves + w; item < num_items; item += waves_total) {
        const int row = item >> a.parts_log2, part = item & (parts - 1);
        int seg_first, in_message;
        const int seg = wave_segments_find(seg_table, row, seg_first, in_message);
        const int le = seg / num_ranks, src = seg - le * num_ranks;
        const int j = row - seg_first;
        const uint8_t* from = a.rows + (int64_t(src) * a.slot_rows + in_message + j) * stride;
        const int64_t out_row = int64_t(le) * slots_per_expert + (row - wave_segments_prefix(seg_table, le * num_ranks));
        uint8_t* to = a.packed_x + out_row * data_bytes;
        int v_begin, v_end;
        row_part_range(num_vec, parts, part, v_begin, v_end);
        const bool carries_tail = part == parts - 1;  // the last part is the shortest
        u32x4 r[kOrderedDepth];
#pragma unroll
        for (int u = 0; u < kOrderedDepth; ++u) {
            const int v = v_begin + u * kWave + lane;
            if (v < v_end) r[u] = load_u32x4<false>(from + int64_t(v) * 16);
        }
        uint32_t tail_scale = 0;
        int32_t tail_info = 0;
        if (carries_tail) {  // scales and source index travel with the payload: one round trip per row
            if (has_scales && lane < scale_dwords) tail_scale = reinterpret_cast<const uint32_t*>(from + data_pad)[lane];
            if (lane == 0) tail_info = *reinterpret_cast<const int32_t*>(from + data_pad + align16(scale_bytes));
        }
#pragma unroll
        for (int u = 0; u < kOrderedDepth; ++u) {
            const int v = v_begin + u * kWave + lane;
            if (v < v_end) store_u32x4<false>(to + int64_t(v) * 16, r[u]);
        }
        wave_copy_vec16<kOrderedDepth, false>(from, to, v_begin + kOrderedDepth * kWave, v_end, lane);
        if (!carries_tail) continue;
        if (has_scales) {
            const uint32_t* s32 = reinterpret_cast<const uint32_t*>(from + data_pad);
            uint32_t* d32 = reinterpret_cast<uint32_t*>(a.packed_scales + out_row * scale_bytes);
            if (lane < scale_dwords) d32[lane] = tail_scale;
            for (int v = kWave + lane; v < scale_dwords; v += kWave) d32[v] = s32[v];
        }
        if (lane == 0) a.src_info[out_row] = tail_info;
    }

    // The records' packed rows, a pair per wave (the first E_l * R waves of the grid, after their copies).
    // Record of row j of pair (e, s): the records of the lower sources (their whole messages, kept or
    // not), then the source's rows for the lower experts, then j.
    if (a.record_packed_row == nullptr) return;
    for (int seg = block * waves + w; seg < num_segments; seg += waves_total) {
        const int le = seg / num_ranks, src = seg - le * num_ranks;
        int lower = 0;  // rows the lower sources sent, all experts
        for (int q = lane; q < num_local * src; q += kWave) lower += sent[(q / src) * num_ranks + q % src];
        const int64_t record0 = int64_t(wave_sum(lower)) + first[seg];
        const int64_t packed0 = int64_t(le) * slots_per_expert +
                                (wave_segments_prefix(seg_table, seg) - wave_segments_prefix(seg_table, le * num_ranks));
        const int n_sent = sent[seg], n_kept = kept[seg];
        for (int j = lane; j < n_sent; j += kWave)
            if (record0 + j < a.row_capacity) a.record_packed_row[record0 + j] = j < n_kept ? int32_t(packed0 + j) : -1;
    }
}

__global__ __launch_bounds__(256) void ll_recv_ordered_kernel(OrderedRecvArgs a) {
    extern __shared__ int32_t ordered_lds[];
    __shared__ int32_t wave_totals[kMaxBlockWaves];
    if (a.num_local_experts * a.num_ranks <= 4 * kWave)
        ordered_recv_impl<4>(a, blockIdx.x, int(gridDim.x) - 1, ordered_lds, wave_totals);
    else
        ordered_recv_impl<16>(a, blockIdx.x, int(gridDim.x) - 1, ordered_lds, wave_totals);
}

}  // namespace deepep

using namespace deepep;

extern "C" {

// Workspace: [flat_total | pad] [chunk histograms: at most ceil(capacity / 512) + R chunks of E_l counts] [descriptors]
static int64_t by_source_head_bytes() { return 256; }
static int64_t by_source_hist_bytes(int num_experts, int64_t row_capacity) {
    const int64_t chunks = (row_capacity + kBySourceThreads - 1) / kBySourceThreads + 1;  // E_l * (chunks + R) <= E * chunks
    return (chunks * num_experts * 4 + 255) & ~int64_t(255);
}

size_t deepep_ll_by_source_workspace_bytes(int num_experts, int64_t row_capacity) {
    const int64_t capacity = row_capacity < 1 ? 1 : row_capacity;
    return size_t(by_source_head_bytes() + by_source_hist_bytes(num_experts, capacity) +
                  capacity * int64_t(sizeof(RowDesc)));
}

int deepep_ll_dispatch_recv_by_source(const void* recv_by_source, int64_t slot_rows, const int32_t* recv_counts,
                                      const uint32_t* source_offset, const uint32_t* num_recv_tokens,
                                      int64_t row_capacity, int hidden, int num_experts, int num_ranks,
                                      int num_max_dispatch_tokens_per_rank, int row_format, void* packed_recv_x,
                                      void* packed_recv_scales, int32_t* packed_recv_src_info,
                                      int64_t* packed_recv_layout_range, int32_t* packed_recv_count,
                                      int32_t* cumulative_local_expert_recv_stats, uint32_t* tokens_per_expert,
                                      int32_t* record_packed_row, int64_t expected_rows, void* workspace,
                                      size_t workspace_bytes, void* stream) {
    clear_error();
    EP_HOST_ASSERT(hidden > 0 && hidden % 128 == 0);
    EP_HOST_ASSERT(num_ranks > 0 && num_ranks <= kBySourceMaxRanks);
    EP_HOST_ASSERT(num_experts > 0 && num_experts % num_ranks == 0);
    const int num_local_experts = num_experts / num_ranks;
    EP_HOST_ASSERT(num_local_experts <= kBySourceMaxLocalExperts && num_experts <= 4096);
    EP_HOST_ASSERT(num_max_dispatch_tokens_per_rank > 0);
    EP_HOST_ASSERT(row_format >= kRowBF16 && row_format <= kRowFP8UE8M0);
    EP_HOST_ASSERT(row_format != kRowFP8UE8M0 || (hidden / 128) % 4 == 0);
    EP_HOST_ASSERT(slot_rows > 0 && slot_rows * num_ranks < (int64_t(1) << 31));
    EP_HOST_ASSERT(row_capacity >= 0 && row_capacity < (int64_t(1) << 31));
    EP_HOST_ASSERT(int64_t(num_experts) * num_max_dispatch_tokens_per_rank < (int64_t(1) << 31));
    EP_HOST_ASSERT(recv_by_source != nullptr && recv_counts != nullptr && num_recv_tokens != nullptr);
    EP_HOST_ASSERT(row_capacity == 0 || source_offset != nullptr);
    EP_HOST_ASSERT(packed_recv_x != nullptr && (row_format == kRowBF16 || packed_recv_scales != nullptr));
    EP_HOST_ASSERT(packed_recv_src_info != nullptr && packed_recv_layout_range != nullptr &&
                   packed_recv_count != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(recv_by_source) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(packed_recv_x) & 15) == 0);
    EP_HOST_ASSERT(workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0);
    EP_HOST_ASSERT(workspace_bytes >= deepep_ll_by_source_workspace_bytes(num_experts, row_capacity));
    // LDS of the index kernel: source prefix, chunk prefix, pair prefix, running counts, per-wave counts
    const size_t index_lds = size_t(2 * (num_ranks + 1) + num_experts + 1 + num_local_experts +
                                    kBySourceWaves * num_local_experts) * sizeof(int32_t);
    EP_HOST_ASSERT(index_lds <= 64 * 1024);

    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
    const int64_t stride = row_stride_bytes(hidden, row_format);
    const int64_t data_bytes = row_data_bytes(hidden, row_format);
    const int64_t scale_bytes = row_scale_bytes(hidden, row_format);
    const int64_t tail_off = align16(data_bytes) + align16(scale_bytes);
    const int64_t buffer_rows = slot_rows * num_ranks;
    const int64_t capacity = row_capacity < 1 ? 1 : row_capacity;
    int32_t* flat_total = reinterpret_cast<int32_t*>(workspace);
    int32_t* hist = reinterpret_cast<int32_t*>(reinterpret_cast<uint8_t*>(workspace) + by_source_head_bytes());
    RowDesc* desc = reinterpret_cast<RowDesc*>(reinterpret_cast<uint8_t*>(workspace) + by_source_head_bytes() +
                                               by_source_hist_bytes(num_experts, capacity));
    const uint8_t* rows_in = reinterpret_cast<const uint8_t*>(recv_by_source);

    // Which form indexes the records depends on how many are expected, not on how many fit: both give the
    // same result, and a buffer sized for its largest batch still takes the short form for a small one.
    const int64_t expected_records = expected_rows > 0 && expected_rows < row_capacity ? expected_rows : row_capacity;
    if (expected_records <= kBySourceSmallRecords) {
        ll_by_source_index_kernel<false><<<num_ranks, kBySourceThreads, index_lds, hs>>>(
            rows_in, stride, tail_off, buffer_rows, int(slot_rows), recv_counts, source_offset, num_recv_tokens,
            row_capacity, num_local_experts, num_ranks, num_max_dispatch_tokens_per_rank, nullptr,
            packed_recv_layout_range, packed_recv_count, cumulative_local_expert_recv_stats, tokens_per_expert,
            record_packed_row, flat_total, desc);
        EP_LAUNCH_CHECK();
    } else {
        // every source's records round up to whole chunks: at most ceil(capacity / 512) + R of them
        const int64_t chunks = (row_capacity + kBySourceThreads - 1) / kBySourceThreads + num_ranks;
        const size_t count_lds = size_t(2 * (num_ranks + 1) + num_local_experts) * sizeof(int32_t);
        ll_by_source_count_kernel<<<unsigned(chunks), kBySourceThreads, count_lds, hs>>>(
            rows_in, stride, tail_off, buffer_rows, int(slot_rows), recv_counts, source_offset, num_recv_tokens,
            row_capacity, num_local_experts, num_ranks, hist);
        EP_LAUNCH_CHECK();
        ll_by_source_index_kernel<true><<<unsigned(chunks), kBySourceThreads, index_lds, hs>>>(
            rows_in, stride, tail_off, buffer_rows, int(slot_rows), recv_counts, source_offset, num_recv_tokens,
            row_capacity, num_local_experts, num_ranks, num_max_dispatch_tokens_per_rank, hist,
            packed_recv_layout_range, packed_recv_count, cumulative_local_expert_recv_stats, tokens_per_expert,
            record_packed_row, flat_total, desc);
        EP_LAUNCH_CHECK();
    }
    if (row_capacity == 0) return 0;
    const int num_vec = int(data_bytes / 16);
    int threads = ((num_vec + 63) / 64) * 64;
    int extra = 64;  // one more wave for scales + source index
    if (threads + extra > 1024) threads = 1024, extra = 0;
    // the copy's grid follows the rows expected, not the capacity: a workgroup that finds no row still costs
    // a fraction of a nanosecond, and a capacity of R slots is many times what a balanced world fills
    const unsigned blocks = flat_grid_blocks(expected_rows > 0 ? expected_rows : row_capacity, row_capacity,
                                             num_max_dispatch_tokens_per_rank);
    ll_rows_flat_kernel<<<blocks, threads + extra, 0, hs>>>(
        flat_total, 0, desc, rows_in, stride, num_vec,
        reinterpret_cast<uint8_t*>(packed_recv_x), nullptr, data_bytes, int(scale_bytes / 4), align16(data_bytes),
        scale_bytes > 0 ? reinterpret_cast<uint8_t*>(packed_recv_scales) : nullptr, tail_off, packed_recv_src_info,
        extra);
    EP_LAUNCH_CHECK();
    return 0;
}

int deepep_ll_dispatch_recv_by_source_ordered(const void* recv_by_source, int64_t slot_rows,
                                              const int32_t* all_num_routed, int hidden, int num_experts,
                                              int num_ranks, int rank, int num_max_dispatch_tokens_per_rank,
                                              int row_format, void* packed_recv_x, void* packed_recv_scales,
                                              int32_t* packed_recv_src_info, int64_t* packed_recv_layout_range,
                                              int32_t* packed_recv_count,
                                              int32_t* cumulative_local_expert_recv_stats,
                                              uint32_t* tokens_per_expert, int32_t* record_packed_row,
                                              int64_t row_capacity, int64_t expected_rows, void* workspace,
                                              size_t workspace_bytes, void* stream) {
    clear_error();
    EP_HOST_ASSERT(hidden > 0 && hidden % 128 == 0);
    EP_HOST_ASSERT(num_ranks > 0 && num_experts > 0 && num_experts % num_ranks == 0);
    EP_HOST_ASSERT(rank >= 0 && rank < num_ranks);
    EP_HOST_ASSERT(num_experts <= kIndexThreads);  // one thread per (local expert, source) pair
    EP_HOST_ASSERT(num_max_dispatch_tokens_per_rank > 0);
    EP_HOST_ASSERT(row_format >= kRowBF16 && row_format <= kRowFP8UE8M0);
    EP_HOST_ASSERT(row_format != kRowFP8UE8M0 || (hidden / 128) % 4 == 0);
    EP_HOST_ASSERT(slot_rows > 0 && slot_rows * num_ranks < (int64_t(1) << 31));
    EP_HOST_ASSERT(row_capacity >= 0 && row_capacity < (int64_t(1) << 31));
    EP_HOST_ASSERT(int64_t(num_experts) * num_max_dispatch_tokens_per_rank < (int64_t(1) << 31));
    EP_HOST_ASSERT(recv_by_source != nullptr && all_num_routed != nullptr);
    EP_HOST_ASSERT(packed_recv_x != nullptr && (row_format == kRowBF16 || packed_recv_scales != nullptr));
    EP_HOST_ASSERT(packed_recv_src_info != nullptr && packed_recv_layout_range != nullptr &&
                   packed_recv_count != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(recv_by_source) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(packed_recv_x) & 15) == 0);
    EP_HOST_ASSERT(workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0);
    // one descriptor per row that can be kept: a source's slot, and an expert's packed slots, bound them
    const int64_t most_rows = std::min<int64_t>(slot_rows * num_ranks,
                                                int64_t(num_experts) * num_max_dispatch_tokens_per_rank);
    EP_HOST_ASSERT(workspace_bytes >= size_t(by_source_head_bytes() + most_rows * int64_t(sizeof(RowDesc))));
    const int num_local_experts = num_experts / num_ranks;
    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
    const int64_t expected = expected_rows > 0 ? expected_rows : most_rows;
    if (expected <= kLargeBatchRows) {  // one launch: every workgroup indexes for itself
        OrderedRecvArgs oa;
        oa.rows = reinterpret_cast<const uint8_t*>(recv_by_source);
        oa.all_num_routed = all_num_routed;
        oa.num_experts = num_experts, oa.num_local_experts = num_local_experts, oa.num_ranks = num_ranks;
        oa.rank = rank, oa.max_tokens = num_max_dispatch_tokens_per_rank;
        oa.hidden = hidden, oa.fmt = row_format;
        oa.parts_log2 = choose_row_parts_log2(expected, row_data_bytes(hidden, row_format));
        oa.slot_rows = slot_rows, oa.row_capacity = row_capacity;
        oa.packed_x = reinterpret_cast<uint8_t*>(packed_recv_x);
        oa.packed_scales = row_format == kRowBF16 ? nullptr : reinterpret_cast<uint8_t*>(packed_recv_scales);
        oa.src_info = packed_recv_src_info, oa.layout_range = packed_recv_layout_range;
        oa.packed_count = packed_recv_count, oa.stats = cumulative_local_expert_recv_stats;
        oa.tokens_per_expert = tokens_per_expert, oa.record_packed_row = record_packed_row;
        int64_t rows = expected + expected / 8 + 16;
        if (rows > most_rows) rows = most_rows;
        int64_t blocks = ((rows << oa.parts_log2) + 3) / 4;
        blocks = blocks < 1 ? 1 : (blocks > 1024 ? 1024 : blocks);
        const size_t lds = size_t(4 * (num_experts + 1)) * sizeof(int32_t);
        ll_recv_ordered_kernel<<<dim3(unsigned(blocks) + 1), 256, lds, hs>>>(oa);  // + the metadata workgroup
        EP_LAUNCH_CHECK();
        return 0;
    }
    int32_t* flat_total = reinterpret_cast<int32_t*>(workspace);
    RowDesc* desc = reinterpret_cast<RowDesc*>(reinterpret_cast<uint8_t*>(workspace) + by_source_head_bytes());
    ll_by_source_ordered_index_kernel<<<num_experts, kIndexThreads, 0, hs>>>(
        all_num_routed, num_experts, num_local_experts, num_ranks, rank, num_max_dispatch_tokens_per_rank,
        int(slot_rows), row_capacity, packed_recv_layout_range, packed_recv_count,
        cumulative_local_expert_recv_stats, tokens_per_expert, record_packed_row, flat_total, desc);
    EP_LAUNCH_CHECK();
    const int64_t data_bytes = row_data_bytes(hidden, row_format);
    const int64_t scale_bytes = row_scale_bytes(hidden, row_format);
    const int num_vec = int(data_bytes / 16);
    int threads = ((num_vec + 63) / 64) * 64;
    int extra = 64;  // one more wave for scales + source index
    if (threads + extra > 1024) threads = 1024, extra = 0;
    const unsigned blocks = flat_grid_blocks(expected_rows > 0 ? expected_rows : most_rows, most_rows,
                                             num_max_dispatch_tokens_per_rank);
    ll_rows_flat_kernel<<<blocks, threads + extra, 0, hs>>>(
        flat_total, 0, desc, reinterpret_cast<const uint8_t*>(recv_by_source), row_stride_bytes(hidden, row_format),
        num_vec, reinterpret_cast<uint8_t*>(packed_recv_x), nullptr, data_bytes, int(scale_bytes / 4),
        align16(data_bytes), scale_bytes > 0 ? reinterpret_cast<uint8_t*>(packed_recv_scales) : nullptr,
        align16(data_bytes) + align16(scale_bytes), packed_recv_src_info, extra);
    EP_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
