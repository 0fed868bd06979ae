// Helpers for kernels that walk a list of variable-length row segments with
// one wavefront per row (part): the segment prefix held in a wave's registers
// with its row -> segment lookup, a workgroup-wide exclusive scan in LDS for the
// metadata pass, the 16-byte-per-lane row copy, and the index + flat-copy pair
// of kernels for large batches.
#pragma once

#include "common.hpp"

namespace deepep {

// ---------------------------------------------------------------------
// Exclusive prefix of n ints held in LDS, by the whole workgroup (a multiple
// of 64 threads, at most 1024).  data[n] receives the total; wave_totals has
// room for 16 ints.
// ---------------------------------------------------------------------
constexpr int kMaxBlockWaves = 16;

__device__ __forceinline__ void block_exclusive_scan(int32_t* data, int n, int32_t* wave_totals) {
    const int tid = threadIdx.x, lane = lane_id(), w = tid >> 6;
    const int threads = blockDim.x, waves = threads >> 6;
    const int per = (n + threads - 1) / threads;
    const int lo = tid * per;
    int sum = 0;
    for (int j = 0; j < per; ++j)
        if (lo + j < n) sum += data[lo + j];
    const int incl = wave_inclusive_sum(sum);
    if (lane == kWave - 1) wave_totals[w] = incl;
    lds_barrier();
    int offset = incl - sum, total = 0;
    for (int w2 = 0; w2 < waves; ++w2) {
        const int t = wave_totals[w2];
        if (w2 < w) offset += t;
        total += t;
    }
    int run = offset;
    for (int j = 0; j < per; ++j)
        if (lo + j < n) {
            const int v = data[lo + j];
            data[lo + j] = run;
            run += v;
        }
    if (tid == 0) data[n] = total;
    lds_barrier();
}

// ---------------------------------------------------------------------
// The same prefix, held by one wave in registers: no LDS and no barrier, so a
// wave can start looking up rows as soon as its own loads of the counts are
// back.  Lane l holds the counts of segments [l * kPer, (l + 1) * kPer) and the
// number of rows in all lower lanes' segments.  kPer is a compile-time 4 (up to
// 256 segments) or 16 (up to 1024) so that every index below is static and the
// arrays stay in registers.
// ---------------------------------------------------------------------
template <int kPer>
struct WaveSegments {
    int cnt[kPer];
    int aux[kPer];  // one caller-defined value per segment, returned by the lookup
    int lane_base;  // rows in the segments held by lower lanes
    int total;      // rows in all segments
};

// Lane l's kPer consecutive values p[l * kPer + u] (0 beyond n), as 16-byte loads where a whole
// vector lies inside the array.  p must be 16-byte aligned.
template <int kPer>
__device__ __forceinline__ void wave_load_int32(const int32_t* __restrict__ p, int n, int lane, int (&out)[kPer]) {
    static_assert(kPer % 4 == 0, "whole 16-byte vectors per lane");
#pragma unroll
    for (int v = 0; v < kPer / 4; ++v) {
        const int s0 = lane * kPer + v * 4;
        if (s0 + 3 < n) {
            const u32x4 q = *reinterpret_cast<const u32x4*>(p + s0);
#pragma unroll
            for (int i = 0; i < 4; ++i) out[v * 4 + i] = int(q[i]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) out[v * 4 + i] = s0 + i < n ? p[s0 + i] : 0;
        }
    }
}

template <int kPer>
__device__ __forceinline__ void wave_load_int64(const int64_t* __restrict__ p, int n, int lane,
                                                int64_t (&out)[kPer]) {
    static_assert(kPer % 2 == 0, "whole 16-byte vectors per lane");
#pragma unroll
    for (int v = 0; v < kPer / 2; ++v) {
        const int s0 = lane * kPer + v * 2;
        if (s0 + 1 < n) {
            const u32x4 q = *reinterpret_cast<const u32x4*>(p + s0);
            out[v * 2] = int64_t((uint64_t(q[1]) << 32) | q[0]);
            out[v * 2 + 1] = int64_t((uint64_t(q[3]) << 32) | q[2]);
        } else {
            out[v * 2] = s0 < n ? p[s0] : 0;
            out[v * 2 + 1] = 0;
        }
    }
}

// Finishes a table whose cnt[] the caller has filled (zero beyond the last segment).
template <int kPer>
__device__ __forceinline__ void wave_segments_finish(WaveSegments<kPer>& t) {
    int mine = 0;
#pragma unroll
    for (int u = 0; u < kPer; ++u) mine += t.cnt[u];
    const int incl = wave_inclusive_sum(mine);
    t.lane_base = incl - mine;
    t.total = __builtin_amdgcn_readlane(incl, kWave - 1);
}

// Rows before segment q (wave-uniform q in [0, 64 * kPer]).
template <int kPer>
__device__ __forceinline__ int wave_segments_prefix(const WaveSegments<kPer>& t, int q) {
    q = __builtin_amdgcn_readfirstlane(q);
    const int owner = q / kPer, within = q % kPer;
    if (owner >= kWave) return t.total;
    int run = t.lane_base;
#pragma unroll
    for (int u = 0; u < kPer; ++u)
        if (u < within) run += t.cnt[u];
    return __builtin_amdgcn_readlane(run, owner);
}

// Segment holding row (wave-uniform, 0 <= row < total); seg_first receives the rows before it,
// seg_aux the segment's aux value.
template <int kPer>
__device__ __forceinline__ int wave_segments_find(const WaveSegments<kPer>& t, int row, int& seg_first,
                                                  int& seg_aux) {
    // the last lane whose base is <= row owns the row (empty lanes share their successor's base)
    const int owner = __builtin_amdgcn_readfirstlane(__popcll(__ballot(t.lane_base <= row)) - 1);
    int run = t.lane_base, found = 0, first = t.lane_base, aux = 0;
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
        if (run <= row && row < run + t.cnt[u]) found = u, first = run, aux = t.aux[u];
        run += t.cnt[u];
    }
    seg_first = __builtin_amdgcn_readlane(first, owner);
    seg_aux = __builtin_amdgcn_readlane(aux, owner);
    return owner * kPer + __builtin_amdgcn_readlane(found, owner);
}

// Copies 16-byte vectors [v_begin, v_end) of a row with one wave, kDepth loads in flight per lane.
template <int kDepth, bool kStream = false>
__device__ __forceinline__ void wave_copy_vec16(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                int v_begin, int v_end, int lane) {
    for (int base = v_begin; base < v_end; base += kWave * kDepth) {
        u32x4 r[kDepth];
#pragma unroll
        for (int u = 0; u < kDepth; ++u) {
            const int v = base + u * kWave + lane;
            if (v < v_end) r[u] = load_u32x4<kStream>(src + int64_t(v) * 16);
        }
#pragma unroll
        for (int u = 0; u < kDepth; ++u) {
            const int v = base + u * kWave + lane;
            if (v < v_end) store_u32x4<kStream>(dst + int64_t(v) * 16, r[u]);
        }
    }
}

// A row of num_vec vectors cut into `parts` runs of whole 64-vector (1 KiB) chunks.
__device__ __forceinline__ void row_part_range(int num_vec, int parts, int part, int& v_begin, int& v_end) {
    const int chunks = (num_vec + kWave - 1) / kWave;
    const int per = (chunks + parts - 1) / parts;
    v_begin = min(part * per * kWave, num_vec);
    v_end = min(v_begin + per * kWave, num_vec);
}

// Host-side choice of the row split (log2 of the parts): small problems cannot fill the chip with
// one wave per row.
inline int choose_row_parts_log2(int64_t estimated_rows, int64_t row_bytes) {
    if (estimated_rows > 8192) return 0;
    return row_bytes > 8192 ? 2 : 1;
}

// ---------------------------------------------------------------------
// Large batches.  A flat copy — one workgroup per row, one 16-byte vector per
// thread, no loop — is what reaches the highest HBM rate on this GPU, but it
// needs the row -> (source, destination) map up front.  ll_segment_index_kernel
// builds it: one workgroup per segment scans the segment counts (<= 1024 ints)
// and writes a descriptor {source row, destination row} for each of its rows.
// ---------------------------------------------------------------------
struct RowDesc {
    int32_t src_row;  // row index in the source buffer; < 0: nothing to copy
    int32_t dst_row;  // >= 0: row index in the primary destination; < 0: -(1 + row) in the secondary one
};

constexpr int kIndexThreads = 1024;

// Exclusive prefix over one value per thread of a 1024-thread workgroup; returns the prefix, sets total.
__device__ __forceinline__ int block_exclusive_scan_1024(int v, int32_t* wave_totals, int& total) {
    const int lane = lane_id(), w = int(threadIdx.x) >> 6;
    const int incl = wave_inclusive_sum(v);
    if (lane == kWave - 1) wave_totals[w] = incl;
    __syncthreads();
    int offset = incl - v;
    total = 0;
    for (int w2 = 0; w2 < kIndexThreads / kWave; ++w2) {
        const int t = wave_totals[w2];
        if (w2 < w) offset += t;
        total += t;
    }
    return offset;
}

// mode 0 (dispatch receive): counts = recv_count; writes layout_range / packed_count / stats;
//        descriptor = {staging row seg*M + j, packed row e_l*N + begin + j}; rank = -1, or the rank
//        whose own rows the send side has already put at their packed position (they keep their
//        place in the ranges, in ascending source order, and get no descriptors).
// mode 1 (combine send; mode 2: the same without this rank's own rows): counts and begins from layout_range;
//        descriptor = {expert-output row e_l*N + begin + j, seg*M + j for other ranks or
//        -(1 + (rank*E_l + e_l)*M + j) for this rank's own rows}.
static __global__ __launch_bounds__(kIndexThreads) void ll_segment_index_kernel(
    int mode, const int32_t* __restrict__ counts32, const int64_t* __restrict__ layout_in, int num_local_experts,
    int num_ranks, int rank, int max_tokens, int64_t* __restrict__ layout_out, int32_t* __restrict__ packed_count,
    int32_t* __restrict__ stats, int32_t* __restrict__ flat_out, RowDesc* __restrict__ desc) {
    __shared__ int32_t flat[kIndexThreads + 1];   // prefix over the rows that get descriptors
    __shared__ int32_t place[kIndexThreads + 1];  // mode 0: prefix over all rows (where a segment lands)
    __shared__ int32_t begin_in[kIndexThreads];
    __shared__ int32_t wave_totals[kIndexThreads / kWave];
    __shared__ int32_t wave_totals_place[kIndexThreads / kWave];
    const int tid = threadIdx.x;
    const int num_segments = num_local_experts * num_ranks;
    int c = 0;
    if (tid < num_segments) {
        if (mode == 0) {
            c = counts32[tid];
        } else {
            const int64_t lr = layout_in[tid];
            c = int(lr & 0xffffffffll);
            begin_in[tid] = int(lr >> 32);
            if (mode == 2 && tid % num_ranks == rank) c = 0;  // own rows stay where they are
        }
        c = c < 0 ? 0 : (c > max_tokens ? max_tokens : c);
    }
    // mode 0 with rank >= 0: the rank's own rows are already in place (reference order: a range
    // begins where the lower source ranks' rows end, csrc/kernels/efa_kernels.cu:991-1010), so
    // they count towards where the later segments land but take no descriptors
    const bool own_placed = mode == 0 && rank >= 0;
    const int c_all = c;
    if (own_placed && tid < num_segments && tid % num_ranks == rank) c = 0;
    int total;
    const int prefix = block_exclusive_scan_1024(c, wave_totals, total);
    if (tid < num_segments) flat[tid] = prefix;
    if (tid == 0) flat[num_segments] = total;
    if (mode == 0) {
        int total_all = total, prefix_all = prefix;
        if (own_placed) prefix_all = block_exclusive_scan_1024(c_all, wave_totals_place, total_all);
        if (tid < num_segments) place[tid] = prefix_all;
        if (tid == 0) place[num_segments] = total_all;
    }
    __syncthreads();
    const int64_t slots_per_expert = int64_t(max_tokens) * num_ranks;
    if (blockIdx.x == 0) {
        for (int s = tid; s <= num_segments; s += kIndexThreads) flat_out[s] = flat[s];
        if (mode == 0) {
            if (tid < num_segments) {
                const int le = tid / num_ranks;
                const int64_t cnt = c_all;
                const int64_t begin = place[tid] - place[le * num_ranks];
                layout_out[tid] = cnt > 0 ? ((begin << 32) | cnt) : 0;
            }
            if (tid < num_local_experts) {
                const int n = place[(tid + 1) * num_ranks] - place[tid * num_ranks];
                packed_count[tid] = n;
                if (stats != nullptr) stats[tid] += n;
            }
        }
    }
    const int seg = blockIdx.x;
    const int le = seg / num_ranks, s = seg - le * num_ranks;
    const int cnt = flat[seg + 1] - flat[seg];
    const int64_t begin = mode == 0 ? place[seg] - place[le * num_ranks] : begin_in[seg];
    if (mode != 0 && (begin < 0 || begin + cnt > slots_per_expert)) return;  // malformed range: emit nothing
    for (int j = tid; j < cnt; j += kIndexThreads) {
        RowDesc d;
        if (mode == 0) {
            d.src_row = seg * max_tokens + j;
            d.dst_row = int32_t(le * slots_per_expert + begin + j);
        } else {
            d.src_row = int32_t(le * slots_per_expert + begin + j);
            d.dst_row = s == rank ? -(1 + (rank * num_local_experts + le) * max_tokens + j) : seg * max_tokens + j;
        }
        desc[flat[seg] + j] = d;
    }
}

// The dispatch-receive index (mode 0 above with the rank's own rows already placed) as one workgroup's
// share inside another launch: the send kernel of a large one-call dispatch carries these workgroups
// beside its own, so the index costs no launch.  The launch that carries it is still writing the
// rank's own counts into recv_count, so they are taken from what that launch reads them from: the
// column sums of the per-chunk expert histograms.  Any workgroup size that is a multiple of 64;
// lds holds 2 * (segments + 1) ints, wave_totals 16.
struct FusedIndexArgs {
    const int32_t* recv_count;  // [E_l][R]; the own column is not read
    const int32_t* chunk_hist;  // [chunks][E] of this rank's own entries
    int num_chunks, num_experts, num_local_experts, num_ranks, rank, max_tokens;
    int64_t* layout_out;
    int32_t* packed_count;
    int32_t* stats;
    int32_t* flat_out;
    RowDesc* desc;
};

__device__ __forceinline__ void recv_index_block(const FusedIndexArgs& a, int seg, int32_t* lds, int32_t* wave_totals) {
    const int tid = threadIdx.x, threads = blockDim.x;
    const int num_ranks = a.num_ranks, max_tokens = a.max_tokens;
    const int num_segments = a.num_local_experts * num_ranks;
    int32_t* flat = lds;                      // prefix over the rows that get descriptors
    int32_t* place = lds + num_segments + 1;  // prefix over all rows: where a segment lands
    for (int s = tid; s < num_segments; s += threads) {
        const int le = s / num_ranks, src = s - le * num_ranks;
        int c = 0;
        if (src == a.rank) {
            const int e = a.rank * a.num_local_experts + le;
            for (int c0 = 0; c0 < a.num_chunks; c0 += 8) {  // eight loads in flight
                int v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    v[u] = c0 + u < a.num_chunks ? a.chunk_hist[int64_t(c0 + u) * a.num_experts + e] : 0;
#pragma unroll
                for (int u = 0; u < 8; ++u) c += v[u];
            }
        } else {
            c = a.recv_count[s];
        }
        c = c < 0 ? 0 : (c > max_tokens ? max_tokens : c);
        place[s] = c;
        flat[s] = src == a.rank ? 0 : c;  // own rows are in place already: no descriptors
    }
    lds_barrier();
    block_exclusive_scan(flat, num_segments, wave_totals);
    block_exclusive_scan(place, num_segments, wave_totals);
    const int64_t slots_per_expert = int64_t(max_tokens) * num_ranks;
    if (seg == 0) {
        for (int s = tid; s <= num_segments; s += threads) a.flat_out[s] = flat[s];
        for (int s = tid; s < num_segments; s += threads) {
            const int le = s / num_ranks;
            const int64_t cnt = place[s + 1] - place[s];
            const int64_t begin = place[s] - place[le * num_ranks];
            a.layout_out[s] = cnt > 0 ? ((begin << 32) | cnt) : 0;
        }
        for (int le = tid; le < a.num_local_experts; le += threads) {
            const int n = place[(le + 1) * num_ranks] - place[le * num_ranks];
            a.packed_count[le] = n;
            if (a.stats != nullptr) a.stats[le] += n;
        }
    }
    const int le = seg / num_ranks;
    const int cnt = flat[seg + 1] - flat[seg];
    const int64_t begin = place[seg] - place[le * num_ranks];
    for (int j = tid; j < cnt; j += threads) {
        RowDesc d;
        d.src_row = seg * max_tokens + j;
        d.dst_row = int32_t(le * slots_per_expert + begin + j);
        a.desc[flat[seg] + j] = d;
    }
}

// One workgroup per described row (looping only if there are more rows than workgroups).  Only
// batches too large for the caches come here, so the payload streams.
static __global__ __launch_bounds__(1024) void ll_rows_flat_kernel(
    const int32_t* __restrict__ flat, int num_segments, const RowDesc* __restrict__ desc,
    const uint8_t* __restrict__ src, int64_t src_stride, int num_vec, uint8_t* __restrict__ dst_primary,
    uint8_t* __restrict__ dst_secondary, int64_t dst_stride, int scale_dwords, int64_t src_scale_off,
    uint8_t* __restrict__ scale_dst, int64_t tail_off, int32_t* __restrict__ src_info, int extra_threads) {
    const int total = flat[num_segments];
    for (int row = blockIdx.x; row < total; row += gridDim.x) {
        const RowDesc d = desc[row];
        if (d.src_row < 0) continue;  // a record that names no row
        const uint8_t* s = src + int64_t(d.src_row) * src_stride;
        uint8_t* o;
        if (d.dst_row >= 0) {
            if (dst_primary == nullptr) continue;
            o = dst_primary + int64_t(d.dst_row) * dst_stride;
        } else {
            o = dst_secondary + int64_t(-(d.dst_row + 1)) * dst_stride;
        }
        // threads [0, data_threads) move the payload; when the launch carries extra threads beyond
        // them, those move scales and the source index in the same pass instead of a second one
        const int data_threads = extra_threads > 0 ? int(blockDim.x) - extra_threads : int(blockDim.x);
        const int tid = threadIdx.x;
        if (tid < data_threads)
            for (int v = tid; v < num_vec; v += data_threads)
                store_u32x4<true>(o + int64_t(v) * 16, load_u32x4<true>(s + int64_t(v) * 16));
        if (extra_threads == 0 || tid >= data_threads) {
            const int t2 = extra_threads > 0 ? tid - data_threads : tid;
            const int step = extra_threads > 0 ? extra_threads : int(blockDim.x);
            if (scale_dst != nullptr) {
                const uint32_t* s32 = reinterpret_cast<const uint32_t*>(s + src_scale_off);
                uint32_t* d32 = reinterpret_cast<uint32_t*>(scale_dst + int64_t(d.dst_row) * scale_dwords * 4);
                for (int v = t2; v < scale_dwords; v += step) d32[v] = s32[v];
            }
            if (src_info != nullptr && t2 == step - 1)
                src_info[d.dst_row] = *reinterpret_cast<const int32_t*>(s + tail_off);
        }
    }
}

__host__ __device__ inline int64_t segment_workspace_bytes(int num_experts, int max_tokens) {
    const int64_t flat_bytes = ((int64_t(num_experts) + 1) * 4 + 255) & ~int64_t(255);
    return flat_bytes + int64_t(num_experts) * max_tokens * int64_t(sizeof(RowDesc));
}

// Estimated rows above this bound take the index + flat-copy pair instead of the single fused kernel.
constexpr int64_t kLargeBatchRows = 8192;

// Rows a call will probably move: the caller's hint or, without one, a guess from the capacity
// (E * M slots, of which a balanced world fills one in 32 at top-8 of 256 experts).  Only the
// choice between equivalent kernels and the grid sizes depend on it.
inline int64_t estimated_rows(int64_t expected_rows, int64_t num_experts, int64_t max_tokens) {
    return expected_rows > 0 ? expected_rows : num_experts * max_tokens / 32;
}

inline unsigned flat_grid_blocks(int64_t expected_rows, int64_t max_rows, int max_tokens) {
    int64_t want = expected_rows > 0 ? expected_rows : int64_t(max_tokens) * 8;
    want += want / 8 + 64;
    if (want > max_rows) want = max_rows;
    if (want > (int64_t(1) << 22)) want = int64_t(1) << 22;
    if (want < 1) want = 1;
    // beyond 64 workgroups per CU two rows per workgroup measured ~5 % faster than one; eight slower
    if (want > 16384) want = want / 2 > 16384 ? want / 2 : 16384;
    return unsigned(want);
}

}  // namespace deepep
