// Low-latency dispatch: route ranking, fused quantise + pack (send side),
// segment compaction (receive side), and the single launch that runs both
// for decode-sized batches.
//
// Data layout in HBM (row stride S = row_stride_bytes(H, format)):
//   recv_staging  [E_l][R][M] rows — slot j of segment (e_l, s) is the j-th
//                 row rank s sent to local expert e_l, in ascending (t,k)
//                 order of the sender.
//   recv_count    [E_l][R] int32 — rows present in each segment.
//   send_slots    [E][M] rows — this rank's rows for remote experts.
// A staged row is [data | pad16][scales | pad16][src_token, k, src_rank, local expert].
//
// Work is cut per wavefront, never per thread block: one wave owns one 1 KiB
// piece of one row, so a 64-lane 16-byte access is one contiguous KiB and no
// LDS or barrier is needed on the copy paths.
#include "common.hpp"
#include "quant.hpp"
#include "segments.hpp"
#include <algorithm>
#include <cstdlib>
#include <mutex>

#include "../../include/deepep_hip.h"

// Route scratch (the chunk histograms of ll_chunk_hist_kernel) for deepep_ll_dispatch_send_static,
// whose callers cannot allocate.  The array is part of the code object: every GPU the library runs
// on holds its own copy, at its own address, until the process ends.  Host code never passes this
// name to a kernel; it passes the device address hipGetSymbolAddress returns (static_route_scratch).
constexpr size_t kStaticScratchBytes = size_t(1) << 20;
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

namespace deepep {

__host__ __device__ inline int64_t align256(int64_t v) { return (v + 255) & ~int64_t(255); }

constexpr int kByDestInBlockEntries = 2048;  // by-destination batches up to here build their tables in the send launch
constexpr int kSweepChunkEntries = 2048;  // a token sweeps at most this many earlier entries itself

// Tokens per sweep chunk: whole tokens, about kSweepChunkEntries entries.
inline int sweep_chunk_tokens(int num_topk) {
    const int t = kSweepChunkEntries / num_topk;
    return t < 1 ? 1 : t;
}

// Per source: the chunk histograms, int32 [chunks][E].
static int64_t route_scratch_bytes(int num_tokens, int num_topk, int num_experts) {
    const int tpc = sweep_chunk_tokens(num_topk);
    const int64_t chunks = (num_tokens + tpc - 1) / tpc;
    return align256((chunks < 1 ? 1 : chunks) * num_experts * 4);
}

// ---------------------------------------------------------------------
// Per-chunk expert histograms for medium and large batches: workgroup c counts the
// entries of tokens [c * tpc, (c + 1) * tpc) per expert.  The send kernel then
// ranks a pair as (entries of earlier chunks naming its expert, summed from these
// rows) + (earlier entries of its own chunk, which it sweeps itself).
// ---------------------------------------------------------------------
__global__ __launch_bounds__(1024) void ll_chunk_hist_kernel(const int64_t* __restrict__ topk_idx, int n,
                                                             int entries_per_chunk, int num_experts,
                                                             int64_t scratch_stride,
                                                             uint8_t* __restrict__ scratch_base) {
    extern __shared__ int32_t hist_lds[];  // [E]
    const int c = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int64_t* my_topk = topk_idx + int64_t(b) * n;
    int32_t* out = reinterpret_cast<int32_t*>(scratch_base + int64_t(b) * scratch_stride) + int64_t(c) * num_experts;
    for (int e = tid; e < num_experts; e += blockDim.x) hist_lds[e] = 0;
    lds_barrier();
    const int begin = c * entries_per_chunk;
    const int end = begin + entries_per_chunk < n ? begin + entries_per_chunk : n;
    for (int i = begin + tid; i < end; i += blockDim.x) {
        const int64_t v = my_topk[i];
        if (v >= 0 && v < num_experts) atomicAdd(&hist_lds[int(v)], 1);
    }
    lds_barrier();
    for (int e = tid; e < num_experts; e += blockDim.x) out[e] = hist_lds[e];
}

// Writes the per-expert totals where the receivers look for them.
__device__ __forceinline__ void emit_expert_count(int e, int total, int num_experts, int num_ranks, int rank,
                                                  int src_rank, int max_tokens, int32_t* recv_count,
                                                  int32_t* send_count) {
    const int cnt = total < max_tokens ? total : max_tokens;
    const int experts_per_rank = num_experts / num_ranks;
    if (send_count != nullptr) send_count[e] = cnt;
    if (e / experts_per_rank == rank) recv_count[(e % experts_per_rank) * num_ranks + src_rank] = cnt;
}

// ---------------------------------------------------------------------
// Fused quantise + pack.  A workgroup owns one token (of one source); each of
// its waves owns one (1 KiB output piece, share of the K selections).
// FP8 formats: the piece is 8 scale groups (1024 channels, 2 KiB of bf16 in);
// each 8-lane cluster owns a group, each lane 16 channels.  The quantised
// 16 bytes stay in registers and are stored once per selection — the row is
// read and quantised once however many experts it goes to
// (reference idea: csrc/kernels/coop_dispatch_send.cuh:572-607).
//
// Per-selection bookkeeping (slot, destination row address, row tail,
// pair_slot) is done once per token by lanes 0..K-1 of wave 0 and handed to the
// other waves through LDS; each wave reads all K destinations with one LDS
// access and takes them back per selection with readlane.  Quantisation runs
// while wave 0 does that.  Barriers fence LDS only, so the row loads stay in
// flight across them.
//
// The slot of a selection is the number of earlier (token,k) entries naming its
// expert (reference: the serial scan of csrc/kernels/efa_kernels.cu:617-637 and
// token_offset / expert_offsets of csrc/kernels/coop_dispatch_send.cuh:360-420).
// The workgroup counts them itself: while the row loads are in flight every
// thread fetches up to four entries that precede the token (more in a loop);
// each wave counts, per selection, its entries naming that selection's expert
// with a ballot and a popcount, and wave 0 adds the waves' counts.  Up to 8192
// entries the sweep covers every earlier entry; beyond, it covers the token's
// own chunk of about 2048 entries and the chunks before it come from the
// histograms of ll_chunk_hist_kernel.  The per-expert totals come from one extra
// workgroup per source.  Deterministic: integer adds and ballots only.
// ---------------------------------------------------------------------
constexpr int kMaxTopk = 64;
constexpr int kFusedMaxEntries = 8192;     // send + receive in one launch up to here
constexpr int kSelfRankMaxEntries = 8192;  // the send kernel ranks its own slots, unaided, up to here
constexpr int kSendMaxWaves = 16;

struct ByDestTables {
    int32_t* expert_prefix;  // [E + 1]
    int32_t* rank_counts;    // [R]
    int64_t* rank_cumsum;    // [R + 1]
};

struct SendArgs {
    const uint8_t* x;
    const int64_t* topk_idx;
    const int32_t* src_ranks;  // null: the rows are this rank's own
    int num_tokens, hidden, num_topk, num_experts, num_ranks, rank, max_tokens;
    int pieces_per_row, split_log2;
    uint32_t rank_of_expert_magic;
    int tokens_per_chunk;  // > 0: scratch holds the per-chunk expert histograms of ll_chunk_hist_kernel
    int64_t scratch_stride;
    const uint8_t* scratch_base;
    uint8_t* recv_staging;
    uint8_t* send_slots;
    int32_t* pair_slot;
    int32_t* recv_count;
    int32_t* send_count;
    // By-destination form: send_slots is one buffer of rows, contiguous per destination rank, and every
    // row (the rank's own included) goes to row expert_prefix[expert] + slot of it.  Null: per-expert slots.
    const int32_t* expert_prefix;
    // Small by-destination batches: no launch builds the tables first.  Every token's workgroup counts
    // the batch's entries per expert itself and scans them in LDS (a few barriers beside its row loads,
    // cheaper than a launch), and the counting row writes the tables out.
    int prefix_in_block;
    ByDestTables by_dest;
};

// Final destination of the rows a rank sends to its own experts, used by the
// one-call dispatch (as one launch or two): they skip the staging area and land
// in the packed tensors behind the rows of the lower source ranks, which is where
// the reference's ascending-source ranges put them.
struct DirectOut {
    uint8_t* packed_x;  // null: stage own rows like everyone else's
    uint8_t* packed_scales;
    int32_t* src_info;
};

struct alignas(16) SendLds {
    int32_t wave_count[kMaxTopk][kSendMaxWaves];  // [k][wave]: the wave's earlier entries naming selection k's expert
    uint64_t sel_row[kMaxTopk];                   // where selection k's payload goes (0: nowhere)
    uint64_t sel_scale[kMaxTopk];                 // where its scales go
};

// hist[e] (LDS, [E + 1]) = entries of topk_idx[0 .. n) naming expert e, clamped to max_tokens, then their
// exclusive prefix over the experts with the total in hist[E]; the whole workgroup takes part.
// counts_out (may be null): the clamped counts.
__device__ __forceinline__ void expert_prefix_in_lds(const int64_t* __restrict__ topk_idx, int n, int num_experts,
                                                     int max_tokens, int32_t* hist, int32_t* wave_totals,
                                                     int32_t* counts_out) {
    const int tid = threadIdx.x, threads = blockDim.x;
    for (int e = tid; e < num_experts; e += threads) hist[e] = 0;
    lds_barrier();
    for (int base = 0; base < n; base += 4 * threads) {  // four loads in flight per thread
        int64_t v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = base + u * threads + tid;
            v[u] = i < n ? topk_idx[i] : -1;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (v[u] >= 0 && v[u] < num_experts) atomicAdd(&hist[int(v[u])], 1);
    }
    lds_barrier();
    for (int e = tid; e < num_experts; e += threads) {
        const int c = hist[e] < max_tokens ? hist[e] : max_tokens;
        hist[e] = c;
        if (counts_out != nullptr) counts_out[e] = c;
    }
    lds_barrier();
    block_exclusive_scan(hist, num_experts, wave_totals);
}

// The per-rank tables of the by-destination form from the prefix in LDS.
__device__ __forceinline__ void by_dest_tables_out(const int32_t* hist, int num_experts, int num_ranks,
                                                   const ByDestTables& out) {
    const int tid = threadIdx.x, threads = blockDim.x;
    for (int e = tid; e <= num_experts; e += threads) out.expert_prefix[e] = hist[e];
    const int experts_per_rank = num_experts / num_ranks;
    for (int r = tid; r < num_ranks; r += threads) {
        out.rank_counts[r] = hist[(r + 1) * experts_per_rank] - hist[r * experts_per_rank];
        out.rank_cumsum[r] = hist[r * experts_per_rank];
    }
    if (tid == 0) out.rank_cumsum[num_ranks] = hist[num_experts];
}

// The per-source counting workgroup.
__device__ __forceinline__ void send_count_block(const SendArgs& a, int b, int32_t* lds_hist) {
    const int tid = threadIdx.x;
    const int n = a.num_tokens * a.num_topk;
    const int src_rank = a.src_ranks != nullptr ? a.src_ranks[b] : a.rank;
    const int64_t* my_topk = a.topk_idx + int64_t(b) * n;
    if (a.tokens_per_chunk > 0) {  // the totals are the column sums of the chunk histograms
        const int32_t* hist = reinterpret_cast<const int32_t*>(a.scratch_base + int64_t(b) * a.scratch_stride);
        const int chunks = (a.num_tokens + a.tokens_per_chunk - 1) / a.tokens_per_chunk;
        for (int e = tid; e < a.num_experts; e += blockDim.x) {
            int total = 0;
            for (int c = 0; c < chunks; ++c) total += hist[int64_t(c) * a.num_experts + e];
            emit_expert_count(e, total, a.num_experts, a.num_ranks, a.rank, src_rank, a.max_tokens, a.recv_count,
                              a.send_count);
        }
        return;
    }
    for (int j = tid; j < a.num_experts; j += blockDim.x) lds_hist[j] = 0;
    lds_barrier();
    for (int i = tid; i < n; i += blockDim.x) {
        const int64_t v = my_topk[i];
        if (v >= 0 && v < a.num_experts) atomicAdd(&lds_hist[int(v)], 1);
    }
    lds_barrier();
    for (int e = tid; e < a.num_experts; e += blockDim.x)
        emit_expert_count(e, lds_hist[e], a.num_experts, a.num_ranks, a.rank, src_rank, a.max_tokens, a.recv_count,
                          a.send_count);
}

// One workgroup's share of token t of source b.  kStream (64 MB of traffic and more): the payload of
// the rows is stored with the non-temporal hint; at 4096 tokens, with the
// destinations in HBM, that takes the send from 73 to 53 us (a row stored the ordinary way is first
// allocated in the memory-side cache and written back later).  The token rows are read, and the
// scales and tails stored, the ordinary way: the hint measured slower on those (63 and 56 us).
template <int kFmt, bool kStream>
__device__ __forceinline__ void send_token_block(const SendArgs& a, const DirectOut& direct, int b, int t,
                                                 int block_in_token, SendLds& lds, int32_t* lds_hist,
                                                 int32_t* lds_wave_totals) {
    const int lane = lane_id(), tid = threadIdx.x;
    const int num_topk = a.num_topk, num_experts = a.num_experts;
    const int n = a.num_tokens * num_topk;
    const int src_rank = a.src_ranks != nullptr ? a.src_ranks[b] : a.rank;
    const int64_t* my_topk = a.topk_idx + int64_t(b) * n;

    const int item = block_in_token * int(blockDim.x >> 6) + wave_in_block();
    const int split = 1 << a.split_log2;
    const bool wave_live = item < (a.pieces_per_row << a.split_log2);
    const int part = item & (split - 1);
    const int piece = item >> a.split_log2;
    const int64_t row_id = int64_t(b) * a.num_tokens + t;
    const int entry0 = t * num_topk;

    const int64_t data_bytes = row_data_bytes(a.hidden, kFmt);
    const int64_t data_pad = align16(data_bytes);
    const int64_t scale_bytes = row_scale_bytes(a.hidden, kFmt);
    const int64_t scale_pad = align16(scale_bytes);
    const int64_t stride = row_stride_bytes(a.hidden, kFmt);

    DEEPEP_PHASE(0);
    // ---- issue this wave's row loads ------------------------------------
    u32x4 lo = {0u, 0u, 0u, 0u}, hi = {0u, 0u, 0u, 0u};
    bool lane_live;
    int group = 0;
    if constexpr (kFmt == kRowBF16) {
        const int64_t off = int64_t(piece) * 1024 + lane * 16;
        lane_live = wave_live && off < data_bytes;
        if (lane_live) lo = load_u32x4<false>(a.x + row_id * data_bytes + off);
    } else {
        group = piece * 8 + (lane >> 3);
        lane_live = wave_live && group < a.hidden / kGroup;
        if (lane_live) {
            const uint8_t* src = a.x + (row_id * a.hidden + int64_t(group) * kGroup + (lane & 7) * 16) * 2;
            lo = load_u32x4<false>(src);
            hi = load_u32x4<false>(src + 16);
        }
    }

    // ---- every index load of the ranking, issued before anything waits -----
    // The loads are unconditional (an index that is not wanted is clamped to one that exists and its
    // value dropped): without branches around them the compiler can count them, so the first wait of
    // wave 0 -- for the token's own selections -- does not also wait out a second round trip for the
    // entries it sweeps.  The wave then has one memory round trip in front of its ballots, not two.
    const int chunk = a.tokens_per_chunk > 0 ? t / a.tokens_per_chunk : 0;
    const int sweep_begin = chunk * a.tokens_per_chunk * num_topk;
    constexpr int kSweepAhead = 4;
    const int64_t own_v = my_topk[entry0 + (tid < num_topk ? tid : num_topk - 1)];     // threads 0..K-1: selection tid
    const int64_t sel_v = my_topk[entry0 + (lane < num_topk ? lane : num_topk - 1)];   // lane k of every wave: selection k
    int64_t ahead_v[kSweepAhead];
#pragma unroll
    for (int r = 0; r < kSweepAhead; ++r) {
        const int i = sweep_begin + tid + r * int(blockDim.x);
        ahead_v[r] = my_topk[i < entry0 ? i : entry0];
    }

    // ---- per-selection bookkeeping, once per token --------------------------
    int my_expert = -1, my_slot = -1, dst_rank = -1, local = 0;  // threads 0..K-1: selection k = tid
    int direct_begin = 0;
    if (tid < num_topk) {
        const int64_t v = own_v;
        if (v >= 0 && v < num_experts) {
            my_expert = int(v);
            // my_expert / E_l by multiply-high; magic 0 stands for E_l == 1
            dst_rank = a.rank_of_expert_magic != 0 ? int(__umulhi(uint32_t(my_expert), a.rank_of_expert_magic))
                                                   : my_expert;
            local = my_expert - dst_rank * (num_experts / a.num_ranks);
        }
    }
    int dest_first = 0;  // by-destination form: where the expert's run of rows begins in the send buffer
    if (a.prefix_in_block) {
        expert_prefix_in_lds(my_topk, n, num_experts, a.max_tokens, lds_hist, lds_wave_totals, nullptr);
        if (my_expert >= 0) dest_first = lds_hist[my_expert];
    } else if (a.expert_prefix != nullptr && my_expert >= 0) {
        dest_first = a.expert_prefix[my_expert];
    }
    if (direct.packed_x != nullptr && tid < kWave) {
        // Rows for this rank's own experts go straight to the packed tensors, at the place the
        // reference's range builder gives them: behind the rows of the lower source ranks
        // (csrc/kernels/efa_kernels.cu:991-1010).  For each such selection wave 0 adds up those
        // ranks' counts of the expert.
        uint64_t to_own = __ballot(my_expert >= 0 && dst_rank == a.rank);
        while (to_own != 0) {
            const int k = __builtin_ctzll(to_own);
            to_own &= to_own - 1;
            const int le = __builtin_amdgcn_readlane(local, k);
            int part = 0;
            for (int s = lane; s < a.rank; s += kWave) {
                const int c = a.recv_count[le * a.num_ranks + s];
                part += c < 0 ? 0 : (c > a.max_tokens ? a.max_tokens : c);
            }
            const int sum = __builtin_amdgcn_readlane(wave_inclusive_sum(part), kWave - 1);
            if (lane == k) direct_begin = sum;
        }
    }
    // Medium and large batches: the token sweeps only the earlier entries of its own chunk; what the
    // chunks before it hold of each selection's expert comes from their histograms.
    int chunk_base = 0;
    if (chunk > 0 && tid < num_topk && my_expert >= 0) {
        const int32_t* hist = reinterpret_cast<const int32_t*>(a.scratch_base + int64_t(b) * a.scratch_stride);
        for (int c0 = 0; c0 < chunk; c0 += 8) {  // eight loads in flight
            int c[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) c[u] = c0 + u < chunk ? hist[int64_t(c0 + u) * num_experts + my_expert] : 0;
#pragma unroll
            for (int u = 0; u < 8; ++u) chunk_base += c[u];
        }
    }
    DEEPEP_PHASE(1);
    u32x4 payload = lo;  // quantised below, while the workgroup's bookkeeping is in flight
    uint32_t scale_bits = 0;
    // Rank the selections.  Each thread takes every blockDim-th entry between the start of the sweep
    // and this token (four fetched up front, so their latency overlaps the loads above); each wave
    // counts, per selection, how many of its entries name that selection's expert (a ballot and a
    // popcount, against the token's own entries read as wave-uniform values) and leaves the counts
    // in LDS.
    int ahead[kSweepAhead];  // -1: no entry
#pragma unroll
    for (int r = 0; r < kSweepAhead; ++r) {
        const int i = sweep_begin + tid + r * int(blockDim.x);
        const int64_t v = ahead_v[r];
        ahead[r] = i < entry0 && v >= 0 && v < num_experts ? int(v) : -1;
    }
    // lane k of every wave holds the token's selection k (-2: none, matches no entry)
    int sel = -2;
    if (lane < num_topk && sel_v >= 0 && sel_v < num_experts) sel = int(sel_v);
    const int w = wave_in_block();
    int my_count = 0;  // lane k: this wave's entries naming selection k's expert
    for (int k = 0; k < num_topk; ++k) {
        const int e = __builtin_amdgcn_readlane(sel, k);
        int count = 0;
#pragma unroll
        for (int r = 0; r < kSweepAhead; ++r) count += __popcll(__ballot(ahead[r] == e));
        if (lane == k) my_count = count;
    }
    for (int base = sweep_begin + kSweepAhead * int(blockDim.x); base < entry0;
         base += kSweepAhead * int(blockDim.x)) {
        int more[kSweepAhead];  // the same again, four loads in flight per thread
#pragma unroll
        for (int r = 0; r < kSweepAhead; ++r) {
            const int i = base + tid + r * int(blockDim.x);
            const int64_t v = i < entry0 ? my_topk[i] : -1;
            more[r] = v >= 0 && v < num_experts ? int(v) : -1;
        }
        for (int k = 0; k < num_topk; ++k) {
            const int e = __builtin_amdgcn_readlane(sel, k);
            int count = 0;
#pragma unroll
            for (int r = 0; r < kSweepAhead; ++r) count += __popcll(__ballot(more[r] == e));
            if (lane == k) my_count += count;
        }
    }
    if (lane < num_topk) lds.wave_count[lane][w] = my_count;
    if constexpr (kFmt != kRowBF16) payload = quantise_16<kFmt>(lo, hi, scale_bits);
    lds_barrier();
    DEEPEP_PHASE(3);
    if (tid < kWave) {  // wave 0: lane k finishes selection k
        const int waves = int(blockDim.x) >> 6;
        int total = 0;
        if (tid < num_topk) {  // one wide read of the row; entries of absent waves are never summed
            static_assert(kSendMaxWaves == 16, "four 16-byte LDS reads");
            u32x4 c[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) c[q] = reinterpret_cast<const u32x4*>(lds.wave_count[tid])[q];
#pragma unroll
            for (int w2 = 0; w2 < kSendMaxWaves; ++w2) total += w2 < waves ? int(c[w2 >> 2][w2 & 3]) : 0;
        }
        for (int k2 = 0; k2 < num_topk; ++k2) {  // the same expert named earlier in this token
            const int other = __builtin_amdgcn_readlane(my_expert, k2);
            if (k2 < tid && other == my_expert) total += 1;
        }
        if (tid < num_topk && my_expert >= 0) my_slot = total + chunk_base;
    }
    if (tid < num_topk) {
        if (my_slot >= a.max_tokens) my_slot = -1;
        uint8_t* row = nullptr;
        uint8_t* scale_row = nullptr;
        bool staged = false;
        if (my_slot >= 0) {
            if (a.expert_prefix != nullptr) {
                row = a.send_slots + (int64_t(dest_first) + my_slot) * stride;
                staged = true;
            } else if (dst_rank == a.rank && direct.packed_x != nullptr) {
                const int64_t out_row = int64_t(local) * a.num_ranks * a.max_tokens + direct_begin + my_slot;
                row = direct.packed_x + out_row * data_bytes;
                scale_row = direct.packed_scales + out_row * scale_bytes;
                if (block_in_token == 0) direct.src_info[out_row] = t;
            } else if (dst_rank == a.rank) {
                row = a.recv_staging + ((int64_t(local) * a.num_ranks + src_rank) * a.max_tokens + my_slot) * stride;
                staged = true;
            } else if (a.send_slots != nullptr) {
                row = a.send_slots + (int64_t(my_expert) * a.max_tokens + my_slot) * stride;
                staged = true;
            }
            if (staged) scale_row = row + data_pad;
        }
        lds.sel_row[tid] = reinterpret_cast<uint64_t>(row);
        lds.sel_scale[tid] = reinterpret_cast<uint64_t>(scale_row);
        if (block_in_token == 0) {
            if (a.pair_slot != nullptr) a.pair_slot[entry0 + tid] = my_slot;
            if (staged) {
                u32x4 tail = {uint32_t(t), uint32_t(tid), uint32_t(src_rank), uint32_t(local)};
                *reinterpret_cast<u32x4*>(row + data_pad + scale_pad) = tail;
            }
        }
    }
    lds_barrier();
    DEEPEP_PHASE(4);
    if (!wave_live) return;

    // ---- one store per selection ----------------------------------------
    const int64_t lane_off = int64_t(piece) * 1024 + lane * 16;
    DEEPEP_PHASE(5);
    // lane k reads selection k's destinations once; the loop takes them back as wave-uniform values
    uint64_t my_row = 0, my_scale_row = 0;
    if (lane < num_topk) {
        my_row = lds.sel_row[lane];
        my_scale_row = lds.sel_scale[lane];
    }
    for (int k = part; k < num_topk; k += split) {
        uint8_t* row = reinterpret_cast<uint8_t*>(
            (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_row >> 32), k))) << 32) |
            uint32_t(__builtin_amdgcn_readlane(int(uint32_t(my_row)), k)));
        if (row == nullptr) continue;
        if (lane_live) store_u32x4<kStream>(row + lane_off, payload);
        if constexpr (kFmt != kRowBF16) {
            uint8_t* scale_row = reinterpret_cast<uint8_t*>(
                (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_scale_row >> 32), k))) << 32) |
                uint32_t(__builtin_amdgcn_readlane(int(uint32_t(my_scale_row)), k)));
            if constexpr (kFmt == kRowFP8UE8M0) {
                if (lane_live && (lane & 7) == 0) store_global_byte(scale_row + group, uint8_t(scale_bits >> 23));
            } else {
                if (lane_live && (lane & 7) == 0) store_global(scale_row + int64_t(group) * 4, scale_bits);
            }
        }
    }
    DEEPEP_PHASE(6);
}

// index_rows > 0: the grid has that many rows in front of the token rows whose workgroups build the
// receive side's row index (one (local expert, source) segment each), so that a large one-call
// dispatch needs no launch for it.
template <int kFmt, bool kStream>
__global__ __launch_bounds__(kSendMaxWaves* kWave) void ll_send_kernel(SendArgs a, DirectOut direct, FusedIndexArgs index,
                                                                       int index_rows) {
    extern __shared__ int32_t lds_hist[];  // counting workgroups: [E]; index workgroups: [2 * (E + 1)]
    __shared__ SendLds lds;
    __shared__ int32_t index_wave_totals[kMaxBlockWaves];
    // Grid rows: first the index rows (started first, so that their few microseconds of scans run beside
    // the token rows instead of behind them), then one row per token, then the counting row.
    const int y = int(blockIdx.y) - index_rows;
    if (y < 0) {
        const int seg = int(blockIdx.y) * int(gridDim.x) + int(blockIdx.x);
        if (seg < index.num_local_experts * index.num_ranks) recv_index_block(index, seg, lds_hist, index_wave_totals);
        return;
    }
    if (y == a.num_tokens) {  // the counting row of the grid
        if (blockIdx.x != 0) return;
        if (a.prefix_in_block) {  // small by-destination batch: this workgroup writes the tables out
            expert_prefix_in_lds(a.topk_idx, a.num_tokens * a.num_topk, a.num_experts, a.max_tokens, lds_hist,
                                 index_wave_totals, a.send_count);
            by_dest_tables_out(lds_hist, a.num_experts, a.num_ranks, a.by_dest);
        } else if (a.expert_prefix == nullptr) {
            send_count_block(a, blockIdx.z, lds_hist);
        }  // else: ll_by_dest_prefix_kernel ran first
        return;
    }
    send_token_block<kFmt, kStream>(a, direct, blockIdx.z, y, blockIdx.x, lds, lds_hist, index_wave_totals);
}

// ---------------------------------------------------------------------
// Receive side.  Every copying wave rebuilds the segment prefix from the E
// counts (a few hundred ints) in its registers, then walks the flat row index
// space: row -> (segment, j) by ballot, one wave per row part.
// Ranges are the reference's: inside an expert's packed range the source ranks
// come in ascending order, begin(e, s) = sum of cnt(e, s') over s' < s
// (csrc/kernels/efa_kernels.cu:991-1010, :1031-1050); the slot order inside a
// segment is fixed by the staging order, not by atomics (:1059-1213 is the
// reference's deterministic scatter).
//
// own_rank >= 0 (one-call dispatch): the rows this rank sends to its own
// experts are not in the staging area — the send side puts them straight into
// the packed tensors, behind the rows of the lower ranks — so the copying waves
// skip the own segments and move the segments of the higher ranks up by the
// expert's own count.  With own_topk (single launch) that count is recounted
// from the rank's own indices, because the launch that reads recv_count's own
// entries is the one that writes them; without it (the send kernel has
// finished) recv_count holds it.
// ---------------------------------------------------------------------
struct RecvArgs {
    const uint8_t* recv_staging;
    const int32_t* recv_count;
    int hidden, num_local_experts, num_ranks, max_tokens, fmt, parts_log2;
    uint8_t* packed_x;
    uint8_t* packed_scales;
    int32_t* src_info;
    int64_t* layout_range;
    int32_t* packed_count;
    int32_t* stats;
};

__device__ __forceinline__ int clamp_count(int c, int max_tokens) {
    return c < 0 ? 0 : (c > max_tokens ? max_tokens : c);
}

// own_cnt[e_l] (LDS, unclamped) = rows this rank sends to its own expert e_l, counted by the whole
// workgroup in two steps so that other loads can be issued in between: `begin` issues the first index
// loads and clears the counters, `finish` counts and ends with a barrier.
constexpr int kOwnAhead = 4;  // index loads in flight per thread

struct OwnCountLoads {
    int64_t v[kOwnAhead];
};

__device__ __forceinline__ void own_row_counts_begin(const RecvArgs& a, const int64_t* own_topk, int own_entries,
                                                     int32_t* own_cnt, OwnCountLoads& loads) {
    const int tid = threadIdx.x, threads = blockDim.x;
    if (own_topk == nullptr) return;
#pragma unroll
    for (int r = 0; r < kOwnAhead; ++r) {
        const int i = tid + r * threads;
        loads.v[r] = i < own_entries ? own_topk[i] : -1;
    }
    for (int le = tid; le < a.num_local_experts; le += threads) own_cnt[le] = 0;
    lds_barrier();
}

__device__ __forceinline__ void own_row_counts_finish(const RecvArgs& a, const int64_t* own_topk, int own_entries,
                                                      int own_rank, int32_t* own_cnt, OwnCountLoads& loads) {
    const int tid = threadIdx.x, threads = blockDim.x;
    if (own_topk == nullptr) {  // the send kernel has finished: recv_count holds the own counts
        for (int le = tid; le < a.num_local_experts; le += threads)
            own_cnt[le] = a.recv_count[le * a.num_ranks + own_rank];
        lds_barrier();
        return;
    }
    const int64_t first = int64_t(own_rank) * a.num_local_experts;
    for (int base = 0; base < own_entries; base += kOwnAhead * threads) {
        int64_t next[kOwnAhead];
#pragma unroll
        for (int r = 0; r < kOwnAhead; ++r) {
            const int i = base + (kOwnAhead + r) * threads + tid;
            next[r] = i < own_entries ? own_topk[i] : -1;
        }
#pragma unroll
        for (int r = 0; r < kOwnAhead; ++r) {
            const int64_t d = loads.v[r] - first;
            if (loads.v[r] >= 0 && d >= 0 && d < a.num_local_experts) atomicAdd(&own_cnt[int(d)], 1);
            loads.v[r] = next[r];
        }
    }
    lds_barrier();
}

// One unit of the copying waves' work: a run of 16-byte vectors of one staged row.
struct RecvItem {
    const uint8_t* src;
    int le, source, slot;  // slot: the row's place among the rows copied for the expert, own rows not counted
    int v_begin, v_end;
    bool carries_tail;  // also moves the row's scales and source index
};

constexpr int kRecvDepth = 4;  // 16-byte loads in flight per lane

// Workgroups [0, num_copy_blocks) copy rows; workgroup num_copy_blocks writes layout_range,
// packed_count and stats and copies nothing.  A copying wave builds the segment prefix in its own
// registers (WaveSegments) from the E counts.  Where a row lands may depend on the own count of its
// expert, where it comes from does not: a wave issues the loads of its first item before the
// workgroup settles the own counts.
// lds: [num_segments + 1 + num_local_experts] ints; wave_totals: 16 ints.
template <int kPer, bool kStream>
__device__ __forceinline__ void recv_rows_impl(const RecvArgs& a, int block, int num_copy_blocks,
                                               const int64_t* own_topk, int own_entries, int own_rank, int32_t* lds,
                                               int32_t* wave_totals) {
    const int tid = threadIdx.x, lane = lane_id(), w = wave_in_block();
    const int threads = blockDim.x, waves = threads >> 6;
    const int num_ranks = a.num_ranks, max_tokens = a.max_tokens;
    const int num_segments = a.num_local_experts * num_ranks;
    const bool own_placed = own_rank >= 0;
    OwnCountLoads own_loads;

    if (block == num_copy_blocks) {  // the metadata workgroup
        int32_t* own_cnt = lds + num_segments + 1;
        if (own_placed) {
            own_row_counts_begin(a, own_topk, own_entries, own_cnt, own_loads);
            own_row_counts_finish(a, own_topk, own_entries, own_rank, own_cnt, own_loads);
        }
        for (int s = tid; s < num_segments; s += threads) {
            const int le = s / num_ranks;
            const bool own = own_placed && s - le * num_ranks == own_rank;
            lds[s] = clamp_count(own ? own_cnt[le] : a.recv_count[s], max_tokens);
        }
        lds_barrier();
        block_exclusive_scan(lds, num_segments, wave_totals);
        for (int s = tid; s < num_segments; s += threads) {
            const int le = s / num_ranks;
            const int64_t cnt = lds[s + 1] - lds[s];
            const int64_t begin = lds[s] - lds[le * num_ranks];
            a.layout_range[s] = cnt > 0 ? ((begin << 32) | cnt) : 0;
        }
        for (int le = tid; le < a.num_local_experts; le += threads) {
            const int c = lds[(le + 1) * num_ranks] - lds[le * num_ranks];
            a.packed_count[le] = c;
            if (a.stats != nullptr) a.stats[le] += c;
        }
        return;
    }

    int32_t* own_cnt = lds;  // [E_l]
    WaveSegments<kPer> seg_table;
    DEEPEP_PHASE(0);
    if (own_placed) own_row_counts_begin(a, own_topk, own_entries, own_cnt, own_loads);
    wave_load_int32<kPer>(a.recv_count, num_segments, lane, seg_table.cnt);
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
        seg_table.aux[u] = 0;
        seg_table.cnt[u] = clamp_count(seg_table.cnt[u], max_tokens);
    }
    if (own_placed) {  // the own segments (le * R + own_rank) hold nothing to copy
        int source = (lane * kPer) % num_ranks;  // source rank of this lane's first segment
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            if (source == own_rank) seg_table.cnt[u] = 0;
            source = source + 1 == num_ranks ? 0 : source + 1;
        }
    }
    wave_segments_finish(seg_table);
    DEEPEP_PHASE(1);

    const int64_t data_bytes = row_data_bytes(a.hidden, a.fmt);
    const int64_t data_pad = align16(data_bytes);
    const int64_t scale_bytes = row_scale_bytes(a.hidden, a.fmt);
    const int64_t stride = row_stride_bytes(a.hidden, a.fmt);
    const int64_t slots_per_expert = int64_t(max_tokens) * num_ranks;
    const int waves_total = num_copy_blocks * waves;
    const int num_vec = int(data_bytes / 16);
    const int parts = 1 << a.parts_log2;
    const int num_items = seg_table.total << a.parts_log2;

    auto decode = [&](int item, RecvItem& it) {
        const int row = item >> a.parts_log2, part = item & (parts - 1);
        int seg_first, unused;
        const int seg = wave_segments_find(seg_table, row, seg_first, unused);
        it.le = seg / num_ranks;
        it.source = seg - it.le * num_ranks;
        it.slot = row - wave_segments_prefix(seg_table, it.le * num_ranks);
        it.src = a.recv_staging + (int64_t(seg) * max_tokens + (row - seg_first)) * stride;
        row_part_range(num_vec, parts, part, it.v_begin, it.v_end);
        it.carries_tail = part == parts - 1;  // the last part is the shortest
    };
    // What the tail-carrying part of a row moves besides payload: one scale word per lane (the first 64;
    // a wider row's remainder is copied after the stores) and, in lane 0, the source index.  They are
    // loaded with the payload, not behind its stores: one round trip per row instead of two.
    const int scale_dwords = int(scale_bytes / 4);
    const bool has_scales = a.packed_scales != nullptr && scale_dwords > 0;
    uint32_t tail_scale = 0;
    int32_t tail_info = 0;
    auto load_first = [&](const RecvItem& it, u32x4 (&r)[kRecvDepth]) {
#pragma unroll
        for (int u = 0; u < kRecvDepth; ++u) {
            const int v = it.v_begin + u * kWave + lane;
            if (v < it.v_end) r[u] = load_u32x4<kStream>(it.src + int64_t(v) * 16);
        }
        if (it.carries_tail) {
            if (has_scales && lane < scale_dwords) tail_scale = reinterpret_cast<const uint32_t*>(it.src + data_pad)[lane];
            if (lane == 0) tail_info = *reinterpret_cast<const int32_t*>(it.src + data_pad + align16(scale_bytes));
        }
    };
    auto finish = [&](const RecvItem& it, const u32x4 (&r)[kRecvDepth]) {
        int slot = it.slot;
        if (own_placed && it.source > own_rank) slot += clamp_count(own_cnt[it.le], max_tokens);
        const int64_t out_row = int64_t(it.le) * slots_per_expert + slot;
        uint8_t* dst = a.packed_x + out_row * data_bytes;
#pragma unroll
        for (int u = 0; u < kRecvDepth; ++u) {
            const int v = it.v_begin + u * kWave + lane;
            if (v < it.v_end) store_u32x4<kStream>(dst + int64_t(v) * 16, r[u]);
        }
        wave_copy_vec16<kRecvDepth, kStream>(it.src, dst, it.v_begin + kRecvDepth * kWave, it.v_end, lane);
        if (!it.carries_tail) return;
        if (has_scales) {
            const uint32_t* s32 = reinterpret_cast<const uint32_t*>(it.src + data_pad);
            uint32_t* d32 = reinterpret_cast<uint32_t*>(a.packed_scales + out_row * scale_bytes);
            if (lane < scale_dwords) d32[lane] = tail_scale;
            for (int v = kWave + lane; v < scale_dwords; v += kWave) d32[v] = s32[v];
        }
        if (lane == 0) a.src_info[out_row] = tail_info;
    };

    RecvItem it;
    u32x4 r[kRecvDepth];
    int item = block * waves + w;
    const bool have_first = item < num_items;
    if (have_first) {
        decode(item, it);
        DEEPEP_PHASE(2);
        load_first(it, r);
    }
    // every wave of the workgroup passes here, with or without rows to copy
    if (own_placed) own_row_counts_finish(a, own_topk, own_entries, own_rank, own_cnt, own_loads);
    if (have_first) {
        finish(it, r);
        DEEPEP_PHASE(3);
        item += waves_total;
    }
    for (; item < num_items; item += waves_total) {
        decode(item, it);
        load_first(it, r);
        finish(it, r);
    }
}

template <bool kStream>
__device__ __forceinline__ void recv_rows(const RecvArgs& a, int block, int num_copy_blocks, const int64_t* own_topk,
                                          int own_entries, int own_rank, int32_t* lds, int32_t* wave_totals) {
    if (a.num_local_experts * a.num_ranks <= 4 * kWave)
        recv_rows_impl<4, kStream>(a, block, num_copy_blocks, own_topk, own_entries, own_rank, lds, wave_totals);
    else
        recv_rows_impl<16, kStream>(a, block, num_copy_blocks, own_topk, own_entries, own_rank, lds, wave_totals);
}

// own_rank >= 0: the send side has already put this rank's own rows at their packed position.
__global__ __launch_bounds__(256) void ll_recv_kernel(RecvArgs a, const int64_t* own_topk, int own_entries,
                                                      int own_rank) {
    extern __shared__ int32_t flat[];  // [num_segments + 1 + E_l]
    __shared__ int32_t wave_totals[kMaxBlockWaves];
    recv_rows<false>(a, blockIdx.x, int(gridDim.x) - 1, own_topk, own_entries, own_rank, flat, wave_totals);
}

// ---------------------------------------------------------------------
// Single-launch dispatch for small batches (T*K <= 8192, at most 8192 expected rows): the send
// workgroups, the counting workgroup and the receive workgroups of the two
// kernels above in one grid.  No workgroup waits on another: the receive
// workgroups copy only the peers' rows (already in the staging area when the
// launch starts); the send workgroups place the rank's rows for its own
// experts at their final packed position, which they find from the lower
// ranks' counts, and the receive workgroups make room for them by recounting
// them from the rank's own indices.  The packed ranges are the reference's
// (ascending source rank, csrc/kernels/efa_kernels.cu:991-1010).
// (The reference's dispatch is one kernel with a send and a receive phase as
// well: csrc/kernels/coop_dispatch_send.cuh:304, coop_dispatch_recv.cuh:42.)
// ---------------------------------------------------------------------
template <int kFmt, bool kStream>
__global__ __launch_bounds__(kSendMaxWaves* kWave) void ll_dispatch_fused_kernel(SendArgs sa, RecvArgs ra, int blocks_per_token,
                                                                                 int num_send_blocks) {
    extern __shared__ int32_t dyn_lds[];  // counting: [E]; receive: [segments + 1 + E_l]
    __shared__ SendLds lds;
    __shared__ int32_t wave_totals[kMaxBlockWaves];
    const int block = blockIdx.x;
    if (block < num_send_blocks) {
        const DirectOut direct = {ra.packed_x, ra.packed_scales, ra.src_info};
        send_token_block<kFmt, kStream>(sa, direct, 0, block / blocks_per_token, block % blocks_per_token, lds, dyn_lds,
                                        wave_totals);
    } else if (block == num_send_blocks) {
        send_count_block(sa, 0, dyn_lds);
    } else {
        recv_rows<kStream>(ra, block - num_send_blocks - 1, int(gridDim.x) - num_send_blocks - 2, sa.topk_idx,
                  sa.num_tokens * sa.num_topk, sa.rank, dyn_lds, wave_totals);
    }
}

// ---------------------------------------------------------------------
// By-destination send (what an all-to-all ships: one contiguous message per
// peer).  Before the send kernel runs (batches of more than kByDestInBlockEntries entries;
// smaller ones build the same tables inside the send launch, every token's workgroup
// for itself), one workgroup turns the route counts into
// the tables the rows are placed by: send_count[e] (clamped to the M slots of a
// pair), its exclusive prefix over the experts -- the first row of every expert's
// run, experts ascending, hence destination ranks ascending -- and the per-rank
// counts and prefix the transport cuts the buffer by.
// Reference: the count + prefix phases of ll_dispatch_route_and_pack_v3
// (csrc/kernels/efa_kernels.cu:2358-2371: ll_dispatch_count_kernel, prefix_sum_kernel).
// ---------------------------------------------------------------------
__global__ __launch_bounds__(1024) void ll_by_dest_prefix_kernel(const int64_t* __restrict__ topk_idx, int n,
                                                                 int num_experts, int num_ranks, int max_tokens,
                                                                 const int32_t* __restrict__ chunk_hist, int num_chunks,
                                                                 int32_t* __restrict__ send_count, ByDestTables out) {
    extern __shared__ int32_t hist[];  // [E + 1]
    __shared__ int32_t wave_totals[kMaxBlockWaves];
    const int tid = threadIdx.x, threads = blockDim.x;
    if (chunk_hist != nullptr) {  // the column sums of the chunk histograms
        for (int e = tid; e < num_experts; e += threads) {
            int total = 0;
            for (int c0 = 0; c0 < num_chunks; c0 += 8) {  // eight loads in flight
                int v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = c0 + u < num_chunks ? chunk_hist[int64_t(c0 + u) * num_experts + e] : 0;
#pragma unroll
                for (int u = 0; u < 8; ++u) total += v[u];
            }
            hist[e] = total;
        }
    } else {
        for (int e = tid; e < num_experts; e += threads) hist[e] = 0;
        lds_barrier();
        for (int base = 0; base < n; base += 4 * threads) {  // four loads in flight per thread
            int64_t v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i = base + u * threads + tid;
                v[u] = i < n ? topk_idx[i] : -1;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (v[u] >= 0 && v[u] < num_experts) atomicAdd(&hist[int(v[u])], 1);
        }
    }
    lds_barrier();
    for (int e = tid; e < num_experts; e += threads) {
        const int c = hist[e] < max_tokens ? hist[e] : max_tokens;
        hist[e] = c;
        send_count[e] = c;
    }
    lds_barrier();
    block_exclusive_scan(hist, num_experts, wave_totals);
    by_dest_tables_out(hist, num_experts, num_ranks, out);
}

// ---------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------
static int check_ll_shape(int num_tokens, int hidden, int num_topk, int num_experts, int num_ranks, int rank,
                          int max_tokens, int row_format) {
    EP_HOST_ASSERT(num_tokens >= 0 && hidden > 0 && num_topk > 0 && num_topk <= kMaxTopk);
    EP_HOST_ASSERT(hidden % 128 == 0);
    EP_HOST_ASSERT(num_ranks > 0 && num_experts > 0 && num_experts % num_ranks == 0);
    EP_HOST_ASSERT(rank >= 0 && rank < num_ranks);
    EP_HOST_ASSERT(max_tokens > 0 && num_tokens <= max_tokens);
    EP_HOST_ASSERT(row_format >= kRowBF16 && row_format <= kRowFP8UE8M0);
    EP_HOST_ASSERT(row_format != kRowFP8UE8M0 || (hidden / 128) % 4 == 0);
    EP_HOST_ASSERT(int64_t(num_tokens) * num_topk < (int64_t(1) << 30));
    EP_HOST_ASSERT(num_experts <= 4096);
    return 0;
}

static int launch_send_side(const void* x, const int64_t* topk_idx, const int32_t* src_ranks, int num_src,
                            int num_tokens, int hidden, int num_topk, int num_experts, int num_ranks, int rank,
                            int max_tokens, int row_format, void* recv_staging, int32_t* recv_count,
                            void* send_slots, int32_t* send_count, int32_t* pair_slot, void* workspace,
                            size_t workspace_bytes, hipStream_t stream, const RecvArgs* fused_recv = nullptr,
                            int64_t fused_recv_wave_items = 0, const DirectOut* own_rows_direct = nullptr,
                            const ByDestTables* by_dest = nullptr, FusedIndexArgs* fused_index = nullptr,
                            bool* index_was_fused = nullptr) {
    const int64_t scratch_bytes = route_scratch_bytes(num_tokens, num_topk, num_experts);
    EP_HOST_ASSERT(workspace != nullptr && workspace_bytes >= size_t(scratch_bytes) * size_t(num_src));
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(workspace) & 15) == 0);
    const int n = num_tokens * num_topk;
    uint8_t* ws = reinterpret_cast<uint8_t*>(workspace);
    // How slots get ranked: up to kSelfRankMaxEntries entries the send kernel sweeps every earlier
    // entry itself; beyond, it sweeps its own chunk on top of the per-chunk histograms.
    const int tpc = n <= kSelfRankMaxEntries || fused_recv != nullptr ? 0 : sweep_chunk_tokens(num_topk);
    if (tpc > 0) {
        const int chunks = (num_tokens + tpc - 1) / tpc;
        ll_chunk_hist_kernel<<<dim3(chunks, num_src), 1024, size_t(num_experts) * sizeof(int32_t), stream>>>(
            topk_idx, n, tpc * num_topk, num_experts, scratch_bytes, ws);
        EP_LAUNCH_CHECK();
    }
    // A small by-destination batch needs no launch for its tables: every token's workgroup counts the
    // batch itself (kByDestInBlockEntries entries are a few loads per thread).
    const bool prefix_in_block = by_dest != nullptr && tpc == 0 && n <= kByDestInBlockEntries;
    if (by_dest != nullptr && !prefix_in_block) {  // the tables the by-destination rows are placed by
        EP_HOST_ASSERT(num_src == 1 && src_ranks == nullptr && fused_recv == nullptr && own_rows_direct == nullptr);
        const int chunks = tpc > 0 ? (num_tokens + tpc - 1) / tpc : 0;
        ll_by_dest_prefix_kernel<<<1, 1024, size_t(num_experts + 1) * sizeof(int32_t), stream>>>(
            topk_idx, n, num_experts, num_ranks, max_tokens, tpc > 0 ? reinterpret_cast<const int32_t*>(ws) : nullptr,
            chunks, send_count, *by_dest);
        EP_LAUNCH_CHECK();
    }

    const int pieces = row_format == kRowBF16 ? (hidden * 2 + 1023) / 1024 : (hidden / kGroup + 7) / 8;
    // A small batch cannot fill 1024 SIMDs with one wave per row piece: give a share of the
    // K stores of each piece to a second wave.
    int split_log2 = int64_t(num_src) * num_tokens * pieces < 4096 && num_topk > 1 ? 1 : 0;
    // In the single launch the receive workgroups share the chip: whole tokens per workgroup, and
    // workgroups small enough that two fit a compute unit.
    if (fused_recv != nullptr) split_log2 = 0;
    const int items = pieces << split_log2;  // waves per token
    const int max_waves = fused_recv != nullptr ? 8 : kSendMaxWaves;
    int waves = items < max_waves ? items : max_waves;
    const int blocks_per_token = (items + waves - 1) / waves;
    if (fused_recv != nullptr && waves < 4) waves = 4;  // the receive workgroups want a few waves each
    EP_HOST_ASSERT(num_tokens < 65535 && num_src <= 65535);
    // floor(e / E_l) == umulhi(e, ceil(2^32 / E_l)) for every e below 2^16.
    const uint32_t experts_per_rank = uint32_t(num_experts / num_ranks);
    const uint32_t magic =
        experts_per_rank == 1 ? 0u : uint32_t(((uint64_t(1) << 32) + experts_per_rank - 1) / experts_per_rank);
    EP_HOST_ASSERT(num_experts < 65536);
    SendArgs sa;
    sa.x = reinterpret_cast<const uint8_t*>(x);
    sa.topk_idx = topk_idx;
    sa.src_ranks = src_ranks;
    sa.num_tokens = num_tokens, sa.hidden = hidden, sa.num_topk = num_topk, sa.num_experts = num_experts;
    sa.num_ranks = num_ranks, sa.rank = rank, sa.max_tokens = max_tokens;
    sa.pieces_per_row = pieces, sa.split_log2 = split_log2;
    sa.rank_of_expert_magic = magic;
    sa.scratch_stride = scratch_bytes, sa.scratch_base = ws;
    sa.tokens_per_chunk = tpc;
    sa.recv_staging = reinterpret_cast<uint8_t*>(recv_staging);
    sa.send_slots = reinterpret_cast<uint8_t*>(send_slots);
    sa.pair_slot = pair_slot, sa.recv_count = recv_count, sa.send_count = send_count;
    sa.expert_prefix = by_dest != nullptr ? by_dest->expert_prefix : nullptr;
    sa.prefix_in_block = prefix_in_block ? 1 : 0;
    sa.by_dest = by_dest != nullptr ? *by_dest : ByDestTables{nullptr, nullptr, nullptr};
    if (by_dest != nullptr)
        EP_HOST_ASSERT(num_src == 1 && src_ranks == nullptr && fused_recv == nullptr && own_rows_direct == nullptr);

    if (fused_recv != nullptr) {  // single launch: send workgroups, the counting workgroup, receive workgroups
        EP_HOST_ASSERT(tpc == 0 && num_src == 1 && src_ranks == nullptr);
        const int num_send_blocks = blocks_per_token * num_tokens;
        int64_t fused_recv_blocks = (fused_recv_wave_items + waves - 1) / waves;
        fused_recv_blocks = fused_recv_blocks < 1 ? 1 : (fused_recv_blocks > 1024 ? 1024 : fused_recv_blocks);
        const int64_t total = int64_t(num_send_blocks) + 1 + fused_recv_blocks + 1;  // + counting, + metadata
        EP_HOST_ASSERT(total < (int64_t(1) << 31));
        const int num_segments = fused_recv->num_local_experts * fused_recv->num_ranks;
        const size_t need_recv = size_t(num_segments + 1 + fused_recv->num_local_experts) * sizeof(int32_t);
        const size_t need_count = size_t(num_experts) * sizeof(int32_t);
        const size_t lds = need_recv > need_count ? need_recv : need_count;
        const RecvArgs ra = *fused_recv;
        // Token rows read and K copies written by the send workgroups, staged rows read and packed rows
        // written by the receive workgroups.  From 64 MB on (about 350 tokens at hidden 7168, top-8) the
        // launch streams: at 512 to 1024 tokens that changes nothing when the caches are clean and takes
        // 11 to 16 % off when they are full of another call's dirty lines (44 against 50 us at 1024 tokens).
        const int64_t payload = row_payload_bytes(hidden, row_format);
        const int64_t fused_traffic = int64_t(num_tokens) * (int64_t(hidden) * 2 + int64_t(num_topk) * payload) +
                                      2 * (fused_recv_wave_items >> ra.parts_log2) * payload;
        const bool fused_streams = fused_traffic > send_stream_bytes();
#define DEEPEP_LAUNCH_FUSED(FMT)                                                                        \
    do {                                                                                                \
        if (fused_streams)                                                                              \
            ll_dispatch_fused_kernel<FMT, true><<<dim3(unsigned(total)), waves * kWave, lds, stream>>>(sa, ra, blocks_per_token, num_send_blocks); \
        else                                                                                            \
            ll_dispatch_fused_kernel<FMT, false><<<dim3(unsigned(total)), waves * kWave, lds, stream>>>(sa, ra, blocks_per_token, num_send_blocks); \
    } while (0)
        switch (row_format) {
            case kRowBF16: DEEPEP_LAUNCH_FUSED(kRowBF16); break;
            case kRowFP8: DEEPEP_LAUNCH_FUSED(kRowFP8); break;
            case kRowFP8Pow2: DEEPEP_LAUNCH_FUSED(kRowFP8Pow2); break;
            default: DEEPEP_LAUNCH_FUSED(kRowFP8UE8M0); break;
        }
#undef DEEPEP_LAUNCH_FUSED
        EP_LAUNCH_CHECK();
        return 0;
    }

    // The receive index rides along when the chunk histograms exist (its own counts come from them)
    FusedIndexArgs index = {};
    int index_rows = 0;
    if (fused_index != nullptr && tpc > 0 && num_src == 1 && own_rows_direct != nullptr) {
        index = *fused_index;
        index.chunk_hist = reinterpret_cast<const int32_t*>(ws);
        index.num_chunks = (num_tokens + tpc - 1) / tpc;
        index_rows = (num_experts + blocks_per_token - 1) / blocks_per_token;
        if (num_tokens + 1 + index_rows > 65535) index_rows = 0, index = FusedIndexArgs{};
    }
    if (index_was_fused != nullptr) *index_was_fused = index_rows > 0;
    const dim3 grid(blocks_per_token, num_tokens + 1 + index_rows, num_src);  // + the counting row, + the index rows
    const size_t lds = size_t(index_rows > 0 ? 2 * (num_experts + 1) : num_experts + 1) * sizeof(int32_t);
    // own_rows_direct (the two-launch form of the one-call dispatch): as in the single launch, the rows
    // for this rank's own experts go straight to their packed position behind the lower ranks' rows
    EP_HOST_ASSERT(own_rows_direct == nullptr || (num_src == 1 && src_ranks == nullptr));
    const DirectOut direct = own_rows_direct != nullptr ? *own_rows_direct : DirectOut{nullptr, nullptr, nullptr};
    // rows read once and written K times (about that many: a dropped selection writes nothing)
    const int64_t traffic = int64_t(num_src) * num_tokens *
                            (int64_t(hidden) * 2 + int64_t(num_topk) * row_payload_bytes(hidden, row_format));
    const bool streams = traffic > send_stream_bytes();
#define DEEPEP_LAUNCH_SEND(FMT)                                                           \
    do {                                                                                  \
        if (streams) ll_send_kernel<FMT, true><<<grid, waves * kWave, lds, stream>>>(sa, direct, index, index_rows);  \
        else ll_send_kernel<FMT, false><<<grid, waves * kWave, lds, stream>>>(sa, direct, index, index_rows);         \
    } while (0)
    switch (row_format) {
        case kRowBF16: DEEPEP_LAUNCH_SEND(kRowBF16); break;
        case kRowFP8: DEEPEP_LAUNCH_SEND(kRowFP8); break;
        case kRowFP8Pow2: DEEPEP_LAUNCH_SEND(kRowFP8Pow2); break;
        default: DEEPEP_LAUNCH_SEND(kRowFP8UE8M0); break;
    }
#undef DEEPEP_LAUNCH_SEND
    EP_LAUNCH_CHECK();
    return 0;
}

}  // namespace deepep

using namespace deepep;

extern "C" {

size_t deepep_ll_row_data_bytes(int hidden, int row_format) { return size_t(row_data_bytes(hidden, row_format)); }
size_t deepep_ll_row_scale_bytes(int hidden, int row_format) { return size_t(row_scale_bytes(hidden, row_format)); }
size_t deepep_ll_row_stride(int hidden, int row_format) { return size_t(row_stride_bytes(hidden, row_format)); }
size_t deepep_ll_row_payload_bytes(int hidden, int row_format) { return size_t(row_payload_bytes(hidden, row_format)); }

size_t deepep_ll_segment_workspace_bytes(int num_experts, int num_max_dispatch_tokens_per_rank) {
    return size_t(segment_workspace_bytes(num_experts, num_max_dispatch_tokens_per_rank));
}

size_t deepep_ll_dispatch_workspace_bytes(int num_tokens, int num_topk, int num_experts) {
    return size_t(route_scratch_bytes(num_tokens, num_topk, num_experts));
}

int deepep_ll_dispatch_send(const void* x, const int64_t* topk_idx, int num_tokens, int hidden, int num_topk,
                            int num_experts, int num_ranks, int rank, int num_max_dispatch_tokens_per_rank,
                            int row_format, void* recv_staging, int32_t* recv_count, void* send_slots,
                            int32_t* send_count, int32_t* pair_slot, void* workspace, size_t workspace_bytes,
                            void* stream) {
    clear_error();
    if (int rc = check_ll_shape(num_tokens, hidden, num_topk, num_experts, num_ranks, rank,
                                num_max_dispatch_tokens_per_rank, row_format))
        return rc;
    EP_HOST_ASSERT(num_tokens == 0 || (x != nullptr && topk_idx != nullptr));
    EP_HOST_ASSERT(recv_staging != nullptr && recv_count != nullptr);
    EP_HOST_ASSERT(send_count != nullptr && pair_slot != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(recv_staging) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(send_slots) & 15) == 0);
    return launch_send_side(x, topk_idx, nullptr, 1, num_tokens, hidden, num_topk, num_experts, num_ranks, rank,
                            num_max_dispatch_tokens_per_rank, row_format, recv_staging, recv_count, send_slots,
                            send_count, pair_slot, workspace, workspace_bytes,
                            reinterpret_cast<hipStream_t>(stream));
}

// Device address of `scratch` on the GPU that `stream` runs on, looked up once per device.
static int static_route_scratch(hipStream_t stream, void** out) {
    constexpr int kMaxDevices = 64;
    static std::mutex mutex;
    static void* address[kMaxDevices] = {};
    int device = -1;
    EP_HIP_CHECK(hipGetDevice(&device));
    EP_HOST_ASSERT(device >= 0 && device < kMaxDevices);
    if (stream != nullptr) {  // the symbol's address is per device: the stream must be the current device's
        int stream_device = -1;
        EP_HIP_CHECK(hipStreamGetDevice(stream, &stream_device));
        EP_HOST_ASSERT(stream_device == device);
    }
    std::lock_guard<std::mutex> lock(mutex);
    if (address[device] == nullptr) {
        void* p = nullptr;
        EP_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        EP_HOST_ASSERT(p != nullptr);
        address[device] = p;
    }
    *out = address[device];
    return 0;
}

int deepep_ll_dispatch_send_static(const void* x, const int64_t* topk_idx, int num_tokens, int hidden, int num_topk,
                                   int num_experts, int num_ranks, int rank, int num_max_dispatch_tokens_per_rank,
                                   int row_format, void* recv_staging, int32_t* recv_count, void* send_slots,
                                   int32_t* send_count, int32_t* pair_slot, void* stream) {
    clear_error();
    if (int rc = check_ll_shape(num_tokens, hidden, num_topk, num_experts, num_ranks, rank,
                                num_max_dispatch_tokens_per_rank, row_format))
        return rc;
    const size_t need = size_t(route_scratch_bytes(num_tokens, num_topk, num_experts));
    if (need > kStaticScratchBytes) {
        set_error("Assertion", __FILE_NAME__, __LINE__,
                  "batch too large for the static route scratch: ceil(num_tokens / floor(2048 / num_topk)) * "
                  "num_experts * 4 bytes must not exceed 1 MiB; use deepep_ll_dispatch_send with a workspace");
        return 1;
    }
    void* route_scratch = nullptr;
    if (int rc = static_route_scratch(reinterpret_cast<hipStream_t>(stream), &route_scratch)) return rc;
    EP_HOST_ASSERT(num_tokens == 0 || (x != nullptr && topk_idx != nullptr));
    EP_HOST_ASSERT(recv_staging != nullptr && recv_count != nullptr);
    EP_HOST_ASSERT(send_count != nullptr && pair_slot != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(recv_staging) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(send_slots) & 15) == 0);
    return launch_send_side(x, topk_idx, nullptr, 1, num_tokens, hidden, num_topk, num_experts, num_ranks, rank,
                            num_max_dispatch_tokens_per_rank, row_format, recv_staging, recv_count, send_slots,
                            send_count, pair_slot, route_scratch, kStaticScratchBytes,
                            reinterpret_cast<hipStream_t>(stream));
}

int deepep_ll_dispatch_send_by_dest(const void* x, const int64_t* topk_idx, int num_tokens, int hidden, int num_topk,
                                    int num_experts, int num_ranks, int rank, int num_max_dispatch_tokens_per_rank,
                                    int row_format, void* send_rows, int64_t send_row_capacity, int32_t* send_count,
                                    int32_t* send_expert_prefix, int32_t* send_counts, int64_t* send_cumsum,
                                    int32_t* pair_slot, void* workspace, size_t workspace_bytes, void* stream) {
    clear_error();
    if (int rc = check_ll_shape(num_tokens, hidden, num_topk, num_experts, num_ranks, rank,
                                num_max_dispatch_tokens_per_rank, row_format))
        return rc;
    EP_HOST_ASSERT(num_tokens == 0 || (x != nullptr && topk_idx != nullptr));
    EP_HOST_ASSERT(send_count != nullptr && send_expert_prefix != nullptr && send_counts != nullptr &&
                   send_cumsum != nullptr && pair_slot != nullptr);
    // every live pair sends one row, and an expert takes at most M of them
    const int64_t most_rows = std::min<int64_t>(int64_t(num_tokens) * num_topk,
                                                int64_t(num_experts) * num_max_dispatch_tokens_per_rank);
    EP_HOST_ASSERT(send_row_capacity >= most_rows);
    EP_HOST_ASSERT(most_rows == 0 || send_rows != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(send_rows) & 15) == 0);
    const ByDestTables tables = {send_expert_prefix, send_counts, send_cumsum};
    return launch_send_side(x, topk_idx, nullptr, 1, num_tokens, hidden, num_topk, num_experts, num_ranks, rank,
                            num_max_dispatch_tokens_per_rank, row_format, nullptr, nullptr, send_rows, send_count,
                            pair_slot, workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream), nullptr, 0,
                            nullptr, &tables);
}

int deepep_loopback_dispatch_from_peers(const void* x, const int64_t* topk_idx, const int32_t* src_ranks,
                                        int num_src, int num_tokens, int hidden, int num_topk, int num_experts,
                                        int num_ranks, int rank, int num_max_dispatch_tokens_per_rank,
                                        int row_format, void* recv_staging, int32_t* recv_count, void* workspace,
                                        size_t workspace_bytes, void* stream) {
    clear_error();
    if (int rc = check_ll_shape(num_tokens, hidden, num_topk, num_experts, num_ranks, rank,
                                num_max_dispatch_tokens_per_rank, row_format))
        return rc;
    EP_HOST_ASSERT(num_src >= 0 && num_src <= 65535);
    if (num_src == 0) return 0;
    EP_HOST_ASSERT(src_ranks != nullptr && recv_staging != nullptr && recv_count != nullptr);
    EP_HOST_ASSERT(num_tokens == 0 || (x != nullptr && topk_idx != nullptr));
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(recv_staging) & 15) == 0);
    return launch_send_side(x, topk_idx, src_ranks, num_src, num_tokens, hidden, num_topk, num_experts, num_ranks,
                            rank, num_max_dispatch_tokens_per_rank, row_format, recv_staging, recv_count, nullptr,
                            nullptr, nullptr, workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream));
}

static int check_recv_args(const void* recv_staging, const int32_t* recv_count, int hidden, int num_experts,
                           int num_ranks, int max_tokens, int row_format, void* packed_recv_x,
                           void* packed_recv_scales, int32_t* packed_recv_src_info, int64_t* packed_recv_layout_range,
                           int32_t* packed_recv_count) {
    EP_HOST_ASSERT(hidden > 0 && hidden % 128 == 0);
    EP_HOST_ASSERT(num_ranks > 0 && num_experts > 0 && num_experts % num_ranks == 0);
    EP_HOST_ASSERT(max_tokens > 0);
    EP_HOST_ASSERT(row_format >= kRowBF16 && row_format <= kRowFP8UE8M0);
    EP_HOST_ASSERT(row_format != kRowFP8UE8M0 || (hidden / 128) % 4 == 0);
    EP_HOST_ASSERT(num_experts <= 1024);
    EP_HOST_ASSERT(recv_staging != nullptr && recv_count != nullptr && packed_recv_x != nullptr);
    EP_HOST_ASSERT(row_format == kRowBF16 || packed_recv_scales != nullptr);
    EP_HOST_ASSERT(packed_recv_src_info != nullptr && packed_recv_layout_range != nullptr &&
                   packed_recv_count != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(recv_staging) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(recv_count) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(packed_recv_x) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(packed_recv_scales) & 3) == 0);
    EP_HOST_ASSERT(int64_t(num_experts) * max_tokens < (int64_t(1) << 31));
    return 0;
}

static RecvArgs make_recv_args(const void* recv_staging, const int32_t* recv_count, int hidden, int num_experts,
                               int num_ranks, int max_tokens, int row_format, void* packed_recv_x,
                               void* packed_recv_scales, int32_t* packed_recv_src_info,
                               int64_t* packed_recv_layout_range, int32_t* packed_recv_count, int32_t* stats,
                               int64_t expected_rows) {
    RecvArgs ra;
    ra.recv_staging = reinterpret_cast<const uint8_t*>(recv_staging);
    ra.recv_count = recv_count;
    ra.hidden = hidden, ra.num_local_experts = num_experts / num_ranks, ra.num_ranks = num_ranks;
    ra.max_tokens = max_tokens, ra.fmt = row_format;
    ra.parts_log2 = choose_row_parts_log2(estimated_rows(expected_rows, num_experts, max_tokens),
                                          row_data_bytes(hidden, row_format));
    ra.packed_x = reinterpret_cast<uint8_t*>(packed_recv_x);
    ra.packed_scales = reinterpret_cast<uint8_t*>(packed_recv_scales);
    ra.src_info = packed_recv_src_info, ra.layout_range = packed_recv_layout_range;
    ra.packed_count = packed_recv_count, ra.stats = stats;
    return ra;
}

// own_rank >= 0: the send kernel, which has finished, put this rank's own rows at their packed
// position and their counts into recv_count; they are not copied again.
static int launch_recv_side(const void* recv_staging, const int32_t* recv_count, int hidden, int num_experts,
                            int num_ranks, int num_max_dispatch_tokens_per_rank, int row_format,
                            void* packed_recv_x, void* packed_recv_scales, int32_t* packed_recv_src_info,
                            int64_t* packed_recv_layout_range, int32_t* packed_recv_count,
                            int32_t* cumulative_local_expert_recv_stats, int64_t expected_rows, void* workspace,
                            size_t workspace_bytes, int own_rank, void* stream, bool index_done = false) {
    if (int rc = check_recv_args(recv_staging, recv_count, hidden, num_experts, num_ranks,
                                 num_max_dispatch_tokens_per_rank, row_format, packed_recv_x, packed_recv_scales,
                                 packed_recv_src_info, packed_recv_layout_range, packed_recv_count))
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
        if (!index_done) {  // (a large one-call dispatch builds the index inside its send launch)
            ll_segment_index_kernel<<<num_experts, kIndexThreads, 0, hs>>>(
                0, recv_count, nullptr, num_local_experts, num_ranks, own_rank, num_max_dispatch_tokens_per_rank,
                packed_recv_layout_range, packed_recv_count, cumulative_local_expert_recv_stats, flat, desc);
            EP_LAUNCH_CHECK();
        }
        const int64_t data_bytes = row_data_bytes(hidden, row_format);
        const int64_t scale_bytes = row_scale_bytes(hidden, row_format);
        const int num_vec = int(data_bytes / 16);
        int threads = ((num_vec + 63) / 64) * 64;
        int extra = 64;  // one more wave for scales + source index
        if (threads + extra > 1024) threads = 1024, extra = 0;
        ll_rows_flat_kernel<<<flat_grid_blocks(expected_rows, max_rows, num_max_dispatch_tokens_per_rank),
                              threads + extra, 0,
                              hs>>>(flat, num_experts, desc, reinterpret_cast<const uint8_t*>(recv_staging),
                                    row_stride_bytes(hidden, row_format), num_vec,
                                    reinterpret_cast<uint8_t*>(packed_recv_x), nullptr, data_bytes,
                                    int(scale_bytes / 4), align16(data_bytes),
                                    scale_bytes > 0 ? reinterpret_cast<uint8_t*>(packed_recv_scales) : nullptr,
                                    align16(data_bytes) + align16(scale_bytes), packed_recv_src_info, extra);
        EP_LAUNCH_CHECK();
        return 0;
    }
    const RecvArgs ra = make_recv_args(recv_staging, recv_count, hidden, num_experts, num_ranks,
                                       num_max_dispatch_tokens_per_rank, row_format, packed_recv_x, packed_recv_scales,
                                       packed_recv_src_info, packed_recv_layout_range, packed_recv_count,
                                       cumulative_local_expert_recv_stats, expected_rows);
    int64_t blocks = ((max_rows << ra.parts_log2) + 3) / 4;
    const int64_t cap = large ? 4096 : 1024;
    if (blocks > cap) blocks = cap;
    const size_t lds = size_t(num_experts + 1 + num_local_experts) * sizeof(int32_t);
    ll_recv_kernel<<<dim3(unsigned(blocks) + 1), 256, lds, hs>>>(ra, nullptr, 0, own_rank);  // + the metadata workgroup
    EP_LAUNCH_CHECK();
    return 0;
}

int deepep_ll_dispatch_recv(const void* recv_staging, const int32_t* recv_count, int hidden, int num_experts,
                            int num_ranks, int num_max_dispatch_tokens_per_rank, int row_format,
                            void* packed_recv_x, void* packed_recv_scales, int32_t* packed_recv_src_info,
                            int64_t* packed_recv_layout_range, int32_t* packed_recv_count,
                            int32_t* cumulative_local_expert_recv_stats, int64_t expected_rows, void* workspace,
                            size_t workspace_bytes, void* stream) {
    clear_error();
    return launch_recv_side(recv_staging, recv_count, hidden, num_experts, num_ranks,
                            num_max_dispatch_tokens_per_rank, row_format, packed_recv_x, packed_recv_scales,
                            packed_recv_src_info, packed_recv_layout_range, packed_recv_count,
                            cumulative_local_expert_recv_stats, expected_rows, workspace, workspace_bytes, -1, stream);
}

int deepep_ll_dispatch_is_single_launch(int num_tokens, int num_topk, int num_experts,
                                        int num_max_dispatch_tokens_per_rank, int64_t expected_rows) {
    return int64_t(num_tokens) * num_topk <= kFusedMaxEntries &&
                   estimated_rows(expected_rows, num_experts, num_max_dispatch_tokens_per_rank) <= kLargeBatchRows
               ? 1
               : 0;
}

int deepep_ll_dispatch(const void* x, const int64_t* topk_idx, int num_tokens, int hidden, int num_topk,
                       int num_experts, int num_ranks, int rank, int num_max_dispatch_tokens_per_rank, int row_format,
                       void* recv_staging, int32_t* recv_count, void* send_slots, int32_t* send_count,
                       int32_t* pair_slot, void* packed_recv_x, void* packed_recv_scales,
                       int32_t* packed_recv_src_info, int64_t* packed_recv_layout_range, int32_t* packed_recv_count,
                       int32_t* cumulative_local_expert_recv_stats, int64_t expected_rows, void* workspace,
                       size_t workspace_bytes, void* segment_workspace, size_t segment_workspace_bytes,
                       void* stream) {
    clear_error();
    const int64_t max_rows = int64_t(num_experts) * num_max_dispatch_tokens_per_rank;
    const bool fused = deepep_ll_dispatch_is_single_launch(num_tokens, num_topk, num_experts,
                                                           num_max_dispatch_tokens_per_rank, expected_rows) != 0;
    if (int rc = check_ll_shape(num_tokens, hidden, num_topk, num_experts, num_ranks, rank,
                                num_max_dispatch_tokens_per_rank, row_format))
        return rc;
    if (!fused) {
        // The two phases back to back, with the single launch's shortcut: the send side writes the
        // rows for this rank's own experts straight to their packed position behind the lower ranks'
        // rows (whose counts are in recv_count already), and the receive side copies the rest.
        EP_HOST_ASSERT(num_tokens == 0 || (x != nullptr && topk_idx != nullptr));
        EP_HOST_ASSERT(recv_staging != nullptr && recv_count != nullptr && pair_slot != nullptr && send_count != nullptr);
        EP_HOST_ASSERT(workspace != nullptr);
        EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(x) & 15) == 0);
        EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(send_slots) & 15) == 0);
        if (int rc = check_recv_args(recv_staging, recv_count, hidden, num_experts, num_ranks,
                                     num_max_dispatch_tokens_per_rank, row_format, packed_recv_x, packed_recv_scales,
                                     packed_recv_src_info, packed_recv_layout_range, packed_recv_count))
            return rc;
        const DirectOut direct = {reinterpret_cast<uint8_t*>(packed_recv_x),
                                  reinterpret_cast<uint8_t*>(packed_recv_scales), packed_recv_src_info};
        // When the receive side will run as index + flat copy, the index is built by extra workgroups of
        // the send launch: three launches (histograms, send + index, copy) instead of four.
        FusedIndexArgs index = {};
        const bool flat_copy =
            segment_workspace != nullptr && num_experts <= 1024 &&
            estimated_rows(expected_rows, num_experts, num_max_dispatch_tokens_per_rank) > kLargeBatchRows;
        if (flat_copy) {
            EP_HOST_ASSERT(segment_workspace_bytes >=
                           size_t(deepep::segment_workspace_bytes(num_experts, num_max_dispatch_tokens_per_rank)));
            EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(segment_workspace) & 15) == 0);
            index.recv_count = recv_count;
            index.num_experts = num_experts, index.num_local_experts = num_experts / num_ranks;
            index.num_ranks = num_ranks, index.rank = rank, index.max_tokens = num_max_dispatch_tokens_per_rank;
            index.layout_out = packed_recv_layout_range, index.packed_count = packed_recv_count;
            index.stats = cumulative_local_expert_recv_stats;
            index.flat_out = reinterpret_cast<int32_t*>(segment_workspace);
            index.desc = reinterpret_cast<RowDesc*>(reinterpret_cast<uint8_t*>(segment_workspace) +
                                                    (((int64_t(num_experts) + 1) * 4 + 255) & ~int64_t(255)));
        }
        bool index_done = false;
        if (int rc = launch_send_side(x, topk_idx, nullptr, 1, num_tokens, hidden, num_topk, num_experts, num_ranks,
                                      rank, num_max_dispatch_tokens_per_rank, row_format, recv_staging, recv_count,
                                      send_slots, send_count, pair_slot, workspace, workspace_bytes,
                                      reinterpret_cast<hipStream_t>(stream), nullptr, 0, &direct, nullptr,
                                      flat_copy ? &index : nullptr, &index_done))
            return rc;
        return launch_recv_side(recv_staging, recv_count, hidden, num_experts, num_ranks,
                                num_max_dispatch_tokens_per_rank, row_format, packed_recv_x, packed_recv_scales,
                                packed_recv_src_info, packed_recv_layout_range, packed_recv_count,
                                cumulative_local_expert_recv_stats, expected_rows, segment_workspace,
                                segment_workspace_bytes, rank, stream, index_done);
    }
    EP_HOST_ASSERT(num_tokens == 0 || (x != nullptr && topk_idx != nullptr));
    EP_HOST_ASSERT(send_count != nullptr && pair_slot != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(send_slots) & 15) == 0);
    if (int rc = check_recv_args(recv_staging, recv_count, hidden, num_experts, num_ranks,
                                 num_max_dispatch_tokens_per_rank, row_format, packed_recv_x, packed_recv_scales,
                                 packed_recv_src_info, packed_recv_layout_range, packed_recv_count))
        return rc;
    const RecvArgs ra = make_recv_args(recv_staging, recv_count, hidden, num_experts, num_ranks,
                                       num_max_dispatch_tokens_per_rank, row_format, packed_recv_x, packed_recv_scales,
                                       packed_recv_src_info, packed_recv_layout_range, packed_recv_count,
                                       cumulative_local_expert_recv_stats, expected_rows);
    int64_t rows = expected_rows > 0 ? expected_rows : int64_t(num_max_dispatch_tokens_per_rank) * num_topk;
    rows += rows / 8 + 16;
    if (rows > max_rows) rows = max_rows;
    return launch_send_side(x, topk_idx, nullptr, 1, num_tokens, hidden, num_topk, num_experts, num_ranks, rank,
                            num_max_dispatch_tokens_per_rank, row_format, recv_staging, recv_count, send_slots,
                            send_count, pair_slot, workspace, workspace_bytes,
                            reinterpret_cast<hipStream_t>(stream), &ra, rows << ra.parts_log2);
}

}  // extern "C"
