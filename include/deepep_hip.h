/*
 * deepep_hip.h — C ABI of the MI355X (gfx950) MoE token dispatch/combine hot path.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (`hipStream_t` passed as `void*`; NULL = the null stream).  Nothing here
 * allocates device memory: outputs, staging buffers and workspaces are
 * owned by the caller.  All work is enqueued on `stream` and is complete in
 * stream order when the call returns; no entry point synchronises the host.
 *
 * Return value: 0 on success.  Non-zero = failure; `deepep_last_error()`
 * then returns a thread-local message shaped like the reference's
 * EPException text, "Failed: Assertion error <file>:<line> '<cond>'"
 * (reference: csrc/kernels/exception.cuh:12-22,46-53).
 *
 * Vocabulary (reference: deep_ep/buffer.py:1836-1842):
 *   T  tokens on this rank            H  hidden size (multiple of 128)
 *   K  top-k                          E  experts in the EP world
 *   R  ranks in the EP world          E_l = E / R local experts per rank
 *   M  num_max_dispatch_tokens_per_rank            N = M * R
 *   G  = H / 128 scale groups per token
 *
 * Expert e lives on rank e / E_l with local id e % E_l
 * (reference: csrc/kernels/efa_kernels.cu:526,628).  topk_idx < 0 means
 * "no selection" (reference: csrc/kernels/layout.cu:36,83).
 */
#ifndef DEEPEP_HIP_H
#define DEEPEP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ */
/* Library                                                            */
/* ------------------------------------------------------------------ */

/* Message of the last failure on the calling thread ("" if none). */
const char* deepep_last_error(void);

/* ABI revision of this header; bumped on any signature change.  deepep_abi_version() returns the
 * revision the library was built from: a binding compares the two before its first call. */
#define DEEPEP_HIP_ABI_VERSION 10
int deepep_abi_version(void);

/* ------------------------------------------------------------------ */
/* Row formats of the low-latency path                                */
/* ------------------------------------------------------------------ */

/* Payload encodings of a dispatched token row.
 * Reference: deep_ep/buffer.py:1647-1667 (data_bpt / scale_bpt / packed_bpt)
 * and csrc/kernels/efa_kernels.cu:155-185 (scale encodings). */
enum {
    DEEPEP_ROW_BF16 = 0,       /* 2H bytes of bf16, no scales                    */
    DEEPEP_ROW_FP8 = 1,        /* H bytes e4m3fn + G float32 scales (amax/448)   */
    DEEPEP_ROW_FP8_POW2 = 2,   /* as FP8, scales rounded up to a power of two    */
    DEEPEP_ROW_FP8_UE8M0 = 3   /* as POW2, scales stored as G exponent bytes     */
};

/* Bytes of the payload part of a row (data only). */
size_t deepep_ll_row_data_bytes(int hidden, int row_format);
/* Bytes of the scale part of a row (0 for bf16). */
size_t deepep_ll_row_scale_bytes(int hidden, int row_format);
/* Payload of one staged row: data and scales each padded to 16 B, plus a
 * 16 B tail {int32 src_token, int32 topk_slot, int32 src_rank, int32 local expert}.
 * 7408 for fp8 at H = 7168 — the stride of the reference's cooperative send
 * (csrc/kernels/coop_dispatch_send.cu:73-75). */
size_t deepep_ll_row_payload_bytes(int hidden, int row_format);
/* Distance between staged rows: the payload rounded up to whole 128-byte cache
 * lines (7424 for fp8 at H = 7168); the bytes behind the tail are never written. */
size_t deepep_ll_row_stride(int hidden, int row_format);

/* Arithmetic of the reference's buffer sizing, kept for API parity.
 * Replaces get_low_latency_rdma_size_hint (csrc/config.hpp:127-193). */
size_t deepep_get_low_latency_rdma_size_hint(int num_max_dispatch_tokens_per_rank, int hidden,
                                             int num_ranks, int num_experts);

/* ------------------------------------------------------------------ */
/* Route counting and layout                                          */
/* ------------------------------------------------------------------ */

/* Bytes of scratch `deepep_get_dispatch_layout` needs for this shape. */
size_t deepep_layout_workspace_bytes(int num_tokens, int num_ranks, int num_experts);

/* Per-expert pair counts, per-rank distinct-token counts, per-node counts
 * and the token×rank membership matrix, in one pass over topk_idx.
 *   topk_idx                  [T, K] int64
 *   num_tokens_per_rank       [R] int32 (out)
 *   num_tokens_per_rdma_rank  [R / 8] int32 (out) or NULL
 *   num_tokens_per_expert     [E] int32 (out)
 *   is_token_in_rank          [T, R] bool bytes (out)
 * Replaces layout::get_dispatch_layout (csrc/kernels/layout.cu:9-149) as
 * called by Buffer::get_dispatch_layout (csrc/deep_ep.cpp:517-581). */
int deepep_get_dispatch_layout(const int64_t* topk_idx, int num_tokens, int num_topk,
                               int num_ranks, int num_experts,
                               int32_t* num_tokens_per_rank, int32_t* num_tokens_per_rdma_rank,
                               int32_t* num_tokens_per_expert, uint8_t* is_token_in_rank,
                               void* workspace, size_t workspace_bytes, void* stream);

/* Bytes of scratch `deepep_moe_routing_sort` needs. */
size_t deepep_routing_sort_workspace_bytes(int num_tokens, int num_ranks);

/* Token ids grouped by destination rank, ascending inside each rank.
 *   is_token_in_rank  [T, R] bool bytes
 *   sorted_token_ids  [T * R] int64 (out; first send_cumsum[R] entries valid)
 *   send_counts       [R] int32 (out)
 *   send_cumsum       [R + 1] int64 (out, exclusive prefix; [R] = total)
 *   row_of_pair       [T, R] int32 (out) or NULL: the inverse of the list, row_of_pair[t, r] = the index
 *                     i with sorted_token_ids[i] == t inside rank r's segment, -1 where token t does
 *                     not go to rank r.  deepep_combine_reduce takes it and then needs one launch.
 * Replaces moe_routing_sort (csrc/kernels/efa_kernels.cu:220-318,1591-1651);
 * the total stays on the device — the caller reads send_cumsum[R]. */
int deepep_moe_routing_sort(const uint8_t* is_token_in_rank, int num_tokens, int num_ranks,
                            int64_t* sorted_token_ids, int32_t* send_counts, int64_t* send_cumsum,
                            int32_t* row_of_pair, void* workspace, size_t workspace_bytes, void* stream);

/* channel_prefix_matrix[d, c] = number of tokens bound for rank d in
 * channels 0..c, channel c owning tokens [min(c*ceil(T/C),T), min(+ceil(T/C),T)).
 *   is_token_in_rank       [T, R] bool bytes
 *   channel_prefix_matrix  [R, C] int32 (out)
 * Replaces blocks >= 1 of intranode::notify_dispatch
 * (csrc/kernels/intranode.cu:90-112, csrc/kernels/utils.cuh:434-438). */
int deepep_channel_prefix_matrix(const uint8_t* is_token_in_rank, int num_tokens, int num_ranks,
                                 int num_channels, int32_t* channel_prefix_matrix, void* stream);

/* Normal-mode pack: dst_row[i] = src_row[sorted_token_ids[i]] for
 * i < *num_rows_dev, rows of `row_bytes` (multiple of 16) bytes.  A second
 * (scale) plane is gathered in the same launch when scale_src != NULL.
 *   max_rows bounds the grid; rows >= *num_rows_dev are not touched.
 * Replaces the torch index gathers x_data[flat_sorted_token_ids] and
 * x_scales[flat_sorted_token_ids] (deep_ep/buffer.py:877,917). */
int deepep_pack_rows(const void* src, const void* scale_src, const int64_t* sorted_token_ids,
                     const int64_t* num_rows_dev, int64_t max_rows, int num_src_rows,
                     int row_bytes, int scale_row_bytes,
                     void* dst, void* scale_dst, void* stream);

/* Top-k of the rows being sent, in the destination rank's expert numbering:
 * for send row i (destination rank d, send_cumsum[d] <= i < send_cumsum[d+1])
 * and selection k, (e - d*E_l, w) if the token's expert e is one of rank d's,
 * else (-1, 0).  Rows i < min(send_cumsum[R], max_send) are written.
 *   topk_idx [T, K] int64       topk_weights [T, K] float32
 *   sorted_token_ids [>= S] int64, send_cumsum [R + 1] int64 (from deepep_moe_routing_sort)
 *   remapped_topk [max_send, K] int64 (out), remapped_weights [max_send, K] float32 (out)
 * Replaces topk_remap (csrc/kernels/efa_kernels.cu:339-387,1653-1691; call site
 * deep_ep/buffer.py:727); the row count stays on the device. */
int deepep_topk_remap(const int64_t* topk_idx, const float* topk_weights,
                      const int64_t* sorted_token_ids, const int64_t* send_cumsum,
                      int num_tokens, int num_topk, int num_ranks, int num_local_experts,
                      int64_t max_send, int64_t* remapped_topk, float* remapped_weights,
                      void* stream);

/* Source metadata of the rows received: row i came from rank s with
 * recv_cumsum[s] <= i < recv_cumsum[s+1]; its 8 bytes are the int32 pair
 * {s / num_local_ranks, 1 << (s % num_local_ranks)}.  Rows
 * i < min(recv_cumsum[R], max_recv_tokens) are written.
 *   recv_cumsum [R + 1] int64     recv_src_meta [max_recv_tokens, 8] bytes (out)
 * Replaces build_recv_src_meta (csrc/kernels/efa_kernels.cu:448-482,1726-1749;
 * call site deep_ep/buffer.py:792). */
int deepep_build_recv_src_meta(const int64_t* recv_cumsum, int num_ranks, int num_local_ranks,
                               int64_t max_recv_tokens, uint8_t* recv_src_meta, void* stream);

/* Bytes of scratch `deepep_combine_reduce` needs. */
size_t deepep_combine_reduce_workspace_bytes(int num_tokens, int num_ranks);

/* Normal-mode combine, receive side: the rows that came back, in the order of
 * the send list (row j of rank r's segment answers token sorted_token_ids[j]),
 * are added per token:
 *   combined_x[t,:] = bf16( sum_{r: is_token_in_rank[t,r]} f32(recv_x[row(t,r),:])
 *                           + bias_0[t,:] + bias_1[t,:] )
 * in float32, ranks ascending, one rounding; the weights likewise in float32.
 * Tokens sent nowhere give the biases (or zeros).
 *   recv_x [>= S, H] bf16          recv_topk_weights [>= S, K] float32 or NULL
 *   sorted_token_ids, send_cumsum  as used for the dispatch pack
 *   is_token_in_rank [T, R] bool bytes
 *   bias_0, bias_1 [T, H] bf16 or NULL
 *   combined_x [T, H] bf16 (out)   combined_topk_weights [T, K] float32 (out) or NULL
 *   max_rows bounds the rows of recv_x that may be read.
 *   row_of_pair  [T, R] int32 from deepep_moe_routing_sort, or NULL: without it the call first
 *                rebuilds that table from the list (a second launch, into `workspace`); with it
 *                `workspace` may be NULL.
 * Replaces the zero_() + index_add_ + bias adds of deep_ep/buffer.py:1542-1557
 * (which accumulate in bf16 through atomics, in arrival order). */
int deepep_combine_reduce(const void* recv_x, const float* recv_topk_weights,
                          const int64_t* sorted_token_ids, const int64_t* send_cumsum,
                          const uint8_t* is_token_in_rank, const void* bias_0, const void* bias_1,
                          int num_tokens, int hidden, int num_topk, int num_ranks, int64_t max_rows,
                          const int32_t* row_of_pair, void* combined_x, float* combined_topk_weights,
                          void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ */
/* FP8 cast                                                           */
/* ------------------------------------------------------------------ */

/* Per token, per 128 channels: amax = max(max|x|, 1e-4), scale = amax/448,
 * q = e4m3fn_rne(clamp(x * (448/amax), ±448)).
 *   x        [M, N] bf16          x_fp8   [M, N] e4m3fn bytes (out)
 *   scales   [M, N/128] float32, or [M, N/512] int32 for UE8M0 (out)
 *   row_format: DEEPEP_ROW_FP8 | _POW2 | _UE8M0
 * Replaces per_token_cast_to_fp8 (csrc/kernels/efa_kernels.cu:104-187,2281-2327;
 * torch form deep_ep/buffer.py:1590-1621). */
int deepep_per_token_cast_to_fp8(const void* x, int num_rows, int num_cols, int row_format,
                                 void* x_fp8, void* scales, void* stream);

/* ------------------------------------------------------------------ */
/* Low-latency dispatch                                               */
/* ------------------------------------------------------------------ */

/* Bytes of the optional scratch of deepep_ll_dispatch_recv / deepep_ll_combine_send. */
size_t deepep_ll_segment_workspace_bytes(int num_experts, int num_max_dispatch_tokens_per_rank);

/* Bytes of scratch `deepep_ll_dispatch_send` needs. */
size_t deepep_ll_dispatch_workspace_bytes(int num_tokens, int num_topk, int num_experts);

/* Send side of the low-latency dispatch, one launch sequence:
 *   route   — send_count[e] = pairs (t,k) with topk_idx[t,k] == e;
 *             pair_slot[t,k] = rank of the pair among this rank's pairs for
 *             that expert in ascending (t,k) order (-1 if no selection);
 *   quantise + pack — each token row is quantised once (row_format) and
 *             written once per selection into slot pair_slot[t,k] of its
 *             expert: rows for this rank's own experts go straight into
 *             recv_staging[(e_l * R + rank) * M + slot] (the self-copy the
 *             reference does on the host side, csrc/transport/ll_pipeline.cpp:1542),
 *             rows for remote experts into send_slots[e * M + slot];
 *   counts  — recv_count[e_l * R + rank] and send_count[e].
 *   x             [T, H] bf16        topk_idx   [T, K] int64
 *   recv_staging  [E_l, R, M] rows of deepep_ll_row_stride bytes (in/out)
 *   recv_count    [E_l, R] int32 (in/out; only column `rank` is written)
 *   send_slots    [E, M] rows (out) or NULL to drop remote rows
 *   send_count    [E] int32 (out)     pair_slot  [T, K] int32 (out)
 * A pair whose slot would reach M (only possible when one token names the
 * same expert twice) is dropped and its pair_slot is -1.
 * Replaces per_token_cast_to_fp8 + ll_dispatch_route_and_pack_v3
 * (csrc/kernels/efa_kernels.cu:2281,2332; kernels :512-845) and the
 * cooperative a2a_dispatch_send (csrc/deep_ep.cpp:3641,
 * csrc/kernels/coop_dispatch_send.cuh:304-790). */
int deepep_ll_dispatch_send(const void* x, const int64_t* topk_idx,
                            int num_tokens, int hidden, int num_topk,
                            int num_experts, int num_ranks, int rank,
                            int num_max_dispatch_tokens_per_rank, int row_format,
                            void* recv_staging, int32_t* recv_count,
                            void* send_slots, int32_t* send_count, int32_t* pair_slot,
                            void* workspace, size_t workspace_bytes, void* stream);

/* deepep_ll_dispatch_send without the workspace arguments: the route scratch is an array inside
 * the library image (1 MiB on every GPU the library runs on, held until the process ends), so the
 * call allocates nothing and needs nothing allocated for it.  No counterpart in the reference; it
 * is for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  Same arguments, outputs and errors as
 * deepep_ll_dispatch_send otherwise.
 *   Limit: deepep_ll_dispatch_workspace_bytes(T, K, E) <= 1 MiB, i.e.
 *   ceil(T / floor(2048 / K)) * E * 4 <= 1048576 (at K = 8, E = 256: T <= 262144); a larger batch
 *   fails with a message that says so.
 *   `stream` must belong to the current device.  The array's address is looked up on the first
 *   call on each device (a host-side query, no device work).
 *   Every call on a GPU shares that GPU's array: two calls that overlap in time on one GPU (on
 *   different streams, or from different threads) race.  Nothing in it has to start at zero: a
 *   call overwrites every word it later reads. */
int deepep_ll_dispatch_send_static(const void* x, const int64_t* topk_idx,
                                   int num_tokens, int hidden, int num_topk, int num_experts,
                                   int num_ranks, int rank, int num_max_dispatch_tokens_per_rank,
                                   int row_format,
                                   void* recv_staging, int32_t* recv_count,
                                   void* send_slots, int32_t* send_count, int32_t* pair_slot,
                                   void* stream);

/* Send side for a transport that ships one contiguous message per peer (an all-to-all): the same
 * route + quantise + pack, but every row -- this rank's own included -- goes into ONE buffer that is
 * contiguous per destination rank, destination ranks ascending.  Inside a destination's message the
 * rows come expert by expert and, inside an expert, in pair_slot order (ascending (token, k)): the
 * per-expert send slots laid end to end without their gaps.  The row of pair (t, k) is
 * send_expert_prefix[topk_idx[t,k]] + pair_slot[t,k].
 *   send_rows           [send_row_capacity] rows of deepep_ll_row_stride bytes (out); the first
 *                       send_cumsum[R] are written; capacity >= min(T * K, E * M)
 *   send_count          [E] int32 (out)      pairs per expert, clamped to M
 *   send_expert_prefix  [E + 1] int32 (out)  exclusive prefix of send_count; [E] = rows sent
 *   send_counts         [R] int32 (out)      rows for each destination rank
 *   send_cumsum         [R + 1] int64 (out)  their exclusive prefix: the message for rank d is rows
 *                       [send_cumsum[d], send_cumsum[d + 1])
 *   pair_slot           [T, K] int32 (out)   as deepep_ll_dispatch_send
 *   workspace           deepep_ll_dispatch_workspace_bytes(T, K, E) bytes
 * Stacked over the ranks, send_count is the all_num_routed of deepep_ll_exchange_metadata.
 * Replaces ll_dispatch_route_and_pack_v3 (csrc/kernels/efa_kernels.cu:2332-2400: send_counts,
 * send_cumsum, rows grouped by destination rank; row tail :797-800), whose output
 * dist.all_to_all_single ships (deep_ep/buffer.py:2297-2301).  The reference leaves the order inside
 * a destination's message to an atomic (:2378-2380); here it is fixed as above. */
int deepep_ll_dispatch_send_by_dest(const void* x, const int64_t* topk_idx,
                                    int num_tokens, int hidden, int num_topk, int num_experts,
                                    int num_ranks, int rank, int num_max_dispatch_tokens_per_rank,
                                    int row_format, void* send_rows, int64_t send_row_capacity,
                                    int32_t* send_count, int32_t* send_expert_prefix,
                                    int32_t* send_counts, int64_t* send_cumsum, int32_t* pair_slot,
                                    void* workspace, size_t workspace_bytes, void* stream);

/* Receive side: compacts the staged rows of every (local expert, source
 * rank) segment into the packed layout.
 *   begin(e,s) = sum_{s' < s} recv_count[e,s'];  rows [begin, begin+cnt)
 *   of expert e hold source rank s's rows in staging order.
 *   packed_recv_x            [E_l, N, H] e4m3fn bytes (or bf16) (out)
 *   packed_recv_scales       [E_l, N, G] float32 / [E_l, N, G/4] int32 (out) or NULL
 *   packed_recv_src_info     [E_l, N] int32 source token index (out)
 *   packed_recv_layout_range [E_l, R] int64 = (begin << 32) | cnt, 0 if cnt == 0 (out)
 *   packed_recv_count        [E_l] int32 (out)
 *   cumulative_local_expert_recv_stats [E_l] int32, += count, or NULL
 * Rows at or beyond packed_recv_count[e] are left untouched.
 *   expected_rows  the number of rows the caller expects this call to move (0 = unknown: E*M/32 is
 *                  assumed); it sizes the grids and picks between equivalent kernels, and any
 *                  value gives the same result.
 *   workspace      deepep_ll_segment_workspace_bytes(E, M) bytes, or NULL.  With it, calls
 *                  expecting more than 8192 rows run as an index kernel plus a flat row copy (faster
 *                  when bandwidth-bound); without it one fused kernel is used at every size.
 * Replaces ll_recv_unpack_v2 (csrc/kernels/efa_kernels.cu:2121-2231;
 * kernels :877-1389) and a2a_dispatch_recv (csrc/deep_ep.cpp:3709,
 * csrc/kernels/coop_dispatch_recv.cuh:39-304). */
int deepep_ll_dispatch_recv(const void* recv_staging, const int32_t* recv_count,
                            int hidden, int num_experts, int num_ranks,
                            int num_max_dispatch_tokens_per_rank, int row_format,
                            void* packed_recv_x, void* packed_recv_scales,
                            int32_t* packed_recv_src_info, int64_t* packed_recv_layout_range,
                            int32_t* packed_recv_count,
                            int32_t* cumulative_local_expert_recv_stats,
                            int64_t expected_rows, void* workspace, size_t workspace_bytes,
                            void* stream);

/* What a rank derives from the gathered per-expert route counts before the
 * exchange, in one launch instead of the reference's host loops over three
 * device-to-host copies.
 *   all_num_routed [R, E] int32: row s = the pairs rank s routed to each expert
 *                  (this rank's own row is the send_count of its dispatch)
 *   send_counts [R] int32 (out): rows this rank sends to each rank
 *   recv_counts [R] int32 (out): rows it receives from each rank
 *   totals      [3] int32 (out): total sent, total received, 1 if the gather was corrupt
 *               (any count above M: every count is then reported as zero, as the reference does)
 *   combine_remote_recv_offset [R] int64 (out): rows peer s sent to the ranks below this one,
 *               i.e. where this rank's returned rows start in peer s's combine buffer
 *   source_rank, source_offset, padded_index, combine_send_offset [row_capacity] uint32 (out):
 *               one record per expected row i, grouped by source rank s in ascending order, the
 *               j-th row of a source getting (s, s * M + j, i, i)
 *   num_recv_tokens [2] uint32 (out): rows expected, records written (the smaller of that and row_capacity)
 *   tokens_per_expert [E_l] uint32 (out): zeroed, as the reference leaves it for the receive kernel
 * Replaces LLPipelineWorker::compute_send_recv_counts and ::upload_recv_metadata
 * (csrc/transport/ll_pipeline.cpp:1204-1269, :1277-1361). */
int deepep_ll_exchange_metadata(const int32_t* all_num_routed, int num_experts, int num_ranks, int rank,
                                int num_max_dispatch_tokens_per_rank, int64_t row_capacity,
                                int32_t* send_counts, int32_t* recv_counts, int32_t* totals,
                                int64_t* combine_remote_recv_offset,
                                uint32_t* source_rank, uint32_t* source_offset, uint32_t* padded_index,
                                uint32_t* combine_send_offset, uint32_t* num_recv_tokens,
                                uint32_t* tokens_per_expert, void* stream);

/* Bytes of scratch deepep_ll_dispatch_recv_by_source needs for `row_capacity` records. */
size_t deepep_ll_by_source_workspace_bytes(int num_experts, int64_t row_capacity);

/* deepep_ll_dispatch_recv for a transport that delivers rows grouped by source rank (what an
 * all-to-all leaves behind): the rows of source s sit in slot s of `recv_by_source`, in the order
 * they arrived, and the records of deepep_ll_exchange_metadata say where each expected row is.
 * Same outputs as deepep_ll_dispatch_recv (ranges in ascending source order; inside an (expert,
 * source) segment the rows keep their arrival order, which for a sender that emits in (token, k)
 * order is the order of the staged form), plus the reference's tokens_per_expert.
 *   recv_by_source  [R * slot_rows] rows of deepep_ll_row_stride bytes in the staged row format;
 *                   the last int32 of a row's tail is its local expert id
 *   slot_rows       rows one source's slot holds (the M the records were built with: record j of
 *                   source s has source_offset = s * M + j); records past it are not copied
 *   recv_counts     [R] int32 rows expected from each rank          } outputs of
 *   source_offset   [row_capacity] uint32 row index of each record  } deepep_ll_exchange_metadata
 *   num_recv_tokens [2] uint32: [1] = records present               }
 *   tokens_per_expert [E_l] uint32 (out) = packed_recv_count, or NULL
 *   record_packed_row [row_capacity] int32 (out) or NULL: for record i, the packed row its row was copied
 *                   to, local_expert * N + position, or -1 if it got none (past its source's slot, no valid
 *                   expert in its tail, past its pair's M rows) -- the reference's recv_expert_ids /
 *                   recv_expert_pos (csrc/kernels/efa_kernels.cu:2121-2231), which the combine needs to
 *                   return the rows in arrival order (deepep_ll_combine_send_by_dest)
 *   expected_rows   rows the caller expects to receive (0 = unknown: row_capacity is assumed); it only
 *                   sizes the copy's grid, and any value gives the same result
 *   workspace       deepep_ll_by_source_workspace_bytes(E, row_capacity) bytes
 * An (expert, source) pair takes at most M rows, as a segment of the staged form does.
 * Replaces ll_recv_unpack_v2 on its flat / slotted input (csrc/kernels/efa_kernels.cu:2121-2231,
 * kernels :877-1052 and :1227-1389, slot addressing :906-913) and consumes the records
 * a2a_dispatch_recv reads (csrc/kernels/coop_dispatch_recv.cuh:42, source_offset). */
int deepep_ll_dispatch_recv_by_source(const void* recv_by_source, int64_t slot_rows,
                                      const int32_t* recv_counts, const uint32_t* source_offset,
                                      const uint32_t* num_recv_tokens, int64_t row_capacity,
                                      int hidden, int num_experts, int num_ranks,
                                      int num_max_dispatch_tokens_per_rank, int row_format,
                                      void* packed_recv_x, void* packed_recv_scales,
                                      int32_t* packed_recv_src_info, int64_t* packed_recv_layout_range,
                                      int32_t* packed_recv_count,
                                      int32_t* cumulative_local_expert_recv_stats,
                                      uint32_t* tokens_per_expert, int32_t* record_packed_row,
                                      int64_t expected_rows,
                                      void* workspace, size_t workspace_bytes, void* stream);

/* deepep_ll_dispatch_recv_by_source for messages whose order is known: every source sent its rows
 * for this rank expert by expert (local experts ascending), an expert's rows in slot order, which is
 * what deepep_ll_dispatch_send_by_dest emits, and its message starts at row s * slot_rows.  With the
 * gathered route counts every row's place then follows by arithmetic -- row j of source s belongs to
 * the expert whose run of that source's column of the counts holds j -- so nothing is read from the
 * rows to index them and no record list is needed: one launch for up to 8192 expected rows, one index
 * launch and the row copy beyond, both sides of every (expert, source) pair contiguous.  Outputs as
 * deepep_ll_dispatch_recv_by_source.
 *   all_num_routed     [R, E] int32, as for deepep_ll_exchange_metadata (counts above M read as M)
 *   record_packed_row  [row_capacity] int32 (out) or NULL, indexed like the records of
 *                      deepep_ll_exchange_metadata: sources ascending, a source's rows in message order
 *   expected_rows      as for deepep_ll_dispatch_recv_by_source
 *   workspace          256 + 8 * min(R * slot_rows, E * M) bytes (deepep_ll_by_source_workspace_bytes(E,
 *                      R * slot_rows) is enough); only read and written past 8192 expected rows
 * Rows of a message beyond the source's slot are lost (their records read -1).
 * Replaces ll_recv_unpack_v2 (csrc/kernels/efa_kernels.cu:2121-2231; ranges :991-1010) for this
 * build's own wire order; the reference cannot take this shortcut because its senders leave the
 * order inside a message to an atomic (:2378-2380). */
int deepep_ll_dispatch_recv_by_source_ordered(const void* recv_by_source, int64_t slot_rows,
                                              const int32_t* all_num_routed,
                                              int hidden, int num_experts, int num_ranks, int rank,
                                              int num_max_dispatch_tokens_per_rank, int row_format,
                                              void* packed_recv_x, void* packed_recv_scales,
                                              int32_t* packed_recv_src_info,
                                              int64_t* packed_recv_layout_range,
                                              int32_t* packed_recv_count,
                                              int32_t* cumulative_local_expert_recv_stats,
                                              uint32_t* tokens_per_expert, int32_t* record_packed_row,
                                              int64_t row_capacity, int64_t expected_rows,
                                              void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ */
/* Low-latency combine                                                */
/* ------------------------------------------------------------------ */

/* Send side: returns every live expert-output row to the rank it came from,
 * in arrival order.  Row j of segment (e_l, s) — x[e_l, begin(e_l,s) + j] —
 * goes to slot j of expert rank*E_l + e_l on rank s: this rank's own rows
 * into combine_staging[(rank * E_l + e_l) * M + j], other ranks' rows into
 * combine_send_slots[(e_l * R + s) * M + j] (NULL drops them).
 *   x                   [E_l, N, H] bf16
 *   layout_range        [E_l, R] int64 from the dispatch
 *   combine_staging     [E, M, H] bf16 (in/out)
 *   combine_send_slots  [E_l, R, M, H] bf16 (out) or NULL
 *   expected_rows, workspace: as for deepep_ll_dispatch_recv.
 * Replaces the two torch gathers of deep_ep/buffer.py:2601-2608 and
 * a2a_combine_send (csrc/deep_ep.cpp:3804, csrc/kernels/coop_combine_send.cuh:34-275). */
int deepep_ll_combine_send(const void* x, const int64_t* layout_range,
                           int hidden, int num_experts, int num_ranks, int rank,
                           int num_max_dispatch_tokens_per_rank,
                           void* combine_staging, void* combine_send_slots,
                           int64_t expected_rows, void* workspace, size_t workspace_bytes,
                           void* stream);

/* Receive side: out[t,:] = bf16( sum_k [pair_slot[t,k] >= 0] * w[t,k] *
 * f32(combine_staging[topk_idx[t,k], pair_slot[t,k], :]) ), accumulated in
 * float32 as acc = fma(row_k, w_k, acc) for k = 0..K-1; tokens with no live
 * selection give zeros.
 *   combine_staging [E, M, H] bf16     topk_idx [T, K] int64
 *   topk_weights    [T, K] float32     pair_slot [T, K] int32 from the dispatch
 *   out             [T, H] bf16 (out; in/out when accumulate != 0: the sum then starts from
 *                   f32(out[t,:]) instead of zero, csrc/kernels/coop_combine_recv.cuh:174-179)
 * Replaces ll_combine_weighted_reduce_v2 (csrc/kernels/efa_kernels.cu:1413-1486,1982-2031)
 * and a2a_combine_recv (csrc/deep_ep.cpp:3850, csrc/kernels/coop_combine_recv.cuh:69-283). */
int deepep_ll_combine_recv(const void* combine_staging, const int64_t* topk_idx,
                           const float* topk_weights, const int32_t* pair_slot,
                           int num_tokens, int hidden, int num_topk, int num_experts,
                           int num_max_dispatch_tokens_per_rank, int accumulate, void* out, void* stream);

/* Send side for an all-to-all shaped transport: every live expert-output row, in arrival order --
 * which is contiguous per destination rank -- in one flat buffer.  For record i of
 * deepep_ll_exchange_metadata (i < num_recv_tokens[1]):
 *   send_flat[combine_send_offset[i], :] = x_rows[record_packed_row[padded_index[i]], :]
 * with x_rows the [E_l * N, H] view of the expert outputs.  The message for rank s is then rows
 * [prefix(recv_counts)[s], prefix(recv_counts)[s + 1]) of send_flat.  A record whose packed row is -1
 * leaves its row untouched.
 *   x                  [E_l, N, H] bf16 expert outputs
 *   record_packed_row  [row_capacity] int32 from deepep_ll_dispatch_recv_by_source
 *   source_rank, padded_index, combine_send_offset [row_capacity] uint32, num_recv_tokens [2] uint32:
 *                      the records of deepep_ll_exchange_metadata
 *   send_flat          [row_capacity, H] bf16 (out); may be NULL with peer_recv_flat
 * Direct delivery (peer_recv_flat != NULL): when the destination ranks' receive buffers are mapped
 * into this GPU's address space (peers on the same node), the row skips send_flat and is stored
 * where the all-to-all would have put it: row combine_remote_recv_offset[s] + j of rank s's buffer, j
 * being the record's place among the rows of source s = source_rank[i].
 *   recv_counts                 [R] int32     } outputs of deepep_ll_exchange_metadata
 *   combine_remote_recv_offset  [R] int64     }
 *   expected_rows   rows the caller expects to return (0 = unknown: row_capacity); sizes the grid only
 *   peer_recv_flat  [R] device array of pointers to the ranks' receive buffers (the buffer
 *                   deepep_ll_combine_recv_flat reads, flat form), peer_recv_rows [R] int64 their rows
 * Replaces the gather + un-sort of deep_ep/buffer.py:2601-2608 and a2a_combine_send
 * (csrc/kernels/coop_combine_send.cuh:37-275: send_buffer[combine_send_offset[i]] =
 * expert_x[padded_index[i]], peer stores :205-246); landing offset
 * csrc/transport/ll_pipeline.cpp:1283-1295. */
int deepep_ll_combine_send_by_dest(const void* x, const int32_t* record_packed_row,
                                   const uint32_t* source_rank, const uint32_t* padded_index,
                                   const uint32_t* combine_send_offset, const uint32_t* num_recv_tokens,
                                   int64_t row_capacity, int hidden, int num_experts, int num_ranks,
                                   int num_max_dispatch_tokens_per_rank, void* send_flat,
                                   const int32_t* recv_counts, const int64_t* combine_remote_recv_offset,
                                   void* const* peer_recv_flat, const int64_t* peer_recv_rows,
                                   int64_t expected_rows, void* stream);

/* deepep_ll_combine_recv reading the answers from the buffer an all-to-all leaves them in: one row
 * per row this rank sent, in send order (deepep_ll_dispatch_send_by_dest), so that pair (t, k) is
 * answered by row send_expert_prefix[topk_idx[t,k]] + pair_slot[t,k].
 *   recv_flat           [recv_flat_rows, H] bf16
 *   slot_rows           0: the rows lie back to back (flat).  > 0: the answers of rank r start at row
 *                       r * slot_rows (one fixed slot per answering rank; the reference's slot_size,
 *                       in rows) and a pair's row is r * slot_rows + (its send index - the first
 *                       send index of rank r)
 *   send_expert_prefix  [E + 1] int32 from deepep_ll_dispatch_send_by_dest
 *   other arguments and the arithmetic as deepep_ll_combine_recv.
 * Replaces ll_combine_weighted_reduce_v2 on its flat / slotted input
 * (csrc/kernels/efa_kernels.cu:1982-2031, kernel :1413-1474, addressing :1449-1466). */
int deepep_ll_combine_recv_flat(const void* recv_flat, int64_t recv_flat_rows, int64_t slot_rows,
                                const int32_t* send_expert_prefix, const int64_t* topk_idx,
                                const float* topk_weights, const int32_t* pair_slot,
                                int num_tokens, int hidden, int num_topk, int num_experts,
                                int num_ranks, int num_max_dispatch_tokens_per_rank, int accumulate,
                                void* out, void* stream);

/* ------------------------------------------------------------------ */
/* Whole dispatch / whole combine in one call                          */
/* ------------------------------------------------------------------ */

/* deepep_ll_dispatch_send followed by deepep_ll_dispatch_recv, for a caller
 * whose peers' rows and counts are already in recv_staging / recv_count when
 * the call is made (the reference's dispatch is one call too:
 * Buffer::low_latency_dispatch, csrc/deep_ep.cpp:1658-1796; its kernel has a
 * send and a receive phase, csrc/kernels/coop_dispatch_send.cuh:304,
 * coop_dispatch_recv.cuh:42).  Arguments and every packed_* output are those
 * of the two calls: inside an expert's range the source ranks come in ascending
 * order, begin(e, s) = sum of the counts of the ranks below s
 * (csrc/kernels/efa_kernels.cu:991-1010).  One thing differs from calling them
 * in turn: this rank's rows for its own experts go straight to their packed
 * position and the own segment of recv_staging is not written; recv_count,
 * send_count, send_slots and pair_slot are written as by
 * deepep_ll_dispatch_send.  Small batches (num_tokens * num_topk <= 8192 and at
 * most 8192 rows expected) run as one kernel launch, larger ones as the send
 * and receive launches back to back; the result is the same.
 *   workspace          as for deepep_ll_dispatch_send
 *   segment_workspace  as the workspace of deepep_ll_dispatch_recv */
/* 1 when deepep_ll_dispatch runs a batch of this shape as one kernel launch, else 0 (the result
 * does not depend on it).  No counterpart in the reference. */
int deepep_ll_dispatch_is_single_launch(int num_tokens, int num_topk, int num_experts,
                                        int num_max_dispatch_tokens_per_rank, int64_t expected_rows);

int deepep_ll_dispatch(const void* x, const int64_t* topk_idx,
                       int num_tokens, int hidden, int num_topk, int num_experts,
                       int num_ranks, int rank, int num_max_dispatch_tokens_per_rank,
                       int row_format,
                       void* recv_staging, int32_t* recv_count,
                       void* send_slots, int32_t* send_count, int32_t* pair_slot,
                       void* packed_recv_x, void* packed_recv_scales,
                       int32_t* packed_recv_src_info, int64_t* packed_recv_layout_range,
                       int32_t* packed_recv_count, int32_t* cumulative_local_expert_recv_stats,
                       int64_t expected_rows, void* workspace, size_t workspace_bytes,
                       void* segment_workspace, size_t segment_workspace_bytes, void* stream);

/* deepep_ll_combine_send followed by deepep_ll_combine_recv, for a caller
 * whose remote experts' answers are already in combine_staging when the call
 * is made (the reference: Buffer::low_latency_combine,
 * csrc/deep_ep.cpp:1798-1920; kernel phases csrc/kernels/coop_combine_send.cuh:37,
 * coop_combine_recv.cuh:72).  `out` is identical to the two calls'.  The
 * answers of this rank's own experts are read from x directly — the own
 * experts' part of combine_staging is neither written nor read.  When at most
 * 8192 rows are expected both phases run as one kernel launch, larger batches
 * launch them back to back.  combine_send_slots may be NULL (the reference's
 * zero_copy, deep_ep/buffer.py:2831-2852: "the next combine kernel can skip the
 * copying"): no row is returned, the call is the reduce alone, and the caller's
 * transport sends the rows of (e_l, s) from where they are,
 * x[e_l, begin .. begin + count) of layout_range[e_l, s], which is contiguous. */
int deepep_ll_combine(const void* x, const int64_t* layout_range,
                      const int64_t* topk_idx, const float* topk_weights,
                      const int32_t* pair_slot,
                      int num_tokens, int hidden, int num_topk, int num_experts,
                      int num_ranks, int rank, int num_max_dispatch_tokens_per_rank, int accumulate,
                      void* combine_staging, void* combine_send_slots, void* out,
                      int64_t expected_rows, void* workspace, size_t workspace_bytes,
                      void* stream);

/* ------------------------------------------------------------------ */
/* Single-GPU loopback: peers synthesised in HBM                      */
/* These stand where the reference has its transport                  */
/* (csrc/transport/, dist.all_to_all_single at deep_ep/buffer.py:2268,2297,2735). */
/* ------------------------------------------------------------------ */

/* Seeded routing for `num_src` ranks: for each (rank, token) draws K distinct
 * experts by repeated inverse-CDF sampling of 32-bit hashes against
 * `expert_cdf` (E uint32 inclusive upper bounds), rejecting repeats.
 *   src_ranks  [num_src] int32 world rank of each batch entry
 *   topk_idx   [num_src, T, K] int64 (out) */
int deepep_synth_topk_idx(const uint32_t* expert_cdf, const int32_t* src_ranks, int num_src,
                          int num_tokens, int num_topk, int num_experts, uint32_t seed,
                          int64_t* topk_idx, void* stream);

/* Seeded bf16 rows, approximately N(0,1): value(seed, row_key, column) is the
 * centred sum of the four bytes of a 32-bit hash times 1/147.8 in float32,
 * rounded to bf16; rows whose key hash is 0 mod `outlier_period` are scaled
 * by 100 first (outlier_period 0 = never).
 *   row_keys  [num_rows] uint32 or NULL (key = first_key + row index)
 *   dst       num_rows rows of `row_stride_bytes`, first 2*hidden bytes written */
int deepep_synth_bf16_rows(void* dst, int64_t num_rows, int hidden, int64_t row_stride_bytes,
                           const uint32_t* row_keys, uint32_t first_key, uint32_t seed,
                           int outlier_period, void* stream);

/* Runs the send side for `num_src` peer ranks and keeps only the rows bound
 * for `rank`: they land in recv_staging[(e_l * R + src) * M + slot] with
 * recv_count[e_l * R + src], exactly where the peers' own sends would put them.
 *   x [num_src, T, H] bf16   topk_idx [num_src, T, K] int64   src_ranks [num_src] int32 (device)
 *   workspace of num_src * deepep_ll_dispatch_workspace_bytes(T, K, E) bytes */
int deepep_loopback_dispatch_from_peers(const void* x, const int64_t* topk_idx,
                                        const int32_t* src_ranks, int num_src,
                                        int num_tokens, int hidden, int num_topk,
                                        int num_experts, int num_ranks, int rank,
                                        int num_max_dispatch_tokens_per_rank, int row_format,
                                        void* recv_staging, int32_t* recv_count,
                                        void* workspace, size_t workspace_bytes, void* stream);

/* Plays the remote experts for this rank's own pairs: for every remote
 * expert e and slot j < send_count[e] writes combine_staging[e, j, :].
 *   mode 0: the dequantised send_slots row (f32(q) * scale -> bf16), i.e. an
 *           identity expert, the recipe of tests/test_low_latency.py:111;
 *   mode 1: a seeded row with key e * M + j (see deepep_synth_bf16_rows). */
int deepep_loopback_combine_from_peers(const void* send_slots, const int32_t* send_count,
                                       int hidden, int num_experts, int num_ranks, int rank,
                                       int num_max_dispatch_tokens_per_rank, int row_format,
                                       int mode, uint32_t seed,
                                       void* combine_staging, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DEEPEP_HIP_H */
