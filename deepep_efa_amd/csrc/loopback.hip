// Single-GPU loopback: the peers of an expert-parallel world synthesised in
// HBM from a seed.  Everything here is integer hashing plus exactly-rounded
// float32 steps, so a CPU can regenerate every byte.
//
//   row_hash(seed, key)    = mix32(seed ^ mix32(key + 0x9e3779b9))
//   value(seed, key, col)  : h = mix32(row_hash ^ (col * 0x9e3779b1 + 0x85ebca6b));
//                            s = sum of the four bytes of h (0..1020, mean 510);
//                            f = float(s - 510) * 0x1.bb68f6p-8 (= 1/147.8 in float32);
//                            rows with mix32(row_hash ^ 0x5bd1e995) % period == 0: f *= 100;
//                            result = bf16_rne(f)
//   topk(seed, rank, t)    : th = row_hash(seed ^ 0x7f4a7c15, rank * T + t);
//                            draw c = 0,1,..: u = mix32(th + c * 0x9e3779b9),
//                            e = first index with cdf[e] >= u, kept unless
//                            already drawn; after 64*K draws the lowest
//                            unused experts fill the rest.
#include "common.hpp"
#include "../../include/deepep_hip.h"

namespace deepep {

constexpr int kMaxSynthTopk = 32;

__host__ __device__ inline uint32_t row_hash(uint32_t seed, uint32_t key) {
    return mix32(seed ^ mix32(key + 0x9e3779b9u));
}

__device__ __forceinline__ float synth_value(uint32_t rh, uint32_t col, float row_scale) {
    const uint32_t h = mix32(rh ^ (col * 0x9e3779b1u + 0x85ebca6bu));
    const int s = int(h & 255u) + int((h >> 8) & 255u) + int((h >> 16) & 255u) + int(h >> 24);
    float f = float(s - 510) * __uint_as_float(0x3bddb47bu);
    return f * row_scale;  // row_scale is 1 or 100: multiplying by 1 is exact
}

__device__ __forceinline__ float synth_row_scale(uint32_t rh, int outlier_period) {
    if (outlier_period > 0 && mix32(rh ^ 0x5bd1e995u) % uint32_t(outlier_period) == 0) return 100.0f;
    return 1.0f;
}

// One wave fills the first 2*hidden bytes of one row, 16 B per lane per step.
__device__ __forceinline__ void wave_fill_synth_row(uint8_t* dst, int hidden, uint32_t rh, int outlier_period,
                                                    int lane) {
    const float rs = synth_row_scale(rh, outlier_period);
    const int num_vec = hidden / 8;
    for (int v = lane; v < num_vec; v += kWave) {
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            o[i] = pack_bf16x2(synth_value(rh, uint32_t(v * 8 + 2 * i), rs),
                               synth_value(rh, uint32_t(v * 8 + 2 * i + 1), rs));
        *reinterpret_cast<u32x4*>(dst + int64_t(v) * 16) = o;
    }
}

__global__ __launch_bounds__(256) void synth_bf16_rows_kernel(uint8_t* __restrict__ dst, int64_t num_rows,
                                                              int hidden, int64_t row_stride,
                                                              const uint32_t* __restrict__ row_keys,
                                                              uint32_t first_key, uint32_t seed,
                                                              int outlier_period) {
    const int lane = lane_id();
    const int64_t waves_total = int64_t(gridDim.x) * 4;
    for (int64_t r = int64_t(blockIdx.x) * 4 + wave_in_block(); r < num_rows; r += waves_total) {
        const uint32_t key = row_keys != nullptr ? row_keys[r] : first_key + uint32_t(r);
        wave_fill_synth_row(dst + r * row_stride, hidden, row_hash(seed, key), outlier_period, lane);
    }
}

__global__ __launch_bounds__(256) void synth_topk_kernel(const uint32_t* __restrict__ cdf,
                                                         const int32_t* __restrict__ src_ranks, int num_src,
                                                         int num_tokens, int num_topk, int num_experts,
                                                         uint32_t seed, int64_t* __restrict__ topk_idx) {
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= int64_t(num_src) * num_tokens) return;
    const int b = int(id / num_tokens);
    const int t = int(id - int64_t(b) * num_tokens);
    const uint32_t th = row_hash(seed ^ 0x7f4a7c15u, uint32_t(src_ranks[b]) * uint32_t(num_tokens) + uint32_t(t));
    int chosen[kMaxSynthTopk];
    int have = 0;
    const int max_draws = 64 * num_topk;
    for (int c = 0; c < max_draws && have < num_topk; ++c) {
        const uint32_t u = mix32(th + uint32_t(c) * 0x9e3779b9u);
        int lo = 0, hi = num_experts - 1;  // first index with cdf[idx] >= u
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (cdf[mid] >= u) hi = mid; else lo = mid + 1;
        }
        bool seen = false;
        for (int j = 0; j < have; ++j) seen |= chosen[j] == lo;
        if (!seen) chosen[have++] = lo;
    }
    for (int e = 0; e < num_experts && have < num_topk; ++e) {
        bool seen = false;
        for (int j = 0; j < have; ++j) seen |= chosen[j] == e;
        if (!seen) chosen[have++] = e;
    }
    int64_t* out = topk_idx + id * num_topk;
    for (int k = 0; k < num_topk; ++k) out[k] = k < have ? chosen[k] : -1;
}

// Remote experts' answers for this rank's own pairs.  One wave per (expert,
// slot); waves past the expert's count, and local experts, exit at once.
__global__ __launch_bounds__(256) void combine_from_peers_kernel(
    const uint8_t* __restrict__ send_slots, const int32_t* __restrict__ send_count, int hidden, int num_experts,
    int num_local_experts, int rank, int max_tokens, int fmt, int mode, uint32_t seed,
    uint8_t* __restrict__ combine_staging) {
    const int lane = lane_id();
    const int64_t item = int64_t(blockIdx.x) * 4 + wave_in_block();
    if (item >= int64_t(num_experts) * max_tokens) return;
    const int e = int(item / max_tokens);
    const int j = int(item - int64_t(e) * max_tokens);
    if (e / num_local_experts == rank) return;
    if (j >= send_count[e]) return;
    uint8_t* dst = combine_staging + item * hidden * 2;
    if (mode == 1) {
        wave_fill_synth_row(dst, hidden, row_hash(seed, uint32_t(item)), 0, lane);
        return;
    }
    const int64_t data_pad = align16(row_data_bytes(hidden, fmt));
    const uint8_t* src = send_slots + item * row_stride_bytes(hidden, fmt);
    const int num_vec = hidden / 8;
    for (int v = lane; v < num_vec; v += kWave) {
        u32x4 o;
        if (fmt == kRowBF16) {
            o = *reinterpret_cast<const u32x4*>(src + int64_t(v) * 16);
        } else {
            const u32x2 q = *reinterpret_cast<const u32x2*>(src + int64_t(v) * 8);
            const int group = v / 16;
            float scale;
            if (fmt == kRowFP8UE8M0)
                scale = __uint_as_float(uint32_t(src[data_pad + group]) << 23);
            else
                scale = *reinterpret_cast<const float*>(src + data_pad + int64_t(group) * 4);
            float f[8];
            f[0] = __builtin_amdgcn_cvt_f32_fp8(int(q[0]), 0);
            f[1] = __builtin_amdgcn_cvt_f32_fp8(int(q[0]), 1);
            f[2] = __builtin_amdgcn_cvt_f32_fp8(int(q[0]), 2);
            f[3] = __builtin_amdgcn_cvt_f32_fp8(int(q[0]), 3);
            f[4] = __builtin_amdgcn_cvt_f32_fp8(int(q[1]), 0);
            f[5] = __builtin_amdgcn_cvt_f32_fp8(int(q[1]), 1);
            f[6] = __builtin_amdgcn_cvt_f32_fp8(int(q[1]), 2);
            f[7] = __builtin_amdgcn_cvt_f32_fp8(int(q[1]), 3);
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] = pack_bf16x2(f[2 * i] * scale, f[2 * i + 1] * scale);
        }
        *reinterpret_cast<u32x4*>(dst + int64_t(v) * 16) = o;
    }
}

}  // namespace deepep

using namespace deepep;

extern "C" {

int deepep_synth_topk_idx(const uint32_t* expert_cdf, const int32_t* src_ranks, int num_src, int num_tokens,
                          int num_topk, int num_experts, uint32_t seed, int64_t* topk_idx, void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_src >= 0 && num_tokens >= 0);
    EP_HOST_ASSERT(num_topk > 0 && num_topk <= kMaxSynthTopk && num_experts >= num_topk);
    const int64_t n = int64_t(num_src) * num_tokens;
    if (n == 0) return 0;
    EP_HOST_ASSERT(expert_cdf != nullptr && src_ranks != nullptr && topk_idx != nullptr);
    const int64_t blocks = (n + 255) / 256;
    EP_HOST_ASSERT(blocks < (int64_t(1) << 31));
    synth_topk_kernel<<<dim3(unsigned(blocks)), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        expert_cdf, src_ranks, num_src, num_tokens, num_topk, num_experts, seed, topk_idx);
    EP_LAUNCH_CHECK();
    return 0;
}

int deepep_synth_bf16_rows(void* dst, int64_t num_rows, int hidden, int64_t row_stride_bytes,
                           const uint32_t* row_keys, uint32_t first_key, uint32_t seed, int outlier_period,
                           void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_rows >= 0 && hidden > 0 && hidden % 8 == 0);
    EP_HOST_ASSERT(row_stride_bytes >= int64_t(hidden) * 2 && row_stride_bytes % 16 == 0);
    EP_HOST_ASSERT(outlier_period >= 0);
    if (num_rows == 0) return 0;
    EP_HOST_ASSERT(dst != nullptr && (reinterpret_cast<uintptr_t>(dst) & 15) == 0);
    int64_t blocks = (num_rows + 3) / 4;
    if (blocks > 16384) blocks = 16384;
    synth_bf16_rows_kernel<<<dim3(unsigned(blocks)), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        reinterpret_cast<uint8_t*>(dst), num_rows, hidden, row_stride_bytes, row_keys, first_key, seed,
        outlier_period);
    EP_LAUNCH_CHECK();
    return 0;
}

int deepep_loopback_combine_from_peers(const void* send_slots, const int32_t* send_count, int hidden,
                                       int num_experts, int num_ranks, int rank,
                                       int num_max_dispatch_tokens_per_rank, int row_format, int mode, uint32_t seed,
                                       void* combine_staging, void* stream) {
    clear_error();
    EP_HOST_ASSERT(hidden > 0 && hidden % 128 == 0);
    EP_HOST_ASSERT(num_ranks > 0 && num_experts > 0 && num_experts % num_ranks == 0);
    EP_HOST_ASSERT(rank >= 0 && rank < num_ranks && num_max_dispatch_tokens_per_rank > 0);
    EP_HOST_ASSERT(row_format >= kRowBF16 && row_format <= kRowFP8UE8M0);
    EP_HOST_ASSERT(mode == 0 || mode == 1);
    EP_HOST_ASSERT(send_count != nullptr && combine_staging != nullptr);
    EP_HOST_ASSERT(mode == 1 || send_slots != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(send_slots) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(combine_staging) & 15) == 0);
    const int64_t items = int64_t(num_experts) * num_max_dispatch_tokens_per_rank;
    const int64_t blocks = (items + 3) / 4;
    EP_HOST_ASSERT(blocks < (int64_t(1) << 31));
    combine_from_peers_kernel<<<dim3(unsigned(blocks)), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        reinterpret_cast<const uint8_t*>(send_slots), send_count, hidden, num_experts, num_experts / num_ranks, rank,
        num_max_dispatch_tokens_per_rank, row_format, mode, seed, reinterpret_cast<uint8_t*>(combine_staging));
    EP_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
