// Host-side error plumbing and device helpers shared by every kernel file.
// gfx950 only: 64-lane wavefronts, DPP lane exchange, hardware OCP-FP8 and
// BF16 pack conversions.
#pragma once
#include <cstdlib>

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace deepep {

// ---------------------------------------------------------------------
// Host errors.  Message format follows the reference's EPException
// (csrc/kernels/exception.cuh:12-22): "Failed: <kind> error <file>:<line> '<what>'".
// ---------------------------------------------------------------------
void set_error(const char* kind, const char* file, int line, const char* what);
void clear_error();

#define EP_HOST_ASSERT(cond)                                                      \
    do {                                                                          \
        if (!(cond)) {                                                            \
            ::deepep::set_error("Assertion", __FILE_NAME__, __LINE__, #cond);     \
            return 1;                                                             \
        }                                                                         \
    } while (0)

#define EP_HIP_CHECK(cmd)                                                                   \
    do {                                                                                    \
        hipError_t e_ = (cmd);                                                              \
        if (e_ != hipSuccess) {                                                             \
            ::deepep::set_error("HIP", __FILE_NAME__, __LINE__, hipGetErrorString(e_));     \
            return 2;                                                                       \
        }                                                                                   \
    } while (0)

#define EP_LAUNCH_CHECK() EP_HIP_CHECK(hipGetLastError())

// Row formats; values are part of the C ABI.
enum RowFormat : int { kRowBF16 = 0, kRowFP8 = 1, kRowFP8Pow2 = 2, kRowFP8UE8M0 = 3 };

// Hook for a timing build: a harness that wants per-phase timestamps defines DEEPEP_PHASE(i)
// before including the kernels; the library compiles it away.
#ifndef DEEPEP_PHASE
#define DEEPEP_PHASE(i)
#endif

constexpr int kWave = 64;
constexpr int kGroup = 128;        // channels per FP8 scale group
constexpr int kRowTailBytes = 16;  // {src_token, topk_slot, src_rank, local expert}

__host__ __device__ inline int64_t align16(int64_t v) { return (v + 15) & ~int64_t(15); }

__host__ __device__ inline int64_t row_data_bytes(int hidden, int fmt) {
    return fmt == kRowBF16 ? int64_t(hidden) * 2 : int64_t(hidden);
}
__host__ __device__ inline int64_t row_scale_bytes(int hidden, int fmt) {
    if (fmt == kRowBF16) return 0;
    const int g = hidden / kGroup;
    return fmt == kRowFP8UE8M0 ? g : int64_t(g) * 4;
}
// Payload of a staged row: [data | pad16][scales | pad16][tail], what the reference's cooperative send
// calls its stride (csrc/kernels/coop_dispatch_send.cu:73-75).
__host__ __device__ inline int64_t row_payload_bytes(int hidden, int fmt) {
    return align16(row_data_bytes(hidden, fmt)) + align16(row_scale_bytes(hidden, fmt)) + kRowTailBytes;
}
// Distance between staged rows: the payload rounded up to whole 128-byte cache lines, so that a row
// never shares a line with its neighbour.  When the rows come from HBM rather than from the caches
// the send kernel and the receive copy run about 4 % faster than at the bare payload size.
constexpr int kRowAlign = 128;
__host__ __device__ inline int64_t row_stride_bytes(int hidden, int fmt) {
    return (row_payload_bytes(hidden, fmt) + kRowAlign - 1) / kRowAlign * kRowAlign;
}

// ---------------------------------------------------------------------
// Device helpers
// ---------------------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int lane_id() { return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

// Wave index inside the workgroup as a scalar, so everything derived from it
// stays in SGPRs and row addresses become scalar loads.
__device__ __forceinline__ int wave_in_block() { return __builtin_amdgcn_readfirstlane(int(threadIdx.x) >> 6); }

// Stores through a pointer the compiler cannot prove to be global memory (one rebuilt from
// integers, say) are emitted as flat stores, which also tick the LDS counter; these say "global".
typedef __attribute__((address_space(1))) u32x4 global_u32x4;
typedef __attribute__((address_space(1))) uint32_t global_u32;
typedef __attribute__((address_space(1))) uint8_t global_u8;
__device__ __forceinline__ void store_global(uint8_t* p, u32x4 v) { *(global_u32x4*)(p) = v; }
__device__ __forceinline__ void store_global(uint8_t* p, uint32_t v) { *(global_u32*)(p) = v; }
__device__ __forceinline__ u32x4 load_global_u32x4(const uint8_t* p) { return *(const global_u32x4*)(p); }
__device__ __forceinline__ void store_global_byte(uint8_t* p, uint8_t v) { *(global_u8*)(p) = v; }

// Streaming variants for kernels whose traffic exceeds what the caches hold: the non-temporal hint
// keeps lines that will not be touched again from displacing others.  On this GPU a plain device
// copy of 512 MiB runs at 6.1 TB/s with ordinary accesses and 6.6 TB/s with these; eight gathered
// loads in flight per lane read at 6.2 against 7.0 TB/s.  kStream == false is the ordinary access.
template <bool kStream>
__device__ __forceinline__ u32x4 load_u32x4(const uint8_t* p) {
    if constexpr (kStream) return __builtin_nontemporal_load((const global_u32x4*)(p));
    else return *(const global_u32x4*)(p);
}
template <bool kStream>
__device__ __forceinline__ void store_u32x4(uint8_t* p, u32x4 v) {
    if constexpr (kStream) __builtin_nontemporal_store(v, (global_u32x4*)(p));
    else *(global_u32x4*)(p) = v;
}
// Traffic above which a kernel streams (the memory-side cache holds 256 MB).
inline int64_t stream_bytes() { return int64_t(192) << 20; }
// The dispatch streams from 64 MB of traffic on (the send side's payload stores; in the single launch
// the receive side's row copies too): with clean caches the hint makes no difference from 512 to 2560
// tokens, with the caches full of another call's dirty lines the send is 18 to 24 % faster with it and
// the single launch 11 to 16 %.  (The single-launch combine measured the other way: slower at 256 and
// 512 tokens with the lower bound, so it keeps the 192 MB.)
inline int64_t send_stream_bytes() { return int64_t(64) << 20; }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
// outstanding global load and store of the wave, which stalls kernels that keep row loads in
// flight across the barrier; use this one where threads exchange data through LDS alone.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// A 64-bit value every lane of the wave holds alike, moved to scalar registers.
__device__ __forceinline__ uint64_t wave_uniform_u64(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane(uint32_t(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(uint32_t(v >> 32));
    return (uint64_t(hi) << 32) | lo;
}

__device__ __forceinline__ uint64_t lanes_below(int lane) { return (uint64_t(1) << lane) - 1; }

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }

// float32 -> bf16 bits, round to nearest even (NaN kept quiet).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}

// max over the 8 lanes that share one 128-channel group (lanes 8i..8i+7):
// two quad permutes and a half-row mirror, all DPP — no LDS traffic.
__device__ __forceinline__ float max_over_8_lanes(float v) {
    int t;
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false);   // quad_perm [1,0,3,2]
    v = fmaxf(v, __int_as_float(t));
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false);   // quad_perm [2,3,0,1]
    v = fmaxf(v, __int_as_float(t));
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, false);  // row_half_mirror
    v = fmaxf(v, __int_as_float(t));
    return v;
}

// Inclusive sum over the wave (lane i gets sum of lanes 0..i), all DPP: a log-step shift-add inside
// each row of 16 lanes, then lane 15 of rows 0 and 2 broadcast into rows 1 and 3, then lane 31 into
// rows 2 and 3.
__device__ __forceinline__ int wave_inclusive_sum(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1, 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2, 3
    return v;
}

__device__ __forceinline__ int wave_sum(int v) {
#pragma unroll
    for (int d = kWave / 2; d >= 1; d >>= 1) v += __shfl_xor(v, d, kWave);
    return v;
}

// 32-bit integer mixer used by the seeded synthesiser (lowbias32 constants).
__host__ __device__ inline uint32_t mix32(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

}  // namespace deepep
