// Per-128-channel FP8 quantisation of one token row, as one 8-lane cluster
// per group: each lane owns 16 consecutive channels (32 B in, 16 B out).
//
// Semantics (reference: csrc/kernels/efa_kernels.cu:143-169,
// deep_ep/buffer.py:1597-1605): amax = max(max|x|, 1e-4); scale = amax/448;
// q = e4m3fn_rne(clamp(x * (448/amax), -448, 448)).  Division is IEEE (hipcc
// keeps fp32 division correctly rounded unless fast-math is asked for).
#pragma once

#include "common.hpp"

namespace deepep {

// Smallest power of two >= s for a positive normal float, from the bit
// pattern (the exact value of exp2(ceil(log2(s)))).
__device__ __forceinline__ uint32_t pow2_ceil_exponent(float s) {
    const uint32_t bits = __float_as_uint(s);
    uint32_t ex = (bits >> 23) & 0xffu;
    if (bits & 0x7fffffu) ex += 1;
    return ex;
}

// in_lo/in_hi: 16 bf16 channels of this lane.  Returns the 16 e4m3 bytes and,
// in every lane of the 8-lane cluster, the group's scale.
//   scale_bits: float32 bit pattern of the scale (formats FP8 / POW2 / UE8M0).
template <int kFmt>
__device__ __forceinline__ u32x4 quantise_16(const u32x4 in_lo, const u32x4 in_hi, uint32_t& scale_bits) {
    float v[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = bf16_lo(in_lo[i]);
        v[2 * i + 1] = bf16_hi(in_lo[i]);
        v[8 + 2 * i] = bf16_lo(in_hi[i]);
        v[8 + 2 * i + 1] = bf16_hi(in_hi[i]);
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(v[i]));
    amax = max_over_8_lanes(amax);
    amax = fmaxf(amax, 1e-4f);

    float inv;
    if constexpr (kFmt == kRowFP8) {
        scale_bits = __float_as_uint(amax / 448.0f);
        inv = 448.0f / amax;
    } else {
        const uint32_t ex = pow2_ceil_exponent(amax / 448.0f);
        scale_bits = ex << 23;
        inv = __uint_as_float((254u - ex) << 23);  // exact reciprocal of a power of two
    }

    u32x4 q;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float a = fminf(fmaxf(v[4 * i + 0] * inv, -448.0f), 448.0f);
        float b = fminf(fmaxf(v[4 * i + 1] * inv, -448.0f), 448.0f);
        float c = fminf(fmaxf(v[4 * i + 2] * inv, -448.0f), 448.0f);
        float d = fminf(fmaxf(v[4 * i + 3] * inv, -448.0f), 448.0f);
        int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
        q[i] = uint32_t(w);
    }
    return q;
}

}  // namespace deepep
