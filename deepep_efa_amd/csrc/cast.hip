// Stand-alone per-token FP8 cast (the dispatch path fuses the same
// arithmetic into its send kernel).  One wave = 8 scale groups of one row.
#include "common.hpp"
#include "quant.hpp"
#include "../../include/deepep_hip.h"

namespace deepep {

// kStream: the rows exceed what the caches are worth spending on (they are read once), so they are loaded
// with the non-temporal hint: 16.5 against 17.5 us at 4096 x 7168 with the rows coming from HBM.  The
// results are stored the ordinary way in either case: whoever packs or sends them next reads them.
template <int kFmt, bool kStream>
__global__ __launch_bounds__(256) void per_token_cast_kernel(const uint8_t* __restrict__ x, int64_t num_rows,
                                                             int num_cols, int pieces_per_row,
                                                             uint8_t* __restrict__ x_fp8,
                                                             uint8_t* __restrict__ scales) {
    const int lane = lane_id();
    const int64_t item = int64_t(blockIdx.x) * 4 + wave_in_block();
    if (item >= num_rows * pieces_per_row) return;
    const int64_t row = item / pieces_per_row;
    const int piece = int(item - row * pieces_per_row);
    const int groups = num_cols / kGroup;
    const int group = piece * 8 + (lane >> 3);
    const bool live = group < groups;
    u32x4 lo = {0u, 0u, 0u, 0u}, hi = {0u, 0u, 0u, 0u};
    if (live) {
        const uint8_t* src = x + (row * num_cols + int64_t(group) * kGroup + (lane & 7) * 16) * 2;
        lo = load_u32x4<kStream>(src);
        hi = load_u32x4<kStream>(src + 16);
    }
    uint32_t scale_bits;
    const u32x4 q = quantise_16<kFmt>(lo, hi, scale_bits);
    if (!live) return;
    *reinterpret_cast<u32x4*>(x_fp8 + row * num_cols + int64_t(group) * kGroup + (lane & 7) * 16) = q;
    if ((lane & 7) == 0) {
        if constexpr (kFmt == kRowFP8UE8M0)
            scales[row * groups + group] = uint8_t(scale_bits >> 23);  // 4 exponent bytes per int32, little endian
        else
            *reinterpret_cast<uint32_t*>(scales + (row * groups + group) * 4) = scale_bits;
    }
}

}  // namespace deepep

using namespace deepep;

extern "C" int deepep_per_token_cast_to_fp8(const void* x, int num_rows, int num_cols, int row_format, void* x_fp8,
                                            void* scales, void* stream) {
    clear_error();
    EP_HOST_ASSERT(num_rows >= 0 && num_cols > 0 && num_cols % 128 == 0);
    EP_HOST_ASSERT(row_format == kRowFP8 || row_format == kRowFP8Pow2 || row_format == kRowFP8UE8M0);
    EP_HOST_ASSERT(row_format != kRowFP8UE8M0 || (num_cols / 128) % 4 == 0);
    if (num_rows == 0) return 0;
    EP_HOST_ASSERT(x != nullptr && x_fp8 != nullptr && scales != nullptr);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(x_fp8) & 15) == 0);
    EP_HOST_ASSERT((reinterpret_cast<uintptr_t>(scales) & 3) == 0);
    const int pieces = (num_cols / kGroup + 7) / 8;
    const int64_t blocks = (int64_t(num_rows) * pieces + 3) / 4;
    EP_HOST_ASSERT(blocks < (int64_t(1) << 31));
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const uint8_t* xb = reinterpret_cast<const uint8_t*>(x);
    uint8_t* qb = reinterpret_cast<uint8_t*>(x_fp8);
    uint8_t* sb = reinterpret_cast<uint8_t*>(scales);
    const bool streams = int64_t(num_rows) * num_cols * 3 > send_stream_bytes();
#define DEEPEP_LAUNCH_CAST(FMT)                                                                                  \
    do {                                                                                                         \
        if (streams)                                                                                             \
            per_token_cast_kernel<FMT, true><<<dim3(unsigned(blocks)), 256, 0, s>>>(xb, num_rows, num_cols, pieces, qb, sb);  \
        else                                                                                                     \
            per_token_cast_kernel<FMT, false><<<dim3(unsigned(blocks)), 256, 0, s>>>(xb, num_rows, num_cols, pieces, qb, sb); \
    } while (0)
    switch (row_format) {
        case kRowFP8: DEEPEP_LAUNCH_CAST(kRowFP8); break;
        case kRowFP8Pow2: DEEPEP_LAUNCH_CAST(kRowFP8Pow2); break;
        default: DEEPEP_LAUNCH_CAST(kRowFP8UE8M0); break;
    }
#undef DEEPEP_LAUNCH_CAST
    EP_LAUNCH_CHECK();
    return 0;
}
