// Measuring sticks for bench.py: kernels with the memory traffic of a hot-path kernel and nothing
// else.  Built into bench_probe.so beside bench.py; not part of libdeepep_hip.so or its header.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "deepep_efa_amd/csrc/common.hpp"

using namespace deepep;

// The dispatch send side's access pattern: one workgroup per token reads the token's row (two 16-byte
// vectors per thread) and stores one vector per thread to each of the token's K destination rows, with
// streaming stores.  No routing, no quantisation, no scales.
__global__ __launch_bounds__(1024) void row_scatter_probe_kernel(const uint8_t* __restrict__ x, int64_t x_row_bytes,
                                                                 const int32_t* __restrict__ dst_rows, int num_topk,
                                                                 uint8_t* __restrict__ dst, int64_t dst_stride,
                                                                 int vecs) {
    const int t = blockIdx.x, tid = threadIdx.x;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (tid < vecs) {
        const uint8_t* src = x + int64_t(t) * x_row_bytes + int64_t(tid) * 32;
        const u32x4 a = *reinterpret_cast<const u32x4*>(src), b = *reinterpret_cast<const u32x4*>(src + 16);
        v = a ^ b;
    }
    for (int k = 0; k < num_topk; ++k) {
        const int row = dst_rows[int64_t(t) * num_topk + k];
        if (row >= 0 && tid < vecs) store_u32x4<true>(dst + int64_t(row) * dst_stride + int64_t(tid) * 16, v);
    }
}

// A plain streaming copy of `bytes` bytes, one 16-byte vector per thread and 1024 threads per
// workgroup: what a contiguous copy reaches on this GPU, for scale beside the row copies.
__global__ __launch_bounds__(1024) void stream_copy_probe_kernel(const uint8_t* __restrict__ src,
                                                                 uint8_t* __restrict__ dst, int64_t vecs) {
    for (int64_t v = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; v < vecs; v += int64_t(gridDim.x) * blockDim.x)
        store_u32x4<true>(dst + v * 16, load_u32x4<true>(src + v * 16));
}

extern "C" {

// x [T, hidden] 2-byte elements; dst_rows [T, K] int32 row index (-1 = none); the first `hidden` bytes of
// each named row of dst (rows of dst_stride_bytes) are written.  Returns 0, or 1 on a bad argument.
int bench_probe_row_scatter(const void* x, int num_tokens, int hidden, const int32_t* dst_rows, int num_topk,
                            void* dst, int64_t dst_stride_bytes, void* stream) {
    if (num_tokens < 0 || hidden <= 0 || hidden % 16 != 0 || hidden / 16 > 1024 || num_topk <= 0) return 1;
    if (dst_stride_bytes < hidden || dst_stride_bytes % 16 != 0) return 1;
    if (num_tokens == 0) return 0;
    if (x == nullptr || dst_rows == nullptr || dst == nullptr) return 1;
    if ((reinterpret_cast<uintptr_t>(x) & 15) != 0 || (reinterpret_cast<uintptr_t>(dst) & 15) != 0) return 1;
    const int vecs = hidden / 16;
    row_scatter_probe_kernel<<<dim3(unsigned(num_tokens)), ((vecs + 63) / 64) * 64, 0,
                               reinterpret_cast<hipStream_t>(stream)>>>(
        reinterpret_cast<const uint8_t*>(x), int64_t(hidden) * 2, dst_rows, num_topk, reinterpret_cast<uint8_t*>(dst),
        dst_stride_bytes, vecs);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

int bench_probe_stream_copy(const void* src, void* dst, int64_t bytes, void* stream) {
    if (bytes < 0 || bytes % 16 != 0 || src == nullptr || dst == nullptr) return 1;
    if ((reinterpret_cast<uintptr_t>(src) & 15) != 0 || (reinterpret_cast<uintptr_t>(dst) & 15) != 0) return 1;
    if (bytes == 0) return 0;
    const int64_t vecs = bytes / 16;
    int64_t blocks = (vecs + 1023) / 1024;
    if (blocks > (int64_t(1) << 20)) blocks = int64_t(1) << 20;
    stream_copy_probe_kernel<<<unsigned(blocks), 1024, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        reinterpret_cast<const uint8_t*>(src), reinterpret_cast<uint8_t*>(dst), vecs);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // extern "C"
