// Helpers for kernels that walk a list of variable-length row segments with
// one wavefront per row: a 256-thread exclusive scan in LDS, the row ->
// segment search, and the 16-byte-per-lane row copy.
#pragma once

#include "common.hpp"

namespace deepep {

// ---------------------------------------------------------------------
// Exclusive prefix of n ints held in LDS, by a 256-thread workgroup.
// data[n] receives the total.
// ---------------------------------------------------------------------
__device__ __forceinline__ void block_exclusive_scan_256(int32_t* data, int n, int32_t* wave_totals) {
    const int tid = threadIdx.x, lane = lane_id(), w = tid >> 6;
    const int per = (n + 255) / 256;
    const int lo = tid * per;
    int sum = 0;
    for (int j = 0; j < per; ++j)
        if (lo + j < n) sum += data[lo + j];
    const int incl = wave_inclusive_sum(sum);
    if (lane == kWave - 1) wave_totals[w] = incl;
    __syncthreads();
    int offset = incl - sum;
    for (int w2 = 0; w2 < w; ++w2) offset += wave_totals[w2];
    int total = 0;
    for (int w2 = 0; w2 < 4; ++w2) total += wave_totals[w2];
    int run = offset;
    for (int j = 0; j < per; ++j)
        if (lo + j < n) {
            const int v = data[lo + j];
            data[lo + j] = run;
            run += v;
        }
    if (tid == 0) data[n] = total;
    __syncthreads();
}

// Largest seg with flat[seg] <= row, for flat[] non-decreasing, flat[0] = 0.
__device__ __forceinline__ int find_segment(const int32_t* flat, int num_segments, int row) {
    int lo = 0, hi = num_segments;  // invariant: flat[lo] <= row < flat[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (flat[mid] <= row) lo = mid; else hi = mid;
    }
    return lo;
}

// Copies `num_vec` 16-byte vectors with one wave, eight loads in flight per lane.
__device__ __forceinline__ void wave_copy_vec16(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                int num_vec, int lane) {
    const u32x4* s = reinterpret_cast<const u32x4*>(src);
    u32x4* d = reinterpret_cast<u32x4*>(dst);
    for (int base = 0; base < num_vec; base += kWave * 8) {
        u32x4 r[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int v = base + u * kWave + lane;
            if (v < num_vec) r[u] = s[v];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int v = base + u * kWave + lane;
            if (v < num_vec) d[v] = r[u];
        }
    }
}

}  // namespace deepep
