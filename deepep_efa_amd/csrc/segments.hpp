// Helpers for kernels that walk a list of variable-length row segments with
// one wavefront per row: a 256-thread exclusive scan in LDS, the row ->
// segment search, and the 16-byte-per-lane row copy.
#pragma once

#include <cstdlib>

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

// Copies 16-byte vectors [v_begin, v_end) of a row with one wave, eight loads
// in flight per lane.
__device__ __forceinline__ void wave_copy_vec16(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                int v_begin, int v_end, int lane) {
    const u32x4* s = reinterpret_cast<const u32x4*>(src);
    u32x4* d = reinterpret_cast<u32x4*>(dst);
    for (int base = v_begin; base < v_end; base += kWave * 8) {
        u32x4 r[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int v = base + u * kWave + lane;
            if (v < v_end) r[u] = s[v];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int v = base + u * kWave + lane;
            if (v < v_end) d[v] = r[u];
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

// Host-side choice of `parts`: small problems cannot fill the chip with one wave per row.
inline int choose_row_parts(int64_t max_rows, int64_t row_bytes) {
    if (const char* s = getenv("DEEPEP_ROW_PARTS")) {
        const int v = atoi(s);
        if (v >= 1 && v <= 8) return v;
    }
    if (max_rows > (int64_t(1) << 18)) return 1;
    return row_bytes > 8192 ? 4 : 2;
}

}  // namespace deepep
