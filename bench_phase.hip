// Timing build of the low-latency kernels for bench.py --phase-marks: the same sources as the library,
// with the DEEPEP_PHASE(i) hook writing the 100 MHz wall clock into a log the harness hands over.
// Per workgroup 16 slots: 0-7 are mark i as wave 0 of the workgroup passes it, 8-15 as its last wave does.
// Nothing in libdeepep_hip.so comes from this file.
#include <hip/hip_runtime.h>
#include <stdint.h>

__device__ uint64_t* g_phase_log = nullptr;

__device__ __forceinline__ void bench_phase_mark(int i) {
    if ((threadIdx.x & 63) == 0 && g_phase_log != nullptr) {
        const int w = threadIdx.x >> 6;
        const int64_t block = (int64_t(blockIdx.z) * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
        if (w == 0) g_phase_log[block * 16 + i] = wall_clock64();
        else if (w == (blockDim.x >> 6) - 1) g_phase_log[block * 16 + 8 + i] = wall_clock64();
    }
}
#define DEEPEP_PHASE(i) bench_phase_mark(i)

#include "deepep_efa_amd/csrc/ll_dispatch.hip"
#include "deepep_efa_amd/csrc/ll_combine.hip"

// log: device memory, [workgroups of the largest launch][16] uint64, zero-filled by the caller before a launch;
// NULL switches the marks off again.
extern "C" int bench_phase_set_log(uint64_t* log) {
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_phase_log), &log, sizeof(log));
}
