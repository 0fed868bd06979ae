// Library-level entry points: error text, ABI revision and the buffer-size
// arithmetic kept for API parity with the reference.
#include <algorithm>
#include <cstdio>
#include <string>

#include "common.hpp"
#include "../../include/deepep_hip.h"

namespace deepep {

static thread_local std::string g_last_error;

void set_error(const char* kind, const char* file, int line, const char* what) {
    g_last_error = std::string("Failed: ") + kind + " error " + file + ":" + std::to_string(line) + " '" + what + "'";
}

void clear_error() { g_last_error.clear(); }

}  // namespace deepep

extern "C" {

const char* deepep_last_error(void) { return deepep::g_last_error.c_str(); }

int deepep_abi_version(void) { return DEEPEP_HIP_ABI_VERSION; }

// Same arithmetic as LowLatencyLayout (reference: csrc/config.hpp:127-193):
// two send buffers, two receive buffers and two 128-byte-aligned signalling
// areas, sized for bf16 messages, rounded up past the next 128 bytes.
size_t deepep_get_low_latency_rdma_size_hint(int num_max_dispatch_tokens_per_rank, int hidden, int num_ranks,
                                             int num_experts) {
    (void)num_ranks;
    const size_t m = size_t(num_max_dispatch_tokens_per_rank), h = size_t(hidden), e = size_t(num_experts);
    const size_t num_scales = h / 128;
    const size_t dispatch_msg = 16 + std::max(h * 2, h + num_scales * 4);
    const size_t combine_msg = num_scales * 4 + h * 2;
    const size_t send_bytes = std::max(m * dispatch_msg, e * m * combine_msg);
    const size_t recv_bytes = std::max(e * m * dispatch_msg, e * m * combine_msg);
    const size_t signal_bytes = ((e * sizeof(int) + 127) / 128) * 128;
    const size_t total = send_bytes * 2 + recv_bytes * 2 + signal_bytes * 2;
    return ((total + 128) / 128) * 128;
}

}  // extern "C"
