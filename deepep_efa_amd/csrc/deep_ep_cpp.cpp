// deep_ep_cpp — pybind11 host module with the reference's Python-visible surface for the
// dispatch/combine hot path (reference bindings: csrc/deep_ep.cpp:4310-4357,4440-4476).
//
// It owns tensors, checks arguments the way the reference's host code does
// (EP_HOST_ASSERT -> "Failed: Assertion error file:line 'cond'"), hands HIP
// streams around, and calls the C ABI of libdeepep_hip.so for every kernel.
// There is no device code in this file and no CPU fallback: a missing or
// failing HIP library is an exception.
#include <torch/extension.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPGraphsC10Utils.h>
#include <pybind11/functional.h>

#include <algorithm>
#include <functional>
#include <memory>
#include <optional>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "../../include/deepep_hip.h"

namespace deep_ep {

// PyTorch-ROCm tags its HIP streams with the CUDA device type; events and tensors expect that tag.
using HostStream = c10::hip::HIPStreamMasqueradingAsCUDA;
using topk_idx_t = int64_t;  // reference: csrc/kernels/configs.cuh:66-72 (TOPK_IDX_BITS = 64)
constexpr int kNumMaxNvlPeers = 8;            // reference: NUM_MAX_NVL_PEERS, csrc/kernels/configs.cuh:3
constexpr int kNumBufferAlignmentBytes = 128;  // reference: csrc/kernels/configs.cuh:7
constexpr int kSourceMetaBytes = 8;            // reference: internode::get_source_meta_bytes()

class EPException : public std::exception {
    std::string message;

public:
    EPException(const char* name, const char* file, int line, const std::string& error) {
        message = std::string("Failed: ") + name + " error " + file + ":" + std::to_string(line) + " '" + error + "'";
    }
    explicit EPException(std::string text) : message(std::move(text)) {}
    const char* what() const noexcept override { return message.c_str(); }
};

#define EP_HOST_ASSERT(cond)                                                          \
    do {                                                                              \
        if (!(cond)) throw ::deep_ep::EPException("Assertion", "deep_ep_cpp.cpp", __LINE__, #cond); \
    } while (0)

// A failed C-ABI call already carries an EPException-shaped message.
static void abi_check(int rc) {
    if (rc != 0) throw EPException(std::string(deepep_last_error()));
}

static hipStream_t current_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

template <typename T>
static T align_up(T a, T b) {
    return (a + b - 1) / b * b;
}

// ---------------------------------------------------------------------------
// Config (reference: csrc/config.hpp:23-105) — arithmetic only.
// ---------------------------------------------------------------------------
struct Config {
    int num_sms;
    int num_max_nvl_chunked_send_tokens;
    int num_max_nvl_chunked_recv_tokens;
    int num_max_rdma_chunked_send_tokens;
    int num_max_rdma_chunked_recv_tokens;

    Config(int num_sms, int nvl_send, int nvl_recv, int rdma_send, int rdma_recv)
        : num_sms(num_sms),
          num_max_nvl_chunked_send_tokens(nvl_send),
          num_max_nvl_chunked_recv_tokens(nvl_recv),
          num_max_rdma_chunked_send_tokens(rdma_send),
          num_max_rdma_chunked_recv_tokens(rdma_recv) {
        EP_HOST_ASSERT(num_sms >= 0);
        EP_HOST_ASSERT(nvl_send > 0 and nvl_recv > 0);
        EP_HOST_ASSERT(nvl_send < nvl_recv);
        EP_HOST_ASSERT(rdma_send > 0 and rdma_recv > 0);
        num_max_rdma_chunked_recv_tokens = align_up<int>(rdma_recv, rdma_send);
        EP_HOST_ASSERT(rdma_send < num_max_rdma_chunked_recv_tokens);
        EP_HOST_ASSERT(rdma_send <= num_max_rdma_chunked_recv_tokens / 2);
    }

    size_t get_nvl_buffer_size_hint(size_t hidden_bytes, int num_ranks) const {
        constexpr size_t kNumMaxTopK = 128, kNumMaxScales = 128;
        EP_HOST_ASSERT(num_ranks < kNumMaxNvlPeers or num_ranks % kNumMaxNvlPeers == 0);
        EP_HOST_ASSERT(num_ranks <= kNumMaxNvlPeers or num_sms % 2 == 0);
        const size_t num_rdma_ranks = std::max(num_ranks / kNumMaxNvlPeers, 1);
        const size_t num_nvl_ranks = std::min(num_ranks, kNumMaxNvlPeers);
        const size_t num_channels = num_sms / 2;
        const size_t recv = num_max_nvl_chunked_recv_tokens;
        size_t num_bytes = 0;
        num_bytes += num_channels * num_nvl_ranks * (2 * num_rdma_ranks + 3) * sizeof(int);
        num_bytes += num_channels * num_nvl_ranks * recv * hidden_bytes;
        num_bytes += num_channels * num_nvl_ranks * recv * kSourceMetaBytes;
        num_bytes += num_channels * num_nvl_ranks * recv * kNumMaxTopK * sizeof(topk_idx_t);
        num_bytes += num_channels * num_nvl_ranks * recv * kNumMaxTopK * sizeof(float);
        num_bytes += num_channels * num_nvl_ranks * recv * kNumMaxScales * sizeof(float);
        return ((num_bytes + 127) / 128) * 128;
    }

    size_t get_rdma_buffer_size_hint(int64_t hidden_bytes, int num_ranks) const {
        if (num_ranks <= kNumMaxNvlPeers) return 0;
        constexpr size_t kNumMaxTopK = 128, kNumMaxScales = 128;
        EP_HOST_ASSERT(num_ranks % kNumMaxNvlPeers == 0);
        EP_HOST_ASSERT(num_sms % 2 == 0);
        const size_t num_rdma_ranks = num_ranks / kNumMaxNvlPeers;
        const size_t num_channels = num_sms / 2;
        const size_t recv = num_max_rdma_chunked_recv_tokens;
        size_t num_bytes = 0;
        num_bytes += num_channels * num_rdma_ranks * (kNumMaxNvlPeers * 2 + 2) * 2 * sizeof(int);
        num_bytes += num_channels * num_rdma_ranks * recv * size_t(hidden_bytes) * 2;
        num_bytes += num_channels * num_rdma_ranks * recv * kSourceMetaBytes * 2;
        num_bytes += num_channels * num_rdma_ranks * recv * kNumMaxTopK * sizeof(topk_idx_t) * 2;
        num_bytes += num_channels * num_rdma_ranks * recv * kNumMaxTopK * sizeof(float) * 2;
        num_bytes += num_channels * num_rdma_ranks * recv * kNumMaxScales * sizeof(float) * 2;
        num_bytes += num_channels * num_rdma_ranks * recv * 16 * 2;
        return ((num_bytes + 127) / 128) * 128;
    }
};

static size_t get_low_latency_rdma_size_hint(int num_max_dispatch_tokens_per_rank, int hidden, int num_ranks,
                                             int num_experts) {
    return deepep_get_low_latency_rdma_size_hint(num_max_dispatch_tokens_per_rank, hidden, num_ranks, num_experts);
}

// ---------------------------------------------------------------------------
// EventHandle (reference: csrc/event.hpp:9-25)
// ---------------------------------------------------------------------------
struct EventHandle {
    std::shared_ptr<torch::Event> event;

    EventHandle() {
        event = std::make_shared<torch::Event>(torch::kCUDA);
        event->record(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA());
    }
    explicit EventHandle(const HostStream& stream) {
        event = std::make_shared<torch::Event>(torch::kCUDA);
        event->record(stream);
    }
    void current_stream_wait() const { c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().unwrap().wait(*event); }
};

static void stream_wait(const HostStream& waiter, const HostStream& other) {
    EP_HOST_ASSERT(waiter.id() != other.id());
    torch::Event ev(torch::kCUDA);
    ev.record(other);
    waiter.unwrap().wait(ev);
}

static void stream_wait(const HostStream& waiter, const EventHandle& event) {
    waiter.unwrap().wait(*event.event);
}

// ---------------------------------------------------------------------------
// Low-latency tensors of one shape (reference: the Python-side cache of
// deep_ep/buffer.py:1623-1813; nothing here is cleared per call)
// ---------------------------------------------------------------------------
struct LowLatencyCache {
    int max_tokens = 0, hidden = 0, num_topk = 0, num_experts = 0, row_format = -1;
    torch::Tensor recv_staging, recv_count, send_slots, send_count, pair_slot, workspace, segment_workspace;
    torch::Tensor packed_recv_x, packed_recv_scales, packed_recv_count, packed_recv_src_info, packed_recv_layout_range;
    torch::Tensor combine_staging, combine_send_slots, combined_x;
    bool dispatched = false;
};

static int row_format_of(bool use_fp8, bool round_scale, bool use_ue8m0) {
    if (!use_fp8) return DEEPEP_ROW_BF16;
    if (use_ue8m0) return DEEPEP_ROW_FP8_UE8M0;
    return round_scale ? DEEPEP_ROW_FP8_POW2 : DEEPEP_ROW_FP8;
}

// ---------------------------------------------------------------------------
// Buffer (reference: csrc/deep_ep.hpp:60-707, csrc/deep_ep.cpp:206-581)
// One process, one GPU.  `num_ranks`/`rank` describe the expert-parallel world
// this GPU plays a part in; the other ranks exist only as tensors handed to
// loopback_set_world().
// ---------------------------------------------------------------------------
struct Buffer {
    int rank, num_ranks, rdma_rank, nvl_rank, num_rdma_ranks, num_nvl_ranks;
    int64_t num_nvl_bytes, num_rdma_bytes;
    bool low_latency_mode, explicitly_destroy, enable_shrink;
    bool available = false, destroyed = false;
    int device_id = 0;
    HostStream comm_stream;
    torch::Tensor nvl_buffer, rdma_buffer, mask_status;
    std::unordered_map<int64_t, torch::Tensor> layout_workspaces;  // one per stream that has run the layout kernel
    static constexpr size_t kMaxLayoutWorkspaces = 8;
    LowLatencyCache ll;
    std::vector<torch::Tensor> combine_input_buffers;
    int combine_buffer_idx = 0;
    // Rows the last large dispatch received, read back without blocking: the next large call is sized by it.
    // (Under skewed routing a rank can receive many times num_tokens * num_topk rows; the row-copy kernels
    // take their grid from the rows expected, and one sized for a balanced world walks such a batch in a slow loop.)
    torch::Tensor observed_count_host;
    std::optional<torch::Event> observed_ready;
    int64_t observed_rows = 0;
    // loopback world
    std::optional<torch::Tensor> world_x, world_topk_idx;
    torch::Tensor ranks_below, ranks_above, peer_workspace;
    int combine_peer_mode = 0;
    uint32_t combine_peer_seed = 0;

    Buffer(int rank, int num_ranks, int64_t num_nvl_bytes, int64_t num_rdma_bytes, bool low_latency_mode,
           bool explicitly_destroy, bool enable_shrink, bool use_fabric)
        : rank(rank),
          num_ranks(num_ranks),
          num_nvl_bytes(num_nvl_bytes),
          num_rdma_bytes(num_rdma_bytes),
          low_latency_mode(low_latency_mode),
          explicitly_destroy(explicitly_destroy),
          enable_shrink(enable_shrink),
          comm_stream(c10::hip::getStreamFromPoolMasqueradingAsCUDA(false)) {  // default priority
        (void)use_fabric;
        EP_HOST_ASSERT(num_ranks > 0 and 0 <= rank and rank < num_ranks);
        EP_HOST_ASSERT(num_nvl_bytes % kNumBufferAlignmentBytes == 0 and num_rdma_bytes % kNumBufferAlignmentBytes == 0);
        EP_HOST_ASSERT(num_ranks <= kNumMaxNvlPeers or num_ranks % kNumMaxNvlPeers == 0 or low_latency_mode);
        rdma_rank = rank / kNumMaxNvlPeers;
        nvl_rank = rank % kNumMaxNvlPeers;
        num_rdma_ranks = std::max(1, num_ranks / kNumMaxNvlPeers);
        num_nvl_ranks = std::min(num_ranks, kNumMaxNvlPeers);
        device_id = c10::hip::current_device();
    }

    ~Buffer() noexcept(false) {
        if (!explicitly_destroy) {
            destroy();
        } else if (!destroyed) {
            printf("WARNING: destroy() was not called before DeepEP buffer destruction, which can leak resources.\n");
            fflush(stdout);
        }
    }

    bool is_available() const { return available; }
    bool is_internode_available() const { return is_available() and num_ranks > kNumMaxNvlPeers; }
    int get_num_rdma_ranks() const { return num_rdma_ranks; }
    int get_rdma_rank() const { return rdma_rank; }
    int get_root_rdma_rank(bool global) const { return global ? nvl_rank : 0; }
    int get_local_device_id() const { return device_id; }
    pybind11::bytearray get_local_ipc_handle() const { return pybind11::bytearray(std::string(64, '\0')); }
    c10::Stream get_comm_stream() const { return comm_stream.unwrap(); }

    // One GPU: nothing to open on peers; the call only marks the buffer usable.
    void sync(const std::vector<int>& device_ids, const std::vector<std::optional<pybind11::bytearray>>& handles,
              const std::optional<pybind11::bytearray>& root_unique_id) {
        (void)handles;
        (void)root_unique_id;
        EP_HOST_ASSERT(not is_available());
        EP_HOST_ASSERT(device_ids.empty() or static_cast<int>(device_ids.size()) == num_ranks or device_ids.size() == 1);
        available = true;
    }

    void destroy() {
        if (destroyed) return;
        if (available) (void)hipDeviceSynchronize();
        nvl_buffer = torch::Tensor();
        rdma_buffer = torch::Tensor();
        layout_workspaces.clear();
        ll = LowLatencyCache();
        observed_ready.reset();
        observed_count_host = torch::Tensor();
        combine_input_buffers.clear();
        world_x.reset();
        world_topk_idx.reset();
        peer_workspace = torch::Tensor();
        destroyed = true;
        available = false;
    }

    torch::Tensor get_local_buffer_tensor(const pybind11::object& dtype, int64_t offset, bool use_rdma_buffer) {
        torch::ScalarType casted = torch::python::detail::py_object_to_dtype(dtype);
        const int64_t element_bytes = static_cast<int64_t>(elementSize(casted));
        torch::Tensor& base = use_rdma_buffer ? rdma_buffer : nvl_buffer;
        const int64_t num_bytes = use_rdma_buffer ? num_rdma_bytes : num_nvl_bytes;
        if (!base.defined())  // allocated on first use; valid until destroy()
            base = torch::empty({std::max<int64_t>(num_bytes, 16)}, torch::dtype(torch::kUInt8).device(torch::kCUDA));
        EP_HOST_ASSERT(offset >= 0 and offset <= num_bytes);
        auto bytes = base.narrow(0, offset, ((num_bytes - offset) / element_bytes) * element_bytes);
        return bytes.view(casted);
    }

    // -- layout ---------------------------------------------------------------
    std::tuple<torch::Tensor, std::optional<torch::Tensor>, torch::Tensor, torch::Tensor, std::optional<EventHandle>>
    get_dispatch_layout(const torch::Tensor& topk_idx, int num_experts, std::optional<EventHandle>& previous_event,
                        bool async, bool allocate_on_comm_stream) {
        EP_HOST_ASSERT(topk_idx.dim() == 2);
        EP_HOST_ASSERT(topk_idx.is_contiguous());
        EP_HOST_ASSERT(topk_idx.is_cuda() and topk_idx.scalar_type() == torch::kInt64);
        EP_HOST_ASSERT(num_experts > 0);

        auto compute_stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
        // A synchronous call with nothing to wait for is ordered on the caller's stream either way: the
        // reference moves the work to its communication stream and back through two events
        // (csrc/deep_ep.cpp:526-537,559-574), which on this GPU costs more than the kernels (27 us against 7);
        // here such a call runs on the caller's stream directly.  Every other form keeps the hand-off.
        const bool in_place = not async and not previous_event.has_value() and not allocate_on_comm_stream;
        auto work_stream = in_place ? compute_stream : comm_stream;
        if (allocate_on_comm_stream) {
            EP_HOST_ASSERT(previous_event.has_value() and async);
            c10::hip::setCurrentHIPStreamMasqueradingAsCUDA(comm_stream);
        }
        if (previous_event.has_value())
            stream_wait(comm_stream, previous_event.value());
        else if (not in_place)
            stream_wait(comm_stream, compute_stream);

        const int num_tokens = static_cast<int>(topk_idx.size(0)), num_topk = static_cast<int>(topk_idx.size(1));
        auto i32 = torch::dtype(torch::kInt32).device(torch::kCUDA);
        auto num_tokens_per_rank = torch::empty({num_ranks}, i32);
        auto num_tokens_per_rdma_rank = std::optional<torch::Tensor>();
        auto num_tokens_per_expert = torch::empty({num_experts}, i32);
        auto is_token_in_rank = torch::empty({num_tokens, num_ranks}, torch::dtype(torch::kBool).device(torch::kCUDA));
        if (is_internode_available()) num_tokens_per_rdma_rank = torch::empty({num_rdma_ranks}, i32);

        const int64_t ws_bytes =
            std::max<int64_t>(256, int64_t(deepep_layout_workspace_bytes(num_tokens, num_ranks, num_experts)));
        // the kernel's scratch belongs to the stream the kernel runs on: a call on the buffer's own stream and
        // one on the caller's stream may be in flight together
        if (layout_workspaces.size() >= kMaxLayoutWorkspaces and layout_workspaces.count(int64_t(work_stream.id())) == 0)
            layout_workspaces.clear();  // a caller cycling through streams does not grow the table without bound
        torch::Tensor& layout_workspace = layout_workspaces[int64_t(work_stream.id())];
        if (!layout_workspace.defined() or layout_workspace.numel() < ws_bytes) {
            // allocated with the kernel's stream current, so that the caching allocator ties the block to that
            // stream: a block dropped here (replaced, or the table cleared) is handed out again only to
            // allocations ordered behind the kernels that used it
            c10::hip::HIPStreamGuardMasqueradingAsCUDA on_work_stream(work_stream.unwrap());
            layout_workspace = torch::empty({ws_bytes}, torch::dtype(torch::kUInt8).device(torch::kCUDA));
        }

        abi_check(deepep_get_dispatch_layout(
            topk_idx.data_ptr<int64_t>(), num_tokens, num_topk, num_ranks, num_experts,
            num_tokens_per_rank.data_ptr<int>(),
            num_tokens_per_rdma_rank.has_value() ? num_tokens_per_rdma_rank->data_ptr<int>() : nullptr,
            num_tokens_per_expert.data_ptr<int>(), reinterpret_cast<uint8_t*>(is_token_in_rank.data_ptr<bool>()),
            layout_workspace.data_ptr(), size_t(layout_workspace.numel()), work_stream.stream()));

        std::optional<EventHandle> event;
        if (async) {
            event = EventHandle(comm_stream);
            for (auto& t : {topk_idx, num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank}) {
                t.record_stream(comm_stream);
                if (allocate_on_comm_stream) t.record_stream(compute_stream);
            }
            if (num_tokens_per_rdma_rank.has_value()) {
                num_tokens_per_rdma_rank->record_stream(comm_stream);
                if (allocate_on_comm_stream) num_tokens_per_rdma_rank->record_stream(compute_stream);
            }
        } else if (not in_place) {
            stream_wait(compute_stream, comm_stream);
        }
        if (allocate_on_comm_stream) c10::hip::setCurrentHIPStreamMasqueradingAsCUDA(compute_stream);
        return {num_tokens_per_rank, num_tokens_per_rdma_rank, num_tokens_per_expert, is_token_in_rank, event};
    }

    // -- loopback world ---------------------------------------------------------
    void loopback_set_world(const torch::Tensor& x_all, const torch::Tensor& topk_idx_all) {
        EP_HOST_ASSERT(x_all.dim() == 3 and x_all.is_contiguous() and x_all.is_cuda());
        EP_HOST_ASSERT(x_all.scalar_type() == torch::kBFloat16);
        EP_HOST_ASSERT(topk_idx_all.dim() == 3 and topk_idx_all.is_contiguous() and topk_idx_all.is_cuda());
        EP_HOST_ASSERT(topk_idx_all.scalar_type() == torch::kInt64);
        EP_HOST_ASSERT(x_all.size(0) == num_ranks and topk_idx_all.size(0) == num_ranks);
        EP_HOST_ASSERT(x_all.size(1) == topk_idx_all.size(1));
        world_x = x_all;
        world_topk_idx = topk_idx_all;
        auto i32 = torch::dtype(torch::kInt32).device(torch::kCUDA);
        ranks_below = torch::arange(0, rank, i32);
        ranks_above = torch::arange(rank + 1, num_ranks, i32);
    }

    void loopback_clear_world() {
        world_x.reset();
        world_topk_idx.reset();
    }

    void loopback_synthesise(int num_tokens, int hidden, int num_topk, int num_experts, const torch::Tensor& expert_cdf,
                             int outlier_period, int64_t seed) {
        EP_HOST_ASSERT(expert_cdf.is_cuda() and expert_cdf.is_contiguous() and expert_cdf.numel() == num_experts);
        EP_HOST_ASSERT(expert_cdf.element_size() == 4);
        auto ranks = torch::arange(0, num_ranks, torch::dtype(torch::kInt32).device(torch::kCUDA));
        auto topk = torch::empty({num_ranks, num_tokens, num_topk}, torch::dtype(torch::kInt64).device(torch::kCUDA));
        auto x = torch::empty({num_ranks, num_tokens, hidden}, torch::dtype(torch::kBFloat16).device(torch::kCUDA));
        abi_check(deepep_synth_topk_idx(reinterpret_cast<const uint32_t*>(expert_cdf.data_ptr()), ranks.data_ptr<int>(),
                                        num_ranks, num_tokens, num_topk, num_experts, uint32_t(seed),
                                        topk.data_ptr<int64_t>(), current_stream()));
        abi_check(deepep_synth_bf16_rows(x.data_ptr(), int64_t(num_ranks) * num_tokens, hidden, int64_t(hidden) * 2,
                                         nullptr, 0, uint32_t(seed), outlier_period, current_stream()));
        loopback_set_world(x, topk);
    }

    std::tuple<torch::Tensor, torch::Tensor> loopback_own_inputs() const {
        EP_HOST_ASSERT(world_x.has_value());
        return {world_x->select(0, rank), world_topk_idx->select(0, rank)};
    }

    std::tuple<torch::Tensor, torch::Tensor> loopback_world() const {
        EP_HOST_ASSERT(world_x.has_value());
        return {*world_x, *world_topk_idx};
    }

    void loopback_set_combine_mode(int mode, int64_t seed) {
        EP_HOST_ASSERT(mode == 0 or mode == 1);
        combine_peer_mode = mode;
        combine_peer_seed = uint32_t(seed);
    }

    // -- low latency ------------------------------------------------------------
    LowLatencyCache& get_ll_cache(int max_tokens, int hidden, int num_topk, int num_experts, int fmt) {
        if (ll.max_tokens == max_tokens and ll.hidden == hidden and ll.num_topk == num_topk and
            ll.num_experts == num_experts and ll.row_format == fmt)
            return ll;
        ll = LowLatencyCache();
        ll.max_tokens = max_tokens, ll.hidden = hidden, ll.num_topk = num_topk, ll.num_experts = num_experts;
        ll.row_format = fmt;
        const int64_t el = num_experts / num_ranks, r = num_ranks, m = max_tokens, e = num_experts, h = hidden;
        const int64_t stride = int64_t(deepep_ll_row_stride(hidden, fmt));
        auto u8 = torch::dtype(torch::kUInt8).device(torch::kCUDA);
        auto i32 = torch::dtype(torch::kInt32).device(torch::kCUDA);
        auto bf16 = torch::dtype(torch::kBFloat16).device(torch::kCUDA);
        ll.recv_staging = torch::empty({el * r * m * stride}, u8);
        ll.recv_count = torch::zeros({el * r}, i32);
        ll.send_slots = torch::empty({e * m * stride}, u8);
        ll.send_count = torch::zeros({e}, i32);
        ll.pair_slot = torch::full({m, num_topk}, -1, i32);
        ll.workspace = torch::empty(
            {std::max<int64_t>(256, int64_t(deepep_ll_dispatch_workspace_bytes(max_tokens, num_topk, num_experts)))}, u8);
        if (int64_t(m) * num_topk > 8192)  // index + flat-copy scratch, only used by large batches
            ll.segment_workspace =
                torch::empty({int64_t(deepep_ll_segment_workspace_bytes(num_experts, max_tokens))}, u8);
        if (fmt == DEEPEP_ROW_BF16) {
            ll.packed_recv_x = torch::empty({el, r * m, h}, bf16);
        } else {
            ll.packed_recv_x = torch::empty({el, r * m, h}, torch::dtype(torch::kFloat8_e4m3fn).device(torch::kCUDA));
            if (fmt == DEEPEP_ROW_FP8_UE8M0)
                ll.packed_recv_scales = torch::empty({el, r * m, h / 512}, i32);
            else
                ll.packed_recv_scales = torch::empty({el, r * m, h / 128}, torch::dtype(torch::kFloat32).device(torch::kCUDA));
        }
        ll.packed_recv_count = torch::zeros({el}, i32);
        ll.packed_recv_src_info = torch::empty({el, r * m}, i32);
        ll.packed_recv_layout_range = torch::zeros({el, r}, torch::dtype(torch::kInt64).device(torch::kCUDA));
        ll.combine_staging = torch::empty({e, m, h}, bf16);
        ll.combine_send_slots = torch::empty({el, r, m, h}, bf16);
        ll.combined_x = torch::empty({m, h}, bf16);
        return ll;
    }

    void stage_peer_rows(LowLatencyCache& c) {
        if (!world_x.has_value()) return;
        const int t = static_cast<int>(world_x->size(1)), h = static_cast<int>(world_x->size(2));
        const int k = static_cast<int>(world_topk_idx->size(2));
        EP_HOST_ASSERT(h == c.hidden and k == c.num_topk and t <= c.max_tokens);
        const int64_t per = int64_t(deepep_ll_dispatch_workspace_bytes(t, k, c.num_experts));
        const int64_t need = std::max<int64_t>(256, per * std::max({rank, num_ranks - 1 - rank, 1}));
        if (!peer_workspace.defined() or peer_workspace.numel() < need)
            peer_workspace = torch::empty({need}, torch::dtype(torch::kUInt8).device(torch::kCUDA));
        const torch::Tensor* groups[2] = {&ranks_below, &ranks_above};
        const int first[2] = {0, rank + 1};
        for (int g = 0; g < 2; ++g) {
            const int n = static_cast<int>(groups[g]->numel());
            if (n == 0) continue;
            abi_check(deepep_loopback_dispatch_from_peers(
                world_x->select(0, first[g]).data_ptr(), world_topk_idx->select(0, first[g]).data_ptr<int64_t>(),
                groups[g]->data_ptr<int>(), n, t, h, k, c.num_experts, num_ranks, rank, c.max_tokens, c.row_format,
                c.recv_staging.data_ptr(), c.recv_count.data_ptr<int>(), peer_workspace.data_ptr(),
                size_t(peer_workspace.numel()), current_stream()));
        }
    }

    std::tuple<torch::Tensor, std::optional<torch::Tensor>, torch::Tensor, torch::Tensor, torch::Tensor,
               std::optional<EventHandle>, std::optional<std::function<void()>>>
    low_latency_dispatch(const torch::Tensor& x, const torch::Tensor& topk_idx,
                         const std::optional<torch::Tensor>& cumulative_local_expert_recv_stats,
                         const std::optional<torch::Tensor>& dispatch_wait_recv_cost_stats,
                         int num_max_dispatch_tokens_per_rank, int num_experts, bool use_fp8, bool round_scale,
                         bool use_ue8m0, bool async, bool return_recv_hook) {
        EP_HOST_ASSERT(low_latency_mode);
        // reference checks: csrc/deep_ep.cpp:1674-1693
        EP_HOST_ASSERT(x.dim() == 2 and x.is_contiguous() and x.scalar_type() == torch::kBFloat16);
        EP_HOST_ASSERT(x.is_cuda() and topk_idx.is_cuda());
        EP_HOST_ASSERT(x.size(1) % 16 == 0 and x.size(1) % 128 == 0);
        EP_HOST_ASSERT(topk_idx.dim() == 2 and topk_idx.is_contiguous());
        EP_HOST_ASSERT(x.size(0) == topk_idx.size(0) and x.size(0) <= num_max_dispatch_tokens_per_rank);
        EP_HOST_ASSERT(topk_idx.scalar_type() == torch::kInt64);
        EP_HOST_ASSERT(num_experts % num_ranks == 0);
        EP_HOST_ASSERT(not use_ue8m0 or round_scale);
        EP_HOST_ASSERT(not use_ue8m0 or (x.size(1) / 128) % 4 == 0);
        if (cumulative_local_expert_recv_stats.has_value()) {
            EP_HOST_ASSERT(cumulative_local_expert_recv_stats->scalar_type() == torch::kInt);
            EP_HOST_ASSERT(cumulative_local_expert_recv_stats->dim() == 1 and
                           cumulative_local_expert_recv_stats->is_contiguous());
            EP_HOST_ASSERT(cumulative_local_expert_recv_stats->size(0) == num_experts / num_ranks);
        }
        if (dispatch_wait_recv_cost_stats.has_value()) {
            EP_HOST_ASSERT(dispatch_wait_recv_cost_stats->scalar_type() == torch::kInt64);
            EP_HOST_ASSERT(dispatch_wait_recv_cost_stats->dim() == 1 and dispatch_wait_recv_cost_stats->is_contiguous());
            EP_HOST_ASSERT(dispatch_wait_recv_cost_stats->size(0) == num_ranks);
        }
        const int num_tokens = static_cast<int>(x.size(0)), hidden = static_cast<int>(x.size(1));
        const int num_topk = static_cast<int>(topk_idx.size(1));
        const int fmt = row_format_of(use_fp8, round_scale, use_ue8m0);
        auto& c = get_ll_cache(num_max_dispatch_tokens_per_rank, hidden, num_topk, num_experts, fmt);
        auto stream = current_stream();

        stage_peer_rows(c);  // what the exchange would have delivered
        // Large batches: the hint is what the dispatch before this one received, if that has arrived on the host
        const bool large = int64_t(num_tokens) * num_topk > 8192;
        int64_t expected_rows = std::max<int64_t>(num_tokens, 1) * num_topk;
        const bool capturing = c10::hip::currentStreamCaptureStatusMayInitCtx() != c10::hip::CaptureStatus::None;
        if (large) {
            // (an event may not be queried while a stream is being captured: a captured call keeps the last hint)
            if (not capturing and observed_ready.has_value() and observed_ready->query()) {
                observed_rows = observed_count_host.sum().item<int64_t>();
                observed_ready.reset();
            }
            expected_rows = std::max(expected_rows, observed_rows);
        }
        // send and receive phase in one call (one kernel launch for decode-sized batches)
        abi_check(deepep_ll_dispatch(
            x.data_ptr(), topk_idx.data_ptr<int64_t>(), num_tokens, hidden, num_topk, num_experts, num_ranks, rank,
            num_max_dispatch_tokens_per_rank, fmt, c.recv_staging.data_ptr(), c.recv_count.data_ptr<int>(),
            c.send_slots.data_ptr(), c.send_count.data_ptr<int>(), c.pair_slot.data_ptr<int>(),
            c.packed_recv_x.data_ptr(), c.packed_recv_scales.defined() ? c.packed_recv_scales.data_ptr() : nullptr,
            c.packed_recv_src_info.data_ptr<int>(), c.packed_recv_layout_range.data_ptr<int64_t>(),
            c.packed_recv_count.data_ptr<int>(),
            cumulative_local_expert_recv_stats.has_value() ? cumulative_local_expert_recv_stats->data_ptr<int>() : nullptr,
            expected_rows, c.workspace.data_ptr(),
            size_t(c.workspace.numel()), c.segment_workspace.defined() ? c.segment_workspace.data_ptr() : nullptr,
            c.segment_workspace.defined() ? size_t(c.segment_workspace.numel()) : 0, stream));
        c.dispatched = true;
        if (large and not capturing and not observed_ready.has_value()) {
            if (!observed_count_host.defined() or observed_count_host.numel() != c.packed_recv_count.numel())
                observed_count_host = torch::empty({c.packed_recv_count.numel()},
                                                   torch::dtype(torch::kInt32).pinned_memory(true));
            observed_count_host.copy_(c.packed_recv_count, /*non_blocking=*/true);
            observed_ready = torch::Event(torch::kCUDA);
            observed_ready->record(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA());
        }

        std::optional<EventHandle> event;
        if (async) event = EventHandle();
        std::optional<std::function<void()>> hook;
        if (return_recv_hook) hook = [] {};
        std::optional<torch::Tensor> scales;
        if (c.packed_recv_scales.defined()) scales = c.packed_recv_scales;
        return {c.packed_recv_x, scales, c.packed_recv_count, c.packed_recv_src_info, c.packed_recv_layout_range,
                event, hook};
    }

    std::tuple<torch::Tensor, std::optional<EventHandle>, std::optional<std::function<void()>>> low_latency_combine(
        const torch::Tensor& x, const torch::Tensor& topk_idx, const torch::Tensor& topk_weights,
        const torch::Tensor& src_info, const torch::Tensor& layout_range,
        const std::optional<torch::Tensor>& combine_wait_recv_cost_stats, int num_max_dispatch_tokens_per_rank,
        int num_experts, bool use_logfmt, bool zero_copy, bool async, bool return_recv_hook,
        const std::optional<torch::Tensor>& out, bool accumulate) {
        (void)use_logfmt;
        // accumulate: the sum starts from what `out` holds (the reference has the flag on its reduce binding,
        // csrc/deep_ep.cpp:3850-3857, kernel csrc/kernels/coop_combine_recv.cuh:174-179)
        EP_HOST_ASSERT(not accumulate or out.has_value());
        EP_HOST_ASSERT(low_latency_mode);
        // reference checks: csrc/deep_ep.cpp:1816-1837
        EP_HOST_ASSERT(x.dim() == 3 and x.is_contiguous() and x.scalar_type() == torch::kBFloat16);
        EP_HOST_ASSERT(x.size(0) == num_experts / num_ranks);
        EP_HOST_ASSERT(x.size(1) == int64_t(num_ranks) * num_max_dispatch_tokens_per_rank);
        EP_HOST_ASSERT(x.size(2) % 16 == 0 and x.size(2) % 128 == 0);
        EP_HOST_ASSERT(topk_idx.dim() == 2 and topk_idx.is_contiguous());
        EP_HOST_ASSERT(topk_idx.size(0) == topk_weights.size(0) and topk_idx.size(1) == topk_weights.size(1));
        EP_HOST_ASSERT(topk_idx.scalar_type() == torch::kInt64);
        EP_HOST_ASSERT(topk_weights.dim() == 2 and topk_weights.is_contiguous());
        EP_HOST_ASSERT(topk_weights.size(0) <= num_max_dispatch_tokens_per_rank);
        EP_HOST_ASSERT(topk_weights.scalar_type() == torch::kFloat32);
        EP_HOST_ASSERT(src_info.dim() == 2 and src_info.is_contiguous());
        EP_HOST_ASSERT(src_info.scalar_type() == torch::kInt32 and x.size(0) == src_info.size(0));
        EP_HOST_ASSERT(layout_range.dim() == 2 and layout_range.is_contiguous());
        EP_HOST_ASSERT(layout_range.scalar_type() == torch::kInt64);
        EP_HOST_ASSERT(layout_range.size(0) == num_experts / num_ranks and layout_range.size(1) == num_ranks);
        if (combine_wait_recv_cost_stats.has_value()) {
            EP_HOST_ASSERT(combine_wait_recv_cost_stats->scalar_type() == torch::kInt64);
            EP_HOST_ASSERT(combine_wait_recv_cost_stats->dim() == 1 and combine_wait_recv_cost_stats->is_contiguous());
            EP_HOST_ASSERT(combine_wait_recv_cost_stats->size(0) == num_ranks);
        }
        const int hidden = static_cast<int>(x.size(2));
        const int num_topk = static_cast<int>(topk_weights.size(1));
        const int num_combined_tokens = static_cast<int>(topk_weights.size(0));
        // the slots of this rank's own pairs were fixed by the dispatch that produced `handle`
        EP_HOST_ASSERT(ll.dispatched and ll.max_tokens == num_max_dispatch_tokens_per_rank and ll.hidden == hidden and
                       ll.num_topk == num_topk and ll.num_experts == num_experts);
        auto& c = ll;
        auto stream = current_stream();

        torch::Tensor src = x;
        // zero_copy: the caller wrote its expert outputs into the buffer handed out earlier, and that buffer is
        // what the transport sends from (the ranges of layout_range are contiguous in it), so the combine skips
        // the row return -- "the next combine kernel can skip the copying", deep_ep/buffer.py:2831-2852
        if (zero_copy) {
            EP_HOST_ASSERT(!combine_input_buffers.empty() and combine_input_buffers[combine_buffer_idx].defined());
            src = combine_input_buffers[combine_buffer_idx];
            EP_HOST_ASSERT(src.size(0) == x.size(0) and src.size(1) == x.size(1) and src.size(2) == x.size(2));
        }
        torch::Tensor combined_x;
        if (out.has_value()) {
            EP_HOST_ASSERT(out->dim() == 2 and out->is_contiguous() and out->scalar_type() == torch::kBFloat16);
            EP_HOST_ASSERT(out->size(0) == num_combined_tokens and out->size(1) == hidden);
            combined_x = out.value();
        } else {
            combined_x = c.combined_x.narrow(0, 0, num_combined_tokens);
        }

        if (world_x.has_value())  // what the remote experts would have returned
            abi_check(deepep_loopback_combine_from_peers(c.send_slots.data_ptr(), c.send_count.data_ptr<int>(), hidden,
                                                         num_experts, num_ranks, rank, num_max_dispatch_tokens_per_rank,
                                                         c.row_format, combine_peer_mode, combine_peer_seed,
                                                         c.combine_staging.data_ptr(), stream));
        // row return and weighted reduce in one call (one kernel launch for decode-sized batches)
        abi_check(deepep_ll_combine(src.data_ptr(), layout_range.data_ptr<int64_t>(), topk_idx.data_ptr<int64_t>(),
                                    topk_weights.data_ptr<float>(), c.pair_slot.data_ptr<int>(), num_combined_tokens,
                                    hidden, num_topk, num_experts, num_ranks, rank, num_max_dispatch_tokens_per_rank,
                                    accumulate ? 1 : 0, c.combine_staging.data_ptr(),
                                    zero_copy ? nullptr : c.combine_send_slots.data_ptr(),
                                    combined_x.data_ptr(),
                                    /*expected_rows=*/std::max<int64_t>(std::max<int64_t>(num_combined_tokens, 1) * num_topk,
                                                                         int64_t(num_combined_tokens) * num_topk > 8192 ? observed_rows : 0),
                                    c.segment_workspace.defined() ? c.segment_workspace.data_ptr() : nullptr,
                                    c.segment_workspace.defined() ? size_t(c.segment_workspace.numel()) : 0, stream));

        std::optional<EventHandle> event;
        if (async) event = EventHandle();
        std::optional<std::function<void()>> hook;
        if (return_recv_hook) hook = [] {};
        return {combined_x, event, hook};
    }

    torch::Tensor get_next_low_latency_combine_buffer(int num_max_dispatch_tokens_per_rank, int hidden, int num_experts) {
        EP_HOST_ASSERT(low_latency_mode);
        if (combine_input_buffers.empty()) combine_input_buffers.resize(2);
        auto& buf = combine_input_buffers[combine_buffer_idx];
        const int64_t el = num_experts / num_ranks, n = int64_t(num_ranks) * num_max_dispatch_tokens_per_rank;
        if (!buf.defined() or buf.size(0) != el or buf.size(1) != n or buf.size(2) != hidden)
            buf = torch::zeros({el, n, hidden}, torch::dtype(torch::kBFloat16).device(torch::kCUDA));
        return buf;
    }

    void clean_low_latency_buffer(int num_max_dispatch_tokens_per_rank, int hidden, int num_experts) {
        (void)num_max_dispatch_tokens_per_rank;
        (void)hidden;
        (void)num_experts;
        EP_HOST_ASSERT(low_latency_mode);
        combine_buffer_idx = 0;
        for (auto& b : combine_input_buffers)
            if (b.defined()) b.zero_();
        if (ll.recv_count.defined()) ll.recv_count.zero_();
        ll.dispatched = false;
    }

    void ensure_mask() {
        if (!mask_status.defined())
            mask_status = torch::zeros({num_ranks}, torch::dtype(torch::kInt32).device(torch::kCUDA));
    }
    void low_latency_update_mask_buffer(int rank_to_mask, bool mask) {
        EP_HOST_ASSERT(rank_to_mask >= 0 and rank_to_mask < num_ranks);
        ensure_mask();
        mask_status.select(0, rank_to_mask).fill_(mask ? 1 : 0);
    }
    void low_latency_query_mask_buffer(torch::Tensor& out) {
        EP_HOST_ASSERT(out.numel() == num_ranks and out.scalar_type() == torch::kInt32);
        ensure_mask();
        out.copy_(mask_status);
    }
    void low_latency_clean_mask_buffer() {
        if (mask_status.defined()) mask_status.zero_();
    }
};

// ---------------------------------------------------------------------------
// Free functions
// ---------------------------------------------------------------------------
// reference: csrc/kernels/efa_kernels.cu:2281-2327
static std::tuple<torch::Tensor, torch::Tensor> per_token_cast_to_fp8(const torch::Tensor& x, bool round_scale,
                                                                      bool use_ue8m0) {
    EP_HOST_ASSERT(x.dim() == 2 && x.is_contiguous() && x.is_cuda());
    EP_HOST_ASSERT(x.scalar_type() == torch::kBFloat16);
    const int m = static_cast<int>(x.size(0)), n = static_cast<int>(x.size(1));
    EP_HOST_ASSERT(n % 128 == 0);
    EP_HOST_ASSERT(not use_ue8m0 or round_scale);
    const int g = n / 128;
    auto x_fp8 = torch::empty({m, n}, torch::dtype(torch::kFloat8_e4m3fn).device(x.device()));
    torch::Tensor scales;
    if (use_ue8m0) {
        EP_HOST_ASSERT(g % 4 == 0);
        scales = torch::empty({m, g / 4}, torch::dtype(torch::kInt32).device(x.device()));
    } else {
        scales = torch::empty({m, g}, torch::dtype(torch::kFloat32).device(x.device()));
    }
    abi_check(deepep_per_token_cast_to_fp8(x.data_ptr(), m, n, row_format_of(true, round_scale, use_ue8m0),
                                           x_fp8.data_ptr(), scales.data_ptr(), current_stream()));
    return {x_fp8, scales};
}

// reference: csrc/kernels/efa_kernels.cu:1591-1651 (the .item() host sync is the reference's)
static std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, int64_t, torch::Tensor> routing_sort_impl(
    const torch::Tensor& is_token_in_rank, bool with_positions) {
    EP_HOST_ASSERT(is_token_in_rank.dim() == 2);
    EP_HOST_ASSERT(is_token_in_rank.scalar_type() == torch::kBool);
    EP_HOST_ASSERT(is_token_in_rank.is_contiguous());
    EP_HOST_ASSERT(is_token_in_rank.is_cuda());
    const int num_tokens = static_cast<int>(is_token_in_rank.size(0)), num_ranks = static_cast<int>(is_token_in_rank.size(1));
    auto dev = is_token_in_rank.device();
    auto send_counts = torch::empty({num_ranks}, torch::dtype(torch::kInt32).device(dev));
    auto send_cumsum = torch::empty({num_ranks + 1}, torch::dtype(torch::kInt64).device(dev));
    auto ids = torch::empty({std::max<int64_t>(1, int64_t(num_tokens) * num_ranks)}, torch::dtype(torch::kInt64).device(dev));
    auto ws = torch::empty({std::max<int64_t>(256, int64_t(deepep_routing_sort_workspace_bytes(num_tokens, num_ranks)))},
                           torch::dtype(torch::kUInt8).device(dev));
    torch::Tensor row_of_pair;
    if (with_positions) row_of_pair = torch::empty({num_tokens, num_ranks}, torch::dtype(torch::kInt32).device(dev));
    abi_check(deepep_moe_routing_sort(reinterpret_cast<const uint8_t*>(is_token_in_rank.data_ptr<bool>()), num_tokens,
                                      num_ranks, ids.data_ptr<int64_t>(), send_counts.data_ptr<int>(),
                                      send_cumsum.data_ptr<int64_t>(),
                                      with_positions and num_tokens > 0 ? row_of_pair.data_ptr<int>() : nullptr,
                                      ws.data_ptr(), size_t(ws.numel()), current_stream()));
    const int64_t total = send_cumsum.select(0, num_ranks).item<int64_t>();
    return {ids.slice(0, 0, total), send_counts, send_cumsum, total, row_of_pair};
}

static std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, int64_t> moe_routing_sort(const torch::Tensor& is_token_in_rank) {
    auto [ids, counts, cumsum, total, unused] = routing_sort_impl(is_token_in_rank, false);
    (void)unused;
    return {ids, counts, cumsum, total};
}

// The same plus row_of_pair [T, R] int32, the inverse of the list, which combine_reduce takes to run as one launch.
static std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, int64_t, torch::Tensor> moe_routing_sort_with_positions(
    const torch::Tensor& is_token_in_rank) {
    return routing_sort_impl(is_token_in_rank, true);
}

// reference: csrc/kernels/intranode.cu:90-112 (the channel part of notify_dispatch)
static torch::Tensor channel_prefix_matrix(const torch::Tensor& is_token_in_rank, int num_channels) {
    EP_HOST_ASSERT(is_token_in_rank.dim() == 2 and is_token_in_rank.is_contiguous() and is_token_in_rank.is_cuda());
    EP_HOST_ASSERT(is_token_in_rank.scalar_type() == torch::kBool);
    EP_HOST_ASSERT(num_channels > 0);
    const int num_tokens = static_cast<int>(is_token_in_rank.size(0)), num_ranks = static_cast<int>(is_token_in_rank.size(1));
    auto cpm = torch::empty({num_ranks, num_channels}, torch::dtype(torch::kInt32).device(is_token_in_rank.device()));
    abi_check(deepep_channel_prefix_matrix(reinterpret_cast<const uint8_t*>(is_token_in_rank.data_ptr<bool>()),
                                           num_tokens, num_ranks, num_channels, cpm.data_ptr<int>(), current_stream()));
    return cpm;
}

// reference: csrc/kernels/efa_kernels.cu:1653-1691 (same arguments, same outputs)
static std::tuple<torch::Tensor, torch::Tensor> topk_remap(const torch::Tensor& topk_idx, const torch::Tensor& topk_weights,
                                                           const torch::Tensor& sorted_token_ids,
                                                           const torch::Tensor& send_cumsum, int64_t total_send,
                                                           int num_ranks, int num_local_experts) {
    EP_HOST_ASSERT(topk_idx.dim() == 2);
    EP_HOST_ASSERT(topk_idx.is_contiguous() && topk_idx.is_cuda());
    EP_HOST_ASSERT(topk_weights.dim() == 2);
    EP_HOST_ASSERT(topk_weights.is_contiguous() && topk_weights.is_cuda());
    EP_HOST_ASSERT(topk_idx.scalar_type() == torch::kInt64 and topk_weights.scalar_type() == torch::kFloat32);
    EP_HOST_ASSERT(topk_weights.size(0) == topk_idx.size(0) and topk_weights.size(1) == topk_idx.size(1));
    EP_HOST_ASSERT(sorted_token_ids.scalar_type() == torch::kInt64 and sorted_token_ids.is_contiguous());
    EP_HOST_ASSERT(send_cumsum.scalar_type() == torch::kInt64 and send_cumsum.is_contiguous());
    EP_HOST_ASSERT(send_cumsum.numel() == num_ranks + 1);
    EP_HOST_ASSERT(total_send >= 0 and total_send <= sorted_token_ids.numel());
    const int num_topk = static_cast<int>(topk_idx.size(1));
    auto remapped_topk = torch::empty({total_send, num_topk}, topk_idx.options());
    auto remapped_weights = torch::empty({total_send, num_topk}, topk_weights.options());
    abi_check(deepep_topk_remap(topk_idx.data_ptr<int64_t>(), topk_weights.data_ptr<float>(),
                                sorted_token_ids.data_ptr<int64_t>(), send_cumsum.data_ptr<int64_t>(),
                                static_cast<int>(topk_idx.size(0)), num_topk, num_ranks, num_local_experts, total_send,
                                remapped_topk.data_ptr<int64_t>(), remapped_weights.data_ptr<float>(), current_stream()));
    return {remapped_topk, remapped_weights};
}

// reference: csrc/kernels/efa_kernels.cu:1726-1749 (recv_counts is accepted and not needed: the prefix has it)
static torch::Tensor build_recv_src_meta(const torch::Tensor& recv_counts, const torch::Tensor& recv_cumsum,
                                         int64_t num_recv_tokens, int num_ranks, int num_local_ranks) {
    EP_HOST_ASSERT(recv_counts.is_cuda() and recv_cumsum.is_cuda());
    EP_HOST_ASSERT(recv_cumsum.scalar_type() == torch::kInt64 and recv_cumsum.is_contiguous());
    EP_HOST_ASSERT(recv_cumsum.numel() == num_ranks + 1 and num_recv_tokens >= 0);
    auto meta = torch::empty({num_recv_tokens, 8}, torch::dtype(torch::kUInt8).device(recv_cumsum.device()));
    abi_check(deepep_build_recv_src_meta(recv_cumsum.data_ptr<int64_t>(), num_ranks, num_local_ranks, num_recv_tokens,
                                         meta.data_ptr<uint8_t>(), current_stream()));
    return meta;
}

// reference: csrc/transport/ll_pipeline.cpp:1204-1269,1277-1361 — the bookkeeping between the gather of the
// route counts and the exchange, on the stream instead of on the host.  Returns (send_counts [R] i32,
// recv_counts [R] i32, totals [3] i32 = sent / received / corrupt, combine_remote_recv_offset [R] i64,
// records [4, row_capacity] i32 = source_rank / source_offset / padded_index / combine_send_offset,
// num_recv_tokens [2] i32, tokens_per_expert [E_l] i32).
static std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor>
ll_exchange_metadata(const torch::Tensor& all_num_routed, int rank, int num_max_dispatch_tokens_per_rank,
                     int64_t row_capacity) {
    EP_HOST_ASSERT(all_num_routed.dim() == 2 and all_num_routed.is_contiguous() and all_num_routed.is_cuda());
    EP_HOST_ASSERT(all_num_routed.scalar_type() == torch::kInt32);
    EP_HOST_ASSERT(row_capacity >= 0);
    const int num_ranks = static_cast<int>(all_num_routed.size(0)), num_experts = static_cast<int>(all_num_routed.size(1));
    EP_HOST_ASSERT(num_ranks > 0 and num_experts % num_ranks == 0);
    const auto i32 = torch::dtype(torch::kInt32).device(all_num_routed.device());
    auto send_counts = torch::empty({num_ranks}, i32), recv_counts = torch::empty({num_ranks}, i32);
    auto totals = torch::empty({3}, i32), num_recv_tokens = torch::empty({2}, i32);
    auto remote = torch::empty({num_ranks}, i32.dtype(torch::kInt64));
    auto records = torch::empty({4, row_capacity}, i32);
    auto tokens_per_expert = torch::empty({num_experts / num_ranks}, i32);
    auto rec = [&](int i) { return reinterpret_cast<uint32_t*>(records.data_ptr<int>()) + int64_t(i) * row_capacity; };
    abi_check(deepep_ll_exchange_metadata(
        all_num_routed.data_ptr<int>(), num_experts, num_ranks, rank, num_max_dispatch_tokens_per_rank, row_capacity,
        send_counts.data_ptr<int>(), recv_counts.data_ptr<int>(), totals.data_ptr<int>(), remote.data_ptr<int64_t>(),
        rec(0), rec(1), rec(2), rec(3), reinterpret_cast<uint32_t*>(num_recv_tokens.data_ptr<int>()),
        reinterpret_cast<uint32_t*>(tokens_per_expert.data_ptr<int>()), current_stream()));
    return {send_counts, recv_counts, totals, remote, records, num_recv_tokens, tokens_per_expert};
}

// reference: deep_ep/buffer.py:1542-1557 — zero_() + index_add_ over the returned rows, then the biases
static std::tuple<torch::Tensor, std::optional<torch::Tensor>> combine_reduce(
    const torch::Tensor& recv_x, const std::optional<torch::Tensor>& recv_topk_weights,
    const torch::Tensor& sorted_token_ids, const torch::Tensor& send_cumsum, const torch::Tensor& is_token_in_rank,
    const std::optional<torch::Tensor>& bias_0, const std::optional<torch::Tensor>& bias_1,
    const std::optional<torch::Tensor>& row_of_pair) {
    EP_HOST_ASSERT(recv_x.dim() == 2 and recv_x.is_contiguous() and recv_x.is_cuda());
    EP_HOST_ASSERT(recv_x.scalar_type() == torch::kBFloat16);
    EP_HOST_ASSERT(is_token_in_rank.dim() == 2 and is_token_in_rank.is_contiguous());
    EP_HOST_ASSERT(is_token_in_rank.scalar_type() == torch::kBool);
    EP_HOST_ASSERT(sorted_token_ids.scalar_type() == torch::kInt64 and sorted_token_ids.is_contiguous());
    EP_HOST_ASSERT(send_cumsum.scalar_type() == torch::kInt64 and send_cumsum.is_contiguous());
    const int num_tokens = static_cast<int>(is_token_in_rank.size(0)), num_ranks = static_cast<int>(is_token_in_rank.size(1));
    const int hidden = static_cast<int>(recv_x.size(1));
    EP_HOST_ASSERT(send_cumsum.numel() == num_ranks + 1);
    const int64_t max_rows = std::min<int64_t>(recv_x.size(0), sorted_token_ids.numel());
    int num_topk = 0;
    if (recv_topk_weights.has_value()) {
        EP_HOST_ASSERT(recv_topk_weights->dim() == 2 and recv_topk_weights->is_contiguous());
        EP_HOST_ASSERT(recv_topk_weights->scalar_type() == torch::kFloat32 and recv_topk_weights->size(0) >= max_rows);
        num_topk = static_cast<int>(recv_topk_weights->size(1));
    }
    for (const auto* b : {&bias_0, &bias_1})
        if (b->has_value()) {
            EP_HOST_ASSERT((*b)->dim() == 2 and (*b)->is_contiguous() and (*b)->scalar_type() == torch::kBFloat16);
            EP_HOST_ASSERT((*b)->size(0) == num_tokens and (*b)->size(1) == hidden);
        }
    if (row_of_pair.has_value()) {
        EP_HOST_ASSERT(row_of_pair->scalar_type() == torch::kInt32 and row_of_pair->is_contiguous() and row_of_pair->is_cuda());
        EP_HOST_ASSERT(row_of_pair->dim() == 2 and row_of_pair->size(0) == num_tokens and row_of_pair->size(1) == num_ranks);
    }
    auto combined_x = torch::empty({num_tokens, hidden}, recv_x.options());
    std::optional<torch::Tensor> combined_w;
    if (recv_topk_weights.has_value()) combined_w = torch::empty({num_tokens, num_topk}, recv_topk_weights->options());
    auto ws = torch::empty({std::max<int64_t>(256, int64_t(deepep_combine_reduce_workspace_bytes(num_tokens, num_ranks)))},
                           torch::dtype(torch::kUInt8).device(recv_x.device()));
    abi_check(deepep_combine_reduce(
        recv_x.data_ptr(), recv_topk_weights.has_value() ? recv_topk_weights->data_ptr<float>() : nullptr,
        sorted_token_ids.data_ptr<int64_t>(), send_cumsum.data_ptr<int64_t>(),
        reinterpret_cast<const uint8_t*>(is_token_in_rank.data_ptr<bool>()),
        bias_0.has_value() ? bias_0->data_ptr() : nullptr, bias_1.has_value() ? bias_1->data_ptr() : nullptr, num_tokens,
        hidden, num_topk, num_ranks, max_rows, row_of_pair.has_value() ? row_of_pair->data_ptr<int>() : nullptr,
        combined_x.data_ptr(),
        combined_w.has_value() ? combined_w->data_ptr<float>() : nullptr, ws.data_ptr(), size_t(ws.numel()),
        current_stream()));
    return {combined_x, combined_w};
}

// reference: deep_ep/buffer.py:877,917 — send_x = x[sorted_ids], send_scales = scales[sorted_ids]
static std::tuple<torch::Tensor, std::optional<torch::Tensor>> pack_rows(const torch::Tensor& x,
                                                                         const std::optional<torch::Tensor>& x_scales,
                                                                         const torch::Tensor& sorted_token_ids,
                                                                         const torch::Tensor& send_cumsum) {
    EP_HOST_ASSERT(x.dim() == 2 and x.is_contiguous() and x.is_cuda());
    EP_HOST_ASSERT(sorted_token_ids.dim() == 1 and sorted_token_ids.is_contiguous());
    EP_HOST_ASSERT(sorted_token_ids.scalar_type() == torch::kInt64);
    EP_HOST_ASSERT(send_cumsum.scalar_type() == torch::kInt64 and send_cumsum.is_contiguous() and send_cumsum.numel() >= 1);
    const int64_t rows = sorted_token_ids.numel();
    const int64_t row_bytes = x.size(1) * x.element_size();
    EP_HOST_ASSERT(row_bytes % 16 == 0);
    auto out = torch::empty({rows, x.size(1)}, x.options());
    std::optional<torch::Tensor> out_scales;
    int64_t scale_row_bytes = 0;
    if (x_scales.has_value()) {
        EP_HOST_ASSERT(x_scales->dim() == 2 and x_scales->is_contiguous() and x_scales->size(0) == x.size(0));
        scale_row_bytes = x_scales->size(1) * x_scales->element_size();
        EP_HOST_ASSERT(scale_row_bytes % 4 == 0);
        out_scales = torch::empty({rows, x_scales->size(1)}, x_scales->options());
    }
    abi_check(deepep_pack_rows(x.data_ptr(), x_scales.has_value() ? x_scales->data_ptr() : nullptr,
                               sorted_token_ids.data_ptr<int64_t>(),
                               send_cumsum.data_ptr<int64_t>() + (send_cumsum.numel() - 1), rows,
                               static_cast<int>(x.size(0)), static_cast<int>(row_bytes), static_cast<int>(scale_row_bytes),
                               out.data_ptr(), out_scales.has_value() ? out_scales->data_ptr() : nullptr,
                               current_stream()));
    return {out, out_scales};
}

static bool is_sm90_compiled() { return true; }  // FP8 paths are always built for gfx950

}  // namespace deep_ep

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "DeepEP dispatch/combine hot path for MI355X (gfx950): host module over libdeepep_hip.so";

    pybind11::register_exception<deep_ep::EPException>(m, "EPException", PyExc_RuntimeError);

    pybind11::class_<deep_ep::Config>(m, "Config")
        .def(pybind11::init<int, int, int, int, int>(), py::arg("num_sms") = 20,
             py::arg("num_max_nvl_chunked_send_tokens") = 6, py::arg("num_max_nvl_chunked_recv_tokens") = 256,
             py::arg("num_max_rdma_chunked_send_tokens") = 6, py::arg("num_max_rdma_chunked_recv_tokens") = 256)
        .def_readonly("num_sms", &deep_ep::Config::num_sms)
        .def_readonly("num_max_nvl_chunked_send_tokens", &deep_ep::Config::num_max_nvl_chunked_send_tokens)
        .def_readonly("num_max_nvl_chunked_recv_tokens", &deep_ep::Config::num_max_nvl_chunked_recv_tokens)
        .def_readonly("num_max_rdma_chunked_send_tokens", &deep_ep::Config::num_max_rdma_chunked_send_tokens)
        .def_readonly("num_max_rdma_chunked_recv_tokens", &deep_ep::Config::num_max_rdma_chunked_recv_tokens)
        .def("get_nvl_buffer_size_hint", &deep_ep::Config::get_nvl_buffer_size_hint)
        .def("get_rdma_buffer_size_hint", &deep_ep::Config::get_rdma_buffer_size_hint);
    m.def("get_low_latency_rdma_size_hint", &deep_ep::get_low_latency_rdma_size_hint);

    pybind11::class_<deep_ep::EventHandle>(m, "EventHandle")
        .def(pybind11::init<>())
        .def("current_stream_wait", &deep_ep::EventHandle::current_stream_wait);

    pybind11::class_<deep_ep::Buffer>(m, "Buffer")
        .def(pybind11::init<int, int, int64_t, int64_t, bool, bool, bool, bool>())
        .def("is_available", &deep_ep::Buffer::is_available)
        .def("get_num_rdma_ranks", &deep_ep::Buffer::get_num_rdma_ranks)
        .def("get_rdma_rank", &deep_ep::Buffer::get_rdma_rank)
        .def("get_root_rdma_rank", &deep_ep::Buffer::get_root_rdma_rank)
        .def("get_local_device_id", &deep_ep::Buffer::get_local_device_id)
        .def("get_local_ipc_handle", &deep_ep::Buffer::get_local_ipc_handle)
        .def("get_local_buffer_tensor", &deep_ep::Buffer::get_local_buffer_tensor)
        .def("get_comm_stream", &deep_ep::Buffer::get_comm_stream)
        .def("sync", &deep_ep::Buffer::sync)
        .def("destroy", &deep_ep::Buffer::destroy)
        .def("get_dispatch_layout", &deep_ep::Buffer::get_dispatch_layout)
        .def("clean_low_latency_buffer", &deep_ep::Buffer::clean_low_latency_buffer)
        .def("low_latency_dispatch", &deep_ep::Buffer::low_latency_dispatch)
        .def("low_latency_combine", &deep_ep::Buffer::low_latency_combine, py::arg("x"), py::arg("topk_idx"),
             py::arg("topk_weights"), py::arg("src_info"), py::arg("layout_range"),
             py::arg("combine_wait_recv_cost_stats"), py::arg("num_max_dispatch_tokens_per_rank"),
             py::arg("num_experts"), py::arg("use_logfmt"), py::arg("zero_copy"), py::arg("async"),
             py::arg("return_recv_hook"), py::arg("out"), py::arg("accumulate") = false)
        .def("low_latency_update_mask_buffer", &deep_ep::Buffer::low_latency_update_mask_buffer)
        .def("low_latency_query_mask_buffer", &deep_ep::Buffer::low_latency_query_mask_buffer)
        .def("low_latency_clean_mask_buffer", &deep_ep::Buffer::low_latency_clean_mask_buffer)
        .def("get_next_low_latency_combine_buffer", &deep_ep::Buffer::get_next_low_latency_combine_buffer)
        .def("loopback_set_world", &deep_ep::Buffer::loopback_set_world)
        .def("loopback_clear_world", &deep_ep::Buffer::loopback_clear_world)
        .def("loopback_synthesise", &deep_ep::Buffer::loopback_synthesise)
        .def("loopback_own_inputs", &deep_ep::Buffer::loopback_own_inputs)
        .def("loopback_world", &deep_ep::Buffer::loopback_world)
        .def("loopback_set_combine_mode", &deep_ep::Buffer::loopback_set_combine_mode);

    m.def("is_sm90_compiled", deep_ep::is_sm90_compiled);
    m.attr("topk_idx_t") = py::reinterpret_borrow<py::object>(
        (PyObject*)torch::getTHPDtype(c10::CppTypeToScalarType<deep_ep::topk_idx_t>::value));

    m.def("per_token_cast_to_fp8", &deep_ep::per_token_cast_to_fp8,
          "Per-token FP8 e4m3 quantisation with 128-channel groups");
    m.def("moe_routing_sort", &deep_ep::moe_routing_sort, "Token ids grouped by destination rank");
    m.def("moe_routing_sort_with_positions", &deep_ep::moe_routing_sort_with_positions,
          "moe_routing_sort plus row_of_pair [T, R], the inverse of the list");
    m.def("channel_prefix_matrix", &deep_ep::channel_prefix_matrix, "Per-rank prefix of token counts over channels");
    m.def("pack_rows", &deep_ep::pack_rows, "Gather rows into per-rank contiguous send buffers");
    m.def("topk_remap", &deep_ep::topk_remap, "Top-k of the send rows in the destination rank's expert numbering");
    m.def("build_recv_src_meta", &deep_ep::build_recv_src_meta, "Source-rank metadata of the received rows");
    m.def("ll_exchange_metadata", &deep_ep::ll_exchange_metadata,
          "Send/receive counts, combine offsets and per-row records from the gathered route counts");
    m.def("combine_reduce", &deep_ep::combine_reduce, "Per-token sum of the rows that came back (normal-mode combine)",
          py::arg("recv_x"), py::arg("recv_topk_weights"), py::arg("sorted_token_ids"), py::arg("send_cumsum"),
          py::arg("is_token_in_rank"), py::arg("bias_0") = py::none(), py::arg("bias_1") = py::none(),
          py::arg("row_of_pair") = py::none());
}
