// What the two host classes of the HIP backend share (`ElasticBuffer`, the V2 surface, and `Buffer`, the V1 surface):
// the exception type, the process-wide launch-shape knobs, the communication stream and the stream choreography of
// one call (csrc/elastic/buffer.hpp:528-586 and csrc/legacy/buffer.hpp:500-520,690-712 in the reference), the
// grow-only workspace, the device status word, and the small "which tensor did this buffer hand out" memory that
// lets the reference's positional calls do without the extra tensors this backend keeps beside a handle.
// Torch types stop in these classes: below them everything goes through the C ABI of include/deep_ep_hip.h.
#pragma once

#include <c10/hip/HIPFunctions.h>
#include <c10/util/intrusive_ptr.h>
#include <pybind11/pybind11.h>
#include <torch/types.h>

#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstdlib>
#include <deque>
#include <optional>
#include <sstream>
#include <stdexcept>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "../../../include/deep_ep_hip.h"
#include "event.hpp"

namespace deep_ep::hip {

// Host checks raise what the reference's EP_HOST_ASSERT raises: an exception Python sees as RuntimeError
// (deep_ep/include/deep_ep/common/exception.cuh:11-34).
class EPException : public std::runtime_error {
public:
    using std::runtime_error::runtime_error;
};

#define EP_HIP_HOST_ASSERT(cond)                                                                      \
    do {                                                                                              \
        if (!(cond)) throw ::deep_ep::hip::EPException(std::string("Assertion failed: ") + #cond);    \
    } while (0)

inline int64_t align_up(int64_t x, int64_t y) { return (x + y - 1) / y * y; }

constexpr int64_t kBufferAlignmentBytes = 2 * 1024 * 1024;   // symmetric::kNumAlignmentBytes (csrc/elastic/buffer.hpp:1363-1365)
constexpr int64_t kRecordAlignBytes = 32;                    // ptx::kNumTMAAlignBytes, used only by the size calculus

// Launch-shape knobs every call passes down (all zero = the library's own choice); seeded from DEEP_EP_HIP_<NAME>.
inline deep_ep_hip_tuning& process_tuning() {
    static deep_ep_hip_tuning tuning = [] {
        deep_ep_hip_tuning t{};
        auto env = [](const char* name) {
            const char* v = std::getenv(name);
            return v != nullptr ? std::atoi(v) : 0;
        };
        t.dispatch_launches = env("DEEP_EP_HIP_DISPATCH_LAUNCHES");
        t.cast_pairs = env("DEEP_EP_HIP_CAST_PAIRS");
        t.copy_vecs = env("DEEP_EP_HIP_COPY_VECS");
        t.plain_loads = env("DEEP_EP_HIP_PLAIN_LOADS");
        t.xcd_remap = env("DEEP_EP_HIP_XCD_REMAP");
        t.combine_vecs = env("DEEP_EP_HIP_COMBINE_VECS");
        t.ll_pairs = env("DEEP_EP_HIP_LL_PAIRS");
        t.ll_threads = env("DEEP_EP_HIP_LL_THREADS");
        t.ll_two_kernels = env("DEEP_EP_HIP_LL_TWO_KERNELS");
        t.ll_combine_vecs = env("DEEP_EP_HIP_LL_COMBINE_VECS");
        t.mover_spin_limit = env("DEEP_EP_HIP_MOVER_SPIN_LIMIT");
        t.move_workgroups_per_cu = env("DEEP_EP_HIP_MOVE_WORKGROUPS_PER_CU");
        t.warm_rounds = env("DEEP_EP_HIP_WARM_ROUNDS");
        t.persistent_movers = env("DEEP_EP_HIP_PERSISTENT_MOVERS");
        return t;
    }();
    return tuning;
}

inline int32_t* tuning_field(const std::string& name) {
    deep_ep_hip_tuning& t = process_tuning();
    if (name == "dispatch_launches") return &t.dispatch_launches;
    if (name == "cast_pairs") return &t.cast_pairs;
    if (name == "copy_vecs") return &t.copy_vecs;
    if (name == "plain_loads") return &t.plain_loads;
    if (name == "xcd_remap") return &t.xcd_remap;
    if (name == "combine_vecs") return &t.combine_vecs;
    if (name == "ll_pairs") return &t.ll_pairs;
    if (name == "ll_threads") return &t.ll_threads;
    if (name == "ll_two_kernels") return &t.ll_two_kernels;
    if (name == "ll_combine_vecs") return &t.ll_combine_vecs;
    if (name == "mover_spin_limit") return &t.mover_spin_limit;
    if (name == "move_workgroups_per_cu") return &t.move_workgroups_per_cu;
    if (name == "warm_rounds") return &t.warm_rounds;
    if (name == "persistent_movers") return &t.persistent_movers;
    throw EPException("unknown tuning field: " + name);
}

inline void check_abi(int rc, const char* what) {
    if (rc != 0) {
        std::ostringstream msg;
        msg << "DeepEP HIP backend: " << what << " failed (code " << rc << "): " << deep_ep_hip_last_error();
        throw EPException(msg.str());
    }
}

template <class T>
inline T* ptr_of(const std::optional<torch::Tensor>& t) {
    return t.has_value() ? static_cast<T*>(t->data_ptr()) : nullptr;
}


// Several output tensors of one call in one device allocation.  Every torch allocation costs the host about a
// microsecond and every view that goes through the dispatcher a third of one, which counts in calls of ten to twenty:
// the tensors are declared first, allocated together (each one 256-byte aligned), and then built directly on the shared
// storage.  Tensors of one pack keep each other's memory alive, so a pack holds what lives and dies together.
class TensorPack {
public:
    explicit TensorPack(const c10::Device& device) : device_(device) {}

    // Declares a tensor (contiguous unless strides are given); returns its index for get().
    int add(c10::ScalarType dtype, std::vector<int64_t> sizes, std::vector<int64_t> strides = {}) {
        if (strides.empty()) {
            strides.resize(sizes.size());
            int64_t running = 1;
            for (int i = static_cast<int>(sizes.size()) - 1; i >= 0; --i) {
                strides[i] = running;
                running *= std::max<int64_t>(sizes[i], 1);
            }
        }
        int64_t span = 1;                                   // elements from the first to one past the last
        for (size_t i = 0; i < sizes.size(); ++i) {
            if (sizes[i] == 0) { span = 0; break; }
            span += (sizes[i] - 1) * strides[i];
        }
        const int64_t bytes = span * static_cast<int64_t>(c10::elementSize(dtype));
        entries_.push_back({dtype, std::move(sizes), std::move(strides), total_bytes_});
        total_bytes_ = align_up(total_bytes_ + bytes, 256);
        return static_cast<int>(entries_.size()) - 1;
    }

    // One allocation for everything declared so far (on the current stream of the caching allocator).
    void allocate() {
        blob_ = torch::empty({std::max<int64_t>(total_bytes_, 1)}, torch::TensorOptions().dtype(torch::kUInt8).device(device_));
    }

    torch::Tensor get(int index) const {
        const Entry& e = entries_[static_cast<size_t>(index)];
        auto impl = c10::make_intrusive<c10::TensorImpl>(c10::Storage(blob_.storage()), blob_.key_set(), c10::scalarTypeToTypeMeta(e.dtype));
        impl->set_storage_offset((blob_.storage_offset() + e.byte_offset) / static_cast<int64_t>(c10::elementSize(e.dtype)));
        impl->set_sizes_and_strides(e.sizes, e.strides);
        return torch::Tensor(std::move(impl));
    }

private:
    struct Entry {
        c10::ScalarType dtype;
        std::vector<int64_t> sizes, strides;
        int64_t byte_offset;
    };
    c10::Device device_;
    std::vector<Entry> entries_;
    int64_t total_bytes_ = 0;
    torch::Tensor blob_;
};

// A few (key tensor -> companion tensor) pairs a buffer remembers about handles it has produced.  The key is held
// weakly and compared by identity, so an entry can only be found through the very tensor object the buffer returned:
// a clone, a view or another tensor that happens to reuse the freed memory misses, and the caller falls back to
// recomputing the companion.
class HandleMemory {
public:
    void remember(const torch::Tensor& key, torch::Tensor companion) {
        forget(key);
        entries_.emplace_front(c10::weak_intrusive_ptr<c10::TensorImpl>(key.getIntrusivePtr()), std::move(companion));
        if (entries_.size() > kCapacity) entries_.pop_back();
    }

    std::optional<torch::Tensor> find(const torch::Tensor& key) const {
        for (const auto& [weak, companion] : entries_)
            if (weak._unsafe_get_target() == key.unsafeGetTensorImpl() and not weak.expired()) return companion;
        return std::nullopt;
    }

    void clear() { entries_.clear(); }

private:
    void forget(const torch::Tensor& key) {
        for (auto it = entries_.begin(); it != entries_.end();)
            it = (it->first._unsafe_get_target() == key.unsafeGetTensorImpl() or it->first.expired()) ? entries_.erase(it) : std::next(it);
    }

    static constexpr size_t kCapacity = 16;
    std::deque<std::pair<c10::weak_intrusive_ptr<c10::TensorImpl>, torch::Tensor>> entries_;
};

class HostRuntime {
public:
    c10::Stream get_comm_stream() const { return comm_stream_.unwrap(); }

    bool is_destroyed() const { return destroyed_; }

    // Synchronise and raise if a kernel flagged bad routing input or a row that did not fit the outputs.
    void check_device_status(const std::string& what) {
        c10::hip::device_synchronize();
        if (workspace_.has_value()) read_and_clear_status(*workspace_, what.c_str());
    }

    // Queues, on the current stream, a copy of the status word into `out` (one int32 in pinned host memory or on the
    // device), clearing it on the way if asked.  Capturable: a graph that holds it refreshes `out` on every replay.
    // The read counts as a use of the workspace: a later call on another stream is ordered behind it.
    void queue_status_read(const torch::Tensor& out, bool clear) {
        EP_HIP_HOST_ASSERT(out.scalar_type() == torch::kInt32 and out.numel() >= 1 and (out.is_cuda() or out.is_pinned()));
        EP_HIP_HOST_ASSERT(workspace_.has_value());                    // a dispatch or combine has run on this buffer
        const Stream stream = current_stream();
        if (last_stream_ != stream) stream_wait(stream, last_stream_);
        check_abi(deep_ep_hip_read_status(workspace_->data_ptr(), out.data_ptr<int32_t>(), clear ? 1 : 0, stream.stream()),
                  "status read");
        last_stream_ = stream;
    }

    // The status check of a loop that never waits for the GPU.  A call that finds no read in flight queues one on the
    // current stream (deep_ep_hip_read_status in its clearing form: a small kernel moves the status word into pinned
    // host memory and leaves the workspace ready for the next launch) and returns false.  A later call returns false
    // while that read is still running; once it has finished, the call throws like check_device_status if a kernel had
    // flagged something since the previous read, and returns true if nothing was flagged.
    bool poll_device_status(const std::string& what) {
        if (not workspace_.has_value()) return true;
        if (not status_read_.has_value()) {
            if (not status_host_.has_value())
                status_host_ = torch::zeros({1}, torch::TensorOptions().dtype(torch::kInt32).pinned_memory(true));
            queue_status_read(*status_host_, true);
            status_read_.emplace(current_stream());
            return false;
        }
        if (not status_read_->event->query()) return false;
        status_read_.reset();
        const int status = *status_host_->data_ptr<int32_t>();
        if (status != 0) throw_status(status, what.c_str());
        return true;
    }

    // The status word as the GPU has it now (every launch queued so far has finished): 0 = nothing flagged.
    int device_status() {
        c10::hip::device_synchronize();
        return workspace_.has_value() ? workspace_->slice(0, 0, 4).view(torch::kInt32).item<int>() : 0;
    }

    // The counters and flags at the head of the workspace (status, launch protocol), copied to the host after a full
    // synchronisation: between launches everything but the status word (word 0), the two row totals (words 2 and 3) and
    // the launch generation (word 32) reads zero.
    torch::Tensor workspace_control_words() {
        c10::hip::device_synchronize();
        const int64_t n = static_cast<int64_t>(deep_ep_hip_workspace_counter_bytes());
        if (not workspace_.has_value()) return torch::zeros({n / 4}, torch::kInt32);
        return workspace_->slice(0, 0, n).view(torch::kInt32).cpu();
    }

    // V1 `Buffer.get_dispatch_layout` (csrc/legacy/buffer.hpp:337-404): (num_tokens_per_rank [R] int32,
    // num_tokens_per_rdma_rank = None, num_tokens_per_expert [E] int32, is_token_in_rank [T, R] bool, event).
    std::tuple<torch::Tensor, std::optional<torch::Tensor>, torch::Tensor, torch::Tensor, std::optional<EventHandle>>
    get_dispatch_layout(const torch::Tensor& topk_idx, int num_experts, const std::optional<EventHandle>& previous_event, bool async,
                        bool allocate_on_comm_stream) {
        EP_HIP_HOST_ASSERT(not destroyed_);
        EP_HIP_HOST_ASSERT(topk_idx.dim() == 2 and topk_idx.is_contiguous() and topk_idx.is_cuda());
        EP_HIP_HOST_ASSERT(topk_idx.scalar_type() == torch::kInt64);
        EP_HIP_HOST_ASSERT(num_experts > 0 and num_experts % num_ranks_ == 0);
        const int num_tokens = static_cast<int>(topk_idx.size(0)), num_topk = static_cast<int>(topk_idx.size(1));
        StreamScope scope(*this, previous_event, allocate_on_comm_stream, async);
        const Stream& run = scope.run_stream;
        torch::Tensor workspace = acquire_workspace(run, num_tokens, num_topk, num_experts);
        c10::hip::HIPStreamGuardMasqueradingAsCUDA on_run(run);          // allocations below belong to the run stream
        const auto i32 = torch::TensorOptions().dtype(torch::kInt32).device(device_);
        torch::Tensor per_rank = torch::empty({num_ranks_}, i32);
        torch::Tensor per_expert = torch::empty({num_experts}, i32);
        torch::Tensor in_rank = torch::empty({num_tokens, num_ranks_}, torch::TensorOptions().dtype(torch::kBool).device(device_));
        deep_ep_hip_layout_args args{};
        args.topk_idx = static_cast<const int64_t*>(topk_idx.data_ptr());
        args.num_tokens = num_tokens; args.num_topk = num_topk; args.num_experts = num_experts; args.num_ranks = num_ranks_;
        args.num_tokens_per_rank = static_cast<int32_t*>(per_rank.data_ptr());
        args.num_tokens_per_expert = static_cast<int32_t*>(per_expert.data_ptr());
        args.is_token_in_rank = static_cast<uint8_t*>(in_rank.data_ptr());
        args.workspace = workspace.data_ptr();
        args.workspace_bytes = static_cast<uint64_t>(workspace.numel());
        check_abi(deep_ep_hip_launch_layout(&args, run.stream()), "get_dispatch_layout");
        std::optional<EventHandle> event = scope.finish({topk_idx, per_rank, per_expert, in_rank, workspace});
        return {per_rank, std::nullopt, per_expert, in_rank, event};
    }

protected:
    HostRuntime(int rank_idx, int num_ranks, bool explicitly_destroy)
        : rank_idx_(rank_idx), num_ranks_(num_ranks), explicitly_destroy_(explicitly_destroy), comm_stream_(make_comm_stream()),
          last_stream_(comm_stream_) {
        EP_HIP_HOST_ASSERT(0 <= rank_idx and rank_idx < num_ranks);
        EP_HIP_HOST_ASSERT(num_ranks <= DEEP_EP_HIP_MAX_RANKS);
        device_ = torch::Device(torch::kCUDA, comm_stream_.device_index());
    }

    void release() {
        EP_HIP_HOST_ASSERT(explicitly_destroy_);
        EP_HIP_HOST_ASSERT(not destroyed_);
        c10::hip::device_synchronize();
        workspace_.reset();
        status_read_.reset();
        destroyed_ = true;
    }

    // The one communication stream of the buffer, at the default priority.  Fails loudly when there is no GPU.
    static Stream make_comm_stream() {
        if (c10::hip::device_count() <= 0) throw EPException("DeepEP HIP backend: no GPU is visible");
        return c10::hip::getStreamFromPoolMasqueradingAsCUDA(false);
    }

    // Stream choreography of one call.  The reference always runs on its comm stream; when nothing asks for overlap
    // the same ordering is had, without two cross-stream waits, by running on the caller's stream.  The destructor
    // restores the current stream whatever happens in between.  `v1_rules`: the argument rule of the V1 calls
    // (allocating on the comm stream needs a previous event and an asynchronous finish, csrc/legacy/buffer.hpp:507-510)
    // instead of the V2 one (a previous event needs allocation on the comm stream, csrc/elastic/buffer.hpp:536).
    struct StreamScope {
        HostRuntime& buffer;
        Stream compute_stream, run_stream;
        bool allocate_on_comm_stream, async_with_compute_stream, switched = false;

        StreamScope(HostRuntime& b, const std::optional<EventHandle>& previous_event, bool allocate_on_comm, bool async,
                    bool v1_rules = false)
            : buffer(b), compute_stream(current_stream()), run_stream(compute_stream), allocate_on_comm_stream(allocate_on_comm),
              async_with_compute_stream(async) {
            if (v1_rules) {
                if (allocate_on_comm_stream) EP_HIP_HOST_ASSERT(previous_event.has_value() and async_with_compute_stream);
            } else if (previous_event.has_value()) {
                EP_HIP_HOST_ASSERT(allocate_on_comm_stream);
            }
            const bool overlap = previous_event.has_value() or allocate_on_comm_stream or async_with_compute_stream;
            if (not overlap) return;
            run_stream = buffer.comm_stream_;
            if (allocate_on_comm_stream) {
                c10::hip::setCurrentHIPStreamMasqueradingAsCUDA(buffer.comm_stream_);
                switched = true;
            }
            if (previous_event.has_value()) stream_wait(run_stream, *previous_event);
            else if (run_stream != compute_stream) stream_wait(run_stream, compute_stream);
        }

        ~StreamScope() {
            if (switched) c10::hip::setCurrentHIPStreamMasqueradingAsCUDA(compute_stream);
        }

        std::optional<EventHandle> finish(std::initializer_list<std::optional<torch::Tensor>> tensors) {
            buffer.last_stream_ = run_stream;
            std::optional<EventHandle> event;
            if (run_stream != compute_stream) {
                if (async_with_compute_stream) {
                    event = EventHandle(run_stream);
                    const char* avoid = std::getenv("EP_AVOID_RECORD_STREAM");
                    if (avoid != nullptr and std::atoi(avoid) != 0) {
                        for (const auto& t : tensors)
                            if (t.has_value()) event->tensors_to_record.push_back(t);
                    } else {
                        for (const auto& t : tensors) {
                            if (t.has_value() and t->is_cuda()) {
                                t->record_stream(compute_stream.unwrap());
                                t->record_stream(run_stream.unwrap());
                            }
                        }
                    }
                } else {
                    stream_wait(compute_stream, run_stream);
                }
            } else if (async_with_compute_stream) {
                event = EventHandle(run_stream);
            }
            return event;
        }
    };

    // The workspace is shared by every call on this buffer and is not re-entrant: a call that runs on another
    // stream than the previous one first waits for everything queued there.  It grows geometrically, so that
    // steady-state calls never allocate; a replaced workspace stays reserved for the stream that last used it.
    torch::Tensor acquire_workspace(const Stream& run, int64_t need) {
        if (last_stream_ != run) stream_wait(run, last_stream_);
        if (not workspace_.has_value() or workspace_->numel() < need) {
            const int64_t size = std::max(need, 2 * (workspace_.has_value() ? workspace_->numel() : int64_t(0)));
            if (workspace_.has_value()) workspace_->record_stream(last_stream_.unwrap());
            c10::hip::HIPStreamGuardMasqueradingAsCUDA on_run(run);
            workspace_ = torch::zeros({size}, torch::TensorOptions().dtype(torch::kUInt8).device(device_));
        }
        return *workspace_;
    }

    // ... sized for dispatches and combines of this routing shape (a combine may have to rebuild the handle's
    // token -> row map in it).
    torch::Tensor acquire_workspace(const Stream& run, int num_tokens, int num_topk, int num_experts) {
        return acquire_workspace(run, static_cast<int64_t>(deep_ep_hip_combine_workspace_bytes(std::max(num_tokens, 1), num_topk,
                                                                                               num_experts, num_ranks_)));
    }

    // The mailbox through which a layout launch tells the host its counts (deep_ep_hip_dispatch_args::host_counts): pinned
    // host memory the kernel writes directly, zeroed here, so that sizing the outputs takes no device-to-host copy and no
    // device synchronisation (the reference's host-mapped counters, csrc/elastic/buffer.hpp:1019-1066).
    int32_t* fresh_mailbox(int entries) {
        if (not mailbox_.has_value())
            mailbox_ = torch::zeros({DEEP_EP_HIP_MAX_RANKS + DEEP_EP_HIP_MAX_EXPERTS + 1},
                                    torch::TensorOptions().dtype(torch::kInt32).pinned_memory(true));
        EP_HIP_HOST_ASSERT(entries <= mailbox_->numel());
        int32_t* box = mailbox_->data_ptr<int32_t>();
        std::fill(box, box + entries, 0);
        return box;
    }

    // Waits (bounded by the buffer's CPU timeout) until the kernel has published all `entries` values; decodes them in
    // place.  Returns false on a timeout.
    static bool await_mailbox(int32_t* box, int entries, int timeout_secs) {
        const auto deadline = std::chrono::steady_clock::now() + std::chrono::seconds(timeout_secs > 0 ? timeout_secs : 300);
        volatile int32_t* watched = box;
        uint32_t spins = 0;
        for (int i = 0; i < entries; ++i) {
            while (watched[i] >= 0) {
                if ((++spins & 0xfffu) == 0 and std::chrono::steady_clock::now() > deadline) return false;
                __builtin_ia32_pause();
            }
            box[i] = -watched[i] - 1;
        }
        return true;
    }

    void read_and_clear_status(const torch::Tensor& workspace, const char* what) {
        const int status = workspace.slice(0, 0, 4).view(torch::kInt32).item<int>();
        if (status == 0) return;
        // also the launch bookkeeping words that follow: a dispatch that gave up has left them mid-protocol
        workspace.slice(0, 0, static_cast<int64_t>(deep_ep_hip_workspace_control_bytes())).zero_();
        throw_status(status, what);
    }

    [[noreturn]] static void throw_status(int status, const char* what) {
        std::string reasons;
        auto add = [&](int bit, const char* text) {
            if (status & bit) reasons += (reasons.empty() ? "" : "; ") + std::string(text);
        };
        add(DEEP_EP_HIP_STATUS_EXPERT_OUT_OF_RANGE, "topk_idx holds an expert id >= num_experts");
        add(DEEP_EP_HIP_STATUS_DUPLICATE_EXPERT, "a token selects the same expert twice");
        add(DEEP_EP_HIP_STATUS_ROW_OVERFLOW, "a received row did not fit the output tensors");
        add(DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT, "a single-launch dispatch gave up waiting for its counting workgroups (outputs invalid)");
        throw EPException(std::string("DeepEP HIP backend: ") + what + ": " + reasons);
    }

    int rank_idx_, num_ranks_;
    bool explicitly_destroy_;
    bool destroyed_ = false;
    Stream comm_stream_;
    Stream last_stream_;                     // stream of the last launch that used the workspace
    torch::Device device_ = torch::Device(torch::kCUDA, 0);
    std::optional<torch::Tensor> workspace_;
    std::optional<torch::Tensor> mailbox_;            // pinned: counts of a layout launch for a call that waits for them
    std::optional<torch::Tensor> status_host_;        // one pinned int32: where poll_device_status has the status copied
    std::optional<EventHandle> status_read_;          // recorded after the read in flight
};

}  // namespace deep_ep::hip
