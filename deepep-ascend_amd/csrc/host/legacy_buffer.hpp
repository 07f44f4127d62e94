// Host side of the V1 surface for the HIP backend: the classes the `deep_ep._C` extension registers as `Config` and
// `Buffer` (the role of csrc/legacy/config.hpp:24-100 and csrc/legacy/buffer.hpp:83-1787 in the reference), for the
// part of V1 that sits on the routing hot path: `get_dispatch_layout`, dispatch / combine inside one scale-up domain
// ("intranode") and the low-latency packed dispatch / combine.  Argument order and returned tuples are the
// reference's, so that its Python wrapper calls land here unchanged; what this backend adds is bound as trailing
// keywords with defaults.
//
// One GPU, logical ranks.  `num_ranks` = R logical ranks, `rank` = this process's logical rank.  `intranode_dispatch`
// moves the tokens of logical source rank `rank`; the received rows are the concatenation over destination ranks d of
// what d gets from this source, in token order.  The packed buffers of `low_latency_dispatch` are those of
// destination rank `rank` (experts [rank * E / R, (rank + 1) * E / R)).  Two input forms are accepted there: `x`
// [T, H] with `topk_idx` [T, K] - the tokens of logical source rank `rank` only - or, as an extension, `x` [R, T, H]
// with `topk_idx` [R, T, K]: the tokens of all R logical source ranks, everything destination `rank` would receive
// in a real R-rank run.  Rows of one expert are filled by source rank ascending, then token ascending.
#pragma once

#include <functional>

#include "runtime_base.hpp"

namespace deep_ep::hip {

// Tuning knobs of the V1 kernels.  Only `num_sms` has a meaning here: it fixes the number of channels (num_sms / 2)
// the handle's channel matrices are laid out for.  The size hints say what the reference would stage; nothing is
// staged on one GPU.
struct Config {
    int num_sms;
    int num_max_nvl_chunked_send_tokens, num_max_nvl_chunked_recv_tokens;
    int num_max_rdma_chunked_send_tokens, num_max_rdma_chunked_recv_tokens;

    static constexpr int kPeersPerDomain = 8;      // LEGACY_NUM_MAX_NVL_PEERS
    static constexpr int64_t kAssumedTopk = 128, kAssumedScales = 128, kSourceRecordBytes = 8;

    Config(int sms, int nvl_send, int nvl_recv, int rdma_send, int rdma_recv)
        : num_sms(sms), num_max_nvl_chunked_send_tokens(nvl_send), num_max_nvl_chunked_recv_tokens(nvl_recv),
          num_max_rdma_chunked_send_tokens(rdma_send), num_max_rdma_chunked_recv_tokens(rdma_recv) {
        EP_HIP_HOST_ASSERT(num_sms >= 0);
        EP_HIP_HOST_ASSERT(0 < nvl_send and nvl_send < nvl_recv);
        EP_HIP_HOST_ASSERT(rdma_send > 0 and rdma_recv > 0);
        num_max_rdma_chunked_recv_tokens = static_cast<int>(align_up(rdma_recv, rdma_send));      // whole send chunks
        EP_HIP_HOST_ASSERT(rdma_send < num_max_rdma_chunked_recv_tokens and rdma_send <= num_max_rdma_chunked_recv_tokens / 2);
    }

    // per queue slot: payload, source record, the assumed maxima of top-k ids, weights and scales
    int64_t slot_bytes(int64_t hidden_bytes) const {
        return hidden_bytes + kSourceRecordBytes + kAssumedTopk * int64_t(sizeof(int64_t)) + kAssumedTopk * 4 + kAssumedScales * 4;
    }

    int64_t get_nvl_buffer_size_hint(int64_t hidden_bytes, int num_ranks) const {
        EP_HIP_HOST_ASSERT(num_ranks < kPeersPerDomain or num_ranks % kPeersPerDomain == 0);
        EP_HIP_HOST_ASSERT(num_ranks <= kPeersPerDomain or num_sms % 2 == 0);
        const int64_t domains = std::max(num_ranks / kPeersPerDomain, 1), peers = std::min(num_ranks, kPeersPerDomain);
        const int64_t queues = int64_t(num_sms / 2) * peers;
        const int64_t bytes = queues * (2 * domains + 3) * 4 + queues * num_max_nvl_chunked_recv_tokens * slot_bytes(hidden_bytes);
        return align_up(bytes, 128);
    }

    int64_t get_rdma_buffer_size_hint(int64_t hidden_bytes, int num_ranks) const {
        if (num_ranks <= kPeersPerDomain) return 0;
        EP_HIP_HOST_ASSERT(num_ranks % kPeersPerDomain == 0 and num_sms % 2 == 0);
        const int64_t queues = int64_t(num_sms / 2) * (num_ranks / kPeersPerDomain);
        const int64_t bytes = queues * (kPeersPerDomain * 2 + 2) * 2 * 4 +
                              queues * num_max_rdma_chunked_recv_tokens * (slot_bytes(hidden_bytes) + 16) * 2;
        return align_up(bytes, 128);
    }
};

// Bytes the reference would reserve for the low-latency buffers (csrc/legacy/config.hpp:131-188): two send, two receive
// and two signalling buffers of one message per (expert, token slot).  Nothing is staged here.
inline int64_t get_low_latency_rdma_size_hint(int num_max_dispatch_tokens_per_rank, int hidden, int /*num_ranks*/, int num_experts) {
    const int64_t num_scales = hidden / 128;
    const int64_t dispatch_msg = 16 + std::max<int64_t>(int64_t(hidden) * 2, hidden + num_scales * 4);
    const int64_t combine_msg = num_scales * 4 + int64_t(hidden) * 2;
    const int64_t M = num_max_dispatch_tokens_per_rank;
    const int64_t send = std::max(M * dispatch_msg, num_experts * M * combine_msg);
    const int64_t recv = num_experts * M * std::max(dispatch_msg, combine_msg);
    return align_up(2 * (send + recv + int64_t(num_experts) * 4), 128);
}

class Buffer : public HostRuntime {
public:
    // rank, num_ranks, num_nvl_bytes, num_rdma_bytes, low_latency_mode, explicitly_destroy, enable_shrink, use_fabric
    // (csrc/legacy/buffer.hpp:83-91).  The byte counts are recorded as given: rows land in the tensors the calls return.
    Buffer(int rank, int num_ranks, int64_t num_nvl_bytes, int64_t num_rdma_bytes, bool low_latency_mode, bool explicitly_destroy,
           bool enable_shrink, bool /*use_fabric*/)
        : HostRuntime(rank, num_ranks, explicitly_destroy), num_nvl_bytes_(num_nvl_bytes), num_rdma_bytes_(num_rdma_bytes),
          low_latency_mode_(low_latency_mode) {
        EP_HIP_HOST_ASSERT(num_nvl_bytes >= 0 and num_rdma_bytes >= 0);
        EP_HIP_HOST_ASSERT(not enable_shrink);      // masking out failed ranks has no meaning on one GPU
    }

    bool is_available() const { return not destroyed_; }
    int get_num_rdma_ranks() const { return 1; }
    int get_rdma_rank() const { return 0; }
    int get_root_rdma_rank(bool /*global*/) const { return 0; }
    int get_local_device_id() const { return device_.index(); }

    void destroy() {
        release();
        ll_workspace_.reset();
        ll_combine_buffer_.reset();
        send_head_of_handle_.clear();
        lane_rows_of_handle_.clear();
    }

    // get_dispatch_layout (csrc/legacy/buffer.hpp:337-404) is inherited: the V2 class offers the same call.

    // ---- intranode dispatch: the 16 arguments and the 11-tuple of csrc/legacy/buffer.hpp:405-717 ----
    // A cached call (rank_prefix_matrix given) replays the routing of an earlier one.  The reference's cached call
    // does not carry the handle's `send_head` (on one GPU: the receive row of every (token, rank) pair): it may be
    // given as a trailing keyword; otherwise the buffer finds the one it produced together with this
    // `rank_prefix_matrix`, and for a handle it has not seen the rows are placed again from `is_token_in_rank`
    // (placement is deterministic, so they land where they landed before).
    std::tuple<torch::Tensor, std::optional<torch::Tensor>, std::optional<torch::Tensor>, std::optional<torch::Tensor>, std::vector<int>,
               torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, std::optional<EventHandle>>
    intranode_dispatch(const torch::Tensor& x, const std::optional<torch::Tensor>& x_scales, const std::optional<torch::Tensor>& topk_idx,
                       const std::optional<torch::Tensor>& topk_weights, const std::optional<torch::Tensor>& num_tokens_per_rank,
                       const torch::Tensor& is_token_in_rank, const std::optional<torch::Tensor>& num_tokens_per_expert,
                       int cached_num_recv_tokens, const std::optional<torch::Tensor>& cached_rank_prefix_matrix,
                       const std::optional<torch::Tensor>& cached_channel_prefix_matrix, int expert_alignment, int num_worst_tokens,
                       const Config& config, const std::optional<EventHandle>& previous_event, bool async, bool allocate_on_comm_stream,
                       const std::optional<torch::Tensor>& cached_send_head_arg) {
        EP_HIP_HOST_ASSERT(not destroyed_);
        const bool cached_mode = cached_rank_prefix_matrix.has_value();
        const int R = num_ranks_;
        EP_HIP_HOST_ASSERT(R <= 64);
        EP_HIP_HOST_ASSERT(config.num_sms % 2 == 0);
        const int num_channels = config.num_sms / 2;
        EP_HIP_HOST_ASSERT(x.dim() == 2 and x.is_cuda() and x.is_contiguous());
        const int num_tokens = static_cast<int>(x.size(0)), hidden = static_cast<int>(x.size(1));
        EP_HIP_HOST_ASSERT((hidden * x.element_size()) % 16 == 0);
        EP_HIP_HOST_ASSERT(is_token_in_rank.scalar_type() == torch::kBool and is_token_in_rank.dim() == 2 and is_token_in_rank.is_contiguous() and
                           is_token_in_rank.size(0) == num_tokens and is_token_in_rank.size(1) == R and is_token_in_rank.is_cuda());
        const auto i32 = torch::TensorOptions().dtype(torch::kInt32).device(device_);

        std::optional<torch::Tensor> cached_send_head = cached_send_head_arg;
        int num_experts = 0;
        if (cached_mode) {
            EP_HIP_HOST_ASSERT(cached_channel_prefix_matrix.has_value());
            EP_HIP_HOST_ASSERT(cached_rank_prefix_matrix->dim() == 2 and cached_rank_prefix_matrix->size(0) == R and
                               cached_rank_prefix_matrix->size(1) == R and cached_rank_prefix_matrix->scalar_type() == torch::kInt32);
            EP_HIP_HOST_ASSERT(cached_channel_prefix_matrix->dim() == 2 and cached_channel_prefix_matrix->size(0) == R and
                               cached_channel_prefix_matrix->size(1) == num_channels and
                               cached_channel_prefix_matrix->scalar_type() == torch::kInt32);
            EP_HIP_HOST_ASSERT(not topk_idx.has_value() and not topk_weights.has_value());      // a cached dispatch takes no top-k tensors
            if (not cached_send_head.has_value()) cached_send_head = send_head_of_handle_.find(*cached_rank_prefix_matrix);
            if (cached_send_head.has_value())
                EP_HIP_HOST_ASSERT(cached_send_head->dim() == 2 and cached_send_head->size(0) == num_tokens and cached_send_head->size(1) == R and
                                   cached_send_head->scalar_type() == torch::kInt32 and cached_send_head->is_contiguous());
        } else {
            EP_HIP_HOST_ASSERT(num_tokens_per_rank.has_value() and num_tokens_per_expert.has_value());
            EP_HIP_HOST_ASSERT(num_tokens_per_rank->scalar_type() == torch::kInt32 and num_tokens_per_rank->dim() == 1 and
                               num_tokens_per_rank->size(0) == R and num_tokens_per_rank->is_contiguous());
            EP_HIP_HOST_ASSERT(num_tokens_per_expert->scalar_type() == torch::kInt32 and num_tokens_per_expert->dim() == 1 and
                               num_tokens_per_expert->is_contiguous());
            num_experts = static_cast<int>(num_tokens_per_expert->size(0));
            EP_HIP_HOST_ASSERT(num_experts % R == 0);
        }
        EP_HIP_HOST_ASSERT(topk_idx.has_value() == topk_weights.has_value());
        int num_topk = 0;
        if (topk_idx.has_value()) {
            num_topk = static_cast<int>(topk_idx->size(1));
            EP_HIP_HOST_ASSERT(num_experts > 0);
            EP_HIP_HOST_ASSERT(topk_idx->dim() == 2 and topk_idx->is_contiguous() and topk_idx->scalar_type() == torch::kInt64 and
                               topk_idx->size(0) == num_tokens and topk_idx->is_cuda());
            EP_HIP_HOST_ASSERT(topk_weights->dim() == 2 and topk_weights->size(0) == num_tokens and topk_weights->size(1) == num_topk and
                               topk_weights->is_contiguous() and topk_weights->scalar_type() == torch::kFloat32);
            EP_HIP_HOST_ASSERT(1 <= num_topk and num_topk <= DEEP_EP_HIP_MAX_TOPK);
            EP_HIP_HOST_ASSERT(num_experts <= DEEP_EP_HIP_MAX_EXPERTS);
        } else {
            EP_HIP_HOST_ASSERT(R <= DEEP_EP_HIP_MAX_TOPK);      // routing by is_token_in_rank alone: one lane per rank
        }
        int payload = DEEP_EP_HIP_PAYLOAD_BF16, num_scales = 0;
        int64_t scale_ts = 0, scale_hs = 0;
        if (x_scales.has_value()) {
            EP_HIP_HOST_ASSERT(x.element_size() == 1);
            EP_HIP_HOST_ASSERT(x_scales->scalar_type() == torch::kFloat32 or x_scales->scalar_type() == torch::kInt32);
            EP_HIP_HOST_ASSERT(x_scales->dim() == 2 and x_scales->size(0) == num_tokens and x_scales->is_cuda());
            num_scales = static_cast<int>(x_scales->size(1));
            scale_ts = x_scales->stride(0); scale_hs = x_scales->stride(1);
            payload = DEEP_EP_HIP_PAYLOAD_FP8;
        } else {
            EP_HIP_HOST_ASSERT(x.scalar_type() == torch::kBFloat16);
        }
        if (num_worst_tokens > 0) EP_HIP_HOST_ASSERT(cached_mode or topk_idx.has_value());

        StreamScope scope(*this, previous_event, allocate_on_comm_stream, async, /*v1_rules=*/true);
        const Stream& run = scope.run_stream;
        const int route_lanes = topk_idx.has_value() ? num_topk : R, route_experts = topk_idx.has_value() ? num_experts : R;
        torch::Tensor workspace = acquire_workspace(run, num_tokens, route_lanes, route_experts);
        c10::hip::HIPStreamGuardMasqueradingAsCUDA on_run(run);          // allocations below belong to the run stream

        deep_ep_hip_intranode_dispatch_args args{};
        args.tuning = process_tuning();
        args.payload = payload;
        args.num_tokens = num_tokens; args.hidden = hidden;
        args.num_topk = num_topk; args.num_experts = topk_idx.has_value() ? num_experts : 0;
        args.num_ranks = R; args.rank_idx = rank_idx_;
        args.num_channels = num_channels; args.expert_alignment = expert_alignment;
        args.x = x.data_ptr(); args.x_scales = x_scales.has_value() ? x_scales->data_ptr() : nullptr;
        args.scale_token_stride = scale_ts; args.scale_hidden_stride = scale_hs; args.num_scales = num_scales;
        args.topk_idx = ptr_of<const int64_t>(topk_idx); args.topk_weights = ptr_of<const float>(topk_weights);
        args.is_token_in_rank = static_cast<const uint8_t*>(is_token_in_rank.data_ptr());
        args.workspace = workspace.data_ptr(); args.workspace_bytes = static_cast<uint64_t>(workspace.numel());
        void* stream_ptr = run.stream();

        int num_recv_tokens;
        std::vector<int> per_expert_list;
        torch::Tensor rank_prefix_matrix, channel_prefix_matrix, recv_channel_prefix_matrix, send_head, recv_src_idx, counts;
        if (cached_mode) {
            num_recv_tokens = cached_num_recv_tokens;
            rank_prefix_matrix = *cached_rank_prefix_matrix;
            channel_prefix_matrix = *cached_channel_prefix_matrix;
            recv_channel_prefix_matrix = torch::empty({R, num_channels}, i32);
            if (cached_send_head.has_value()) {
                send_head = *cached_send_head;
                args.cached = 1;
                args.phases = DEEP_EP_HIP_PHASE_MOVE;
            } else {
                // place the rows again from the mask: layout and move in one call, the handle tensors it would
                // fill are scratch
                send_head = torch::empty({num_tokens, R}, i32);
                counts = torch::empty({R}, i32);
                args.psum_num_recv_tokens_per_rank = static_cast<int32_t*>(counts.data_ptr());
                args.phases = DEEP_EP_HIP_PHASE_LAYOUT | DEEP_EP_HIP_PHASE_MOVE;
            }
        } else {
            rank_prefix_matrix = torch::empty({R, R}, i32);
            channel_prefix_matrix = torch::empty({R, num_channels}, i32);
            recv_channel_prefix_matrix = torch::empty({R, num_channels}, i32);
            send_head = torch::empty({num_tokens, R}, i32);
            counts = torch::empty({R + std::max(num_experts, 1)}, i32);
            args.rank_prefix_matrix = static_cast<int32_t*>(rank_prefix_matrix.data_ptr());
            args.channel_prefix_matrix = static_cast<int32_t*>(channel_prefix_matrix.data_ptr());
            args.recv_channel_prefix_matrix = static_cast<int32_t*>(recv_channel_prefix_matrix.data_ptr());
            args.psum_num_recv_tokens_per_rank = static_cast<int32_t*>(counts.data_ptr());
            args.num_recv_tokens_per_expert = topk_idx.has_value() ? static_cast<int32_t*>(counts.data_ptr()) + R : nullptr;
            if (num_worst_tokens > 0) {
                num_recv_tokens = num_worst_tokens;
                args.phases = DEEP_EP_HIP_PHASE_LAYOUT | DEEP_EP_HIP_PHASE_MOVE;
                args.fill_unused_topk_idx = 1;
            } else {
                // The host waits for the counts of the layout launch, as the reference does on its host-mapped counters
                // (csrc/legacy/buffer.hpp:580-600).  With top-k tensors they arrive in the pinned mailbox; without,
                // the per-expert counts are the caller's tensor and are copied back with the per-rank ones.
                args.phases = DEEP_EP_HIP_PHASE_LAYOUT;
                per_expert_list.resize(num_experts);
                if (topk_idx.has_value()) {
                    int32_t* box = fresh_mailbox(R + num_experts + 1);
                    args.host_counts = box;
                    check_abi(deep_ep_hip_launch_intranode_dispatch(&args, stream_ptr), "intranode dispatch layout");
                    args.host_counts = nullptr;
                    if (not await_mailbox(box, R + num_experts + 1, 300))
                        throw EPException("DeepEP HIP backend: dispatch: timed out waiting for the layout counts");
                    if (box[R + num_experts] != 0) read_and_clear_status(workspace, "dispatch");      // raises
                    num_recv_tokens = 0;
                    for (int r = 0; r < R; ++r) num_recv_tokens += box[r];
                    std::copy(box + R, box + R + num_experts, per_expert_list.begin());               // aligned counts
                } else {
                    check_abi(deep_ep_hip_launch_intranode_dispatch(&args, stream_ptr), "intranode dispatch layout");
                    const torch::Tensor host = torch::cat({counts.slice(0, 0, R), *num_tokens_per_expert}).cpu();
                    const int32_t* h = host.data_ptr<int32_t>();
                    num_recv_tokens = h[R - 1];
                    for (int e = 0; e < num_experts; ++e)
                        per_expert_list[e] = (h[R + e] + expert_alignment - 1) / expert_alignment * expert_alignment;
                }
                args.phases = DEEP_EP_HIP_PHASE_MOVE;
            }
        }
        recv_src_idx = torch::empty({num_recv_tokens}, i32);

        torch::Tensor recv_x = torch::empty({num_recv_tokens, hidden}, x.options());
        std::optional<torch::Tensor> recv_x_scales, recv_topk_idx, recv_topk_weights;
        if (topk_idx.has_value()) {
            recv_topk_idx = torch::empty({num_recv_tokens, num_topk}, topk_idx->options());
            recv_topk_weights = torch::empty({num_recv_tokens, num_topk}, topk_weights->options());
        }
        if (x_scales.has_value()) {
            recv_x_scales = torch::empty({num_recv_tokens, num_scales}, x_scales->options().memory_format(torch::MemoryFormat::Contiguous));
            args.recv_scale_token_stride = num_scales; args.recv_scale_hidden_stride = 1;
        }
        args.send_head = static_cast<int32_t*>(send_head.data_ptr());
        args.recv_src_idx = (cached_mode and cached_send_head.has_value()) ? nullptr : static_cast<int32_t*>(recv_src_idx.data_ptr());
        args.recv_x = recv_x.data_ptr();
        args.recv_x_scales = recv_x_scales.has_value() ? recv_x_scales->data_ptr() : nullptr;
        args.recv_topk_idx = ptr_of<int64_t>(recv_topk_idx); args.recv_topk_weights = ptr_of<float>(recv_topk_weights);
        args.recv_capacity = num_recv_tokens;
        check_abi(deep_ep_hip_launch_intranode_dispatch(&args, stream_ptr), "intranode dispatch");
        if (not cached_mode) send_head_of_handle_.remember(rank_prefix_matrix, send_head);

        std::optional<EventHandle> event = scope.finish(
            {x, x_scales, topk_idx, topk_weights, num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank, rank_prefix_matrix,
             channel_prefix_matrix, recv_channel_prefix_matrix, recv_x, recv_x_scales, recv_src_idx, recv_topk_idx, recv_topk_weights,
             send_head, counts.defined() ? std::optional<torch::Tensor>(counts) : std::nullopt, workspace});
        return {recv_x, recv_x_scales, recv_topk_idx, recv_topk_weights, per_expert_list, rank_prefix_matrix, channel_prefix_matrix,
                recv_channel_prefix_matrix, recv_src_idx, send_head, event};
    }

    // ---- intranode combine: the 12 arguments and the 3-tuple of csrc/legacy/buffer.hpp:719-860 ----
    std::tuple<torch::Tensor, std::optional<torch::Tensor>, std::optional<EventHandle>>
    intranode_combine(const torch::Tensor& x, const std::optional<torch::Tensor>& topk_weights, const std::optional<torch::Tensor>& bias_0,
                      const std::optional<torch::Tensor>& bias_1, const torch::Tensor& src_idx, const torch::Tensor& rank_prefix_matrix,
                      const torch::Tensor& channel_prefix_matrix, const torch::Tensor& send_head, const Config& /*config*/,
                      const std::optional<EventHandle>& previous_event, bool async, bool allocate_on_comm_stream) {
        EP_HIP_HOST_ASSERT(not destroyed_);
        const int R = num_ranks_;
        EP_HIP_HOST_ASSERT(x.dim() == 2 and x.is_cuda() and x.is_contiguous() and x.scalar_type() == torch::kBFloat16);
        const int64_t num_x_rows = x.size(0);
        const int hidden = static_cast<int>(x.size(1));
        EP_HIP_HOST_ASSERT((hidden * 2) % 16 == 0);
        EP_HIP_HOST_ASSERT(src_idx.dim() == 1 and src_idx.size(0) == num_x_rows and src_idx.scalar_type() == torch::kInt32);
        EP_HIP_HOST_ASSERT(send_head.dim() == 2 and send_head.size(1) == R and send_head.scalar_type() == torch::kInt32 and
                           send_head.is_contiguous());
        EP_HIP_HOST_ASSERT(rank_prefix_matrix.dim() == 2 and rank_prefix_matrix.size(0) == R and rank_prefix_matrix.size(1) == R and
                           rank_prefix_matrix.scalar_type() == torch::kInt32);
        EP_HIP_HOST_ASSERT(channel_prefix_matrix.dim() == 2 and channel_prefix_matrix.size(0) == R);
        const int num_tokens = static_cast<int>(send_head.size(0));
        int num_topk = 0;
        if (topk_weights.has_value()) {
            EP_HIP_HOST_ASSERT(topk_weights->dim() == 2 and topk_weights->size(0) == num_x_rows and topk_weights->is_contiguous() and
                               topk_weights->scalar_type() == torch::kFloat32 and topk_weights->is_cuda());
            num_topk = static_cast<int>(topk_weights->size(1));
            EP_HIP_HOST_ASSERT(num_topk <= DEEP_EP_HIP_MAX_TOPK);
        }
        for (const auto* b : {&bias_0, &bias_1})
            if (b->has_value())
                EP_HIP_HOST_ASSERT((*b)->scalar_type() == x.scalar_type() and (*b)->dim() == 2 and (*b)->size(0) == num_tokens and
                                   (*b)->size(1) == hidden and (*b)->is_cuda() and (*b)->is_contiguous());
        EP_HIP_HOST_ASSERT(bias_0.has_value() or not bias_1.has_value());

        StreamScope scope(*this, previous_event, allocate_on_comm_stream, async, /*v1_rules=*/true);
        const Stream& run = scope.run_stream;
        torch::Tensor workspace = acquire_workspace(run, int64_t(4096));
        c10::hip::HIPStreamGuardMasqueradingAsCUDA on_run(run);
        torch::Tensor combined_x = torch::empty({num_tokens, hidden}, x.options());
        std::optional<torch::Tensor> combined_topk_weights;
        if (topk_weights.has_value()) combined_topk_weights = torch::empty({num_tokens, num_topk}, topk_weights->options());
        deep_ep_hip_intranode_combine_args args{};
        args.tuning = process_tuning();
        args.num_tokens = num_tokens; args.hidden = hidden; args.num_ranks = R; args.num_topk = num_topk;
        args.x = x.data_ptr(); args.num_x_rows = num_x_rows;
        args.topk_weights = ptr_of<const float>(topk_weights);
        args.bias_0 = bias_0.has_value() ? bias_0->data_ptr() : nullptr;
        args.bias_1 = bias_1.has_value() ? bias_1->data_ptr() : nullptr;
        args.send_head = static_cast<const int32_t*>(send_head.data_ptr());
        args.combined_x = combined_x.data_ptr(); args.combined_topk_weights = ptr_of<float>(combined_topk_weights);
        args.workspace = workspace.data_ptr(); args.workspace_bytes = static_cast<uint64_t>(workspace.numel());
        check_abi(deep_ep_hip_launch_intranode_combine(&args, run.stream()), "intranode combine");
        std::optional<EventHandle> event = scope.finish({x, topk_weights, bias_0, bias_1, src_idx, send_head, rank_prefix_matrix,
                                                         channel_prefix_matrix, combined_x, combined_topk_weights, workspace});
        return {combined_x, combined_topk_weights, event};
    }

    void internode_unsupported() const {
        PyErr_SetString(PyExc_NotImplementedError, "the HIP backend has one scale-up domain: there are no RDMA ranks to dispatch to or combine from");
        throw pybind11::error_already_set();
    }

    // Nothing is staged between calls on one GPU, so there is nothing to clean (csrc/legacy/buffer.hpp:1431-1461).
    void clean_low_latency_buffer(int /*num_max_dispatch_tokens_per_rank*/, int /*hidden*/, int /*num_experts*/) {}

    // ---- low-latency dispatch: the 11 arguments and the 7-tuple of csrc/legacy/buffer.hpp:1455-1596 ----
    // FP8 scales are amax * fp32(1 / 448), as the reference's kernel stores them (csrc/kernels/legacy/utils.cuh:499-501);
    // with `round_scale` they are rounded up to powers of two (:481-498) and with `use_ue8m0` returned as exponent bytes
    // packed four to an int32: [E / R, R * M, hidden / 512].  Scale tensors are column-major in their last two dimensions.
    // Layout ranges of source ranks that do not send in a call read (begin 0, count 0).  The hook, when asked for, does
    // nothing: the reference splits send and receive around it; on one GPU everything is already enqueued.
    std::tuple<torch::Tensor, std::optional<torch::Tensor>, torch::Tensor, torch::Tensor, torch::Tensor, std::optional<EventHandle>,
               std::optional<std::function<void()>>>
    low_latency_dispatch(const torch::Tensor& x, const torch::Tensor& topk_idx,
                         const std::optional<torch::Tensor>& cumulative_local_expert_recv_stats,
                         const std::optional<torch::Tensor>& /*dispatch_wait_recv_cost_stats*/, int num_max_dispatch_tokens_per_rank,
                         int num_experts, bool use_fp8, bool round_scale, bool use_ue8m0, bool async, bool return_recv_hook) {
        EP_HIP_HOST_ASSERT(not destroyed_);
        EP_HIP_HOST_ASSERT(not round_scale or use_fp8);
        EP_HIP_HOST_ASSERT(not use_ue8m0 or round_scale);
        EP_HIP_HOST_ASSERT(not (return_recv_hook and async));
        const int R = num_ranks_, M = num_max_dispatch_tokens_per_rank;
        EP_HIP_HOST_ASSERT(x.scalar_type() == torch::kBFloat16 and x.is_contiguous() and x.is_cuda());
        EP_HIP_HOST_ASSERT(topk_idx.is_contiguous() and topk_idx.scalar_type() == torch::kInt64 and topk_idx.is_cuda());
        EP_HIP_HOST_ASSERT(num_experts % R == 0);
        int S, T, H, src_begin;
        if (x.dim() == 3) {                       // all logical source ranks stacked
            S = static_cast<int>(x.size(0)); T = static_cast<int>(x.size(1)); H = static_cast<int>(x.size(2));
            EP_HIP_HOST_ASSERT(S == R and topk_idx.dim() == 3 and topk_idx.size(0) == S and topk_idx.size(1) == T);
            src_begin = 0;
        } else {
            EP_HIP_HOST_ASSERT(x.dim() == 2 and topk_idx.dim() == 2 and x.size(0) == topk_idx.size(0));
            S = 1; T = static_cast<int>(x.size(0)); H = static_cast<int>(x.size(1));
            src_begin = rank_idx_;
        }
        const int K = static_cast<int>(topk_idx.size(-1));
        EP_HIP_HOST_ASSERT(T <= M and H % 16 == 0 and (not use_fp8 or H % 128 == 0));
        EP_HIP_HOST_ASSERT((int64_t(R) * M) % 4 == 0);           // rows per expert, for the column-major scales
        EP_HIP_HOST_ASSERT(not use_ue8m0 or H % 512 == 0);
        const int E_l = num_experts / R;
        const int64_t rows = int64_t(R) * M;
        if (cumulative_local_expert_recv_stats.has_value())
            EP_HIP_HOST_ASSERT(cumulative_local_expert_recv_stats->scalar_type() == torch::kInt32 and
                               cumulative_local_expert_recv_stats->dim() == 1 and cumulative_local_expert_recv_stats->size(0) == E_l);

        StreamScope scope(*this, std::nullopt, false, async);
        const Stream& run = scope.run_stream;
        if (ll_last_stream_ != run) stream_wait(run, ll_last_stream_);       // the low-latency workspace is shared too
        c10::hip::HIPStreamGuardMasqueradingAsCUDA on_run(run);
        const auto dev = torch::TensorOptions().device(device_);
        // Two allocations: the payload with its scales, and the small outputs (ranges first, for their 8-byte
        // alignment).  The kernel writes every range, (begin 0, count 0) for source ranks that do not send in this call.
        TensorPack payload(device_), small(device_);
        const int i_x = payload.add(use_fp8 ? torch::kFloat8_e4m3fn : torch::kBFloat16, {E_l, rows, H});
        int i_scales = -1;                                              // [E_l, rows, groups], column-major in the last two
        if (use_fp8 and use_ue8m0) i_scales = payload.add(torch::kInt32, {E_l, rows, H / 512}, {int64_t(H / 512) * rows, 1, rows});
        else if (use_fp8) i_scales = payload.add(torch::kFloat32, {E_l, rows, H / 128}, {int64_t(H / 128) * rows, 1, rows});
        const int i_range = small.add(torch::kInt64, {E_l, R});
        const int i_info = small.add(torch::kInt32, {E_l, rows});
        const int i_count = small.add(torch::kInt32, {E_l});
        const int i_lane = small.add(torch::kInt32, {int64_t(S) * T, K});
        payload.allocate();
        small.allocate();
        torch::Tensor packed_recv_x = payload.get(i_x);
        std::optional<torch::Tensor> packed_recv_x_scales;
        if (i_scales >= 0) packed_recv_x_scales = payload.get(i_scales);
        torch::Tensor packed_recv_layout_range = small.get(i_range);
        torch::Tensor packed_recv_src_info = small.get(i_info);
        torch::Tensor packed_recv_count = small.get(i_count);
        torch::Tensor lane_rows = small.get(i_lane);
        if (T > 0) {
            const int64_t need = static_cast<int64_t>(deep_ep_hip_ll_workspace_bytes(S, T, K, E_l));
            if (not ll_workspace_.has_value() or ll_workspace_->numel() < need)
                ll_workspace_ = torch::zeros({std::max<int64_t>(need, 4096)}, dev.dtype(torch::kUInt8));
            deep_ep_hip_ll_dispatch_args args{};
            args.tuning = process_tuning();
            args.use_fp8 = use_fp8; args.round_scale = round_scale; args.use_ue8m0 = use_ue8m0;
            args.num_src_ranks = S; args.src_rank_begin = src_begin; args.src_token_stride = T;
            args.hidden = H; args.num_topk = K; args.num_experts = num_experts;
            args.expert_begin = rank_idx_ * E_l; args.num_local_experts = E_l;
            args.num_ranks = R; args.num_max_dispatch_tokens_per_rank = M;
            args.x = x.data_ptr(); args.topk_idx = static_cast<const int64_t*>(topk_idx.data_ptr());
            args.packed_recv_x = packed_recv_x.data_ptr();
            args.packed_recv_x_scales = packed_recv_x_scales.has_value() ? static_cast<float*>(packed_recv_x_scales->data_ptr()) : nullptr;
            args.packed_recv_count = static_cast<int32_t*>(packed_recv_count.data_ptr());
            args.packed_recv_src_info = static_cast<int32_t*>(packed_recv_src_info.data_ptr());
            args.packed_recv_layout_range = static_cast<int64_t*>(packed_recv_layout_range.data_ptr());
            args.cumulative_local_expert_recv_stats = ptr_of<int32_t>(cumulative_local_expert_recv_stats);
            args.lane_rows = static_cast<int32_t*>(lane_rows.data_ptr());
            args.workspace = ll_workspace_->data_ptr(); args.workspace_bytes = static_cast<uint64_t>(ll_workspace_->numel());
            check_abi(deep_ep_hip_launch_ll_dispatch(&args, run.stream()), "low_latency_dispatch");
            // the packed row of every (token, lane) rides beside the handle: the combine of this very handle skips
            // its search through src_info
            lane_rows_of_handle_.remember(packed_recv_src_info, lane_rows);
        } else {
            packed_recv_layout_range.zero_();
            packed_recv_count.zero_();
        }
        ll_last_stream_ = run;
        std::optional<EventHandle> event = scope.finish({x, topk_idx, packed_recv_x, packed_recv_x_scales, packed_recv_count,
                                                         packed_recv_src_info, packed_recv_layout_range,
                                                         cumulative_local_expert_recv_stats, lane_rows, ll_workspace_});
        std::optional<std::function<void()>> hook;
        if (return_recv_hook) hook = [] {};
        return {packed_recv_x, packed_recv_x_scales, packed_recv_count, packed_recv_src_info, packed_recv_layout_range, event, hook};
    }

    // [E / R, R * M, hidden] BF16 buffer a caller may fill instead of passing `x` to low_latency_combine with zero_copy
    // (csrc/legacy/buffer.hpp:1717-1729).
    torch::Tensor get_next_low_latency_combine_buffer(int num_max_dispatch_tokens_per_rank, int hidden, int num_experts) {
        const std::vector<int64_t> shape = {num_experts / num_ranks_, int64_t(num_ranks_) * num_max_dispatch_tokens_per_rank, hidden};
        if (not ll_combine_buffer_.has_value() or ll_combine_buffer_->sizes().vec() != shape)
            ll_combine_buffer_ = torch::empty(shape, torch::TensorOptions().dtype(torch::kBFloat16).device(device_));
        return *ll_combine_buffer_;
    }

    // ---- low-latency combine: the 13 arguments and the 3-tuple of csrc/legacy/buffer.hpp:1598-1715 ----
    // Each token sums, in lane order and in fp32, weight * row over its lanes whose expert lives on this rank, then
    // rounds once to BF16.  `use_logfmt`: every row first passes through the LogFMT-10 codec (the reference compresses
    // the rows it sends this way, csrc/kernels/legacy/internode_ll.cu:556-712); needs hidden % 512 == 0 and excludes
    // `zero_copy` (:1182).
    std::tuple<torch::Tensor, std::optional<EventHandle>, std::optional<std::function<void()>>>
    low_latency_combine(const torch::Tensor& x_arg, const torch::Tensor& topk_idx, const torch::Tensor& topk_weights,
                        const torch::Tensor& src_info, const torch::Tensor& layout_range,
                        const std::optional<torch::Tensor>& /*combine_wait_recv_cost_stats*/, int num_max_dispatch_tokens_per_rank,
                        int num_experts, bool use_logfmt, bool zero_copy, bool async, bool return_recv_hook,
                        const std::optional<torch::Tensor>& out) {
        EP_HIP_HOST_ASSERT(not destroyed_);
        EP_HIP_HOST_ASSERT(not (zero_copy and use_logfmt));
        EP_HIP_HOST_ASSERT(not (return_recv_hook and async));
        const int R = num_ranks_, M = num_max_dispatch_tokens_per_rank, E_l = num_experts / R;
        torch::Tensor x = x_arg;
        if (zero_copy) {
            EP_HIP_HOST_ASSERT(ll_combine_buffer_.has_value());       // get_next_low_latency_combine_buffer() comes first
            x = *ll_combine_buffer_;
        }
        EP_HIP_HOST_ASSERT(x.dim() == 3 and x.is_contiguous() and x.scalar_type() == torch::kBFloat16 and x.is_cuda());
        EP_HIP_HOST_ASSERT(x.size(0) == E_l and x.size(1) == int64_t(R) * M);
        const int H = static_cast<int>(x.size(2));
        EP_HIP_HOST_ASSERT(topk_idx.is_contiguous() and topk_idx.scalar_type() == torch::kInt64);
        EP_HIP_HOST_ASSERT(topk_weights.is_contiguous() and topk_weights.scalar_type() == torch::kFloat32);
        EP_HIP_HOST_ASSERT(topk_idx.sizes() == topk_weights.sizes());
        EP_HIP_HOST_ASSERT(src_info.dim() == 2 and src_info.is_contiguous() and src_info.scalar_type() == torch::kInt32 and
                           src_info.size(0) == E_l);
        EP_HIP_HOST_ASSERT(layout_range.dim() == 2 and layout_range.is_contiguous() and layout_range.scalar_type() == torch::kInt64 and
                           layout_range.size(0) == E_l and layout_range.size(1) == R);
        int S, T, K, src_begin;
        std::vector<int64_t> out_shape;
        if (topk_idx.dim() == 3) {
            S = static_cast<int>(topk_idx.size(0)); T = static_cast<int>(topk_idx.size(1)); K = static_cast<int>(topk_idx.size(2));
            EP_HIP_HOST_ASSERT(S == R);
            src_begin = 0;
            out_shape = {S, T, H};
        } else {
            EP_HIP_HOST_ASSERT(topk_idx.dim() == 2);
            S = 1; T = static_cast<int>(topk_idx.size(0)); K = static_cast<int>(topk_idx.size(1));
            src_begin = rank_idx_;
            out_shape = {T, H};
        }
        EP_HIP_HOST_ASSERT(T <= M);

        StreamScope scope(*this, std::nullopt, false, async);
        const Stream& run = scope.run_stream;
        if (ll_last_stream_ != run) stream_wait(run, ll_last_stream_);
        c10::hip::HIPStreamGuardMasqueradingAsCUDA on_run(run);
        torch::Tensor combined_x;
        if (out.has_value()) {
            EP_HIP_HOST_ASSERT(out->sizes().vec() == out_shape and out->scalar_type() == torch::kBFloat16 and out->is_contiguous());
            combined_x = *out;
        } else {
            combined_x = torch::empty(out_shape, x.options());
        }
        if (T > 0) {
            if (not ll_workspace_.has_value())
                ll_workspace_ = torch::zeros({4096}, torch::TensorOptions().dtype(torch::kUInt8).device(device_));
            deep_ep_hip_ll_combine_args args{};
            args.tuning = process_tuning();
            args.num_src_ranks = S; args.src_rank_begin = src_begin; args.src_token_stride = T;
            args.use_logfmt = use_logfmt;
            args.hidden = H; args.num_topk = K; args.num_experts = num_experts;
            args.expert_begin = rank_idx_ * E_l; args.num_local_experts = E_l; args.num_ranks = R;
            args.num_max_dispatch_tokens_per_rank = M;
            args.x = x.data_ptr();
            args.topk_idx = static_cast<const int64_t*>(topk_idx.data_ptr());
            args.topk_weights = static_cast<const float*>(topk_weights.data_ptr());
            args.packed_recv_src_info = static_cast<const int32_t*>(src_info.data_ptr());
            args.packed_recv_layout_range = static_cast<const int64_t*>(layout_range.data_ptr());
            const std::optional<torch::Tensor> lane_rows = lane_rows_of_handle_.find(src_info);
            if (lane_rows.has_value() and lane_rows->size(0) == int64_t(S) * T and lane_rows->size(1) == K)
                args.lane_rows = static_cast<const int32_t*>(lane_rows->data_ptr());
            args.combined_x = combined_x.data_ptr();
            args.workspace = ll_workspace_->data_ptr(); args.workspace_bytes = static_cast<uint64_t>(ll_workspace_->numel());
            check_abi(deep_ep_hip_launch_ll_combine(&args, run.stream()), "low_latency_combine");
        }
        ll_last_stream_ = run;
        std::optional<EventHandle> event = scope.finish({x, topk_idx, topk_weights, src_info, layout_range, combined_x, ll_workspace_});
        std::optional<std::function<void()>> hook;
        if (return_recv_hook) hook = [] {};
        return {combined_x, event, hook};
    }

private:
    int64_t num_nvl_bytes_, num_rdma_bytes_;
    bool low_latency_mode_;
    std::optional<torch::Tensor> ll_workspace_, ll_combine_buffer_;
    Stream ll_last_stream_ = comm_stream_;      // stream of the last launch that used the low-latency workspace
    HandleMemory send_head_of_handle_;          // rank_prefix_matrix of a dispatch -> its send_head
    HandleMemory lane_rows_of_handle_;          // packed_recv_src_info of a low-latency dispatch -> packed row of every (token, lane)
};

}  // namespace deep_ep::hip
