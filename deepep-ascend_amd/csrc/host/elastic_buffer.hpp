// Host side of dispatch / combine for the HIP backend: the class the `deep_ep._C` extension registers as
// `ElasticBuffer` (the role of csrc/elastic/buffer.hpp:83-1345 on CUDA and csrc/backends/ascend/elastic_buffer.hpp on
// Ascend).  It checks arguments, allocates the outputs, sequences the launches on the right stream and returns the
// reference's tuples.
//
// One GPU, logical ranks: `num_ranks` only decides which bucket (destination rank) an expert belongs to; every
// bucket lives in this GPU's HBM.  One call moves the tokens of the logical source rank `rank_idx`.
#pragma once

#include "runtime_base.hpp"

namespace deep_ep::hip {

class ElasticBuffer : public HostRuntime {
public:
    using cpu_comm_t = pybind11::object;      // there is no CPU communicator on one GPU; whatever is passed is ignored

    ElasticBuffer(int rank_idx, int num_ranks, int64_t /*comm_handle*/, cpu_comm_t /*cpu_comm*/, int64_t num_buffer_bytes,
                  int64_t num_cpu_buffer_bytes, bool allow_hybrid_mode, bool allow_multiple_reduction,
                  bool prefer_overlap_with_compute, int /*sl_idx*/, int /*num_allocated_qps*/, int num_cpu_timeout_secs,
                  int /*num_gpu_timeout_secs*/, bool explicitly_destroy)
        : HostRuntime(rank_idx, num_ranks, explicitly_destroy), num_buffer_bytes_(num_buffer_bytes),
          allow_hybrid_mode_(allow_hybrid_mode), allow_multiple_reduction_(allow_multiple_reduction),
          prefer_overlap_with_compute_(prefer_overlap_with_compute), num_cpu_timeout_secs_(num_cpu_timeout_secs) {
        EP_HIP_HOST_ASSERT(num_buffer_bytes > 0 and num_buffer_bytes % kBufferAlignmentBytes == 0);
        EP_HIP_HOST_ASSERT(num_cpu_buffer_bytes == 0);      // CPU buffers are not supported by the HIP backend
    }

    // ---- lifetime ----
    void destroy() {
        release();
        slots_of_handle_.clear();
    }

    // (RDMA ranks, load/store-reachable ranks): every logical rank is local
    std::tuple<int, int> get_physical_domain_size() const { return {1, num_ranks_}; }

    // (scale-out ranks, scale-up ranks)
    std::tuple<int, int> get_logical_domain_size() const { return {1, num_ranks_}; }

    void barrier(bool use_comm_stream, bool with_cpu_sync, bool /*sequential*/) {
        // One process, one GPU: ordering between logical ranks is stream ordering.
        if (with_cpu_sync) c10::hip::device_synchronize();
        if (use_comm_stream) {
            const Stream compute = current_stream();
            if (compute != comm_stream_) {
                stream_wait(comm_stream_, compute);
                stream_wait(compute, comm_stream_);
            }
        }
        if (with_cpu_sync) c10::hip::device_synchronize();
    }

    // Size the reference would ask for (csrc/elastic/buffer.hpp:588-688, direct mode, peers reachable by load/store).
    // This backend scatters straight into the output tensors and needs no staging buffer; the number is kept so that
    // `num_bytes` / `get_buffer_size_hint` stay drop-in.  `comm_handle` is the logical rank count here.
    static int64_t calculate_buffer_size(int64_t comm_handle, int num_max_tokens_per_rank, int hidden, int num_topk,
                                         bool use_fp8_dispatch, bool /*allow_hybrid_mode*/, bool allow_multiple_reduction) {
        EP_HIP_HOST_ASSERT(num_max_tokens_per_rank > 0 and hidden > 0);
        EP_HIP_HOST_ASSERT((hidden + 31) / 32 * 4 <= hidden);
        const int64_t ranks = comm_handle > 0 ? comm_handle : 1;
        const int64_t topk = num_topk == 0 ? 32 : num_topk;
        auto record = [&](int64_t hidden_bytes, int64_t sf_bytes, bool with_metadata) {
            // deep_ep/include/deep_ep/common/layout.cuh:187-208
            const int64_t meta = topk * 8 + (with_metadata ? (1 + topk) * 4 : 0);
            return align_up(hidden_bytes, kRecordAlignBytes) + align_up(sf_bytes, kRecordAlignBytes) + align_up(meta, kRecordAlignBytes);
        };
        const int64_t sf_packs = use_fp8_dispatch ? (hidden + 31) / 32 : 0;
        const int64_t dispatch_bytes = ranks * num_max_tokens_per_rank * record(int64_t(hidden) * (use_fp8_dispatch ? 1 : 2), sf_packs * 4, true);
        const int64_t tokens_in_layout = allow_multiple_reduction ? std::min<int64_t>(ranks, topk) : topk;
        const int64_t combine_bytes = tokens_in_layout * num_max_tokens_per_rank * record(int64_t(hidden) * 2, 0, false);
        return align_up(std::max(dispatch_bytes, combine_bytes), kBufferAlignmentBytes);
    }

    // ---- dispatch: argument order and the 16-tuple follow csrc/elastic/buffer.hpp:695-728,1166-1178 ----
    // The 29 arguments are the reference's, in its order; `cast_to_fp8` is an extension bound as a trailing keyword
    // with a default: `x` is BF16 and the FP8 e4m3 cast with per-1x128 fp32 scales is fused into the scatter; the
    // result equals casting first and dispatching the pair.
    std::tuple<torch::Tensor, std::optional<torch::Tensor>, std::optional<torch::Tensor>, std::optional<torch::Tensor>,
               std::optional<torch::Tensor>, int, int, std::vector<int>, torch::Tensor, torch::Tensor, torch::Tensor,
               torch::Tensor, torch::Tensor, std::optional<torch::Tensor>, std::optional<torch::Tensor>,
               std::optional<EventHandle>>
    dispatch(const torch::Tensor& x, const std::optional<torch::Tensor>& sf, const torch::Tensor& topk_idx,
             const std::optional<torch::Tensor>& topk_weights,
             const std::optional<torch::Tensor>& cumulative_local_expert_recv_stats,
             const std::optional<int>& cached_num_recv_tokens, const std::optional<int>& cached_num_expanded_tokens,
             const std::optional<std::vector<int>>& cached_num_recv_tokens_per_expert_list,
             const std::optional<torch::Tensor>& cached_psum_num_recv_tokens_per_scaleup_rank,
             const std::optional<torch::Tensor>& cached_psum_num_recv_tokens_per_expert,
             const std::optional<torch::Tensor>& cached_num_unaligned_recv_tokens_per_expert,
             const std::optional<torch::Tensor>& cached_dst_buffer_slot_idx,
             const std::optional<torch::Tensor>& /*cached_token_metadata_at_forward*/,
             const std::optional<torch::Tensor>& cached_recv_src_metadata,
             const std::optional<torch::Tensor>& /*cached_channel_linked_list*/, int num_max_tokens_per_rank,
             int num_experts, int expert_alignment, int /*num_sms*/, int /*num_qps*/,
             const std::optional<EventHandle>& previous_event,
             const std::optional<EventHandle>& previous_event_before_epilogue, bool async_with_compute_stream,
             bool allocate_on_comm_stream, bool do_handle_copy, bool do_cpu_sync, bool do_expand, bool do_zero_padding,
             bool use_tma_aligned_col_major_sf, bool cast_to_fp8) {
        EP_HIP_HOST_ASSERT(not destroyed_);
        EP_HIP_HOST_ASSERT(not do_zero_padding or do_expand);
        const bool cached_mode = cached_num_recv_tokens.has_value();
        if (cached_mode) {
            EP_HIP_HOST_ASSERT(cached_num_recv_tokens_per_expert_list.has_value());
            EP_HIP_HOST_ASSERT(cached_num_expanded_tokens.has_value());
            EP_HIP_HOST_ASSERT(cached_psum_num_recv_tokens_per_scaleup_rank.has_value());
            EP_HIP_HOST_ASSERT(cached_psum_num_recv_tokens_per_expert.has_value());
            EP_HIP_HOST_ASSERT(cached_num_unaligned_recv_tokens_per_expert.has_value());
            EP_HIP_HOST_ASSERT(cached_dst_buffer_slot_idx.has_value());
            EP_HIP_HOST_ASSERT(cached_recv_src_metadata.has_value());
            EP_HIP_HOST_ASSERT(not do_cpu_sync);                                       // no CPU sync with a cached handle
            EP_HIP_HOST_ASSERT(not cumulative_local_expert_recv_stats.has_value());    // statistics need a fresh layout
        }

        EP_HIP_HOST_ASSERT(x.dim() == 2 and x.is_cuda() and x.is_contiguous());
        const int num_tokens = static_cast<int>(x.size(0)), hidden = static_cast<int>(x.size(1));
        EP_HIP_HOST_ASSERT((hidden * x.element_size()) % 16 == 0);
        EP_HIP_HOST_ASSERT(num_tokens <= num_max_tokens_per_rank);
        const int R = num_ranks_;
        EP_HIP_HOST_ASSERT(num_experts % R == 0);
        EP_HIP_HOST_ASSERT(num_experts <= DEEP_EP_HIP_MAX_EXPERTS);

        int payload, num_sf_packs = 0;
        int64_t sf_ts = 0, sf_hs = 0;
        torch::ScalarType out_dtype = x.scalar_type();
        std::optional<torch::ScalarType> sf_dtype;
        if (cast_to_fp8) {
            EP_HIP_HOST_ASSERT(not sf.has_value() and x.scalar_type() == torch::kBFloat16);
            EP_HIP_HOST_ASSERT(hidden % 128 == 0);
            payload = DEEP_EP_HIP_PAYLOAD_CAST_FP8;
            num_sf_packs = hidden / 128;
            out_dtype = torch::kFloat8_e4m3fn;
            sf_dtype = torch::kFloat32;
        } else if (sf.has_value()) {
            EP_HIP_HOST_ASSERT(x.element_size() == 1);
            EP_HIP_HOST_ASSERT(sf->dim() == 2 and sf->is_cuda() and sf->size(0) == num_tokens);
            EP_HIP_HOST_ASSERT(sf->element_size() == 4);                 // fp32, or four packed UE8M0 exponents
            payload = DEEP_EP_HIP_PAYLOAD_FP8;
            num_sf_packs = static_cast<int>(sf->size(1));
            sf_dtype = sf->scalar_type();
            sf_ts = sf->stride(0);
            sf_hs = sf->stride(1);
        } else {
            EP_HIP_HOST_ASSERT(x.scalar_type() == torch::kBFloat16);
            payload = DEEP_EP_HIP_PAYLOAD_BF16;
        }

        EP_HIP_HOST_ASSERT(topk_idx.dim() == 2 and topk_idx.size(0) == num_tokens);
        const int num_topk = static_cast<int>(topk_idx.size(1));
        EP_HIP_HOST_ASSERT(1 <= num_topk and num_topk <= DEEP_EP_HIP_MAX_TOPK);
        EP_HIP_HOST_ASSERT(topk_idx.scalar_type() == torch::kInt64);
        EP_HIP_HOST_ASSERT(topk_idx.is_cuda() and topk_idx.is_contiguous());
        if (topk_weights.has_value()) {
            EP_HIP_HOST_ASSERT(topk_weights->dim() == 2 and topk_weights->size(0) == num_tokens and topk_weights->size(1) == num_topk);
            EP_HIP_HOST_ASSERT(topk_weights->is_cuda() and topk_weights->is_contiguous() and topk_weights->scalar_type() == torch::kFloat32);
        }
        if (cumulative_local_expert_recv_stats.has_value()) {
            const auto& s = *cumulative_local_expert_recv_stats;
            EP_HIP_HOST_ASSERT(s.dim() == 1 and s.size(0) == num_experts and s.scalar_type() == torch::kInt32 and s.is_cuda() and s.is_contiguous());
        }

        StreamScope scope(*this, previous_event, allocate_on_comm_stream, async_with_compute_stream);
        const Stream& run = scope.run_stream;
        const auto i32 = torch::TensorOptions().dtype(torch::kInt32).device(device_);
        torch::Tensor workspace = acquire_workspace(run, num_tokens, num_topk, num_experts);

        torch::Tensor psum_rank, psum_expert, num_unaligned, dst_slot;
        std::optional<torch::Tensor> copied_topk_idx;
        {
            c10::hip::HIPStreamGuardMasqueradingAsCUDA on_run(run);      // allocations below belong to the run stream
            if (cached_mode) {
                psum_rank = *cached_psum_num_recv_tokens_per_scaleup_rank;
                psum_expert = *cached_psum_num_recv_tokens_per_expert;
                num_unaligned = *cached_num_unaligned_recv_tokens_per_expert;
                EP_HIP_HOST_ASSERT(psum_rank.dim() == 1 and psum_rank.size(0) == R and psum_rank.scalar_type() == torch::kInt32 and psum_rank.is_cuda());
                EP_HIP_HOST_ASSERT(psum_expert.dim() == 1 and psum_expert.size(0) == num_experts and psum_expert.scalar_type() == torch::kInt32);
                EP_HIP_HOST_ASSERT(num_unaligned.dim() == 1 and num_unaligned.size(0) == num_experts);
                dst_slot = *cached_dst_buffer_slot_idx;
                EP_HIP_HOST_ASSERT(dst_slot.dim() == 2 and dst_slot.size(0) == num_tokens and dst_slot.size(1) == num_topk and
                                   dst_slot.scalar_type() == torch::kInt32 and dst_slot.is_contiguous());
            } else {
                // what the handle keeps, in one allocation
                TensorPack pack(device_);
                const int i_rank = pack.add(torch::kInt32, {R});
                const int i_expert = pack.add(torch::kInt32, {num_experts});
                const int i_unaligned = pack.add(torch::kInt32, {num_experts});
                const int i_slot = pack.add(torch::kInt32, {num_tokens, num_topk});
                const int i_copy = do_handle_copy ? pack.add(torch::kInt64, {num_tokens, num_topk}) : -1;
                pack.allocate();
                psum_rank = pack.get(i_rank);
                psum_expert = pack.get(i_expert);
                num_unaligned = pack.get(i_unaligned);
                dst_slot = pack.get(i_slot);
                if (do_handle_copy) copied_topk_idx = pack.get(i_copy);
            }
        }

        deep_ep_hip_dispatch_args args{};
        args.payload = payload;
        args.cached = cached_mode ? 1 : 0;
        args.do_expand = do_expand ? 1 : 0;
        args.do_zero_padding = do_zero_padding ? 1 : 0;
        args.num_tokens = num_tokens; args.hidden = hidden; args.num_topk = num_topk;
        args.num_experts = num_experts; args.num_ranks = R; args.rank_idx = rank_idx_;
        args.num_max_tokens_per_rank = num_max_tokens_per_rank;
        args.expert_alignment = expert_alignment;
        args.x = x.data_ptr();
        args.sf = sf.has_value() ? sf->data_ptr() : nullptr;
        args.sf_token_stride = sf_ts; args.sf_hidden_stride = sf_hs;
        args.num_sf_packs = num_sf_packs;
        args.topk_idx = static_cast<const int64_t*>(topk_idx.data_ptr());
        args.topk_weights = ptr_of<const float>(topk_weights);
        args.copied_topk_idx = ptr_of<int64_t>(copied_topk_idx);
        args.psum_num_recv_tokens_per_rank = static_cast<int32_t*>(psum_rank.data_ptr());
        args.psum_num_recv_tokens_per_expert = static_cast<int32_t*>(psum_expert.data_ptr());
        args.num_unaligned_recv_tokens_per_expert = static_cast<int32_t*>(num_unaligned.data_ptr());
        args.cumulative_local_expert_recv_stats = ptr_of<int32_t>(cumulative_local_expert_recv_stats);
        args.host_counts = nullptr;
        args.dst_buffer_slot_idx = static_cast<int32_t*>(dst_slot.data_ptr());
        args.workspace = workspace.data_ptr();
        args.workspace_bytes = static_cast<uint64_t>(workspace.numel());
        args.tuning = process_tuning();
        void* stream_ptr = run.stream();

        // Sizes of the outputs
        int num_recv_tokens, num_expanded_tokens;
        std::vector<int> per_expert_list;
        if (cached_mode) {
            num_recv_tokens = *cached_num_recv_tokens;
            num_expanded_tokens = *cached_num_expanded_tokens;
            per_expert_list = *cached_num_recv_tokens_per_expert_list;
        } else if (do_cpu_sync) {
            // layout launch, then the host waits for the counts in its mailbox (no copy, no device synchronisation)
            int32_t* box = fresh_mailbox(R + num_experts + 1);
            args.phases = DEEP_EP_HIP_PHASE_LAYOUT;
            args.host_counts = box;
            check_abi(deep_ep_hip_launch_dispatch(&args, stream_ptr), "dispatch layout");
            args.host_counts = nullptr;
            if (not await_mailbox(box, R + num_experts + 1, num_cpu_timeout_secs_))
                throw EPException("DeepEP HIP backend: dispatch: timed out waiting for the layout counts");
            if (box[R + num_experts] != 0) {
                c10::hip::HIPStreamGuardMasqueradingAsCUDA on_run(run);
                read_and_clear_status(workspace, "dispatch");          // raises, and leaves the workspace ready again
            }
            num_recv_tokens = 0;
            for (int r = 0; r < R; ++r) num_recv_tokens += box[r];
            num_expanded_tokens = 0;
            per_expert_list.assign(box + R, box + R + num_experts);         // aligned counts
            for (int e = 0; e < num_experts; ++e) num_expanded_tokens += per_expert_list[e];
        } else {
            num_recv_tokens = num_max_tokens_per_rank * R;
            num_expanded_tokens = num_max_tokens_per_rank * std::min(num_topk, num_experts) + (expert_alignment - 1) * num_experts;
            num_expanded_tokens = static_cast<int>(align_up(num_expanded_tokens, expert_alignment));
        }

        const int64_t num_allocated = do_expand ? num_expanded_tokens : num_recv_tokens;
        torch::Tensor recv_x, recv_src_metadata;
        std::optional<torch::Tensor> recv_sf, recv_topk_idx, recv_topk_weights;
        int64_t rsf_ts = 0, rsf_hs = 0;
        {
            c10::hip::HIPStreamGuardMasqueradingAsCUDA on_run(run);
            recv_x = torch::empty({num_allocated, hidden}, torch::TensorOptions().dtype(out_dtype).device(device_));
            recv_src_metadata = cached_mode ? *cached_recv_src_metadata : torch::empty({num_recv_tokens, num_topk + 2}, i32);
            // what travels beside the payload (scales, indices, weights), in one allocation; the payload and the
            // handle's metadata stay on their own, because callers keep them for different spans
            TensorPack beside(device_);
            int i_sf = -1, i_idx = -1, i_w = -1;
            if (sf_dtype.has_value()) {
                if (not use_tma_aligned_col_major_sf) {
                    rsf_ts = num_sf_packs; rsf_hs = 1;
                } else {
                    rsf_ts = 1; rsf_hs = align_up(num_allocated, 4);        // column-major, rows padded to 4 (csrc/elastic/buffer.hpp:1092-1101)
                }
                i_sf = beside.add(*sf_dtype, {num_allocated, num_sf_packs}, {rsf_ts, rsf_hs});
            }
            if (not do_expand) i_idx = beside.add(torch::kInt64, {num_allocated, num_topk});
            if (topk_weights.has_value())
                i_w = do_expand ? beside.add(torch::kFloat32, {num_allocated}) : beside.add(torch::kFloat32, {num_allocated, num_topk});
            if (i_sf >= 0 or i_idx >= 0 or i_w >= 0) beside.allocate();
            if (i_sf >= 0) recv_sf = beside.get(i_sf);
            if (i_idx >= 0) recv_topk_idx = beside.get(i_idx);
            if (i_w >= 0) recv_topk_weights = beside.get(i_w);
        }

        if (previous_event_before_epilogue.has_value()) stream_wait(run, *previous_event_before_epilogue);

        args.phases = (cached_mode or do_cpu_sync) ? DEEP_EP_HIP_PHASE_MOVE : (DEEP_EP_HIP_PHASE_LAYOUT | DEEP_EP_HIP_PHASE_MOVE);
        args.recv_src_metadata = static_cast<int32_t*>(recv_src_metadata.data_ptr());
        args.recv_x = recv_x.data_ptr();
        args.recv_sf = recv_sf.has_value() ? recv_sf->data_ptr() : nullptr;
        args.recv_sf_token_stride = rsf_ts; args.recv_sf_hidden_stride = rsf_hs;
        args.recv_topk_idx = ptr_of<int64_t>(recv_topk_idx);
        args.recv_topk_weights = ptr_of<float>(recv_topk_weights);
        args.recv_capacity = recv_src_metadata.size(0);
        args.expanded_capacity = do_expand ? num_expanded_tokens : 0;
        check_abi(deep_ep_hip_launch_dispatch(&args, stream_ptr), "dispatch");
        if (not cached_mode) slots_of_handle_.remember(recv_src_metadata, dst_slot);

        std::optional<EventHandle> event = scope.finish(
            {x, sf, topk_idx, topk_weights, recv_x, recv_sf, recv_topk_idx, recv_topk_weights,
             cumulative_local_expert_recv_stats, copied_topk_idx, psum_rank, psum_expert, num_unaligned, recv_src_metadata,
             dst_slot, workspace});
        return {recv_x, recv_sf, recv_topk_idx, recv_topk_weights, copied_topk_idx, num_recv_tokens, num_expanded_tokens,
                per_expert_list, psum_rank, psum_expert, num_unaligned, recv_src_metadata, dst_slot, std::nullopt,
                std::nullopt, event};
    }

    // ---- combine: argument order and the 3-tuple follow csrc/elastic/buffer.hpp:1181-1198,1344 ----
    // The 18 arguments are the reference's, in its order.  A single GPU gathers rows through the handle's token ->
    // received-row map (`dst_buffer_slot_idx`) instead of routing them back through a buffer, and the reference's
    // signature does not carry that tensor: it may be given as a trailing keyword; otherwise the buffer finds the one
    // it produced together with this `src_metadata`, and for a handle it has not seen (or whose tensors were cloned)
    // the library rebuilds the map from `src_metadata[:, 0:2]` and the per-rank prefix, a scatter of one entry per
    // received row.
    std::tuple<torch::Tensor, std::optional<torch::Tensor>, std::optional<EventHandle>>
    combine(const torch::Tensor& x, const std::optional<torch::Tensor>& topk_weights, const std::optional<torch::Tensor>& bias_0,
            const std::optional<torch::Tensor>& bias_1, const torch::Tensor& src_metadata, const torch::Tensor& combined_topk_idx,
            const torch::Tensor& psum_num_recv_tokens_per_scaleup_rank,
            const std::optional<torch::Tensor>& /*token_metadata_at_forward*/,
            const std::optional<torch::Tensor>& /*channel_linked_list*/, int num_experts, int num_max_tokens_per_rank,
            int /*num_sms*/, int /*num_qps*/, const std::optional<EventHandle>& previous_event,
            const std::optional<EventHandle>& previous_event_before_epilogue, bool async_with_compute_stream,
            bool allocate_on_comm_stream, bool use_expanded_layout, const std::optional<torch::Tensor>& dst_buffer_slot_idx_arg) {
        EP_HIP_HOST_ASSERT(not destroyed_);
        EP_HIP_HOST_ASSERT(src_metadata.is_cuda() and src_metadata.is_contiguous() and src_metadata.scalar_type() == torch::kInt32);
        std::optional<torch::Tensor> dst_buffer_slot_idx = dst_buffer_slot_idx_arg;
        if (not dst_buffer_slot_idx.has_value()) dst_buffer_slot_idx = slots_of_handle_.find(src_metadata);
        EP_HIP_HOST_ASSERT(x.dim() == 2 and x.is_cuda() and x.is_contiguous());
        EP_HIP_HOST_ASSERT(x.scalar_type() == torch::kBFloat16);
        const int64_t num_x_rows = x.size(0);
        const int hidden = static_cast<int>(x.size(1));
        EP_HIP_HOST_ASSERT((hidden * 2) % 16 == 0);
        EP_HIP_HOST_ASSERT(combined_topk_idx.dim() == 2 and combined_topk_idx.scalar_type() == torch::kInt64 and combined_topk_idx.is_contiguous());
        const int num_tokens = static_cast<int>(combined_topk_idx.size(0)), num_topk = static_cast<int>(combined_topk_idx.size(1));
        if (dst_buffer_slot_idx.has_value())
            EP_HIP_HOST_ASSERT(dst_buffer_slot_idx->dim() == 2 and dst_buffer_slot_idx->size(0) == num_tokens and
                               dst_buffer_slot_idx->size(1) == num_topk and dst_buffer_slot_idx->scalar_type() == torch::kInt32 and
                               dst_buffer_slot_idx->is_contiguous());
        EP_HIP_HOST_ASSERT(psum_num_recv_tokens_per_scaleup_rank.dim() == 1 and psum_num_recv_tokens_per_scaleup_rank.size(0) == num_ranks_ and
                           psum_num_recv_tokens_per_scaleup_rank.scalar_type() == torch::kInt32);
        EP_HIP_HOST_ASSERT(src_metadata.dim() == 2 and src_metadata.size(1) == num_topk + 2);
        if (topk_weights.has_value()) {
            EP_HIP_HOST_ASSERT(topk_weights->scalar_type() == torch::kFloat32 and topk_weights->is_cuda() and topk_weights->is_contiguous());
            if (use_expanded_layout) EP_HIP_HOST_ASSERT(topk_weights->dim() == 1 and topk_weights->size(0) == num_x_rows);
            else EP_HIP_HOST_ASSERT(topk_weights->dim() == 2 and topk_weights->size(0) == num_x_rows and topk_weights->size(1) == num_topk);
        }
        for (const auto* b : {&bias_0, &bias_1}) {
            if (b->has_value()) {
                const auto& t = **b;
                EP_HIP_HOST_ASSERT(t.scalar_type() == x.scalar_type() and t.dim() == 2 and t.size(0) == num_tokens and t.size(1) == hidden and
                                   t.is_cuda() and t.is_contiguous());
            }
        }
        EP_HIP_HOST_ASSERT(bias_0.has_value() or not bias_1.has_value());

        StreamScope scope(*this, previous_event, allocate_on_comm_stream, async_with_compute_stream);
        const Stream& run = scope.run_stream;
        torch::Tensor workspace = acquire_workspace(run, num_tokens, num_topk, num_experts);
        torch::Tensor combined_x;
        std::optional<torch::Tensor> combined_topk_weights;
        {
            c10::hip::HIPStreamGuardMasqueradingAsCUDA on_run(run);
            combined_x = torch::empty({num_tokens, hidden}, x.options());
            if (topk_weights.has_value())
                combined_topk_weights = torch::empty({num_tokens, num_topk}, torch::TensorOptions().dtype(torch::kFloat32).device(device_));
        }
        if (previous_event_before_epilogue.has_value()) stream_wait(run, *previous_event_before_epilogue);

        deep_ep_hip_combine_args args{};
        args.do_expand = use_expanded_layout ? 1 : 0;
        args.allow_multiple_reduction = allow_multiple_reduction_ ? 1 : 0;
        args.num_tokens = num_tokens; args.hidden = hidden; args.num_topk = num_topk;
        args.num_experts = num_experts; args.num_ranks = num_ranks_;
        args.rank_idx = rank_idx_; args.num_max_tokens_per_rank = num_max_tokens_per_rank;
        args.x = x.data_ptr();
        args.num_x_rows = num_x_rows;
        args.topk_weights = ptr_of<const float>(topk_weights);
        args.bias_0 = bias_0.has_value() ? bias_0->data_ptr() : nullptr;
        args.bias_1 = bias_1.has_value() ? bias_1->data_ptr() : nullptr;
        args.topk_idx = static_cast<const int64_t*>(combined_topk_idx.data_ptr());
        args.dst_buffer_slot_idx = ptr_of<const int32_t>(dst_buffer_slot_idx);     // NULL: rebuilt in the workspace
        args.recv_src_metadata = static_cast<const int32_t*>(src_metadata.data_ptr());
        args.num_recv_rows = src_metadata.size(0);
        args.psum_num_recv_tokens_per_rank = static_cast<const int32_t*>(psum_num_recv_tokens_per_scaleup_rank.data_ptr());
        args.combined_x = combined_x.data_ptr();
        args.combined_topk_weights = ptr_of<float>(combined_topk_weights);
        args.workspace = workspace.data_ptr();
        args.workspace_bytes = static_cast<uint64_t>(workspace.numel());
        args.tuning = process_tuning();
        check_abi(deep_ep_hip_launch_combine(&args, run.stream()), "combine");

        std::optional<EventHandle> event = scope.finish({x, topk_weights, bias_0, bias_1, src_metadata, combined_topk_idx,
                                                         psum_num_recv_tokens_per_scaleup_rank, dst_buffer_slot_idx, combined_x,
                                                         combined_topk_weights, workspace});
        return {combined_x, combined_topk_weights, event};
    }

    // V1 `get_dispatch_layout` on this buffer is inherited from HostRuntime.

private:
    int64_t num_buffer_bytes_;
    bool allow_hybrid_mode_, allow_multiple_reduction_, prefer_overlap_with_compute_;
    int num_cpu_timeout_secs_;
    // recv_src_metadata of the dispatches of this buffer -> their dst_buffer_slot_idx: the token -> received-row map a
    // combine gathers through, which the reference's combine signature has no argument for
    HandleMemory slots_of_handle_;
};

}  // namespace deep_ep::hip
