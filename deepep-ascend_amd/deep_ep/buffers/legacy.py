"""`Buffer`: the part of the V1 Python surface that sits on the routing hot path —
`get_dispatch_layout`, `dispatch` / `combine` inside one scale-up domain, and the low-latency packed
dispatch / combine (reference deep_ep/buffers/legacy.py:293-455, 553-689).  The work is done by the compiled
host class `deep_ep._C.Buffer` (csrc/host/legacy_buffer.hpp), which takes the reference's positional arguments.

`dispatch` moves the tokens of logical source rank `group.rank()`; the received rows are the concatenation
over destination ranks d of what d gets from this source, in token order (rows of destination d start at
`rank_prefix_matrix[-1][:d].sum()`).  The handle is the reference's 6-tuple; its `send_head` holds receive
rows instead of queue positions (opaque to callers either way).

Logical ranks on one GPU.  `group.size()` = R logical ranks, `group.rank()` = this process's logical
rank.  The packed buffers returned by `low_latency_dispatch` are those of destination rank
`group.rank()` (experts [rank*E/R, (rank+1)*E/R)), shaped exactly as in the reference:
`[E/R, R * num_max_dispatch_tokens_per_rank, hidden]`.  Two input forms are accepted:
  * `x` `[T, H]`, `topk_idx` `[T, K]`: the tokens of logical source rank `group.rank()` only;
  * `x` `[R, T, H]`, `topk_idx` `[R, T, K]` (extension): the tokens of all R logical source ranks,
    i.e. everything destination rank `group.rank()` would receive in a real R-rank run.
Rows of one expert are filled by source rank ascending, then token ascending.
"""
from typing import Optional, Tuple, Union

import torch

from .. import _binding as _C
from ..platform import unwrap_event
from ..utils.event import EventOverlap


class Buffer:
    num_sms: int = 20

    def __init__(self, group, num_nvl_bytes: int = 0, num_rdma_bytes: int = 0, low_latency_mode: bool = False,
                 num_qps_per_rank: int = 24, allow_nvlink_for_low_latency_mode: bool = True,
                 allow_mnnvl: bool = False, explicitly_destroy: bool = False, enable_shrink: bool = False,
                 comm=None) -> None:
        self.group, self.rank, self.group_size = group, group.rank(), group.size()
        # sizes and mode are recorded as given; the rows land in the tensors the calls return, not in these buffers
        self.num_nvl_bytes, self.num_rdma_bytes, self.low_latency_mode = num_nvl_bytes, num_rdma_bytes, low_latency_mode
        self.explicitly_destroy = explicitly_destroy
        self.runtime = _C.Buffer(self.rank, self.group_size, num_nvl_bytes, num_rdma_bytes, low_latency_mode,
                                 explicitly_destroy, enable_shrink, False)

    def destroy(self) -> None:
        assert self.explicitly_destroy, 'construct with explicitly_destroy=True to release by hand'
        runtime, self.runtime = self.runtime, None
        runtime.destroy()

    @staticmethod
    def capture() -> EventOverlap:
        return EventOverlap(_C.EventHandle())

    @staticmethod
    def is_sm90_compiled() -> bool:
        """The reference gates its FP8 paths on this (deep_ep/buffers/legacy.py:149-151); they are always built here."""
        return True

    def get_comm_stream(self) -> torch.cuda.Stream:
        ts = self.runtime.get_comm_stream()
        return torch.cuda.Stream(stream_id=ts.stream_id, device_index=ts.device_index, device_type=ts.device_type)

    def get_local_buffer_tensor(self, *args, **kwargs):
        raise NotImplementedError('the HIP backend stages nothing: there is no buffer to look into')

    def clean_low_latency_buffer(self, num_max_dispatch_tokens_per_rank: int, hidden: int, num_experts: int) -> None:
        """Nothing is staged between calls on one GPU, so there is nothing to clean
        (deep_ep/buffers/legacy.py:538-551)."""
        self.runtime.clean_low_latency_buffer(num_max_dispatch_tokens_per_rank, hidden, num_experts)

    # ---- mask buffers of the shrink mode (deep_ep/buffers/legacy.py:672-698): a rank is masked when it stops answering.
    # On one GPU every logical rank lives in the calling process and cannot time out, so no rank is ever masked.
    def low_latency_update_mask_buffer(self, rank_to_mask: int, mask: bool = False) -> None:
        if mask:
            raise NotImplementedError('the HIP backend has no peers to mask: every logical rank runs on this GPU')

    def low_latency_query_mask_buffer(self, mask_status: torch.Tensor) -> None:
        mask_status.zero_()

    def low_latency_clean_mask_buffer(self) -> None:
        pass

    def internode_dispatch(self, *args, **kwargs):
        return self.runtime.internode_dispatch(*args, **kwargs)        # raises NotImplementedError

    def internode_combine(self, *args, **kwargs):
        return self.runtime.internode_combine(*args, **kwargs)         # raises NotImplementedError

    @staticmethod
    def get_low_latency_rdma_size_hint(num_max_dispatch_tokens_per_rank: int, hidden: int, num_ranks: int,
                                       num_experts: int) -> int:
        """Bytes the reference would reserve (csrc/legacy/config.hpp:131-188); nothing is staged here."""
        return _C.get_low_latency_rdma_size_hint(num_max_dispatch_tokens_per_rank, hidden, num_ranks, num_experts)

    def get_dispatch_layout(self, topk_idx: torch.Tensor, num_experts: int,
                            previous_event: Optional[EventOverlap] = None, async_finish: bool = False,
                            allocate_on_comm_stream: bool = False):
        """Counts a dispatch needs.

        Returns:
            num_tokens_per_rank: `[num_ranks]` int32, tokens that go to each rank (once per rank).
            num_tokens_per_rdma_rank: None (single scale-up domain).
            num_tokens_per_expert: `[num_experts]` int32.
            is_token_in_rank: `[num_tokens, num_ranks]` bool.
            event: valid if `async_finish`.
        """
        a, b, c, d, event = self.runtime.get_dispatch_layout(topk_idx, num_experts, unwrap_event(previous_event),
                                                             async_finish, allocate_on_comm_stream)
        return a, b, c, d, EventOverlap(event)

    @staticmethod
    def set_num_sms(new_num_sms: int) -> None:
        assert new_num_sms % 2 == 0, 'The SM count must be even'
        Buffer.num_sms = new_num_sms

    @staticmethod
    def get_dispatch_config(num_ranks: int) -> '_C.Config':
        """Default tuning config (deep_ep/buffers/legacy.py:243-266).  Only `num_sms` matters here: it fixes the
        channel count of the handle's channel matrices."""
        return _C.Config(Buffer.num_sms, 6, 256, 6, 128)

    @staticmethod
    def get_combine_config(num_ranks: int) -> '_C.Config':
        return _C.Config(Buffer.num_sms, 6, 256, 6, 128)

    @staticmethod
    def _unpack_bias(bias):
        """None, one tensor or a pair of tensors -> always a pair."""
        if bias is None or isinstance(bias, torch.Tensor):
            return bias, None
        first, second = bias            # anything else must be exactly two tensors
        return first, second

    def dispatch(self, x: Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]],
                 handle: Optional[Tuple] = None,
                 num_tokens_per_rank: Optional[torch.Tensor] = None,
                 num_tokens_per_rdma_rank: Optional[torch.Tensor] = None,
                 is_token_in_rank: Optional[torch.Tensor] = None,
                 num_tokens_per_expert: Optional[torch.Tensor] = None,
                 topk_idx: Optional[torch.Tensor] = None, topk_weights: Optional[torch.Tensor] = None,
                 expert_alignment: int = 1, num_worst_tokens: int = 0, config=None,
                 previous_event: Optional[EventOverlap] = None, async_finish: bool = False,
                 allocate_on_comm_stream: bool = False):
        """Dispatch tokens to the ranks that own their experts (signature and returns of
        deep_ep/buffers/legacy.py:322-404).

        Returns (recv_x or (recv_x, recv_x_scales), recv_topk_idx, recv_topk_weights,
        num_recv_tokens_per_expert_list, handle, event).  `recv_topk_idx` holds ids local to the receiving
        rank or -1; `recv_topk_weights` is 0 where `recv_topk_idx` is -1.  The list has one aligned count per
        expert of every destination rank (empty with `num_worst_tokens`).  With `handle=` the layout is reused
        and only `recv_x` is returned.
        """
        config = config or self.get_dispatch_config(self.group_size)
        payload, scales = x if isinstance(x, tuple) else (x, None)
        streams = (unwrap_event(previous_event), async_finish, allocate_on_comm_stream)
        pack = (lambda rows, row_scales: rows) if scales is None else (lambda rows, row_scales: (rows, row_scales))

        if handle is not None:
            # cached: the six handle tensors stand in for the layout; only the payload moves
            assert topk_idx is None and topk_weights is None, 'A cached dispatch takes its routing from the handle'
            rank_prefix, channel_prefix, _, recv_src_idx, in_rank, send_head = handle
            out = self.runtime.intranode_dispatch(payload, scales, None, None, None, in_rank, None, recv_src_idx.size(0),
                                                  rank_prefix, channel_prefix, expert_alignment, num_worst_tokens, config,
                                                  *streams, cached_send_head=send_head)
            return pack(out[0], out[1]), None, None, None, None, EventOverlap(out[-1])

        assert all(t is not None for t in (num_tokens_per_rank, is_token_in_rank, num_tokens_per_expert)), \
            'A fresh dispatch needs the three outputs of get_dispatch_layout'
        (rows, row_scales, recv_topk_idx, recv_topk_weights, per_expert_list, rank_prefix, channel_prefix,
         recv_channel_prefix, recv_src_idx, send_head, event) = self.runtime.intranode_dispatch(
            payload, scales, topk_idx, topk_weights, num_tokens_per_rank, is_token_in_rank, num_tokens_per_expert, 0,
            None, None, expert_alignment, num_worst_tokens, config, *streams)
        handle = (rank_prefix, channel_prefix, recv_channel_prefix, recv_src_idx, is_token_in_rank, send_head)
        return pack(rows, row_scales), recv_topk_idx, recv_topk_weights, per_expert_list, handle, EventOverlap(event)

    def combine(self, x: torch.Tensor, handle: Tuple, topk_weights: Optional[torch.Tensor] = None,
                bias: Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor], None] = None, config=None,
                previous_event: Optional[EventOverlap] = None, async_finish: bool = False,
                allocate_on_comm_stream: bool = False):
        """Reduce (add, **without** weights) the rows of every token back to its origin
        (deep_ep/buffers/legacy.py:407-455): fp32 sum of the biases and of the token's rows in ascending rank
        order, one rounding to BF16; `topk_weights` rows are summed the same way.
        Returns (combined_x, combined_topk_weights, event)."""
        config = config or self.get_combine_config(self.group_size)
        rank_prefix, _, channel_prefix, src_idx, _, send_head = handle
        first_bias, second_bias = self._unpack_bias(bias)
        combined_x, combined_topk_weights, event = self.runtime.intranode_combine(
            x, topk_weights, first_bias, second_bias, src_idx, rank_prefix, channel_prefix, send_head, config,
            unwrap_event(previous_event), async_finish, allocate_on_comm_stream)
        return combined_x, combined_topk_weights, EventOverlap(event)

    def low_latency_dispatch(self, x: torch.Tensor, topk_idx: torch.Tensor,
                             num_max_dispatch_tokens_per_rank: int, num_experts: int,
                             cumulative_local_expert_recv_stats: Optional[torch.Tensor] = None,
                             dispatch_wait_recv_cost_stats: Optional[torch.Tensor] = None,
                             use_fp8: bool = True, round_scale: bool = False, use_ue8m0: bool = False,
                             async_finish: bool = False, return_recv_hook: bool = False):
        """Dispatch into packed per-local-expert buffers.

        Returns (recv_x or (recv_x, recv_x_scales), recv_count, handle, event, hook) with
            recv_x: `[E/R, R*M, hidden]` FP8 e4m3 (or BF16 with `use_fp8=False`); rows at or beyond
                `recv_count[e]` are unspecified;
            recv_x_scales: `[E/R, R*M, hidden // 128]` fp32, column-major in the last two dimensions;
            recv_count: `[E/R]` int32;
            handle: `(src_info [E/R, R*M] int32, layout_range [E/R, R] int64 = (begin << 32) | count,
                      num_max_dispatch_tokens_per_rank, hidden, num_experts)`;
            hook: with `return_recv_hook`, a callable to invoke before reading the outputs (the reference splits
                send and receive around it; on one GPU everything is already enqueued and it does nothing).
        FP8 scales are amax * fp32(1/448), as the reference's kernel stores them (csrc/kernels/legacy/utils.cuh:499-501);
        with `round_scale` they are rounded up
        to powers of two (csrc/kernels/legacy/utils.cuh:481-503) and with `use_ue8m0` returned as exponent bytes
        packed four to an int32: `[E/R, R*M, hidden // 512]`, column-major in the last two dimensions.
        """
        (packed_recv_x, packed_recv_x_scales, packed_recv_count, packed_recv_src_info, packed_recv_layout_range, event,
         hook) = self.runtime.low_latency_dispatch(x, topk_idx, cumulative_local_expert_recv_stats,
                                                   dispatch_wait_recv_cost_stats, num_max_dispatch_tokens_per_rank,
                                                   num_experts, use_fp8, round_scale, use_ue8m0, async_finish,
                                                   return_recv_hook)
        handle = (packed_recv_src_info, packed_recv_layout_range, num_max_dispatch_tokens_per_rank, x.size(-1), num_experts)
        tensors = (x, topk_idx, packed_recv_x, packed_recv_x_scales, packed_recv_count, packed_recv_src_info,
                   packed_recv_layout_range, cumulative_local_expert_recv_stats)
        recv = (packed_recv_x, packed_recv_x_scales) if use_fp8 else packed_recv_x
        return recv, packed_recv_count, handle, EventOverlap(event, tensors if async_finish else None), hook

    def get_next_low_latency_combine_buffer(self, handle: tuple) -> torch.Tensor:
        """`[E/R, R*M, hidden]` BF16 buffer a caller may fill instead of passing `x` to `low_latency_combine`
        (`zero_copy=True`), deep_ep/buffers/legacy.py:673-689."""
        src_info, layout_range, num_max_dispatch_tokens_per_rank, hidden, num_experts = handle
        return self.runtime.get_next_low_latency_combine_buffer(num_max_dispatch_tokens_per_rank, hidden, num_experts)

    def low_latency_combine(self, x: torch.Tensor, topk_idx: torch.Tensor, topk_weights: torch.Tensor,
                            handle: tuple, use_logfmt: bool = False, zero_copy: bool = False,
                            async_finish: bool = False, return_recv_hook: bool = False,
                            out: Optional[torch.Tensor] = None,
                            combine_wait_recv_cost_stats: Optional[torch.Tensor] = None):
        """Weighted reduce of expert outputs back to token order.

        `x` is `[E/R, R*M, hidden]` BF16 laid out like the dispatched buffers; `topk_idx` / `topk_weights` are
        those of the dispatched tokens (`[T, K]`, or `[R, T, K]` for the stacked form).  Each token sums, in lane
        order and in fp32, `weight * row` over its lanes whose expert lives on this rank, then rounds once to
        BF16.  Returns (combined_x, event, hook); `hook` is a no-op callable with `return_recv_hook`, else None.
        With `zero_copy` the rows are read from `get_next_low_latency_combine_buffer(handle)` instead of `x`.
        `use_logfmt`: every row passes through the LogFMT-10 codec before it is accumulated (the reference compresses
        the rows it sends this way, csrc/kernels/legacy/internode_ll.cu:556-712): chunks of 1024 channels (512 if hidden
        is not a multiple of 1024) whose 128-channel groups all have amax < 1 come back as 9-bit logarithmic codes,
        the others unchanged.  Needs hidden % 512 == 0 and excludes `zero_copy` (internode_ll.cu:1182).
        """
        src_info, layout_range, num_max_dispatch_tokens_per_rank, hidden, num_experts = handle
        combined_x, event, hook = self.runtime.low_latency_combine(
            x, topk_idx, topk_weights, src_info, layout_range, combine_wait_recv_cost_stats,
            num_max_dispatch_tokens_per_rank, num_experts, use_logfmt, zero_copy, async_finish, return_recv_hook, out)
        tensors = (x, topk_idx, topk_weights, src_info, layout_range, combined_x)
        return combined_x, EventOverlap(event, tensors if async_finish else None), hook
