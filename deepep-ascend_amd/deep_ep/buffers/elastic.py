"""`ElasticBuffer` / `EPHandle`: the V2 Python surface (reference deep_ep/buffers/elastic.py:40-113,
331-553, 884-911, 1391-1712) over the single-GPU HIP runtime.

Logical ranks.  `group.size()` is the logical expert-parallel width R and `group.rank()` the logical
source rank of the tokens this process dispatches.  Destination rank d owns experts
[d*E/R, (d+1)*E/R); all R destination buckets live in this GPU's HBM.  A dispatch returns the
concatenation over d of "what d receives from this source": compact rows are ordered by
(d, token); expanded rows are grouped by global expert id.  Per-expert handle tensors therefore
have `num_experts` entries.  With R = 1 every shape and value equals the reference's at world
size 1.  Placement is scan based, hence already deterministic: `deterministic=True` changes nothing.
"""
import os
from dataclasses import dataclass, field
from typing import List, Optional, Tuple, Union

import torch

from .. import _binding as _C
from .._binding import EventHandle
from ..platform import capture_event, unwrap_event
from ..utils.event import EventOverlap
from ..utils.semantic import value_or


class LogicalGroup:
    """Stand-in for a `torch.distributed` group when the ranks are logical: anything with
    `rank()` and `size()` is accepted by `ElasticBuffer`."""

    def __init__(self, rank: int, size: int):
        assert 0 <= rank < size
        self._rank, self._size = rank, size

    def rank(self) -> int:
        return self._rank

    def size(self) -> int:
        return self._size

    def barrier(self) -> None:
        pass


@dataclass(eq=False)
class EPHandle:
    """What `dispatch` returns for `combine` and for cached re-dispatch.  Constructor arguments, in order, are the
    fields up to `channel_linked_list` (reference deep_ep/buffers/elastic.py:40-113).

    Fields:
        do_expand: whether the expanded (one row per (token, expert)) layout is used.
        num_experts, expert_alignment, num_max_tokens_per_rank, num_sms: the dispatch settings.
        topk_idx: the routing the handle was built from, `[num_tokens, num_topk]`.
        num_recv_tokens, num_expanded_tokens: row counts (upper bounds without CPU sync).
        num_recv_tokens_per_expert_list: aligned rows per expert as a Python list (empty without CPU sync).
        psum_num_recv_tokens_per_scaleup_rank: inclusive prefix of rows per destination rank, `[num_ranks]`.
        psum_num_recv_tokens_per_expert: per expert, inclusive prefix of aligned counts (compact) or
            region start + actual count (expanded), `[num_experts]`.
        num_unaligned_recv_tokens_per_expert: actual rows per expert, `[num_experts]`.
        recv_src_metadata: `[num_recv_tokens, num_topk + 2]`: source token, source rank * num_topk + master
            lane, then the expanded row of each lane (-1 if none).
        dst_buffer_slot_idx: `[num_tokens, num_topk]`: rank_idx * num_max_tokens_per_rank + slot inside the
            destination bucket on each destination's master (highest) lane, -1 elsewhere.
        token_metadata_at_forward, channel_linked_list: hybrid-mode fields, always None here.
        cached_recv_src_metadata_before_sort: deterministic-mode scratch of the reference, always None here.
    """
    do_expand: bool
    num_experts: int
    expert_alignment: int
    num_max_tokens_per_rank: int
    num_sms: int
    topk_idx: torch.Tensor
    num_recv_tokens: int
    num_expanded_tokens: int
    num_recv_tokens_per_expert_list: list
    psum_num_recv_tokens_per_scaleup_rank: torch.Tensor
    psum_num_recv_tokens_per_expert: torch.Tensor
    num_unaligned_recv_tokens_per_expert: torch.Tensor
    recv_src_metadata: torch.Tensor
    dst_buffer_slot_idx: torch.Tensor
    token_metadata_at_forward: Optional[torch.Tensor]
    channel_linked_list: Optional[torch.Tensor]
    cached_recv_src_metadata_before_sort: Optional[torch.Tensor] = field(default=None, init=False)

    def __post_init__(self):
        assert self.topk_idx is not None, "a handle always carries the routing it was built from"
        self.cached_recv_src_metadata_before_sort = None        # an instance attribute, as in the reference

    def deterministic_sort(self, do_cpu_sync: bool, is_cached_dispatch: bool, recv_x: torch.Tensor,
                           recv_sf: Optional[torch.Tensor], recv_topk_idx: Optional[torch.Tensor],
                           recv_topk_weights: Optional[torch.Tensor], channel_linked_list: Optional[torch.Tensor]) -> None:
        """The reference sorts what it received by source token to undo its arrival order
        (deep_ep/buffers/elastic.py:115-207).  Here rows are placed by a scan, in source-token order inside every
        bucket and every expert region, so the sorted order is the order the tensors already have: nothing moves."""
        return None

    def layout_fields(self) -> tuple:
        """The ten values a cached dispatch hands back to the runtime, in the runtime's argument order."""
        return (self.num_recv_tokens, self.num_expanded_tokens, self.num_recv_tokens_per_expert_list,
                self.psum_num_recv_tokens_per_scaleup_rank, self.psum_num_recv_tokens_per_expert,
                self.num_unaligned_recv_tokens_per_expert, self.dst_buffer_slot_idx,
                self.token_metadata_at_forward, self.recv_src_metadata, self.channel_linked_list)


class ElasticBuffer:
    """Expert-parallel dispatch / combine on one MI355X.

    Attributes:
        group, rank_idx, num_ranks: the (logical) communication group.
        allow_hybrid_mode, allow_multiple_reduction, prefer_overlap_with_compute, deterministic: as given.
        num_bytes: the buffer size the reference would reserve (kept for compatibility; unused).
        num_max_tokens_per_rank: default capacity per rank.
        num_scaleout_ranks / num_scaleup_ranks, scaleout_rank_idx / scaleup_rank_idx,
        num_rdma_ranks / num_nvlink_ranks: domain sizes (everything is one scale-up domain).
        runtime: the host runtime (`deep_ep._C.ElasticBuffer`).
    """

    def __init__(self, group, num_bytes: Optional[int] = None, num_cpu_bytes: int = 0,
                 num_max_tokens_per_rank: int = 0, hidden: int = 0, num_topk: int = 0,
                 use_fp8_dispatch: bool = False, deterministic: bool = False,
                 allow_hybrid_mode: bool = True, allow_multiple_reduction: bool = True,
                 prefer_overlap_with_compute: bool = True, sl_idx: int = 3, num_allocated_qps: int = 0,
                 num_cpu_timeout_secs: int = 300, num_gpu_timeout_secs: int = 100,
                 explicitly_destroy: bool = False):
        self.group, self.rank_idx, self.num_ranks = group, group.rank(), group.size()
        self.comm_handle = None                     # the reference's communicator handle: there is none
        self.deterministic = deterministic
        self.allow_hybrid_mode, self.allow_multiple_reduction = allow_hybrid_mode, allow_multiple_reduction
        self.prefer_overlap_with_compute = prefer_overlap_with_compute
        self.num_max_tokens_per_rank, self.num_allocated_qps = num_max_tokens_per_rank, num_allocated_qps
        self.explicitly_destroy = explicitly_destroy

        # Sizing is kept for compatibility: the rows land in the tensors dispatch returns, not in a staging buffer.
        self.num_bytes = num_bytes if num_bytes is not None else self.get_buffer_size_hint(
            group, num_max_tokens_per_rank, hidden, num_topk, use_fp8_dispatch, allow_hybrid_mode, allow_multiple_reduction)
        if os.environ.get('EP_BUFFER_DEBUG'):
            print(f'EP elastic buffer, logical rank {self.rank_idx} of {self.num_ranks}: {self.num_bytes} bytes '
                  f'(+ {num_cpu_bytes} on the host)')
        self.runtime = _C.ElasticBuffer(self.rank_idx, self.num_ranks, 0, None, self.num_bytes, num_cpu_bytes,
                                        allow_hybrid_mode, allow_multiple_reduction, prefer_overlap_with_compute,
                                        sl_idx, num_allocated_qps, num_cpu_timeout_secs, num_gpu_timeout_secs,
                                        explicitly_destroy)

        # One scale-up domain holds every logical rank.
        self.num_scaleout_ranks, self.num_scaleup_ranks = self.get_logical_domain_size()
        self.scaleout_rank_idx, self.scaleup_rank_idx = divmod(self.rank_idx, self.num_scaleup_ranks)
        self.num_rdma_ranks, self.num_nvlink_ranks = self.get_physical_domain_size()

    def destroy(self) -> None:
        """Release the runtime. Requires `explicitly_destroy=True` at construction."""
        assert self.explicitly_destroy, 'construct with explicitly_destroy=True to release by hand'
        runtime, self.runtime = self.runtime, None
        if runtime is not None:
            runtime.destroy()

    @staticmethod
    def get_buffer_size_hint(group, num_max_tokens_per_rank: int, hidden: int, num_topk: int = 0,
                             use_fp8_dispatch: bool = False, allow_hybrid_mode: bool = True,
                             allow_multiple_reduction: bool = True) -> int:
        """The 2 MB-aligned size the reference would recommend for these MoE settings."""
        return _C.calculate_elastic_buffer_size(group.size(), num_max_tokens_per_rank, hidden, num_topk,
                                                use_fp8_dispatch, allow_hybrid_mode, allow_multiple_reduction)

    def barrier(self, use_comm_stream: bool = True, with_cpu_sync: bool = False, sequential: bool = True) -> None:
        self.runtime.barrier(use_comm_stream, with_cpu_sync, sequential)

    @staticmethod
    def capture() -> EventHandle:
        """Record an event on the current stream."""
        return capture_event()

    def get_comm_stream(self) -> torch.cuda.Stream:
        ts = self.runtime.get_comm_stream()
        return torch.cuda.Stream(stream_id=ts.stream_id, device_index=ts.device_index, device_type=ts.device_type)

    def get_physical_domain_size(self) -> Tuple[int, int]:
        return self.runtime.get_physical_domain_size()

    def get_logical_domain_size(self) -> Tuple[int, int]:
        return self.runtime.get_logical_domain_size()

    def get_theoretical_num_qps(self, num_sms: int) -> int:
        """RDMA queue pairs the reference would recommend (deep_ep/buffers/elastic.py:1371-1389): nothing here crosses
        a network, so none."""
        return 0

    def get_theoretical_num_sms(self, num_experts: int, num_topk: int, *args, **kwargs) -> int:
        """The routing kernels are bandwidth bound and always launched over the whole GPU."""
        return torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count

    def get_dispatch_layout(self, topk_idx: torch.Tensor, num_experts: int,
                            previous_event: Optional[EventOverlap] = None, async_finish: bool = False,
                            allocate_on_comm_stream: bool = False):
        """V1 `Buffer.get_dispatch_layout` (reference deep_ep/buffers/legacy.py:293-319) on this buffer:
        returns (num_tokens_per_rank[R] int32, None, num_tokens_per_expert[E] int32,
        is_token_in_rank[T, R] bool, EventOverlap)."""
        a, b, c, d, event = self.runtime.get_dispatch_layout(topk_idx, num_experts, unwrap_event(previous_event),
                                                             async_finish, allocate_on_comm_stream)
        return a, b, c, d, EventOverlap(event)

    def dispatch(self, x: Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]],
                 topk_idx: Optional[torch.Tensor] = None, topk_weights: Optional[torch.Tensor] = None,
                 cumulative_local_expert_recv_stats: Optional[torch.Tensor] = None,
                 num_experts: Optional[int] = None, num_max_tokens_per_rank: Optional[int] = None,
                 expert_alignment: Optional[int] = None, num_sms: int = 0, num_qps: int = 0,
                 previous_event: Optional[EventHandle] = None,
                 previous_event_before_epilogue: Optional[EventHandle] = None,
                 async_with_compute_stream: bool = False, allocate_on_comm_stream: bool = False,
                 handle: Optional[EPHandle] = None, do_handle_copy: bool = True,
                 do_cpu_sync: Optional[bool] = None, do_expand: bool = False, do_zero_padding: bool = False,
                 use_tma_aligned_col_major_sf: bool = False, cast_to_fp8: bool = False):
        """Dispatch tokens to the logical destination ranks.

        Arguments follow the reference (`deep_ep/buffers/elastic.py:1391-1412`):
            x: BF16 `[num_tokens, hidden]`, or a pair (FP8 e4m3 `[num_tokens, hidden]`, scale factors).
            topk_idx / topk_weights: `[num_tokens, num_topk]` (`deep_ep.topk_idx_t` / float); must be None with `handle`
                (weights may still be given with a cached handle).
            cumulative_local_expert_recv_stats: int32 `[num_experts]`, incremented by the per-expert counts.
            num_experts, num_max_tokens_per_rank, expert_alignment: taken from `handle` / the constructor when None.
            num_sms, num_qps: accepted and ignored (the kernels use the whole GPU; there are no queue pairs).
            previous_event, previous_event_before_epilogue, async_with_compute_stream, allocate_on_comm_stream:
                stream control, as in the reference.
            handle: a cached `EPHandle` to skip the layout computation.
            do_handle_copy: clone `topk_idx` into the handle.
            do_cpu_sync: wait for exact counts and size the outputs exactly (default True unless cached);
                otherwise outputs have worst-case sizes.
            do_expand / do_zero_padding / use_tma_aligned_col_major_sf: output layout options.
            cast_to_fp8 (extension): `x` is BF16; the per-1x128 FP8 e4m3 cast is fused into the scatter and
                `recv_x` comes back as (FP8, fp32 scales).

        Returns (recv_x or (recv_x, recv_sf), recv_topk_idx, recv_topk_weights, handle, event).
        """
        payload, scale_factors = x if isinstance(x, tuple) else (x, None)

        cached = (None,) * 10
        if handle is not None:
            # A cached dispatch replays the handle's routing: its settings may be repeated but not changed.
            assert topk_idx is None, 'A cached dispatch takes its routing from the handle'
            assert not do_cpu_sync, 'Cannot do CPU sync with cached handle'
            assert do_expand == handle.do_expand, 'The cached handle was built for the other layout'
            settings = (value_or(num_experts, handle.num_experts), value_or(expert_alignment, handle.expert_alignment),
                        value_or(num_max_tokens_per_rank, handle.num_max_tokens_per_rank))
            assert settings == (handle.num_experts, handle.expert_alignment, handle.num_max_tokens_per_rank), \
                'A cached dispatch cannot change num_experts, expert_alignment or num_max_tokens_per_rank'
            num_experts, expert_alignment, num_max_tokens_per_rank = settings
            topk_idx, do_cpu_sync, cached = handle.topk_idx, False, handle.layout_fields()
        else:
            assert num_experts is not None, '`num_experts` is required'
            num_max_tokens_per_rank = value_or(num_max_tokens_per_rank, self.num_max_tokens_per_rank)
            expert_alignment, do_cpu_sync = value_or(expert_alignment, 1), value_or(do_cpu_sync, True)
        num_sms = num_sms or self.get_theoretical_num_sms(num_experts, 0)

        (recv_x, recv_sf, recv_topk_idx, recv_topk_weights, cloned_topk_idx,
         num_recv_tokens, num_expanded_tokens, num_recv_tokens_per_expert_list,
         psum_num_recv_tokens_per_scaleup_rank, psum_num_recv_tokens_per_expert,
         num_unaligned_recv_tokens_per_expert, recv_src_metadata, dst_buffer_slot_idx,
         token_metadata_at_forward, channel_linked_list, event) = self.runtime.dispatch(
            payload, scale_factors, topk_idx, topk_weights, cumulative_local_expert_recv_stats,
            *cached,
            num_max_tokens_per_rank, num_experts, expert_alignment, num_sms, num_qps,
            unwrap_event(previous_event), unwrap_event(previous_event_before_epilogue),
            async_with_compute_stream, allocate_on_comm_stream,
            do_handle_copy, do_cpu_sync, do_expand, do_zero_padding, use_tma_aligned_col_major_sf,
            cast_to_fp8=cast_to_fp8)

        if handle is None:
            kept_topk_idx = cloned_topk_idx if do_handle_copy else topk_idx      # without a copy the handle aliases the caller's tensor
            handle = EPHandle(do_expand, num_experts, expert_alignment, num_max_tokens_per_rank, num_sms, kept_topk_idx,
                              num_recv_tokens, num_expanded_tokens, num_recv_tokens_per_expert_list,
                              psum_num_recv_tokens_per_scaleup_rank, psum_num_recv_tokens_per_expert,
                              num_unaligned_recv_tokens_per_expert, recv_src_metadata, dst_buffer_slot_idx,
                              token_metadata_at_forward, channel_linked_list)
        received = recv_x if recv_sf is None else (recv_x, recv_sf)
        return received, recv_topk_idx, recv_topk_weights, handle, EventOverlap(event)

    @staticmethod
    def _unpack_bias(bias) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        """None, one tensor or a pair of tensors -> always a pair."""
        if bias is None or isinstance(bias, torch.Tensor):
            return bias, None
        first, second = bias            # anything else must be exactly two tensors
        return first, second

    def combine(self, x: torch.Tensor, handle: EPHandle, topk_weights: Optional[torch.Tensor] = None,
                bias: Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]] = None,
                num_sms: int = 0, num_qps: int = 0, previous_event: EventHandle = None,
                previous_event_before_epilogue: Optional[EventHandle] = None,
                async_with_compute_stream: bool = False, allocate_on_comm_stream: bool = False):
        """Reduce received rows back to their origin tokens.

        Arguments follow the reference (`deep_ep/buffers/elastic.py:1616-1626`):
            x: BF16 `[num_recv_tokens, hidden]` (compact) or `[num_expanded_tokens, hidden]` (expanded).
            handle: the handle `dispatch` returned.
            topk_weights: float `[num_recv_tokens, num_topk]` (compact) or `[num_expanded_tokens]` (expanded);
                routed back unchanged, never multiplied into `x`.
            bias: zero, one or two BF16 `[num_tokens, hidden]` tensors added once to the output.

        Returns (combined_x BF16 `[num_tokens, hidden]`, combined_topk_weights float `[num_tokens, num_topk]`
        or None, event).  Accumulation is fp32 with one round-to-nearest-even BF16 store.
        """
        first_bias, second_bias = self._unpack_bias(bias)
        combined_x, combined_topk_weights, event = self.runtime.combine(
            x, topk_weights, first_bias, second_bias, handle.recv_src_metadata, handle.topk_idx,
            handle.psum_num_recv_tokens_per_scaleup_rank, handle.token_metadata_at_forward,
            handle.channel_linked_list, handle.num_experts, handle.num_max_tokens_per_rank,
            num_sms or handle.num_sms, num_qps, unwrap_event(previous_event), unwrap_event(previous_event_before_epilogue),
            async_with_compute_stream, allocate_on_comm_stream, handle.do_expand,
            dst_buffer_slot_idx=handle.dst_buffer_slot_idx)
        return combined_x, combined_topk_weights, EventOverlap(event)

    def check_device_status(self) -> None:
        """Synchronise and raise if a kernel flagged bad routing input (an expert id outside
        [0, num_experts), one expert named twice by a token) or a row that did not fit the outputs.
        Calls with `do_cpu_sync=True` check this themselves."""
        self.runtime.check_device_status("routing")

    def poll_device_status(self) -> bool:
        """The same check without waiting for the GPU, for loops that run without host synchronisation (for example
        `do_cpu_sync=False` dispatches replayed from a graph).  The first call queues a read of the status word on the
        current stream and returns False; later calls return False until that read has finished, then raise as
        `check_device_status` does if something was flagged, or return True (the next call queues a new read)."""
        return self.runtime.poll_device_status("routing")

    def queue_status_read(self, out: torch.Tensor, clear: bool = True) -> None:
        """Queues, on the current stream, a copy of the device status word into `out` (one int32, pinned host memory or
        device memory) without any host wait; with `clear` the word is reset on the way, so `out` holds what was
        flagged since the previous clearing read (0 = nothing; bits as in `deep_ep_hip.h`).  May be captured into a
        graph together with `do_cpu_sync=False` dispatches: every replay then refreshes `out`."""
        self.runtime.queue_status_read(out, clear)
