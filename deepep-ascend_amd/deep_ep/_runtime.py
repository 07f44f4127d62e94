"""Host runtime of the HIP backend in Python, over the ctypes binding of the C ABI (include/deep_ep_hip.h): a second
binding of the same ABI beside the compiled `deep_ep._C` extension (csrc/host/), with the same names and the same
argument and tuple contracts (csrc/python_api.cpp:37-54, csrc/elastic/binding.hpp:9-44 of the reference).  The V2
`ElasticBuffer` uses the compiled extension when it is built and this module otherwise (or when
DEEP_EP_HIP_BINDING=ctypes); the V1 `Buffer` surface (intranode dispatch / combine, low latency) always runs on this
module.  PyTorch supplies device memory and streams only.

Public names: `get_platform`, `topk_idx_t`, `EventHandle`, `ElasticBuffer`, `calculate_elastic_buffer_size`,
`get_elastic_buffer_alignment`, `Config`.

One GPU, logical ranks: `num_ranks` only decides which bucket (destination rank) an expert
belongs to; every bucket lives in this GPU's HBM.  One call moves the tokens of the logical
source rank `rank_idx`.
"""
import ctypes
import os
from typing import List, Optional, Tuple

import torch

from . import _abi

topk_idx_t = torch.int64          # EP_NUM_TOPK_IDX_BITS default (csrc/python_api.cpp:21-35)
_ALIGNMENT_BYTES = 2 * 1024 * 1024  # symmetric::kNumAlignmentBytes (csrc/elastic/buffer.hpp:1363-1365)
_TMA_ALIGN = 32                     # ptx::kNumTMAAlignBytes, used only by the size calculus


def get_platform() -> str:
    return "hip"


def get_elastic_buffer_alignment() -> int:
    return _ALIGNMENT_BYTES


def _align(x: int, y: int) -> int:
    return (x + y - 1) // y * y


def _host_assert(cond: bool, what: str) -> None:
    # EP_HOST_ASSERT raises EPException -> RuntimeError in Python (exception.cuh:11-34)
    if not cond:
        raise RuntimeError(f"Assertion failed: {what}")


class EventHandle:
    """An event recorded on a stream at construction (csrc/utils/event.hpp:10-42)."""

    def __init__(self, stream: Optional[torch.cuda.Stream] = None):
        self.event = torch.cuda.Event()
        self.event.record(stream if stream is not None else torch.cuda.current_stream())
        self.tensors_to_record: list = []

    def __copy__(self):
        other = EventHandle.__new__(EventHandle)
        other.event = self.event
        other.tensors_to_record = list(self.tensors_to_record)
        return other

    def current_stream_wait(self) -> None:
        torch.cuda.current_stream().wait_event(self.event)


def _stream_wait_event(stream: torch.cuda.Stream, event) -> None:
    """`stream` waits for `event`, an EventHandle of this module or of the compiled extension."""
    with torch.cuda.stream(stream):
        event.current_stream_wait()


def _token_record_bytes(hidden_bytes: int, sf_bytes: int, num_topk: int, with_metadata: bool) -> int:
    # deep_ep/include/deep_ep/common/layout.cuh:187-208
    meta = num_topk * 8 + ((1 + num_topk) * 4 if with_metadata else 0)
    return _align(hidden_bytes, _TMA_ALIGN) + _align(sf_bytes, _TMA_ALIGN) + _align(meta, _TMA_ALIGN)


def calculate_elastic_buffer_size(comm_handle, num_max_tokens_per_rank: int, hidden: int, num_topk: int,
                                  use_fp8_dispatch: bool, allow_hybrid_mode: bool,
                                  allow_multiple_reduction: bool, num_ranks: Optional[int] = None) -> int:
    """Size the reference would ask for (csrc/elastic/buffer.hpp:588-688, direct mode, peers reachable
    by load/store).  The HIP backend scatters straight into the output tensors and needs no staging
    buffer; the number is kept so `num_bytes` / `get_buffer_size_hint` stay drop-in.
    `comm_handle` is the logical rank count here (there is no communicator)."""
    _host_assert(num_max_tokens_per_rank > 0 and hidden > 0, "num_max_tokens_per_rank > 0 and hidden > 0")
    _host_assert(-(-hidden // 32) * 4 <= hidden, "ceil_div(hidden, 32) * sizeof(float) <= hidden")
    ranks = int(num_ranks if num_ranks is not None else (comm_handle if comm_handle else 1))
    topk = 32 if num_topk == 0 else num_topk
    elem = 1 if use_fp8_dispatch else 2
    sf_packs = -(-hidden // 32) if use_fp8_dispatch else 0
    dispatch_record = _token_record_bytes(hidden * elem, sf_packs * 4, topk, True)
    dispatch_bytes = ranks * num_max_tokens_per_rank * dispatch_record
    combine_record = _token_record_bytes(hidden * 2, 0, topk, False)
    tokens_in_layout = min(ranks, topk) if allow_multiple_reduction else topk
    combine_bytes = tokens_in_layout * num_max_tokens_per_rank * combine_record
    return _align(max(dispatch_bytes, combine_bytes), _ALIGNMENT_BYTES)


class ElasticBuffer:
    """Host side of dispatch / combine (the role of csrc/elastic/buffer.hpp:83-1345 on CUDA and of
    csrc/backends/ascend/elastic_buffer.hpp on Ascend): checks arguments, allocates outputs,
    sequences the kernels on the right stream and returns the reference's tuples."""

    cpu_comm_t = list

    def __init__(self, rank_idx: int, num_ranks: int, comm_handle: int, cpu_comm,
                 num_buffer_bytes: int, num_cpu_buffer_bytes: int,
                 allow_hybrid_mode: bool, allow_multiple_reduction: bool,
                 prefer_overlap_with_compute: bool, sl_idx: int, num_allocated_qps: int,
                 num_cpu_timeout_secs: int, num_gpu_timeout_secs: int, explicitly_destroy: bool):
        _host_assert(0 <= rank_idx < num_ranks, "0 <= rank_idx < num_ranks")
        _host_assert(num_ranks <= _abi.MAX_RANKS, f"num_ranks <= {_abi.MAX_RANKS}")
        _host_assert(num_buffer_bytes > 0 and num_buffer_bytes % _ALIGNMENT_BYTES == 0,
                     "num_buffer_bytes > 0 and num_buffer_bytes % kNumAlignmentBytes == 0")
        _host_assert(num_cpu_buffer_bytes == 0, "CPU buffers are not supported by the HIP backend")
        if not torch.cuda.is_available():
            raise RuntimeError("DeepEP HIP backend: no GPU is visible")
        self.rank_idx = rank_idx
        self.num_ranks = num_ranks
        self.num_buffer_bytes = num_buffer_bytes
        self.allow_hybrid_mode = allow_hybrid_mode
        self.allow_multiple_reduction = allow_multiple_reduction
        self.prefer_overlap_with_compute = prefer_overlap_with_compute
        self.num_cpu_timeout_secs = num_cpu_timeout_secs
        self.explicitly_destroy = explicitly_destroy
        self.device = torch.device("cuda", torch.cuda.current_device())
        self.comm_stream = torch.cuda.Stream(device=self.device)
        self._workspace: Optional[torch.Tensor] = None
        self._last_stream: Optional[torch.cuda.Stream] = None      # stream of the last launch that used the workspace
        self._status_host: Optional[torch.Tensor] = None           # one pinned int32: where poll_device_status has the status copied
        self._status_read: Optional[torch.cuda.Event] = None       # recorded after the status read in flight
        self._destroyed = False

    # ---- lifetime ----
    def destroy(self) -> None:
        _host_assert(self.explicitly_destroy, "explicitly_destroy")
        _host_assert(not self._destroyed, "not destroyed")
        torch.cuda.synchronize(self.device)
        self._workspace = None
        self._status_read = None
        self._destroyed = True

    def is_destroyed(self) -> bool:
        return self._destroyed

    def get_comm_stream(self) -> torch.cuda.Stream:
        return self.comm_stream

    def get_physical_domain_size(self) -> Tuple[int, int]:
        # (RDMA ranks, load/store-reachable ranks): every logical rank is local
        return 1, self.num_ranks

    def get_logical_domain_size(self) -> Tuple[int, int]:
        # (scale-out ranks, scale-up ranks)
        return 1, self.num_ranks

    def barrier(self, use_comm_stream: bool = True, with_cpu_sync: bool = False, sequential: bool = True) -> None:
        # One process, one GPU: ordering between logical ranks is stream ordering.
        if with_cpu_sync:
            torch.cuda.synchronize(self.device)
        if use_comm_stream:
            self.comm_stream.wait_stream(torch.cuda.current_stream())
            torch.cuda.current_stream().wait_stream(self.comm_stream)
        if with_cpu_sync:
            torch.cuda.synchronize(self.device)

    # ---- helpers ----
    def _get_workspace(self, run_stream: torch.cuda.Stream, num_tokens: int, num_topk: int, num_experts: int) -> torch.Tensor:
        """The workspace is shared by every call on this buffer and is not re-entrant: a call that runs on another
        stream than the previous one first waits for everything queued there.  It grows geometrically, so that
        steady-state calls never allocate; a replaced workspace stays reserved for the stream that last used it."""
        if self._last_stream is not None and self._last_stream != run_stream:
            run_stream.wait_stream(self._last_stream)
        need = _abi.lib.deep_ep_hip_workspace_bytes(max(num_tokens, 1), num_topk, num_experts, self.num_ranks)
        if self._workspace is None or self._workspace.numel() < need:
            size = max(need, 2 * (self._workspace.numel() if self._workspace is not None else 0))
            if self._workspace is not None and self._last_stream is not None:
                self._workspace.record_stream(self._last_stream)
            with torch.cuda.stream(run_stream):
                self._workspace = torch.zeros(size, dtype=torch.uint8, device=self.device)
        self._last_stream = run_stream
        return self._workspace

    def check_device_status(self, what: str = "routing") -> None:
        """Synchronise and raise if a kernel flagged bad routing input or a row that did not fit the outputs."""
        torch.cuda.synchronize(self.device)
        if self._workspace is not None:
            self._read_and_clear_status(what)

    def queue_status_read(self, out: torch.Tensor, clear: bool = True) -> None:
        """Queues, on the current stream, a copy of the status word into `out` (one int32 in pinned host memory or on
        the device), clearing it on the way if asked.  Capturable: a graph that holds it refreshes `out` on every
        replay."""
        _host_assert(out.dtype == torch.int32 and out.numel() >= 1 and (out.is_cuda or out.is_pinned()), "out: int32, pinned or on the device")
        _host_assert(self._workspace is not None, "a dispatch or combine has run on this buffer")
        stream = torch.cuda.current_stream()
        if self._last_stream is not None and self._last_stream != stream:
            stream.wait_stream(self._last_stream)
        _abi.check(_abi.lib.deep_ep_hip_read_status(self._workspace.data_ptr(), out.data_ptr(), int(clear), stream.cuda_stream),
                   "status read")

    def poll_device_status(self, what: str = "routing") -> bool:
        """The status check of a loop that never waits for the GPU.  A call that finds no read in flight queues one on
        the current stream (deep_ep_hip_read_status in its clearing form: a small kernel moves the status word into
        pinned host memory and leaves the workspace ready for the next launch) and returns False.  A later call
        returns False while that read is still running; once it has finished, the call raises like
        check_device_status if a kernel had flagged something since the previous read, and returns True if nothing
        was flagged."""
        if self._workspace is None:
            return True
        if self._status_read is None:
            if self._status_host is None:
                self._status_host = torch.zeros(1, dtype=torch.int32, pin_memory=True)
            self.queue_status_read(self._status_host, True)
            self._status_read = torch.cuda.Event()
            self._status_read.record(torch.cuda.current_stream())
            return False
        if not self._status_read.query():
            return False
        self._status_read = None
        status = int(self._status_host[0])
        if status != 0:
            self._raise_status(status, what)
        return True

    def workspace_control_words(self) -> torch.Tensor:
        """The counters and flags at the head of the workspace (status, launch protocol), copied to the host after a full
        synchronisation: between launches everything but the status word (word 0), the two row totals (words 2 and 3) and
        the launch generation (word 32) reads zero."""
        torch.cuda.synchronize(self.device)
        n = _abi.lib.deep_ep_hip_workspace_counter_bytes()
        if self._workspace is None:
            return torch.zeros(n // 4, dtype=torch.int32)
        return self._workspace[:n].view(torch.int32).cpu()

    def device_status(self) -> int:
        torch.cuda.synchronize(self.device)
        return 0 if self._workspace is None else int(self._workspace[:4].view(torch.int32).item())

    def _read_and_clear_status(self, what: str) -> None:
        status = int(self._workspace[:4].view(torch.int32).item())
        if status != 0:
            # also the launch bookkeeping words that follow: a dispatch that gave up has left them mid-protocol
            self._workspace[:_abi.lib.deep_ep_hip_workspace_control_bytes()].zero_()
            self._raise_status(status, what)

    @staticmethod
    def _raise_status(status: int, what: str) -> None:
        reasons = []
        if status & _abi.STATUS_EXPERT_OUT_OF_RANGE:
            reasons.append("topk_idx holds an expert id >= num_experts")
        if status & _abi.STATUS_DUPLICATE_EXPERT:
            reasons.append("a token selects the same expert twice")
        if status & _abi.STATUS_ROW_OVERFLOW:
            reasons.append("a received row did not fit the output tensors")
        if status & _abi.STATUS_LAYOUT_TIMEOUT:
            reasons.append("a single-launch dispatch gave up waiting for its counting workgroups (outputs invalid)")
        raise RuntimeError(f"DeepEP HIP backend: {what}: " + "; ".join(reasons))

    def _prologue(self, previous_event, allocate_on_comm_stream: bool, async_with_compute_stream: bool,
                  v1_rules: bool = False):
        """Returns (compute_stream, run_stream).  The reference always runs on its comm stream
        (csrc/elastic/buffer.hpp:528-551); when nothing asks for overlap the same ordering is had,
        without two cross-stream waits, by running on the caller's stream."""
        compute_stream = torch.cuda.current_stream()
        if previous_event is not None and not v1_rules:
            _host_assert(allocate_on_comm_stream, "allocate_on_comm_stream")
        if v1_rules and allocate_on_comm_stream:
            # csrc/legacy/buffer.hpp:507-510
            _host_assert(previous_event is not None and async_with_compute_stream, "previous_event.has_value() and async")
        overlap = previous_event is not None or allocate_on_comm_stream or async_with_compute_stream
        if not overlap:
            return compute_stream, compute_stream
        if allocate_on_comm_stream:
            torch.cuda.set_stream(self.comm_stream)
        if previous_event is not None:
            _stream_wait_event(self.comm_stream, previous_event)
        else:
            self.comm_stream.wait_stream(compute_stream)
        return compute_stream, self.comm_stream

    def _epilogue(self, tensors, compute_stream, run_stream, allocate_on_comm_stream: bool,
                  async_with_compute_stream: bool) -> Optional[EventHandle]:
        event = None
        if run_stream is not compute_stream:
            if async_with_compute_stream:
                event = EventHandle(run_stream)
                if int(os.environ.get("EP_AVOID_RECORD_STREAM", "0")):
                    event.tensors_to_record = [t for t in tensors if t is not None]
                else:
                    for t in tensors:
                        if t is not None and t.is_cuda:
                            t.record_stream(compute_stream)
                            t.record_stream(run_stream)
            else:
                compute_stream.wait_stream(run_stream)
        elif async_with_compute_stream:
            event = EventHandle(run_stream)
        return event

    # ---- dispatch ----
    def dispatch(self, x: torch.Tensor, sf: Optional[torch.Tensor],
                 topk_idx: torch.Tensor, topk_weights: Optional[torch.Tensor],
                 cumulative_local_expert_recv_stats: Optional[torch.Tensor],
                 cached_num_recv_tokens: Optional[int],
                 cached_num_expanded_tokens: Optional[int],
                 cached_num_recv_tokens_per_expert_list: Optional[List[int]],
                 cached_psum_num_recv_tokens_per_scaleup_rank: Optional[torch.Tensor],
                 cached_psum_num_recv_tokens_per_expert: Optional[torch.Tensor],
                 cached_num_unaligned_recv_tokens_per_expert: Optional[torch.Tensor],
                 cached_dst_buffer_slot_idx: Optional[torch.Tensor],
                 cached_token_metadata_at_forward: Optional[torch.Tensor],
                 cached_recv_src_metadata: Optional[torch.Tensor],
                 cached_channel_linked_list: Optional[torch.Tensor],
                 num_max_tokens_per_rank: int, num_experts: int, expert_alignment: int,
                 num_sms: int, num_qps: int,
                 previous_event: Optional[EventHandle],
                 previous_event_before_epilogue: Optional[EventHandle],
                 async_with_compute_stream: bool, allocate_on_comm_stream: bool,
                 do_handle_copy: bool, do_cpu_sync: bool, do_expand: bool, do_zero_padding: bool,
                 use_tma_aligned_col_major_sf: bool, cast_to_fp8: bool = False):
        """Argument order and the 16-tuple returned follow csrc/elastic/buffer.hpp:695-728,1166-1178.
        `cast_to_fp8` (extension): `x` is BF16 and the FP8 e4m3 cast with per-1x128 fp32 scales is
        fused into the scatter; the result equals casting first and dispatching the pair."""
        _host_assert(not self._destroyed, "buffer is destroyed")
        _host_assert(not do_zero_padding or do_expand, "not do_zero_padding or do_expand")
        cached_mode = cached_num_recv_tokens is not None
        if cached_mode:
            _host_assert(cached_num_recv_tokens_per_expert_list is not None, "cached_num_recv_tokens_per_expert_list")
            _host_assert(cached_num_expanded_tokens is not None, "cached_num_expanded_tokens")
            _host_assert(cached_psum_num_recv_tokens_per_scaleup_rank is not None, "cached psum per rank")
            _host_assert(cached_psum_num_recv_tokens_per_expert is not None, "cached psum per expert")
            _host_assert(cached_dst_buffer_slot_idx is not None, "cached_dst_buffer_slot_idx")
            _host_assert(cached_recv_src_metadata is not None, "cached_recv_src_metadata")
            _host_assert(not do_cpu_sync, "Cannot do CPU sync with cached mode")
            _host_assert(cumulative_local_expert_recv_stats is None, "statistics need a non-cached dispatch")

        _host_assert(x.dim() == 2 and x.is_cuda and x.is_contiguous(), "x is a contiguous 2-D device tensor")
        num_tokens, hidden = x.shape
        _host_assert((hidden * x.element_size()) % 16 == 0, "(x.size(1) * x.element_size()) % sizeof(int4) == 0")
        _host_assert(num_tokens <= num_max_tokens_per_rank, "num_tokens <= num_max_tokens_per_rank")
        R = self.num_ranks
        _host_assert(num_experts % R == 0, "num_experts % num_ranks == 0")
        _host_assert(num_experts <= _abi.MAX_EXPERTS, f"num_experts <= {_abi.MAX_EXPERTS}")

        if cast_to_fp8:
            _host_assert(sf is None and x.dtype == torch.bfloat16, "cast_to_fp8 takes a BF16 tensor without scales")
            _host_assert(hidden % 128 == 0, "cast_to_fp8 needs hidden % 128 == 0")
            payload = _abi.PAYLOAD_CAST_FP8
            num_sf_packs = hidden // 128
            out_dtype, sf_dtype = torch.float8_e4m3fn, torch.float32
            sf_ts = sf_hs = 0
        elif sf is not None:
            _host_assert(x.element_size() == 1, "x with scale factors must be a 1-byte type")
            _host_assert(sf.dim() == 2 and sf.is_cuda and sf.shape[0] == num_tokens, "sf is [num_tokens, num_sf_packs] on device")
            _host_assert(sf.element_size() == 4, "sf.element_size() == sizeof(sf_pack_t)")
            payload = _abi.PAYLOAD_FP8
            num_sf_packs = sf.shape[1]
            out_dtype, sf_dtype = x.dtype, sf.dtype
            sf_ts, sf_hs = sf.stride(0), sf.stride(1)
        else:
            _host_assert(x.dtype == torch.bfloat16, "x without scale factors must be BF16")
            payload = _abi.PAYLOAD_BF16
            num_sf_packs = 0
            out_dtype, sf_dtype = x.dtype, None
            sf_ts = sf_hs = 0

        _host_assert(topk_idx is not None and topk_idx.dim() == 2 and topk_idx.shape[0] == num_tokens,
                     "topk_idx is [num_tokens, num_topk]")
        num_topk = topk_idx.shape[1]
        _host_assert(1 <= num_topk <= _abi.MAX_TOPK, f"1 <= num_topk <= {_abi.MAX_TOPK}")
        _host_assert(topk_idx.dtype == topk_idx_t, "topk_idx.scalar_type() == topk_idx_t")
        _host_assert(topk_idx.is_cuda and topk_idx.is_contiguous(), "topk_idx is contiguous on device")
        if topk_weights is not None:
            _host_assert(tuple(topk_weights.shape) == (num_tokens, num_topk), "topk_weights is [num_tokens, num_topk]")
            _host_assert(topk_weights.is_cuda and topk_weights.is_contiguous() and topk_weights.dtype == torch.float32,
                         "topk_weights is contiguous FP32 on device")
        if cumulative_local_expert_recv_stats is not None:
            s = cumulative_local_expert_recv_stats
            _host_assert(s.dim() == 1 and s.shape[0] == num_experts and s.dtype == torch.int32 and s.is_cuda and
                         s.is_contiguous(), "cumulative_local_expert_recv_stats is int32 [num_experts] on device")

        compute_stream, run_stream = self._prologue(previous_event, allocate_on_comm_stream, async_with_compute_stream)
        try:
            dev = self.device
            i32 = dict(dtype=torch.int32, device=dev)
            workspace = self._get_workspace(run_stream, num_tokens, num_topk, num_experts)

            with torch.cuda.stream(run_stream):
                if cached_mode:
                    psum_rank = cached_psum_num_recv_tokens_per_scaleup_rank
                    psum_expert = cached_psum_num_recv_tokens_per_expert
                    num_unaligned = cached_num_unaligned_recv_tokens_per_expert
                    _host_assert(psum_rank.shape == (R,) and psum_rank.dtype == torch.int32 and psum_rank.is_cuda,
                                 "cached psum per rank is int32 [num_ranks]")
                    _host_assert(psum_expert.shape == (num_experts,) and psum_expert.dtype == torch.int32,
                                 "cached psum per expert is int32 [num_experts]")
                    _host_assert(num_unaligned is not None and num_unaligned.shape == (num_experts,),
                                 "cached unaligned counts are int32 [num_experts]")
                    dst_slot = cached_dst_buffer_slot_idx
                    _host_assert(tuple(dst_slot.shape) == (num_tokens, num_topk) and dst_slot.dtype == torch.int32 and
                                 dst_slot.is_contiguous(), "cached dst_buffer_slot_idx is int32 [num_tokens, num_topk]")
                    copied_topk_idx = None
                else:
                    counts = torch.empty(R + 2 * num_experts, **i32)   # one allocation, one D2H copy when syncing
                    psum_rank = counts[:R]
                    psum_expert = counts[R:R + num_experts]
                    num_unaligned = counts[R + num_experts:]
                    dst_slot = torch.empty((num_tokens, num_topk), **i32)
                    copied_topk_idx = torch.empty_like(topk_idx) if do_handle_copy else None

                args = _abi.DispatchArgs()

                args.tuning = _abi.tuning
                args.payload = payload
                args.cached = int(cached_mode)
                args.do_expand = int(do_expand)
                args.do_zero_padding = int(do_zero_padding)
                args.num_tokens, args.hidden, args.num_topk = num_tokens, hidden, num_topk
                args.num_experts, args.num_ranks, args.rank_idx = num_experts, R, self.rank_idx
                args.num_max_tokens_per_rank = num_max_tokens_per_rank
                args.expert_alignment = expert_alignment
                args.x = _abi.ptr(x)
                args.sf = _abi.ptr(sf)
                args.sf_token_stride, args.sf_hidden_stride = sf_ts, sf_hs
                args.num_sf_packs = num_sf_packs
                args.topk_idx = _abi.ptr(topk_idx)
                args.topk_weights = _abi.ptr(topk_weights)
                args.copied_topk_idx = _abi.ptr(copied_topk_idx)
                args.psum_num_recv_tokens_per_rank = _abi.ptr(psum_rank)
                args.psum_num_recv_tokens_per_expert = _abi.ptr(psum_expert)
                args.num_unaligned_recv_tokens_per_expert = _abi.ptr(num_unaligned)
                args.cumulative_local_expert_recv_stats = _abi.ptr(cumulative_local_expert_recv_stats)
                args.host_counts = 0
                args.dst_buffer_slot_idx = _abi.ptr(dst_slot)
                args.workspace = _abi.ptr(workspace)
                args.workspace_bytes = workspace.numel()
                stream_ptr = run_stream.cuda_stream

                # Sizes of the outputs
                if cached_mode:
                    num_recv_tokens = cached_num_recv_tokens
                    num_expanded_tokens = cached_num_expanded_tokens
                    per_expert_list = list(cached_num_recv_tokens_per_expert_list)
                elif do_cpu_sync:
                    args.phases = _abi.PHASE_LAYOUT
                    _abi.check(_abi.lib.deep_ep_hip_launch_dispatch(ctypes.byref(args), stream_ptr), "dispatch layout")
                    host = counts.cpu()                                  # waits for the layout kernel
                    self._read_and_clear_status("dispatch")
                    num_recv_tokens = int(host[R - 1])
                    unaligned = host[R + num_experts:]
                    aligned = (unaligned + (expert_alignment - 1)) // expert_alignment * expert_alignment
                    per_expert_list = aligned.tolist()
                    num_expanded_tokens = int(aligned.sum())
                else:
                    num_recv_tokens = num_max_tokens_per_rank * R
                    num_expanded_tokens = num_max_tokens_per_rank * min(num_topk, num_experts) + \
                        (expert_alignment - 1) * num_experts
                    num_expanded_tokens = _align(num_expanded_tokens, expert_alignment)
                    per_expert_list = []

                num_allocated = num_expanded_tokens if do_expand else num_recv_tokens
                recv_x = torch.empty((num_allocated, hidden), dtype=out_dtype, device=dev)
                recv_src_metadata = cached_recv_src_metadata if cached_mode else \
                    torch.empty((num_recv_tokens, num_topk + 2), **i32)
                recv_sf = None
                rsf_ts = rsf_hs = 0
                if sf_dtype is not None:
                    if not use_tma_aligned_col_major_sf:
                        rsf_ts, rsf_hs = num_sf_packs, 1
                    else:
                        rsf_ts, rsf_hs = 1, _align(num_allocated, 4)
                    recv_sf = torch.empty_strided((num_allocated, num_sf_packs), (rsf_ts, rsf_hs), dtype=sf_dtype, device=dev)
                recv_topk_idx = torch.empty((num_allocated, num_topk), dtype=topk_idx.dtype, device=dev) if not do_expand else None
                recv_topk_weights = None
                if topk_weights is not None:
                    recv_topk_weights = torch.empty((num_allocated,) if do_expand else (num_allocated, num_topk),
                                                    dtype=torch.float32, device=dev)

                if previous_event_before_epilogue is not None:
                    _stream_wait_event(run_stream, previous_event_before_epilogue)

                args.phases = _abi.PHASE_MOVE if (cached_mode or do_cpu_sync) else (_abi.PHASE_LAYOUT | _abi.PHASE_MOVE)
                args.recv_src_metadata = _abi.ptr(recv_src_metadata)
                args.recv_x = _abi.ptr(recv_x)
                args.recv_sf = _abi.ptr(recv_sf)
                args.recv_sf_token_stride, args.recv_sf_hidden_stride = rsf_ts, rsf_hs
                args.recv_topk_idx = _abi.ptr(recv_topk_idx)
                args.recv_topk_weights = _abi.ptr(recv_topk_weights)
                args.recv_capacity = recv_src_metadata.shape[0]
                args.expanded_capacity = num_expanded_tokens if do_expand else 0
                _abi.check(_abi.lib.deep_ep_hip_launch_dispatch(ctypes.byref(args), stream_ptr), "dispatch")

            event = self._epilogue(
                [x, sf, topk_idx, topk_weights, recv_x, recv_sf, recv_topk_idx, recv_topk_weights,
                 cumulative_local_expert_recv_stats, copied_topk_idx, psum_rank, psum_expert, num_unaligned,
                 recv_src_metadata, dst_slot, workspace],
                compute_stream, run_stream, allocate_on_comm_stream, async_with_compute_stream)

            return (recv_x, recv_sf, recv_topk_idx, recv_topk_weights, copied_topk_idx,
                    num_recv_tokens, num_expanded_tokens, per_expert_list,
                    psum_rank, psum_expert, num_unaligned, recv_src_metadata, dst_slot,
                    None, None, event)
        finally:
            if allocate_on_comm_stream:
                torch.cuda.set_stream(compute_stream)

    # ---- combine ----
    def combine(self, x: torch.Tensor, topk_weights: Optional[torch.Tensor],
                bias_0: Optional[torch.Tensor], bias_1: Optional[torch.Tensor],
                src_metadata: torch.Tensor, combined_topk_idx: torch.Tensor,
                psum_num_recv_tokens_per_scaleup_rank: torch.Tensor,
                token_metadata_at_forward: Optional[torch.Tensor],
                channel_linked_list: Optional[torch.Tensor],
                num_experts: int, num_max_tokens_per_rank: int,
                num_sms: int, num_qps: int,
                previous_event: Optional[EventHandle],
                previous_event_before_epilogue: Optional[EventHandle],
                async_with_compute_stream: bool, allocate_on_comm_stream: bool,
                use_expanded_layout: bool, dst_buffer_slot_idx: Optional[torch.Tensor] = None):
        """Argument order and the 3-tuple returned follow csrc/elastic/buffer.hpp:1181-1198,1344.
        `dst_buffer_slot_idx` (the handle's token -> received-row map) is what lets a single GPU
        gather instead of routing rows back through a buffer; the Python wrapper passes it."""
        _host_assert(not self._destroyed, "buffer is destroyed")
        _host_assert(dst_buffer_slot_idx is not None, "combine needs the handle's dst_buffer_slot_idx")
        _host_assert(x.dim() == 2 and x.is_cuda and x.is_contiguous(), "x is a contiguous 2-D device tensor")
        _host_assert(x.dtype == torch.bfloat16, "x.scalar_type() == torch::kBFloat16")
        num_x_rows, hidden = x.shape
        _host_assert((hidden * 2) % 16 == 0, "(hidden * sizeof(bf16)) % sizeof(int4) == 0")
        num_tokens, num_topk = combined_topk_idx.shape
        _host_assert(combined_topk_idx.dtype == topk_idx_t and combined_topk_idx.is_contiguous(), "handle topk_idx")
        _host_assert(tuple(dst_buffer_slot_idx.shape) == (num_tokens, num_topk), "handle dst_buffer_slot_idx shape")
        _host_assert(src_metadata.dim() == 2 and src_metadata.shape[1] == num_topk + 2, "handle recv_src_metadata shape")
        if topk_weights is not None:
            _host_assert(topk_weights.dtype == torch.float32 and topk_weights.is_cuda and topk_weights.is_contiguous(),
                         "topk_weights is contiguous FP32 on device")
            if use_expanded_layout:
                _host_assert(topk_weights.dim() == 1 and topk_weights.shape[0] == num_x_rows, "expanded weights are [num_rows]")
            else:
                _host_assert(tuple(topk_weights.shape) == (num_x_rows, num_topk), "weights are [num_rows, num_topk]")
        for b in (bias_0, bias_1):
            if b is not None:
                _host_assert(b.dtype == x.dtype and tuple(b.shape) == (num_tokens, hidden) and b.is_cuda and
                             b.is_contiguous(), "bias is BF16 [num_combined_tokens, hidden]")
        _host_assert(bias_0 is not None or bias_1 is None, "bias_1 needs bias_0")

        compute_stream, run_stream = self._prologue(previous_event, allocate_on_comm_stream, async_with_compute_stream)
        try:
            workspace = self._get_workspace(run_stream, num_tokens, num_topk, num_experts)
            with torch.cuda.stream(run_stream):
                combined_x = torch.empty((num_tokens, hidden), dtype=x.dtype, device=self.device)
                combined_topk_weights = None
                if topk_weights is not None:
                    combined_topk_weights = torch.empty((num_tokens, num_topk), dtype=torch.float32, device=self.device)
                if previous_event_before_epilogue is not None:
                    _stream_wait_event(run_stream, previous_event_before_epilogue)
                args = _abi.CombineArgs()
                args.tuning = _abi.tuning
                args.do_expand = int(use_expanded_layout)
                args.allow_multiple_reduction = int(self.allow_multiple_reduction)
                args.num_tokens, args.hidden, args.num_topk = num_tokens, hidden, num_topk
                args.num_experts, args.num_ranks = num_experts, self.num_ranks
                args.rank_idx, args.num_max_tokens_per_rank = self.rank_idx, num_max_tokens_per_rank
                args.x = _abi.ptr(x)
                args.num_x_rows = num_x_rows
                args.topk_weights = _abi.ptr(topk_weights)
                args.bias_0, args.bias_1 = _abi.ptr(bias_0), _abi.ptr(bias_1)
                args.topk_idx = _abi.ptr(combined_topk_idx)
                args.dst_buffer_slot_idx = _abi.ptr(dst_buffer_slot_idx)
                args.recv_src_metadata = _abi.ptr(src_metadata)
                args.num_recv_rows = src_metadata.shape[0]
                args.psum_num_recv_tokens_per_rank = _abi.ptr(psum_num_recv_tokens_per_scaleup_rank)
                args.combined_x = _abi.ptr(combined_x)
                args.combined_topk_weights = _abi.ptr(combined_topk_weights)
                args.workspace = _abi.ptr(workspace)
                args.workspace_bytes = workspace.numel()
                _abi.check(_abi.lib.deep_ep_hip_launch_combine(ctypes.byref(args), run_stream.cuda_stream), "combine")

            event = self._epilogue(
                [x, topk_weights, bias_0, bias_1, src_metadata, combined_topk_idx,
                 psum_num_recv_tokens_per_scaleup_rank, dst_buffer_slot_idx, combined_x, combined_topk_weights, workspace],
                compute_stream, run_stream, allocate_on_comm_stream, async_with_compute_stream)
            return combined_x, combined_topk_weights, event
        finally:
            if allocate_on_comm_stream:
                torch.cuda.set_stream(compute_stream)

    # ---- V1 surface kept on the same runtime ----
    def get_dispatch_layout(self, topk_idx: torch.Tensor, num_experts: int,
                            previous_event: Optional[EventHandle], async_finish: bool,
                            allocate_on_comm_stream: bool):
        """csrc/legacy/buffer.hpp:337-404: (num_tokens_per_rank, num_tokens_per_rdma_rank=None,
        num_tokens_per_expert, is_token_in_rank, event)."""
        _host_assert(topk_idx.dim() == 2 and topk_idx.is_contiguous() and topk_idx.is_cuda, "topk_idx is contiguous 2-D on device")
        _host_assert(topk_idx.dtype == topk_idx_t, "topk_idx.scalar_type() == topk_idx_t")
        _host_assert(num_experts > 0 and num_experts % self.num_ranks == 0, "num_experts % num_ranks == 0")
        num_tokens, num_topk = topk_idx.shape
        compute_stream, run_stream = self._prologue(previous_event, allocate_on_comm_stream, async_finish)
        try:
            workspace = self._get_workspace(run_stream, num_tokens, num_topk, num_experts)
            with torch.cuda.stream(run_stream):
                num_tokens_per_rank = torch.empty((self.num_ranks,), dtype=torch.int32, device=self.device)
                num_tokens_per_expert = torch.empty((num_experts,), dtype=torch.int32, device=self.device)
                is_token_in_rank = torch.empty((num_tokens, self.num_ranks), dtype=torch.bool, device=self.device)
                args = _abi.LayoutArgs()
                args.topk_idx = _abi.ptr(topk_idx)
                args.num_tokens, args.num_topk, args.num_experts, args.num_ranks = num_tokens, num_topk, num_experts, self.num_ranks
                args.num_tokens_per_rank = _abi.ptr(num_tokens_per_rank)
                args.num_tokens_per_expert = _abi.ptr(num_tokens_per_expert)
                args.is_token_in_rank = _abi.ptr(is_token_in_rank)
                args.workspace = _abi.ptr(workspace)
                args.workspace_bytes = workspace.numel()
                _abi.check(_abi.lib.deep_ep_hip_launch_layout(ctypes.byref(args), run_stream.cuda_stream), "get_dispatch_layout")
            event = self._epilogue([topk_idx, num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank, workspace],
                                   compute_stream, run_stream, allocate_on_comm_stream, async_finish)
            return num_tokens_per_rank, None, num_tokens_per_expert, is_token_in_rank, event
        finally:
            if allocate_on_comm_stream:
                torch.cuda.set_stream(compute_stream)

    def intranode_dispatch(self, x: torch.Tensor, x_scales: Optional[torch.Tensor],
                           topk_idx: Optional[torch.Tensor], topk_weights: Optional[torch.Tensor],
                           num_tokens_per_rank: Optional[torch.Tensor], is_token_in_rank: torch.Tensor,
                           num_tokens_per_expert: Optional[torch.Tensor], cached_num_recv_tokens: int,
                           cached_rank_prefix_matrix: Optional[torch.Tensor],
                           cached_channel_prefix_matrix: Optional[torch.Tensor],
                           expert_alignment: int, num_worst_tokens: int, config,
                           previous_event: Optional[EventHandle], async_finish: bool, allocate_on_comm_stream: bool,
                           cached_send_head: Optional[torch.Tensor] = None):
        """Argument order and the 11-tuple returned follow csrc/legacy/buffer.hpp:417-717.
        `cached_send_head` (the handle's token -> receive-row map) is the one addition: on one GPU a
        cached dispatch scatters through it instead of replaying per-channel queues."""
        _host_assert(not self._destroyed, "buffer is destroyed")
        cached_mode = cached_rank_prefix_matrix is not None
        R = self.num_ranks
        _host_assert(R <= 64, "num_ranks <= 64 for the V1 dispatch")
        _host_assert(config.num_sms % 2 == 0, "config.num_sms % 2 == 0")
        num_channels = config.num_sms // 2
        _host_assert(x.dim() == 2 and x.is_cuda and x.is_contiguous(), "x.dim() == 2 and x.is_contiguous()")
        num_tokens, hidden = x.shape
        _host_assert((hidden * x.element_size()) % 16 == 0, "(x.size(1) * x.element_size()) % sizeof(int4) == 0")
        _host_assert(is_token_in_rank.dtype == torch.bool and is_token_in_rank.dim() == 2 and
                     is_token_in_rank.is_contiguous() and tuple(is_token_in_rank.shape) == (num_tokens, R),
                     "is_token_in_rank is a contiguous bool [num_tokens, num_ranks]")
        i32 = dict(dtype=torch.int32, device=self.device)
        if cached_mode:
            _host_assert(cached_channel_prefix_matrix is not None and cached_send_head is not None, "cached handle tensors")
            _host_assert(tuple(cached_rank_prefix_matrix.shape) == (R, R) and cached_rank_prefix_matrix.dtype == torch.int32,
                         "cached_rank_prefix_matrix is int32 [num_ranks, num_ranks]")
            _host_assert(tuple(cached_channel_prefix_matrix.shape) == (R, num_channels) and
                         cached_channel_prefix_matrix.dtype == torch.int32,
                         "cached_channel_prefix_matrix is int32 [num_ranks, num_channels]")
            _host_assert(tuple(cached_send_head.shape) == (num_tokens, R) and cached_send_head.dtype == torch.int32 and
                         cached_send_head.is_contiguous(), "cached send_head is int32 [num_tokens, num_ranks]")
            _host_assert(topk_idx is None and topk_weights is None, "a cached dispatch takes no top-k tensors")
            num_experts = 0
        else:
            _host_assert(num_tokens_per_rank is not None and num_tokens_per_expert is not None,
                         "num_tokens_per_rank and num_tokens_per_expert")
            _host_assert(num_tokens_per_rank.dtype == torch.int32 and tuple(num_tokens_per_rank.shape) == (R,) and
                         num_tokens_per_rank.is_contiguous(), "num_tokens_per_rank is int32 [num_ranks]")
            _host_assert(num_tokens_per_expert.dtype == torch.int32 and num_tokens_per_expert.dim() == 1 and
                         num_tokens_per_expert.is_contiguous(), "num_tokens_per_expert is int32 [num_experts]")
            num_experts = num_tokens_per_expert.shape[0]
            _host_assert(num_experts % R == 0, "num_tokens_per_expert.size(0) % num_ranks == 0")
        _host_assert((topk_idx is None) == (topk_weights is None), "topk_idx.has_value() == topk_weights.has_value()")
        num_topk = 0
        if topk_idx is not None:
            num_topk = topk_idx.shape[1]
            _host_assert(num_experts > 0, "num_experts > 0")
            _host_assert(topk_idx.dim() == 2 and topk_idx.is_contiguous() and topk_idx.dtype == topk_idx_t and
                         topk_idx.shape[0] == num_tokens, "topk_idx is a contiguous [num_tokens, num_topk] tensor")
            _host_assert(tuple(topk_weights.shape) == (num_tokens, num_topk) and topk_weights.is_contiguous() and
                         topk_weights.dtype == torch.float32, "topk_weights is contiguous FP32 [num_tokens, num_topk]")
            _host_assert(1 <= num_topk <= _abi.MAX_TOPK, f"1 <= num_topk <= {_abi.MAX_TOPK}")
            _host_assert(num_experts <= _abi.MAX_EXPERTS, f"num_experts <= {_abi.MAX_EXPERTS}")
        else:
            _host_assert(R <= _abi.MAX_TOPK, f"num_ranks <= {_abi.MAX_TOPK} without top-k tensors")
        num_scales, scale_ts, scale_hs = 0, 0, 0
        if x_scales is not None:
            _host_assert(x.element_size() == 1, "x.element_size() == 1")
            _host_assert(x_scales.dtype in (torch.float32, torch.int32), "x_scales is FP32 or int32")
            _host_assert(x_scales.dim() == 2 and x_scales.shape[0] == num_tokens and x_scales.is_cuda, "x_scales is [num_tokens, num_scales]")
            num_scales, scale_ts, scale_hs = x_scales.shape[1], x_scales.stride(0), x_scales.stride(1)
            payload = _abi.PAYLOAD_FP8
        else:
            _host_assert(x.dtype == torch.bfloat16, "x without scales must be BF16")
            payload = _abi.PAYLOAD_BF16
        if num_worst_tokens > 0:
            _host_assert(cached_mode or topk_idx is not None, "num_worst_tokens needs the top-k tensors")

        compute_stream, run_stream = self._prologue(previous_event, allocate_on_comm_stream, async_finish, v1_rules=True)
        try:
            route_lanes = num_topk if topk_idx is not None else R
            route_experts = num_experts if topk_idx is not None else R
            workspace = self._get_workspace(run_stream, num_tokens, route_lanes, route_experts)
            per_expert_list: List[int] = []
            with torch.cuda.stream(run_stream):
                args = _abi.IntranodeDispatchArgs()
                args.tuning = _abi.tuning
                args.payload, args.cached = payload, int(cached_mode)
                args.num_tokens, args.hidden = num_tokens, hidden
                args.num_topk, args.num_experts = num_topk, (num_experts if topk_idx is not None else 0)
                args.num_ranks, args.rank_idx = R, self.rank_idx
                args.num_channels, args.expert_alignment = num_channels, expert_alignment
                args.x, args.x_scales = _abi.ptr(x), _abi.ptr(x_scales)
                args.scale_token_stride, args.scale_hidden_stride, args.num_scales = scale_ts, scale_hs, num_scales
                args.topk_idx, args.topk_weights = _abi.ptr(topk_idx), _abi.ptr(topk_weights)
                args.is_token_in_rank = _abi.ptr(is_token_in_rank)
                args.workspace, args.workspace_bytes = _abi.ptr(workspace), workspace.numel()
                stream_ptr = run_stream.cuda_stream

                if cached_mode:
                    num_recv_tokens = cached_num_recv_tokens
                    rank_prefix_matrix, channel_prefix_matrix = cached_rank_prefix_matrix, cached_channel_prefix_matrix
                    recv_channel_prefix_matrix = torch.empty((R, num_channels), **i32)
                    send_head = cached_send_head
                    recv_src_idx = torch.empty((num_recv_tokens,), **i32)
                    args.phases = _abi.PHASE_MOVE
                else:
                    rank_prefix_matrix = torch.empty((R, R), **i32)
                    channel_prefix_matrix = torch.empty((R, num_channels), **i32)
                    recv_channel_prefix_matrix = torch.empty((R, num_channels), **i32)
                    send_head = torch.empty((num_tokens, R), **i32)
                    counts = torch.empty(R + max(num_experts, 1), **i32)
                    args.rank_prefix_matrix = _abi.ptr(rank_prefix_matrix)
                    args.channel_prefix_matrix = _abi.ptr(channel_prefix_matrix)
                    args.recv_channel_prefix_matrix = _abi.ptr(recv_channel_prefix_matrix)
                    args.psum_num_recv_tokens_per_rank = _abi.ptr(counts)
                    args.num_recv_tokens_per_expert = _abi.ptr(counts[R:]) if topk_idx is not None else 0
                    if num_worst_tokens > 0:
                        num_recv_tokens = num_worst_tokens
                        args.phases = _abi.PHASE_LAYOUT | _abi.PHASE_MOVE
                        args.fill_unused_topk_idx = 1
                    else:
                        # The reference spins on host-mapped counters here (csrc/legacy/buffer.hpp:580-600)
                        args.phases = _abi.PHASE_LAYOUT
                        _abi.check(_abi.lib.deep_ep_hip_launch_intranode_dispatch(ctypes.byref(args), stream_ptr),
                                   "intranode dispatch layout")
                        if topk_idx is None:
                            host = torch.cat([counts[:R], num_tokens_per_expert]).cpu()
                        else:
                            host = counts.cpu()
                            self._read_and_clear_status("dispatch")
                        num_recv_tokens = int(host[R - 1])
                        per_expert = host[R:R + num_experts]
                        per_expert_list = ((per_expert + (expert_alignment - 1)) // expert_alignment * expert_alignment).tolist()
                        args.phases = _abi.PHASE_MOVE
                    recv_src_idx = torch.empty((num_recv_tokens,), **i32)

                recv_x = torch.empty((num_recv_tokens, hidden), dtype=x.dtype, device=self.device)
                recv_x_scales = recv_topk_idx = recv_topk_weights = None
                if topk_idx is not None:
                    recv_topk_idx = torch.empty((num_recv_tokens, num_topk), dtype=topk_idx.dtype, device=self.device)
                    recv_topk_weights = torch.empty((num_recv_tokens, num_topk), dtype=torch.float32, device=self.device)
                if x_scales is not None:
                    recv_x_scales = torch.empty((num_recv_tokens, num_scales), dtype=x_scales.dtype, device=self.device)
                    args.recv_scale_token_stride, args.recv_scale_hidden_stride = num_scales, 1
                args.send_head = _abi.ptr(send_head)
                args.recv_src_idx = _abi.ptr(recv_src_idx)
                args.recv_x, args.recv_x_scales = _abi.ptr(recv_x), _abi.ptr(recv_x_scales)
                args.recv_topk_idx, args.recv_topk_weights = _abi.ptr(recv_topk_idx), _abi.ptr(recv_topk_weights)
                args.recv_capacity = num_recv_tokens
                _abi.check(_abi.lib.deep_ep_hip_launch_intranode_dispatch(ctypes.byref(args), stream_ptr), "intranode dispatch")

            event = self._epilogue(
                [x, x_scales, topk_idx, topk_weights, num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank,
                 rank_prefix_matrix, channel_prefix_matrix, recv_channel_prefix_matrix, recv_x, recv_x_scales, recv_src_idx,
                 recv_topk_idx, recv_topk_weights, send_head, workspace],
                compute_stream, run_stream, allocate_on_comm_stream, async_finish)
            return (recv_x, recv_x_scales, recv_topk_idx, recv_topk_weights, per_expert_list, rank_prefix_matrix,
                    channel_prefix_matrix, recv_channel_prefix_matrix, recv_src_idx, send_head, event)
        finally:
            if allocate_on_comm_stream:
                torch.cuda.set_stream(compute_stream)

    def intranode_combine(self, x: torch.Tensor, topk_weights: Optional[torch.Tensor],
                          bias_0: Optional[torch.Tensor], bias_1: Optional[torch.Tensor],
                          src_idx: torch.Tensor, rank_prefix_matrix: torch.Tensor,
                          channel_prefix_matrix: torch.Tensor, send_head: torch.Tensor, config,
                          previous_event: Optional[EventHandle], async_finish: bool, allocate_on_comm_stream: bool):
        """Argument order and the 3-tuple returned follow csrc/legacy/buffer.hpp:719-860."""
        _host_assert(not self._destroyed, "buffer is destroyed")
        R = self.num_ranks
        _host_assert(x.dim() == 2 and x.is_cuda and x.is_contiguous() and x.dtype == torch.bfloat16,
                     "x is a contiguous BF16 [num_tokens, hidden] device tensor")
        num_x_rows, hidden = x.shape
        _host_assert((hidden * 2) % 16 == 0, "(hidden * sizeof(bf16)) % sizeof(int4) == 0")
        _host_assert(src_idx.dim() == 1 and src_idx.shape[0] == num_x_rows and src_idx.dtype == torch.int32,
                     "src_idx is int32 [num_tokens]")
        _host_assert(send_head.dim() == 2 and send_head.shape[1] == R and send_head.dtype == torch.int32 and
                     send_head.is_contiguous(), "send_head is int32 [num_recv_tokens, num_ranks]")
        _host_assert(tuple(rank_prefix_matrix.shape) == (R, R) and rank_prefix_matrix.dtype == torch.int32,
                     "rank_prefix_matrix is int32 [num_ranks, num_ranks]")
        num_tokens = send_head.shape[0]
        num_topk = 0
        if topk_weights is not None:
            _host_assert(topk_weights.dim() == 2 and topk_weights.shape[0] == num_x_rows and topk_weights.is_contiguous() and
                         topk_weights.dtype == torch.float32 and topk_weights.is_cuda, "topk_weights is FP32 [num_tokens, num_topk]")
            num_topk = topk_weights.shape[1]
            _host_assert(num_topk <= _abi.MAX_TOPK, f"num_topk <= {_abi.MAX_TOPK}")
        for b in (bias_0, bias_1):
            if b is not None:
                _host_assert(b.dtype == x.dtype and tuple(b.shape) == (num_tokens, hidden) and b.is_cuda and
                             b.is_contiguous(), "bias is BF16 [num_recv_tokens, hidden]")
        _host_assert(bias_0 is not None or bias_1 is None, "bias_1 needs bias_0")

        compute_stream, run_stream = self._prologue(previous_event, allocate_on_comm_stream, async_finish, v1_rules=True)
        try:
            workspace = self._get_workspace(run_stream, 1, 1, R)
            with torch.cuda.stream(run_stream):
                recv_x = torch.empty((num_tokens, hidden), dtype=x.dtype, device=self.device)
                recv_topk_weights = None
                if topk_weights is not None:
                    recv_topk_weights = torch.empty((num_tokens, num_topk), dtype=torch.float32, device=self.device)
                args = _abi.IntranodeCombineArgs()
                args.tuning = _abi.tuning
                args.num_tokens, args.hidden, args.num_ranks, args.num_topk = num_tokens, hidden, R, num_topk
                args.x, args.num_x_rows = _abi.ptr(x), num_x_rows
                args.topk_weights = _abi.ptr(topk_weights)
                args.bias_0, args.bias_1 = _abi.ptr(bias_0), _abi.ptr(bias_1)
                args.send_head = _abi.ptr(send_head)
                args.combined_x, args.combined_topk_weights = _abi.ptr(recv_x), _abi.ptr(recv_topk_weights)
                args.workspace, args.workspace_bytes = _abi.ptr(workspace), workspace.numel()
                _abi.check(_abi.lib.deep_ep_hip_launch_intranode_combine(ctypes.byref(args), run_stream.cuda_stream),
                           "intranode combine")
            event = self._epilogue([x, topk_weights, bias_0, bias_1, src_idx, send_head, rank_prefix_matrix,
                                    channel_prefix_matrix, recv_x, recv_topk_weights, workspace],
                                   compute_stream, run_stream, allocate_on_comm_stream, async_finish)
            return recv_x, recv_topk_weights, event
        finally:
            if allocate_on_comm_stream:
                torch.cuda.set_stream(compute_stream)


class Config:
    """Tuning knobs of the V1 kernels (csrc/legacy/config.hpp:24-60).  Only `num_sms` has a meaning here: it
    fixes the number of channels (num_sms / 2) the handle's channel matrices are laid out for."""

    def __init__(self, num_sms: int = 20, num_max_nvl_chunked_send_tokens: int = 6,
                 num_max_nvl_chunked_recv_tokens: int = 256, num_max_rdma_chunked_send_tokens: int = 6,
                 num_max_rdma_chunked_recv_tokens: int = 256):
        _host_assert(num_sms >= 0, "num_sms >= 0")
        _host_assert(0 < num_max_nvl_chunked_send_tokens < num_max_nvl_chunked_recv_tokens,
                     "0 < num_max_nvl_chunked_send_tokens < num_max_nvl_chunked_recv_tokens")
        _host_assert(0 < num_max_rdma_chunked_send_tokens < num_max_rdma_chunked_recv_tokens,
                     "0 < num_max_rdma_chunked_send_tokens < num_max_rdma_chunked_recv_tokens")
        self.num_sms = num_sms
        self.num_max_nvl_chunked_send_tokens = num_max_nvl_chunked_send_tokens
        self.num_max_nvl_chunked_recv_tokens = num_max_nvl_chunked_recv_tokens
        self.num_max_rdma_chunked_send_tokens = num_max_rdma_chunked_send_tokens
        self.num_max_rdma_chunked_recv_tokens = num_max_rdma_chunked_recv_tokens

    def get_nvl_buffer_size_hint(self, hidden_bytes: int, num_ranks: int) -> int:
        """Bytes the reference would stage per rank (csrc/legacy/config.hpp:53-73); nothing is staged here."""
        nvl_ranks, rdma_ranks = min(num_ranks, 8), max(num_ranks // 8, 1)
        slots = (self.num_sms // 2) * nvl_ranks * self.num_max_nvl_chunked_recv_tokens
        # per queue slot: payload, 8-byte source record, 128 top-k ids and weights, 128 scales (the assumed maxima)
        per_slot = hidden_bytes + 8 + 128 * 8 + 128 * 4 + 128 * 4
        total = (self.num_sms // 2) * nvl_ranks * (2 * rdma_ranks + 3) * 4 + slots * per_slot
        return (total + 127) // 128 * 128
