"""ctypes binding of the C ABI declared in include/deep_ep_hip.h.

The shared library is the product path: if it cannot be loaded the import fails loudly; there is
no CPU or eager-PyTorch fallback.  Build it with `python deepep-ascend_amd/build.py`.
"""
import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_int, c_int32, c_int64, c_size_t, c_uint64, c_void_p

LIB_NAME = "libdeep_ep_hip.so"
ABI_VERSION = 4

PHASE_LAYOUT = 1
PHASE_MOVE = 2
PAYLOAD_BF16 = 0
PAYLOAD_FP8 = 1
PAYLOAD_CAST_FP8 = 2

STATUS_EXPERT_OUT_OF_RANGE = 1
STATUS_DUPLICATE_EXPERT = 2
STATUS_ROW_OVERFLOW = 4
STATUS_LAYOUT_TIMEOUT = 8

MAX_TOPK = 32
MAX_EXPERTS = 1024
MAX_RANKS = 512
STATIC_WORKSPACE_BYTES = 1 << 20


class Tuning(Structure):
    """Launch-shape knobs carried by every argument block (all zero = the library's own choice).  The C library reads
    no environment variables; this package seeds its process-wide default (`deep_ep.tuning`) from
    DEEP_EP_HIP_<FIELD NAME IN CAPITALS> once at import."""
    _fields_ = [
        ("dispatch_launches", c_int32), ("cast_pairs", c_int32), ("copy_vecs", c_int32), ("plain_loads", c_int32),
        ("xcd_remap", c_int32), ("combine_vecs", c_int32), ("ll_pairs", c_int32), ("ll_threads", c_int32),
        ("ll_two_kernels", c_int32), ("ll_combine_vecs", c_int32), ("mover_spin_limit", c_int32),
        ("move_workgroups_per_cu", c_int32), ("warm_rounds", c_int32), ("persistent_movers", c_int32), ("reserved", c_int32 * 2),
    ]

    @classmethod
    def from_env(cls) -> "Tuning":
        t = cls()
        for name, _ in cls._fields_:
            if name != "reserved":
                setattr(t, name, int(os.environ.get("DEEP_EP_HIP_" + name.upper(), "0")))
        return t


tuning = Tuning.from_env()


class LayoutArgs(Structure):
    _fields_ = [
        ("topk_idx", c_void_p),
        ("num_tokens", c_int32), ("num_topk", c_int32), ("num_experts", c_int32), ("num_ranks", c_int32),
        ("num_tokens_per_rank", c_void_p),
        ("num_tokens_per_expert", c_void_p),
        ("is_token_in_rank", c_void_p),
        ("workspace", c_void_p),
        ("workspace_bytes", c_uint64),
    ]


class DispatchArgs(Structure):
    _fields_ = [
        ("phases", c_int32), ("payload", c_int32), ("cached", c_int32), ("do_expand", c_int32),
        ("do_zero_padding", c_int32),
        ("num_tokens", c_int32), ("hidden", c_int32), ("num_topk", c_int32), ("num_experts", c_int32),
        ("num_ranks", c_int32),
        ("rank_idx", c_int32), ("num_max_tokens_per_rank", c_int32), ("expert_alignment", c_int32),
        ("x", c_void_p),
        ("sf", c_void_p),
        ("sf_token_stride", c_int64), ("sf_hidden_stride", c_int64),
        ("num_sf_packs", c_int32),
        ("topk_idx", c_void_p),
        ("topk_weights", c_void_p),
        ("copied_topk_idx", c_void_p),
        ("psum_num_recv_tokens_per_rank", c_void_p),
        ("psum_num_recv_tokens_per_expert", c_void_p),
        ("num_unaligned_recv_tokens_per_expert", c_void_p),
        ("cumulative_local_expert_recv_stats", c_void_p),
        ("host_counts", c_void_p),
        ("dst_buffer_slot_idx", c_void_p),
        ("recv_src_metadata", c_void_p),
        ("recv_x", c_void_p),
        ("recv_sf", c_void_p),
        ("recv_sf_token_stride", c_int64), ("recv_sf_hidden_stride", c_int64),
        ("recv_topk_idx", c_void_p),
        ("recv_topk_weights", c_void_p),
        ("recv_capacity", c_int64),
        ("expanded_capacity", c_int64),
        ("workspace", c_void_p),
        ("workspace_bytes", c_uint64),
        ("tuning", Tuning),
    ]


class CombineArgs(Structure):
    _fields_ = [
        ("do_expand", c_int32), ("allow_multiple_reduction", c_int32),
        ("num_tokens", c_int32), ("hidden", c_int32), ("num_topk", c_int32), ("num_experts", c_int32),
        ("num_ranks", c_int32),
        ("rank_idx", c_int32), ("num_max_tokens_per_rank", c_int32),
        ("x", c_void_p),
        ("num_x_rows", c_int64),
        ("topk_weights", c_void_p),
        ("bias_0", c_void_p),
        ("bias_1", c_void_p),
        ("topk_idx", c_void_p),
        ("dst_buffer_slot_idx", c_void_p),
        ("recv_src_metadata", c_void_p),
        ("num_recv_rows", c_int64),
        ("psum_num_recv_tokens_per_rank", c_void_p),
        ("combined_x", c_void_p),
        ("combined_topk_weights", c_void_p),
        ("workspace", c_void_p),
        ("workspace_bytes", c_uint64),
        ("tuning", Tuning),
    ]


class IntranodeDispatchArgs(Structure):
    _fields_ = [
        ("phases", c_int32), ("payload", c_int32), ("cached", c_int32),
        ("num_tokens", c_int32), ("hidden", c_int32),
        ("num_topk", c_int32),
        ("num_experts", c_int32),
        ("num_ranks", c_int32), ("rank_idx", c_int32),
        ("num_channels", c_int32),
        ("expert_alignment", c_int32),
        ("fill_unused_topk_idx", c_int32),
        ("x", c_void_p),
        ("x_scales", c_void_p),
        ("scale_token_stride", c_int64), ("scale_hidden_stride", c_int64),
        ("num_scales", c_int32),
        ("topk_idx", c_void_p),
        ("topk_weights", c_void_p),
        ("is_token_in_rank", c_void_p),
        ("rank_prefix_matrix", c_void_p),
        ("channel_prefix_matrix", c_void_p),
        ("recv_channel_prefix_matrix", c_void_p),
        ("psum_num_recv_tokens_per_rank", c_void_p),
        ("num_recv_tokens_per_expert", c_void_p),
        ("host_counts", c_void_p),
        ("send_head", c_void_p),
        ("recv_src_idx", c_void_p),
        ("recv_x", c_void_p),
        ("recv_x_scales", c_void_p),
        ("recv_scale_token_stride", c_int64), ("recv_scale_hidden_stride", c_int64),
        ("recv_topk_idx", c_void_p),
        ("recv_topk_weights", c_void_p),
        ("recv_capacity", c_int64),
        ("workspace", c_void_p),
        ("workspace_bytes", c_uint64),
        ("tuning", Tuning),
    ]


class IntranodeCombineArgs(Structure):
    _fields_ = [
        ("num_tokens", c_int32), ("hidden", c_int32), ("num_ranks", c_int32),
        ("num_topk", c_int32),
        ("x", c_void_p),
        ("num_x_rows", c_int64),
        ("topk_weights", c_void_p),
        ("bias_0", c_void_p),
        ("bias_1", c_void_p),
        ("send_head", c_void_p),
        ("combined_x", c_void_p),
        ("combined_topk_weights", c_void_p),
        ("workspace", c_void_p),
        ("workspace_bytes", c_uint64),
        ("tuning", Tuning),
    ]


class LLDispatchArgs(Structure):
    _fields_ = [
        ("use_fp8", c_int32),
        ("round_scale", c_int32),
        ("use_ue8m0", c_int32),
        ("num_src_ranks", c_int32), ("src_rank_begin", c_int32),
        ("src_token_stride", c_int32),
        ("num_tokens_per_src", c_void_p),
        ("hidden", c_int32), ("num_topk", c_int32), ("num_experts", c_int32),
        ("expert_begin", c_int32), ("num_local_experts", c_int32),
        ("num_ranks", c_int32),
        ("num_max_dispatch_tokens_per_rank", c_int32),
        ("x", c_void_p),
        ("topk_idx", c_void_p),
        ("packed_recv_x", c_void_p),
        ("packed_recv_x_scales", c_void_p),
        ("packed_recv_count", c_void_p),
        ("packed_recv_src_info", c_void_p),
        ("packed_recv_layout_range", c_void_p),
        ("cumulative_local_expert_recv_stats", c_void_p),
        ("lane_rows", c_void_p),
        ("workspace", c_void_p),
        ("workspace_bytes", c_uint64),
        ("tuning", Tuning),
    ]


class LLCombineArgs(Structure):
    _fields_ = [
        ("num_src_ranks", c_int32), ("src_rank_begin", c_int32),
        ("src_token_stride", c_int32),
        ("use_logfmt", c_int32),
        ("num_tokens_per_src", c_void_p),
        ("hidden", c_int32), ("num_topk", c_int32), ("num_experts", c_int32),
        ("expert_begin", c_int32), ("num_local_experts", c_int32), ("num_ranks", c_int32),
        ("num_max_dispatch_tokens_per_rank", c_int32),
        ("x", c_void_p),
        ("topk_idx", c_void_p),
        ("topk_weights", c_void_p),
        ("packed_recv_src_info", c_void_p),
        ("packed_recv_layout_range", c_void_p),
        ("lane_rows", c_void_p),
        ("combined_x", c_void_p),
        ("workspace", c_void_p),
        ("workspace_bytes", c_uint64),
        ("tuning", Tuning),
    ]


class CastArgs(Structure):
    _fields_ = [
        ("x", c_void_p),
        ("out", c_void_p),
        ("scales", c_void_p),
        ("num_tokens", c_int32), ("hidden", c_int32),
    ]


# name -> (restype, argtypes): every symbol include/deep_ep_hip.h declares
EXPORTS = {
    "deep_ep_hip_abi_version": (c_int, []),
    "deep_ep_hip_last_error": (c_char_p, []),
    "deep_ep_hip_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "deep_ep_hip_workspace_status_offset": (c_size_t, []),
    "deep_ep_hip_workspace_control_bytes": (c_size_t, []),
    "deep_ep_hip_workspace_counter_bytes": (c_size_t, []),
    "deep_ep_hip_read_status": (c_int, [c_void_p, c_void_p, c_int, c_void_p]),
    "deep_ep_hip_launch_layout": (c_int, [POINTER(LayoutArgs), c_void_p]),
    "deep_ep_hip_launch_dispatch": (c_int, [POINTER(DispatchArgs), c_void_p]),
    "deep_ep_hip_launch_dispatch_static": (c_int, [POINTER(DispatchArgs), c_void_p]),
    "deep_ep_hip_dispatch_kernel_launches": (c_int, [POINTER(DispatchArgs)]),
    "deep_ep_hip_launch_combine": (c_int, [POINTER(CombineArgs), c_void_p]),
    "deep_ep_hip_combine_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "deep_ep_hip_launch_intranode_dispatch": (c_int, [POINTER(IntranodeDispatchArgs), c_void_p]),
    "deep_ep_hip_launch_intranode_combine": (c_int, [POINTER(IntranodeCombineArgs), c_void_p]),
    "deep_ep_hip_ll_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "deep_ep_hip_launch_ll_dispatch": (c_int, [POINTER(LLDispatchArgs), c_void_p]),
    "deep_ep_hip_launch_ll_combine": (c_int, [POINTER(LLCombineArgs), c_void_p]),
    "deep_ep_hip_launch_cast_fp8": (c_int, [POINTER(CastArgs), c_void_p]),
}


def library_path() -> str:
    override = os.environ.get("DEEP_EP_HIP_LIBRARY")
    if override:
        return override
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)


def _load():
    path = library_path()
    if not os.path.exists(path):
        raise ImportError(
            f"deep_ep: the HIP kernel library {path} is missing. Build it with "
            f"`python deepep-ascend_amd/build.py` (needs hipcc); there is no fallback path.")
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in EXPORTS.items():
        fn = getattr(lib, name)          # AttributeError if the library does not export it
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.deep_ep_hip_abi_version()
    if got != ABI_VERSION:
        raise ImportError(f"deep_ep: {path} has ABI version {got}, this package needs {ABI_VERSION}")
    return lib


lib = _load()


def last_error() -> str:
    msg = lib.deep_ep_hip_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def check(rc: int, what: str) -> None:
    """Raise the reference's error type (RuntimeError, csrc exception.cuh:11-34) on failure."""
    if rc != 0:
        raise RuntimeError(f"DeepEP HIP backend: {what} failed (code {rc}): {last_error()}")


def ptr(t) -> int:
    """Device address of a tensor, or NULL for None."""
    return 0 if t is None else t.data_ptr()
