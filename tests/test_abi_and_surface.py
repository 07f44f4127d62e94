"""CPU-side checks of the boundary: the C ABI exports what include/deep_ep_hip.h declares, the ctypes
mirrors have the header's struct layouts, arguments are validated before anything is launched, and
the Python surface has the reference's names and signatures.  No GPU work happens here."""
import ctypes
import inspect
import os
import re
import subprocess
import sys
import tempfile

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "deep_ep_hip.h")

import deep_ep
from deep_ep import _C, _abi


def header_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(deep_ep_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = header_functions()
    assert len(names) >= 11
    for name in names:
        assert hasattr(_abi.lib, name), f"{name} is declared in the header but not exported"
    assert sorted(_abi.EXPORTS) == names, "ctypes binding table and header disagree"
    assert _abi.lib.deep_ep_hip_abi_version() == _abi.ABI_VERSION == 4


def test_measurement_build_exports_the_same_abi_plus_the_stamp_reader():
    """libdeep_ep_hip_stamps.so (bench.py --wave-spans) is the product's sources with time stamps in the mover wavefronts:
    the declared ABI and one more function to read the stamps, which the product library does not have."""
    import ctypes
    import os
    stamps = ctypes.CDLL(os.path.join(os.path.dirname(_abi.library_path()), "libdeep_ep_hip_stamps.so"))
    for name in header_functions():
        assert hasattr(stamps, name), f"{name} is missing from the measurement build"
    assert hasattr(stamps, "deep_ep_hip_debug_wave_stamps")
    assert not hasattr(_abi.lib, "deep_ep_hip_debug_wave_stamps")


def test_ctypes_structs_match_the_header_layout():
    structs = {"deep_ep_hip_layout_args": _abi.LayoutArgs, "deep_ep_hip_dispatch_args": _abi.DispatchArgs,
               "deep_ep_hip_combine_args": _abi.CombineArgs,
               "deep_ep_hip_intranode_dispatch_args": _abi.IntranodeDispatchArgs,
               "deep_ep_hip_intranode_combine_args": _abi.IntranodeCombineArgs, "deep_ep_hip_ll_dispatch_args": _abi.LLDispatchArgs,
               "deep_ep_hip_ll_combine_args": _abi.LLCombineArgs, "deep_ep_hip_cast_args": _abi.CastArgs,
               "deep_ep_hip_tuning": _abi.Tuning}
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', "int main(void) {"]
    for cname, cls in structs.items():
        lines.append(f'  printf("{cname} %zu\\n", sizeof({cname}));')
        for field, _ in cls._fields_:
            lines.append(f'  printf("{cname}.{field} %zu\\n", offsetof({cname}, {field}));')
    lines += ["  return 0;", "}"]
    with tempfile.TemporaryDirectory() as tmp:
        src, exe = os.path.join(tmp, "layout.c"), os.path.join(tmp, "layout")
        open(src, "w").write("\n".join(lines))
        subprocess.run(["gcc", "-std=c11", "-o", exe, src], check=True, capture_output=True)
        out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout
    got = dict(line.split() for line in out.strip().splitlines())
    for cname, cls in structs.items():
        assert int(got[cname]) == ctypes.sizeof(cls), cname
        for field, _ in cls._fields_:
            assert int(got[f"{cname}.{field}"]) == getattr(cls, field).offset, f"{cname}.{field}"


def test_header_limits_match_python_constants():
    text = open(HEADER).read()
    for name, value in (("DEEP_EP_HIP_MAX_TOPK", _abi.MAX_TOPK), ("DEEP_EP_HIP_MAX_EXPERTS", _abi.MAX_EXPERTS),
                        ("DEEP_EP_HIP_MAX_RANKS", _abi.MAX_RANKS), ("DEEP_EP_HIP_PHASE_LAYOUT", _abi.PHASE_LAYOUT),
                        ("DEEP_EP_HIP_PHASE_MOVE", _abi.PHASE_MOVE), ("DEEP_EP_HIP_PAYLOAD_CAST_FP8", _abi.PAYLOAD_CAST_FP8),
                        ("DEEP_EP_HIP_STATUS_ROW_OVERFLOW", _abi.STATUS_ROW_OVERFLOW),
                        ("DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT", _abi.STATUS_LAYOUT_TIMEOUT)):
        assert re.search(rf"#define {name} {value}\b", text), name


def _dispatch_args(**kw):
    a = _abi.DispatchArgs()
    a.phases = _abi.PHASE_LAYOUT
    a.num_tokens, a.hidden, a.num_topk, a.num_experts, a.num_ranks = 16, 256, 2, 8, 2
    a.num_max_tokens_per_rank, a.expert_alignment = 16, 1
    # never dereferenced: every case below is rejected before a launch
    a.topk_idx = a.workspace = a.psum_num_recv_tokens_per_rank = 0x1000
    a.psum_num_recv_tokens_per_expert = a.num_unaligned_recv_tokens_per_expert = 0x1000
    a.workspace_bytes = 1 << 30
    for k, v in kw.items():
        setattr(a, k, v)
    return a


@pytest.mark.parametrize("kw,fragment", [
    (dict(num_topk=0), "num_topk"), (dict(num_topk=33), "num_topk"), (dict(num_experts=9), "divisible"),
    (dict(num_ranks=0), "num_ranks"), (dict(num_tokens=17), "num_max_tokens_per_rank"), (dict(rank_idx=2), "rank_idx"),
    (dict(phases=0), "phases"), (dict(cached=1), "cached"), (dict(do_zero_padding=1), "do_expand"),
    (dict(expert_alignment=0), "expert_alignment"), (dict(payload=7), "payload"), (dict(workspace=0), "workspace"),
    (dict(num_experts=2048, num_ranks=2), "num_experts"),
    (dict(phases=_abi.PHASE_MOVE, hidden=100, payload=_abi.PAYLOAD_FP8), "16 bytes"),
    (dict(phases=_abi.PHASE_MOVE, hidden=192, payload=_abi.PAYLOAD_CAST_FP8, x=0x1000, recv_x=0x1000, recv_src_metadata=0x1000,
          dst_buffer_slot_idx=0x1000), "128"),
    # a BF16 payload carries no scale factors: neither tensor nor pack count may be set
    (dict(phases=_abi.PHASE_MOVE, x=0x1000, recv_x=0x1000, recv_src_metadata=0x1000, dst_buffer_slot_idx=0x1000, sf=0x1000),
     "no scale factors"),
    (dict(phases=_abi.PHASE_MOVE, x=0x1000, recv_x=0x1000, recv_src_metadata=0x1000, dst_buffer_slot_idx=0x1000, recv_sf=0x1000),
     "no scale factors"),
    (dict(phases=_abi.PHASE_MOVE, x=0x1000, recv_x=0x1000, recv_src_metadata=0x1000, dst_buffer_slot_idx=0x1000, num_sf_packs=2),
     "no scale factors"),
    # FP8 rows with scale-factor packs need both scale-factor tensors, unless the outputs are empty
    (dict(phases=_abi.PHASE_MOVE, payload=_abi.PAYLOAD_FP8, x=0x1000, recv_x=0x1000, recv_src_metadata=0x1000,
          dst_buffer_slot_idx=0x1000, num_sf_packs=2, recv_sf=0x1000, recv_capacity=4), "sf is NULL"),
    (dict(phases=_abi.PHASE_MOVE, payload=_abi.PAYLOAD_FP8, x=0x1000, recv_x=0x1000, recv_src_metadata=0x1000,
          dst_buffer_slot_idx=0x1000, num_sf_packs=2, sf=0x1000, recv_capacity=4), "recv_sf is NULL"),
])
def test_dispatch_rejects_bad_arguments_before_launch(kw, fragment):
    rc = _abi.lib.deep_ep_hip_launch_dispatch(ctypes.byref(_dispatch_args(**kw)), None)
    assert rc == -1, kw
    assert fragment in _abi.last_error(), _abi.last_error()


def _launches(T=8192, H=7168, K=8, E=256, R=8, payload=None, phases=None, **kw):
    a = _abi.DispatchArgs()
    a.phases = _abi.PHASE_LAYOUT | _abi.PHASE_MOVE if phases is None else phases
    a.payload = _abi.PAYLOAD_CAST_FP8 if payload is None else payload
    a.num_tokens, a.hidden, a.num_topk, a.num_experts, a.num_ranks = T, H, K, E, R
    a.num_max_tokens_per_rank, a.expert_alignment = T, 1
    for k, v in kw.items():
        if k.startswith("tuning_"):
            setattr(a.tuning, k[len("tuning_"):], v)
        else:
            setattr(a, k, v)
    return _abi.lib.deep_ep_hip_dispatch_kernel_launches(ctypes.byref(a))


def test_launch_plan_of_a_dispatch():
    """Which shapes share one launch between layout and move (no pointer is read, nothing is launched)."""
    assert _launches() == 1                                             # the headline shape: fused cast, compact
    assert _launches(T=16384) == 1 and _launches(T=16385) == 2          # up to 131072 (token, lane) pairs
    assert _launches(K=9, E=288) == 2 and _launches(E=512, R=8) == 2    # top-k <= 8, ranks + experts <= 512
    assert _launches(do_expand=1) == 2 and _launches(T=4096, do_expand=1) == 1   # expanded: two launches from 64 MB of input on
    assert _launches(T=4096, do_expand=1, tuning_dispatch_launches=2) == 2
    assert _launches(do_expand=1, tuning_dispatch_launches=1) == 1
    assert _launches(payload=_abi.PAYLOAD_BF16) == 2                    # 28672 mover workgroups: more than the single launch takes
    assert _launches(payload=_abi.PAYLOAD_BF16, tuning_dispatch_launches=1) == 1
    assert _launches(T=4096, H=2048, K=6, E=64, payload=_abi.PAYLOAD_BF16) == 1
    assert _launches(tuning_cast_pairs=4) == 2                          # wide cast tiles have no single-launch kernel
    assert _launches(phases=_abi.PHASE_LAYOUT) == 1 and _launches(phases=_abi.PHASE_MOVE) == 1
    assert _launches(T=0) == 1 and _launches(T=0, phases=_abi.PHASE_MOVE) == 0
    assert _launches(phases=0) == -1 and _launches(payload=9) == -1 and _launches(E=255) == -1


def test_workspace_size_contract():
    rc = _abi.lib.deep_ep_hip_launch_dispatch(ctypes.byref(_dispatch_args(workspace_bytes=64)), None)
    assert rc == -2 and "needed" in _abi.last_error()
    need = _abi.lib.deep_ep_hip_workspace_bytes
    assert need(0, 2, 8, 2) > 0 and need(8192, 8, 256, 8) >= need(4096, 8, 256, 8) >= need(128, 2, 8, 2)
    assert need(8192, 8, 256, 8) % 256 == 0 and need(8192, 8, 256, 8) < (1 << 21)
    assert need(-1, 8, 256, 8) == 0 and _abi.lib.deep_ep_hip_ll_workspace_bytes(8, 128, 8, 32) > 0
    # a combine that rebuilds the handle's token -> row map keeps it behind the dispatch tables
    assert _abi.lib.deep_ep_hip_combine_workspace_bytes(8192, 8, 256, 8) == need(8192, 8, 256, 8) + 8192 * 8 * 4
    with pytest.raises(RuntimeError, match="DeepEP HIP backend"):
        _abi.check(-1, "probe")


def test_other_entry_points_validate():
    a = _abi.LayoutArgs()
    a.num_tokens, a.num_topk, a.num_experts, a.num_ranks = 4, 2, 8, 3
    assert _abi.lib.deep_ep_hip_launch_layout(ctypes.byref(a), None) == -1
    c = _abi.CombineArgs()
    c.num_tokens, c.hidden, c.num_topk, c.num_experts, c.num_ranks = 4, 100, 2, 8, 2       # 200-byte rows
    assert _abi.lib.deep_ep_hip_launch_combine(ctypes.byref(c), None) == -1 and "16 bytes" in _abi.last_error()
    l = _abi.LLDispatchArgs()
    l.num_src_ranks, l.src_token_stride, l.num_topk, l.num_experts, l.num_local_experts = 1, 8, 2, 8, 4
    l.expert_begin, l.num_ranks, l.num_max_dispatch_tokens_per_rank, l.hidden, l.use_fp8 = 6, 2, 8, 192, 1
    assert _abi.lib.deep_ep_hip_launch_ll_dispatch(ctypes.byref(l), None) == -1
    assert _abi.lib.deep_ep_hip_launch_cast_fp8(None, None) == -1


def _intranode_args(**kw):
    a = _abi.IntranodeDispatchArgs()
    a.phases = _abi.PHASE_LAYOUT
    a.num_tokens, a.hidden, a.num_ranks, a.num_channels, a.expert_alignment = 16, 256, 2, 4, 1
    a.is_token_in_rank = a.workspace = a.psum_num_recv_tokens_per_rank = 0x1000   # never dereferenced
    a.workspace_bytes = 1 << 30
    for k, v in kw.items():
        setattr(a, k, v)
    return a


@pytest.mark.parametrize("kw,fragment", [
    (dict(num_ranks=65), "num_ranks"), (dict(num_ranks=0), "num_ranks"),
    (dict(topk_idx=0x1000, num_topk=2, num_experts=8), "go together"),
    (dict(cached=1, topk_idx=0x1000, topk_weights=0x1000, num_topk=2, num_experts=8), "cached"),
    (dict(cached=1), "layout phase"), (dict(rank_idx=2), "rank_idx"), (dict(phases=0), "phases"),
    (dict(expert_alignment=0), "expert_alignment"), (dict(is_token_in_rank=0), "is_token_in_rank"),
    (dict(workspace=0), "workspace"), (dict(payload=9), "payload"),
    (dict(topk_idx=0x1000, topk_weights=0x1000, num_topk=2, num_experts=9), "divisible"),
    (dict(num_ranks=40, num_tokens=4), "up to 32 ranks"),
    (dict(phases=_abi.PHASE_MOVE, hidden=100, payload=_abi.PAYLOAD_FP8), "16 bytes"),
    (dict(phases=_abi.PHASE_MOVE, x=0x1000, recv_x=0x1000, recv_capacity=8), "send_head"),
    (dict(rank_prefix_matrix=0x1000, num_channels=0), "num_channels"),
])
def test_intranode_dispatch_rejects_bad_arguments_before_launch(kw, fragment):
    rc = _abi.lib.deep_ep_hip_launch_intranode_dispatch(ctypes.byref(_intranode_args(**kw)), None)
    assert rc == -1, kw
    assert fragment in _abi.last_error(), _abi.last_error()


def test_intranode_combine_and_low_latency_validate():
    c = _abi.IntranodeCombineArgs()
    c.num_tokens, c.hidden, c.num_ranks, c.num_topk = 4, 100, 2, 0
    assert _abi.lib.deep_ep_hip_launch_intranode_combine(ctypes.byref(c), None) == -1 and "16 bytes" in _abi.last_error()
    c.hidden, c.num_ranks = 128, 65
    assert _abi.lib.deep_ep_hip_launch_intranode_combine(ctypes.byref(c), None) == -1 and "num_ranks" in _abi.last_error()
    c.num_ranks, c.num_topk = 2, 33
    assert _abi.lib.deep_ep_hip_launch_intranode_combine(ctypes.byref(c), None) == -1 and "num_topk" in _abi.last_error()
    l = _abi.LLDispatchArgs()
    l.num_src_ranks, l.src_token_stride, l.num_topk, l.num_experts, l.num_local_experts = 1, 8, 2, 8, 4
    l.expert_begin, l.num_ranks, l.num_max_dispatch_tokens_per_rank, l.hidden = 4, 2, 8, 256
    l.x = l.topk_idx = l.packed_recv_x = l.packed_recv_count = l.packed_recv_src_info = l.packed_recv_layout_range = 0x1000
    l.use_fp8, l.round_scale = 0, 1
    assert _abi.lib.deep_ep_hip_launch_ll_dispatch(ctypes.byref(l), None) == -1 and "round_scale" in _abi.last_error()
    l.use_fp8, l.use_ue8m0, l.packed_recv_x_scales = 1, 1, 0x1000          # 256 is not a multiple of 512
    assert _abi.lib.deep_ep_hip_launch_ll_dispatch(ctypes.byref(l), None) == -1 and "use_ue8m0" in _abi.last_error()


def test_missing_library_fails_loudly():
    env = dict(os.environ, DEEP_EP_HIP_LIBRARY="/nonexistent/libdeep_ep_hip.so",
               PYTHONPATH=os.path.join(ROOT, "deepep-ascend_amd"))
    res = subprocess.run([sys.executable, "-c", "import deep_ep"], env=env, capture_output=True, text=True)
    assert res.returncode != 0 and "ImportError" in res.stderr and "no fallback" in res.stderr


def test_no_product_module_touches_the_oracle():
    pkg = os.path.join(ROOT, "deepep-ascend_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".hpp", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "routing_oracle" not in text and "fp8_ref" not in text and "/oracle" not in text, f


# ---- Python surface (names and signatures of the reference: deep_ep/__init__.py:92-109,
# deep_ep/buffers/elastic.py:331-349,1391-1412,1616-1626; binding contract tests/platform/api_contract.py:1-42)
# The reference's binding contract (tests/platform/api_contract.py:1-42): names every platform's `_C` has, and what
# this platform adds (the Ascend build adds `is_destroyed` in the same way).
COMMON_MODULE_NAMES = {"get_platform", "topk_idx_t", "EventHandle", "ElasticBuffer", "calculate_elastic_buffer_size"}
# V1 names of the reference's extension (csrc/legacy/buffer.hpp:1751-1787) and the `Buffer` methods that exist on one
# GPU; sync / IPC / NVSHMEM handles and the mask-buffer calls of shrink mode have no meaning here and are absent.
LEGACY_MODULE_NAMES = {"Config", "Buffer", "get_low_latency_rdma_size_hint"}
LEGACY_BUFFER_METHODS = {"is_available", "get_num_rdma_ranks", "get_rdma_rank", "get_root_rdma_rank", "get_local_device_id",
                         "get_comm_stream", "destroy", "get_dispatch_layout", "intranode_dispatch", "intranode_combine",
                         "internode_dispatch", "internode_combine", "clean_low_latency_buffer", "low_latency_dispatch",
                         "low_latency_combine", "get_next_low_latency_combine_buffer"}
REFERENCE_LEGACY_METHODS_ABSENT = {"get_local_ipc_handle", "get_local_nvshmem_unique_id", "get_local_buffer_tensor", "sync",
                                   "low_latency_update_mask_buffer", "low_latency_query_mask_buffer",
                                   "low_latency_clean_mask_buffer"}
STATUS_METHODS = {"is_destroyed", "check_device_status", "poll_device_status", "queue_status_read", "device_status",
                  "workspace_control_words"}
COMMON_BUFFER_METHODS = {"destroy", "get_comm_stream", "get_physical_domain_size", "get_logical_domain_size", "barrier",
                         "dispatch", "combine"}
HIP_ONLY_MODULE_NAMES = {"EPException", "get_elastic_buffer_alignment", "set_tuning", "get_tuning", "abi_version"}
HIP_ONLY_BUFFER_METHODS = {"get_dispatch_layout"} | STATUS_METHODS


def _public(obj):
    return {n for n in dir(obj) if not n.startswith("_")}


def test_compiled_extension_has_exactly_the_contract_names():
    """`deep_ep._C` is the compiled extension (csrc/host/binding.cpp), loaded by file like the reference's contract
    test loads a built extension; its public names are the common contract plus this platform's additions."""
    assert _C.__file__.endswith(".so") and deep_ep._binding.name == "pybind" and deep_ep._binding.compiled is _C
    assert _C.get_platform() == "hip" and deep_ep.platform.get_platform() == "hip"
    assert _C.topk_idx_t == torch.int64 == deep_ep.topk_idx_t
    assert _public(_C) == COMMON_MODULE_NAMES | LEGACY_MODULE_NAMES | HIP_ONLY_MODULE_NAMES
    assert _public(_C.ElasticBuffer) == COMMON_BUFFER_METHODS | HIP_ONLY_BUFFER_METHODS
    assert _public(_C.Buffer) == LEGACY_BUFFER_METHODS | STATUS_METHODS
    assert not (_public(_C.Buffer) & REFERENCE_LEGACY_METHODS_ABSENT)
    assert _public(_C.Config) == {"num_sms", "get_nvl_buffer_size_hint", "get_rdma_buffer_size_hint"}
    assert _public(_C.EventHandle) == {"current_stream_wait"} and hasattr(_C.EventHandle, "__copy__")
    assert _C.abi_version() == _abi.ABI_VERSION
    with pytest.raises(RuntimeError):          # host checks surface as RuntimeError (exception.cuh:11-34)
        _C.calculate_elastic_buffer_size(8, 0, 7168, 8, False, True, True)
    with pytest.raises(TypeError):             # the 14-argument constructor of binding.hpp:24-27
        _C.ElasticBuffer(0, 8)
    _C.set_tuning("cast_pairs", 4)
    assert _C.get_tuning("cast_pairs") == 4
    _C.set_tuning("cast_pairs", 0)
    with pytest.raises(RuntimeError):
        _C.set_tuning("no_such_knob", 1)


def test_missing_extension_fails_loudly():
    """There is one host runtime: without the compiled extension the package does not import (no silent second path)."""
    with tempfile.TemporaryDirectory() as tmp:
        pkg = os.path.join(tmp, "deep_ep")
        os.makedirs(os.path.join(pkg, "buffers")); os.makedirs(os.path.join(pkg, "utils"))
        src = os.path.join(ROOT, "deepep-ascend_amd", "deep_ep")
        for dirpath, _, files in os.walk(src):
            for f in files:
                if f.endswith(".py") or f == _abi.LIB_NAME:
                    rel = os.path.relpath(os.path.join(dirpath, f), src)
                    os.symlink(os.path.join(dirpath, f), os.path.join(pkg, rel))
        res = subprocess.run([sys.executable, "-c", "import deep_ep"], env=dict(os.environ, PYTHONPATH=tmp), capture_output=True, text=True)
    assert res.returncode != 0 and "ImportError" in res.stderr and "deep_ep._C" in res.stderr and "no fallback" in res.stderr


def test_module_surface():
    for name in ("ElasticBuffer", "EPHandle", "EventOverlap", "EventHandle", "Buffer", "Config", "topk_idx_t", "__version__"):
        assert hasattr(deep_ep, name)
    assert deep_ep.topk_idx_t == torch.int64
    assert deep_ep.Config is _C.Config and deep_ep.EventHandle is _C.EventHandle
    assert callable(_C.EventHandle.current_stream_wait) and hasattr(_C.EventHandle, "__copy__")
    assert not hasattr(deep_ep, "_runtime")


def test_tuning_reaches_the_runtime_and_the_raw_abi_block():
    deep_ep.tuning.combine_vecs = 4
    try:
        assert _abi.tuning.combine_vecs == 4 and _C.get_tuning("combine_vecs") == 4 and deep_ep.tuning.combine_vecs == 4
    finally:
        deep_ep.tuning.combine_vecs = 0
    with pytest.raises(AttributeError):
        deep_ep.tuning.no_such_knob = 1


def _params(fn):
    return [p for p in inspect.signature(fn).parameters if p != "self"]


def test_signatures_are_drop_in():
    ctor = ["group", "num_bytes", "num_cpu_bytes", "num_max_tokens_per_rank", "hidden", "num_topk", "use_fp8_dispatch",
            "deterministic", "allow_hybrid_mode", "allow_multiple_reduction", "prefer_overlap_with_compute", "sl_idx",
            "num_allocated_qps", "num_cpu_timeout_secs", "num_gpu_timeout_secs", "explicitly_destroy"]
    assert _params(deep_ep.ElasticBuffer.__init__) == ctor
    dispatch = ["x", "topk_idx", "topk_weights", "cumulative_local_expert_recv_stats", "num_experts",
                "num_max_tokens_per_rank", "expert_alignment", "num_sms", "num_qps", "previous_event",
                "previous_event_before_epilogue", "async_with_compute_stream", "allocate_on_comm_stream", "handle",
                "do_handle_copy", "do_cpu_sync", "do_expand", "do_zero_padding", "use_tma_aligned_col_major_sf"]
    got = _params(deep_ep.ElasticBuffer.dispatch)
    assert got[:len(dispatch)] == dispatch and got[len(dispatch):] == ["cast_to_fp8"]
    combine = ["x", "handle", "topk_weights", "bias", "num_sms", "num_qps", "previous_event",
               "previous_event_before_epilogue", "async_with_compute_stream", "allocate_on_comm_stream"]
    assert _params(deep_ep.ElasticBuffer.combine) == combine
    assert _params(deep_ep.ElasticBuffer.get_buffer_size_hint) == ["group", "num_max_tokens_per_rank", "hidden", "num_topk",
                                                                  "use_fp8_dispatch", "allow_hybrid_mode",
                                                                  "allow_multiple_reduction"]
    assert _params(deep_ep.Buffer.get_dispatch_layout) == ["topk_idx", "num_experts", "previous_event", "async_finish",
                                                           "allocate_on_comm_stream"]
    assert _params(deep_ep.Buffer.low_latency_dispatch) == ["x", "topk_idx", "num_max_dispatch_tokens_per_rank", "num_experts",
                                                            "cumulative_local_expert_recv_stats", "dispatch_wait_recv_cost_stats",
                                                            "use_fp8", "round_scale", "use_ue8m0", "async_finish", "return_recv_hook"]
    assert _params(deep_ep.Buffer.low_latency_combine) == ["x", "topk_idx", "topk_weights", "handle", "use_logfmt", "zero_copy",
                                                           "async_finish", "return_recv_hook", "out", "combine_wait_recv_cost_stats"]
    # V1 pair: deep_ep/buffers/legacy.py:322-331 and :408-413
    assert _params(deep_ep.Buffer.dispatch) == ["x", "handle", "num_tokens_per_rank", "num_tokens_per_rdma_rank",
                                                "is_token_in_rank", "num_tokens_per_expert", "topk_idx", "topk_weights",
                                                "expert_alignment", "num_worst_tokens", "config", "previous_event",
                                                "async_finish", "allocate_on_comm_stream"]
    assert _params(deep_ep.Buffer.combine) == ["x", "handle", "topk_weights", "bias", "config", "previous_event",
                                               "async_finish", "allocate_on_comm_stream"]
    assert deep_ep.Buffer.is_sm90_compiled() and deep_ep.Config(20, 6, 256).num_sms == 20


def _arg_names(method):
    text = method.__doc__.split(" -> ")[0]
    return [n for n in re.findall(r"(\w+): ", text) if n != "self"]


def test_compiled_signatures_take_the_reference_positional_calls():
    """The reference calls its extension positionally: 29 arguments for `ElasticBuffer.dispatch`
    (csrc/elastic/buffer.hpp:704-728, deep_ep/buffers/elastic.py:1517-1549), 18 for `combine` (:1182-1198, :1695-1710),
    16 / 12 for the V1 pair (csrc/legacy/buffer.hpp:417-432, :719-731), 11 / 13 for the low-latency pair (:1463-1473,
    :1598-1611), 8 for the `Buffer` constructor (:83-91), 14 for `ElasticBuffer` (csrc/elastic/binding.hpp:24-27).
    What this backend adds comes after those, as keywords with defaults."""
    E, B = _C.ElasticBuffer, _C.Buffer
    d = _arg_names(E.dispatch)
    assert len(d) == 30 and d[-1] == "cast_to_fp8" and d[28] == "use_tma_aligned_col_major_sf" and d[0:3] == ["x", "sf", "topk_idx"]
    assert "cast_to_fp8: bool = False" in E.dispatch.__doc__
    c = _arg_names(E.combine)
    assert len(c) == 19 and c[-1] == "dst_buffer_slot_idx" and c[17] == "use_expanded_layout"
    assert re.search(r"dst_buffer_slot_idx: .* = None", E.combine.__doc__)
    i = _arg_names(B.intranode_dispatch)
    assert len(i) == 17 and i[-1] == "cached_send_head" and i[15] == "allocate_on_comm_stream"
    assert re.search(r"cached_send_head: .* = None", B.intranode_dispatch.__doc__)
    assert B.intranode_combine.__doc__.split(" -> ")[0].count("arg") == 12
    assert B.low_latency_dispatch.__doc__.split(" -> ")[0].count("arg") == 11
    l = _arg_names(B.low_latency_combine)
    assert len(l) == 13 and l[-1] == "out" and re.search(r"out: .* = None", B.low_latency_combine.__doc__)
    assert B.__init__.__doc__.split(" -> ")[0].count("arg") == 8
    assert E.__init__.__doc__.split(" -> ")[0].count("arg") == 14
    assert B.get_dispatch_layout.__doc__.split(" -> ")[0].count("arg") == 5
    assert B.get_next_low_latency_combine_buffer.__doc__.split(" -> ")[0].count("arg") == 3
    cfg = _C.Config()
    assert (cfg.num_sms, _C.Config(24, 6, 256, 6, 128).num_sms) == (20, 24)
    with pytest.raises(RuntimeError):
        _C.Config(20, 256, 6, 6, 128)          # send chunk not below receive chunk (csrc/legacy/config.hpp:42-44)
    # size hints: what the reference would reserve, closed forms of csrc/legacy/config.hpp:53-100,131-188
    assert cfg.get_rdma_buffer_size_hint(7168 * 2, 8) == 0
    per_slot = 7168 * 2 + 8 + 128 * 8 + 128 * 4 + 128 * 4
    assert cfg.get_nvl_buffer_size_hint(7168 * 2, 8) == (10 * 8 * 5 * 4 + 10 * 8 * 256 * per_slot + 127) // 128 * 128
    msg, cmsg = 16 + 7168 * 2, 56 * 4 + 7168 * 2
    assert _C.get_low_latency_rdma_size_hint(128, 7168, 8, 256) == \
        (2 * (max(128 * msg, 256 * 128 * cmsg) + 256 * 128 * max(msg, cmsg) + 256 * 4) + 127) // 128 * 128
    assert deep_ep.Buffer.get_low_latency_rdma_size_hint(128, 7168, 8, 256) == _C.get_low_latency_rdma_size_hint(128, 7168, 8, 256)


def test_handle_fields():
    idx = torch.zeros((2, 2), dtype=torch.int64)
    h = deep_ep.EPHandle(False, 8, 1, 16, 4, idx, 3, 3, [1, 2], idx, idx, idx, idx, idx, None, None)
    expected = {"do_expand", "num_experts", "expert_alignment", "num_max_tokens_per_rank", "num_sms", "topk_idx",
                "psum_num_recv_tokens_per_scaleup_rank", "psum_num_recv_tokens_per_expert",
                "num_unaligned_recv_tokens_per_expert", "num_recv_tokens_per_expert_list", "recv_src_metadata",
                "dst_buffer_slot_idx", "token_metadata_at_forward", "channel_linked_list", "num_recv_tokens",
                "num_expanded_tokens", "cached_recv_src_metadata_before_sort"}
    assert set(vars(h)) == expected      # field set asserted by the reference at run_two_rank_dispatch.py:594-606


def test_buffer_size_calculus_worked_numbers():
    # T=8192 per rank, H=7168, K=8, R=8 (Appendix A of the reference's calculus): BF16 904 MiB, FP8 max(512, 900) MiB
    mib = 1 << 20
    rt = _C
    assert rt.calculate_elastic_buffer_size(8, 8192, 7168, 8, False, True, True) == 904 * mib
    assert rt.calculate_elastic_buffer_size(8, 8192, 7168, 8, True, True, True) == 900 * mib
    assert rt.calculate_elastic_buffer_size(8, 128, 1024, 0, False, True, True) % rt.get_elastic_buffer_alignment() == 0
    with pytest.raises(RuntimeError):
        rt.calculate_elastic_buffer_size(8, 0, 7168, 8, False, True, True)
    g = deep_ep.LogicalGroup(3, 8)
    assert (g.rank(), g.size()) == (3, 8)
    assert deep_ep.ElasticBuffer.get_buffer_size_hint(g, 8192, 7168, 8) == 904 * mib


def test_event_overlap_hooks_without_gpu():
    class FakeEvent:
        waits = 0
        def current_stream_wait(self):
            FakeEvent.waits += 1
    calls = []
    ev = deep_ep.EventOverlap(FakeEvent())
    ev.register_hook_after_wait(lambda: calls.append(1))
    with pytest.raises(AssertionError):
        ev.register_hook_after_wait(lambda: None)
    with ev(release_handle=True):
        pass
    assert FakeEvent.waits == 1 and calls == [1] and ev.event is None and ev.hook_after_wait is None


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-GPU failure mode")
def test_runtime_fails_loudly_without_gpu():
    with pytest.raises(RuntimeError, match="no GPU"):
        deep_ep.ElasticBuffer(deep_ep.LogicalGroup(0, 2), num_max_tokens_per_rank=16, hidden=256, num_topk=2)


def test_package_imports_in_a_fresh_interpreter_before_torch():
    """`import deep_ep` as the first import of a process: the compiled extension needs torch's Python module, and the
    package loads it itself."""
    import subprocess
    import sys
    code = "import sys; sys.path.insert(0, %r); import deep_ep; print(deep_ep.ElasticBuffer.__name__)" % os.path.join(ROOT, "deepep-ascend_amd")
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-600:]
    assert res.stdout.strip() == "ElasticBuffer"
