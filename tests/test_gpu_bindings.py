"""The compiled extension `deep_ep._C` takes the reference's own positional calls and gives the oracle's results.

The argument lists below are those of the reference's Python wrappers, in their order and with nothing added:
`ElasticBuffer.dispatch` 29 arguments (deep_ep/buffers/elastic.py:1517-1549 -> csrc/elastic/buffer.hpp:704-728),
`ElasticBuffer.combine` 18 (:1695-1710 -> :1182-1198), `Buffer.intranode_dispatch` 16 and `intranode_combine` 12
(deep_ep/buffers/legacy.py:386-399, 451-454 -> csrc/legacy/buffer.hpp:417-432, 719-731), `low_latency_dispatch` 11 and
`low_latency_combine` 13 (legacy.py:608-613, 667-669 -> buffer.hpp:1463-1473, 1598-1611).  None of them carries the
tensors this backend keeps beside a handle (the token -> row map of a V2 handle, `send_head` on a cached V1 dispatch,
the packed rows of a low-latency handle): each call is made once through a handle the buffer has seen, which it
remembers them for, and once through clones of the handle tensors, for which they are recomputed.
"""
import pytest
import torch

import routing_cases as rc
import routing_oracle as oracle
from test_gpu_parity import assert_equal

pytestmark = pytest.mark.gpu

MIB2 = 2 * 1024 * 1024


def _elastic(rank, R, multi_red=True):
    from deep_ep import _C
    # rank_idx, num_ranks, comm_handle, cpu_comm, num_buffer_bytes, num_cpu_buffer_bytes, allow_hybrid_mode,
    # allow_multiple_reduction, prefer_overlap_with_compute, sl_idx, num_allocated_qps, num_cpu_timeout_secs,
    # num_gpu_timeout_secs, explicitly_destroy (csrc/elastic/binding.hpp:24-27)
    return _C.ElasticBuffer(rank, R, 0, None, MIB2, 0, True, multi_red, True, 3, 0, 300, 100, False)


@pytest.mark.parametrize("do_expand", [False, True])
@pytest.mark.parametrize("do_cpu_sync", [True, False])
def test_elastic_dispatch_29_and_combine_18_positional_arguments(do_expand, do_cpu_sync):
    case = rc.small("positional", 777, 1024, 32, 4, 6, seed=5, masked_ratio=0.1)
    rank, A = 1, 4
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    ref = oracle.dispatch(case.x, case.topk_idx, case.topk_weights, case.E, case.R, rank, case.M, do_expand=do_expand,
                          expert_alignment=A)
    rt = _elastic(rank, case.R)
    out = rt.dispatch(x, None, idx, w, None,                                            # x, sf, topk_idx, topk_weights, stats
                      None, None, None, None, None, None, None, None, None, None,       # the ten cached handle fields
                      case.M, case.E, A, 0, 0,                                          # M, E, alignment, num_sms, num_qps
                      None, None, False, False,                                         # events, async, allocate_on_comm_stream
                      True, do_cpu_sync, do_expand, do_expand, False)                   # copy, sync, expand, zero padding, col-major SF
    assert len(out) == 16
    (recv_x, recv_sf, recv_idx, recv_w, copied_idx, num_recv, num_expanded, per_expert_list, psum_rank, psum_expert, unaligned,
     meta, slots, token_meta, linked_list, event) = out
    assert recv_sf is None and token_meta is None and linked_list is None and event is None
    n = ref.num_expanded_tokens if do_expand else ref.num_recv_tokens
    if do_cpu_sync:
        assert (num_recv, recv_x.shape[0]) == (ref.num_recv_tokens, n) and per_expert_list == ref.num_recv_tokens_per_expert_list
    assert_equal(recv_x[:n], ref.recv_x, "recv_x")
    assert_equal(copied_idx, case.topk_idx, "copied topk_idx")
    assert_equal(meta[:ref.num_recv_tokens, :2], ref.recv_src_metadata[:, :2], "recv_src_metadata")
    assert_equal(slots, ref.dst_buffer_slot_idx, "dst_buffer_slot_idx")
    assert_equal(psum_rank, ref.psum_num_recv_tokens_per_scaleup_rank, "psum per rank")

    y = torch.zeros((recv_x.shape[0], case.H), dtype=torch.bfloat16)
    y[:n] = (ref.recv_x.float() * 1.25).to(torch.bfloat16)
    y_d = y.cuda()
    ref_out, ref_w = oracle.combine(y[:n], case.topk_idx, ref.recv_src_metadata, ref.dst_buffer_slot_idx,
                                    ref.psum_num_recv_tokens_per_scaleup_rank, case.E, case.R, rank, case.M,
                                    topk_weights=ref.recv_topk_weights, do_expand=do_expand)

    def combine(runtime, metadata, handle_idx, psum):
        res = runtime.combine(y_d, recv_w, None, None, metadata, handle_idx, psum, None, None,       # x, weights, biases, handle tensors
                              case.E, case.M, 0, 0, None, None, False, False, do_expand)           # E, M, sms, qps, events, flags, layout
        assert len(res) == 3 and res[2] is None
        assert_equal(res[0] + 0.0, ref_out + 0.0, "combined_x")
        assert_equal(res[1], ref_w, "combined_topk_weights")

    combine(rt, meta, copied_idx, psum_rank)                                   # a handle this buffer has seen
    combine(rt, meta.clone(), copied_idx.clone(), psum_rank.clone())           # the same handle as tensors it has not seen
    combine(_elastic(rank, case.R), meta, copied_idx, psum_rank)               # another buffer: nothing remembered
    rt.check_device_status("positional")


def test_rebuilt_slot_map_equals_the_handles_through_the_c_abi():
    """deep_ep_hip_launch_combine with dst_buffer_slot_idx == NULL rebuilds the map behind the dispatch tables of the
    workspace: the rebuilt words equal the handle's own, and a workspace that is too small is refused."""
    import ctypes
    import deep_ep
    from deep_ep import _abi
    case = rc.small("rebuild", 1500, 512, 64, 8, 8, seed=9, masked_ratio=0.2)
    buf = deep_ep.ElasticBuffer(deep_ep.LogicalGroup(3, case.R), num_max_tokens_per_rank=case.M, hidden=case.H, num_topk=case.K)
    recv_x, recv_idx, recv_w, handle, _ = buf.dispatch(case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda(), num_experts=case.E)
    need = _abi.lib.deep_ep_hip_combine_workspace_bytes(case.T, case.K, case.E, case.R)
    tables = _abi.lib.deep_ep_hip_workspace_bytes(case.T, case.K, case.E, case.R)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    out = torch.empty((case.T, case.H), dtype=torch.bfloat16, device="cuda")
    c = _abi.CombineArgs()
    c.num_tokens, c.hidden, c.num_topk, c.num_experts, c.num_ranks = case.T, case.H, case.K, case.E, case.R
    c.rank_idx, c.num_max_tokens_per_rank, c.allow_multiple_reduction = 3, case.M, 1
    c.x, c.num_x_rows = recv_x.data_ptr(), recv_x.shape[0]
    c.topk_idx = handle.topk_idx.data_ptr()
    c.recv_src_metadata, c.num_recv_rows = handle.recv_src_metadata.data_ptr(), handle.recv_src_metadata.shape[0]
    c.psum_num_recv_tokens_per_rank = handle.psum_num_recv_tokens_per_scaleup_rank.data_ptr()
    c.combined_x = out.data_ptr()
    c.workspace, c.workspace_bytes = ws.data_ptr(), need - 256
    sp = torch.cuda.current_stream().cuda_stream
    assert _abi.lib.deep_ep_hip_launch_combine(ctypes.byref(c), sp) == -2 and "rebuild" in _abi.last_error()
    c.workspace_bytes = need
    _abi.check(_abi.lib.deep_ep_hip_launch_combine(ctypes.byref(c), sp), "combine")
    torch.cuda.synchronize()
    rebuilt = ws[tables:tables + case.T * case.K * 4].view(torch.int32).view(case.T, case.K)
    assert_equal(rebuilt, handle.dst_buffer_slot_idx.cpu(), "rebuilt dst_buffer_slot_idx")
    expect, _, _ = buf.combine(recv_x, handle)
    assert_equal(out, expect.cpu(), "combined_x through the rebuilt map")
    assert int(ws[:4].view(torch.int32).item()) == 0


@pytest.mark.parametrize("with_topk", [True, False])
def test_legacy_buffer_reference_positional_calls(with_topk):
    from deep_ep import _C
    c = rc.skewed_masked_case("v1 positional", 1000, 512, 32, 4, 5, 0, masked_ratio=0.3)
    rank, A, C = 2, 4, 6
    rt = _C.Buffer(rank, c.R, 0, 0, False, False, False, False)      # rank, num_ranks, nvl bytes, rdma bytes, ll mode, destroy, shrink, fabric
    assert rt.is_available() and rt.get_num_rdma_ranks() == 1 and rt.get_rdma_rank() == 0
    config = _C.Config(2 * C, 6, 256, 6, 128)
    idx_d, w_d, x_d = c.topk_idx.cuda(), c.topk_weights.cuda(), c.x.cuda()
    per_rank, per_rdma_rank, per_expert, mask_d, event = rt.get_dispatch_layout(idx_d, c.E, None, False, False)
    assert per_rdma_rank is None and event is None
    mask = oracle.layout(c.topk_idx, c.E, c.R)[2]
    assert_equal(mask_d, mask, "is_token_in_rank")
    ref = oracle.intranode_dispatch(c.x, mask, c.topk_idx if with_topk else None, c.topk_weights if with_topk else None,
                                    c.E, c.R, rank, A, C)
    out = rt.intranode_dispatch(x_d, None, idx_d if with_topk else None, w_d if with_topk else None, per_rank, mask_d, per_expert,
                                0, None, None, A, 0, config, None, False, False)
    assert len(out) == 11
    (recv_x, recv_scales, recv_idx, recv_w, per_expert_list, rank_prefix, channel_prefix, recv_channel_prefix, recv_src_idx,
     send_head, event) = out
    assert recv_scales is None and event is None
    assert_equal(recv_x, ref.recv_x, "recv_x")
    assert_equal(send_head, ref.send_head, "send_head")
    assert_equal(rank_prefix, ref.rank_prefix_matrix, "rank_prefix_matrix")
    assert_equal(recv_src_idx, ref.recv_src_idx, "recv_src_idx")
    if with_topk:
        assert_equal(recv_idx, ref.recv_topk_idx, "recv_topk_idx")
        assert per_expert_list == ref.num_recv_tokens_per_expert_list

    # cached dispatch of another payload, as the reference's wrapper calls it: no top-k tensors, no counts, no send_head
    g = torch.Generator().manual_seed(3)
    x2 = torch.randn(c.x.shape, generator=g).to(torch.bfloat16)
    ref2 = oracle.intranode_dispatch(x2, mask, None, None, c.E, c.R, rank, A, C).recv_x
    for prefix, channels, in_rank in ((rank_prefix, channel_prefix, mask_d),                       # the handle the buffer has seen
                                      (rank_prefix.clone(), channel_prefix.clone(), mask_d.clone())):    # the same handle, unseen tensors
        cached = rt.intranode_dispatch(x2.cuda(), None, None, None, None, in_rank, None, recv_src_idx.size(0), prefix, channels,
                                       A, 0, config, None, False, False)
        assert cached[2] is None and cached[3] is None and cached[4] == []
        assert_equal(cached[0], ref2, "cached recv_x")

    y = (ref.recv_x.float() * 0.5).to(torch.bfloat16)
    bias = torch.randn(c.x.shape, generator=g).to(torch.bfloat16)
    w_in = ref.recv_topk_weights if with_topk else None
    res = rt.intranode_combine(y.cuda(), None if w_in is None else w_in.cuda(), bias.cuda(), None, recv_src_idx, rank_prefix,
                               recv_channel_prefix, send_head, config, None, False, False)
    ref_out, ref_w = oracle.intranode_combine(y, ref.send_head, w_in, bias)
    assert len(res) == 3 and res[2] is None
    assert_equal(res[0] + 0.0, ref_out + 0.0, "combined_x")
    if with_topk:
        assert_equal(res[1], ref_w, "combined_topk_weights")
    with pytest.raises(NotImplementedError):
        rt.internode_dispatch(x_d)
    rt.check_device_status("v1 positional")


@pytest.mark.parametrize("use_fp8", [True, False])
def test_low_latency_reference_positional_calls(use_fp8):
    from deep_ep import _C
    R, T, H, E, K, M = 4, 96, 1024, 32, 6, 128
    rank, E_l = 1, E // R
    xs, idxs, ws = rc.c5_sources(seed=2, R=R, T=T, H=H, E=E, K=K)
    rt = _C.Buffer(rank, R, 0, _C.get_low_latency_rdma_size_hint(M, H, R, E), True, False, False, False)
    x, idx, w = xs[rank].contiguous(), idxs[rank].contiguous(), ws[rank].contiguous()
    out = rt.low_latency_dispatch(x.cuda(), idx.cuda(), None, None, M, E, use_fp8, False, False, False, True)
    assert len(out) == 7
    packed_x, packed_scales, count, src_info, layout_range, event, hook = out
    assert event is None and callable(hook) and hook() is None
    assert (packed_scales is not None) == use_fp8
    sources = [x if s == rank else None for s in range(R)]                 # only this logical rank sends in a 2-D call
    ref_x, ref_s, ref_cnt, ref_info, ref_range = oracle.ll_dispatch(sources, list(idxs), M, E, R, rank, use_fp8)
    assert_equal(count, ref_cnt, "packed_recv_count")
    assert_equal(layout_range, ref_range, "packed_recv_layout_range")
    for e in range(E_l):
        n = int(ref_cnt[e])
        assert_equal(src_info[e, :n], ref_info[e, :n], "src_info")
        assert_equal(packed_x[e, :n], ref_x[e, :n], "packed_recv_x")
        if use_fp8:
            assert_equal(packed_scales[e, :n], ref_s[e, :n], "packed_recv_x_scales")

    y = torch.randn((E_l, R * M, H), generator=torch.Generator().manual_seed(7)).to(torch.bfloat16)
    expect = oracle.ll_combine(y, idx, w, ref_info, ref_range, rank, E, R, rank)
    y_d, idx_d, w_d = y.cuda(), idx.cuda(), w.cuda()
    for info in (src_info, src_info.clone()):             # the handle's own tensor (packed rows remembered), then an unseen one (searched)
        res = rt.low_latency_combine(y_d, idx_d, w_d, info, layout_range, None, M, E, False, False, False, False, None)
        assert len(res) == 3 and res[1] is None and res[2] is None
        assert_equal(res[0], expect, "combined_x")
    buf = rt.get_next_low_latency_combine_buffer(M, H, E)
    assert tuple(buf.shape) == (E_l, R * M, H) and buf.dtype == torch.bfloat16
    buf.copy_(y_d)
    res = rt.low_latency_combine(torch.empty_like(y_d), idx_d, w_d, src_info, layout_range, None, M, E, False, True, False, False, None)
    assert_equal(res[0], expect, "combined_x (zero copy)")
    rt.clean_low_latency_buffer(M, H, E)
