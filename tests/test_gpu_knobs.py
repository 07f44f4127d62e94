"""Every tuning knob (a field of the `tuning` member of the argument blocks, set here through the package-wide
default `deep_ep.tuning`) selects another instantiation or code path of the same kernels; the results must stay
bit-identical to the oracle."""
import pytest
import torch

import routing_cases as rc
import routing_oracle as oracle
from test_gpu_parity import _buffer, assert_equal

pytestmark = pytest.mark.gpu

KNOBS = [
    ("xcd_remap", 1), ("plain_loads", 1), ("dispatch_launches", 1), ("dispatch_launches", 2),
    ("cast_pairs", 1), ("cast_pairs", 4), ("cast_pairs", 7), ("cast_pairs", 8), ("copy_vecs", 1), ("copy_vecs", 2),
    ("copy_vecs", 7), ("copy_vecs", 8), ("combine_vecs", 1), ("combine_vecs", 4),
    ("move_workgroups_per_cu", 3), ("move_workgroups_per_cu", 8), ("warm_rounds", -1), ("warm_rounds", 1),
    ("persistent_movers", 4), ("persistent_movers", 8), ("persistent_movers", 15),
]


@pytest.fixture
def knob(request, monkeypatch):
    import deep_ep
    name, value = request.param
    monkeypatch.setattr(deep_ep.tuning, name, value)
    return name, value


@pytest.mark.parametrize("knob", KNOBS, indirect=True, ids=[f"{n}={v}" for n, v in KNOBS])
def test_dispatch_and_combine_under_knob(knob):
    case = rc.small("knobs", 700, 2304, 64, 8, 6, seed=40, masked_ratio=0.1)        # 2304 = 2.25 x 1024 channels: ragged tiles
    buf = _buffer(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    q = oracle.per_token_cast_to_fp8(case.x)
    for do_expand in (False, True):
        ref = oracle.dispatch(q, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M, do_expand=do_expand)
        (rx, rsf), ridx, rw, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E, cast_to_fp8=True, do_expand=do_expand,
                                                      do_cpu_sync=False)
        n = ref.num_expanded_tokens if do_expand else ref.num_recv_tokens
        valid = ref.expanded_row_is_valid if do_expand else torch.ones(n, dtype=torch.bool)
        assert_equal(rx[:n].cpu()[valid], ref.recv_x[valid], "fused FP8 payload")
        assert_equal(rsf[:n].cpu()[valid], ref.recv_sf[valid], "fused FP8 scales")
        assert_equal(handle.dst_buffer_slot_idx, ref.dst_buffer_slot_idx, "dst_buffer_slot_idx")
    ref = oracle.dispatch(case.x, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M)
    rx, ridx, rw, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E)
    assert_equal(rx, ref.recv_x, "BF16 payload")
    assert_equal(ridx, ref.recv_topk_idx, "recv_topk_idx")
    assert_equal(rw, ref.recv_topk_weights, "recv_topk_weights")
    g = torch.Generator().manual_seed(41)
    y = (ref.recv_x.float() * (0.5 + torch.rand((ref.num_recv_tokens, 1), generator=g))).to(torch.bfloat16)
    out, out_w, _ = buf.combine(y.cuda(), handle, topk_weights=rw)
    ref_out, ref_w = oracle.combine(y, case.topk_idx, ref.recv_src_metadata, ref.dst_buffer_slot_idx,
                                    ref.psum_num_recv_tokens_per_scaleup_rank, case.E, case.R, 0, case.M,
                                    topk_weights=ref.recv_topk_weights)
    assert_equal(out + 0.0, ref_out + 0.0, "combined_x")
    assert_equal(out_w, ref_w, "combined_topk_weights")
    buf.check_device_status()


@pytest.mark.parametrize("tokens,hidden", [(1, 1024), (37, 2304), (5000, 7168)], ids=["one_token", "under_one_chunk", "dynamic_chunks"])
def test_persistent_movers_work_queue(tokens, hidden, monkeypatch):
    """The persistent move kernel draws its items from counters that it has to leave at zero, and it shares them with the
    single-launch dispatch: launches of both kinds, one after the other on one buffer, from a call smaller than one chunk
    to one that goes round the global counter many times."""
    import deep_ep
    case = rc.small("queue", tokens, hidden, 64, 8, 6, seed=44, masked_ratio=0.1)
    buf = _buffer(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    q = oracle.per_token_cast_to_fp8(case.x)
    ref = oracle.dispatch(q, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M)
    n = ref.num_recv_tokens
    for movers in (8, 0, 15, 4, 0, 8):
        monkeypatch.setattr(deep_ep.tuning, "persistent_movers", movers)
        (rx, rsf), ridx, rw, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E, cast_to_fp8=True, do_cpu_sync=False)
        assert_equal(rx[:n], ref.recv_x, f"fused FP8 payload, {movers} movers")
        assert_equal(rsf[:n], ref.recv_sf, f"fused FP8 scales, {movers} movers")
        assert_equal(ridx[:n], ref.recv_topk_idx, f"recv_topk_idx, {movers} movers")
        assert_equal(rw[:n], ref.recv_topk_weights, f"recv_topk_weights, {movers} movers")
        assert_equal(handle.dst_buffer_slot_idx, ref.dst_buffer_slot_idx, f"dst_buffer_slot_idx, {movers} movers")
        assert_equal(handle.recv_src_metadata[:n], ref.recv_src_metadata, f"recv_src_metadata, {movers} movers")
        buf.check_device_status()


LL_KNOBS = [("ll_threads", 256), ("ll_threads", 1024), ("ll_pairs", 1), ("ll_pairs", 2), ("ll_two_kernels", 1),
            ("ll_combine_vecs", 1), ("ll_combine_vecs", 2), ("ll_combine_vecs", 4), ("ll_combine_vecs", 7)]


@pytest.mark.parametrize("knob", LL_KNOBS, indirect=True, ids=[f"{n}={v}" for n, v in LL_KNOBS])
def test_low_latency_under_knob(knob):
    import deep_ep
    R, T, H, E, K, M = 4, 100, 2560, 32, 5, 128
    x, idx, w = rc.c5_sources(seed=42, R=R, T=T, H=H, E=E, K=K)
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(2, R), low_latency_mode=True)
    recv, count, handle, _, _ = buf.low_latency_dispatch(x.cuda(), idx.cuda(), M, E, use_fp8=True)
    ref_x, ref_s, ref_cnt, ref_info, ref_range = oracle.ll_dispatch(list(x), list(idx), M, E, R, 2, True)
    assert_equal(count, ref_cnt, "packed_recv_count")
    assert_equal(handle[1], ref_range, "packed_recv_layout_range")
    y = torch.zeros((E // R, R * M, H), dtype=torch.bfloat16)
    for e in range(E // R):
        n = int(ref_cnt[e])
        assert_equal(recv[0][e, :n], ref_x[e, :n], f"packed_recv_x[{e}]")
        assert_equal(recv[1][e, :n], ref_s[e, :n], f"scales[{e}]")
        assert_equal(handle[0][e, :n], ref_info[e, :n], f"src_info[{e}]")
        y[e, :n] = oracle.per_token_cast_back(ref_x[e, :n], ref_s[e, :n])
    out, _, _ = buf.low_latency_combine(y.cuda(), idx.cuda(), w.cuda(), handle)
    for s in range(R):
        assert_equal(out[s] + 0.0, oracle.ll_combine(y, idx[s], w[s], ref_info, ref_range, s, E, R, 2) + 0.0, f"combined_x of source {s}")
