"""GPU parity: the HIP path (through the C ABI, via the deep_ep package) against the CPU oracle.

Bars: layout counts / indices, dispatched payload, scales and metadata are bit-exact; combine is
compared bit-exactly with the fp32-accumulated oracle too (the stated tolerance of the path is
1 BF16 ulp; the deterministic accumulation order makes it exact, signed zeros aside).
"""
import pytest
import torch

import routing_cases as rc
import routing_oracle as oracle

pytestmark = pytest.mark.gpu


def _buffer(case, rank=0, **kw):
    import deep_ep
    return deep_ep.ElasticBuffer(deep_ep.LogicalGroup(rank, case.R), num_max_tokens_per_rank=case.M,
                                 hidden=case.H, num_topk=case.K, **kw)


def _dev(t):
    return None if t is None else t.cuda()


def assert_equal(a, b, what):
    a, b = a.cpu(), b.cpu()
    assert a.shape == b.shape, f"{what}: shape {tuple(a.shape)} != {tuple(b.shape)}"
    assert a.dtype == b.dtype, f"{what}: dtype {a.dtype} != {b.dtype}"
    if a.dtype in (torch.float8_e4m3fn,):
        a, b = a.view(torch.uint8), b.view(torch.uint8)
    if a.dtype in (torch.bfloat16,):
        a, b = a.view(torch.int16), b.view(torch.int16)
    if a.dtype == torch.float32:
        a, b = a.contiguous().view(torch.int32), b.contiguous().view(torch.int32)
    if not torch.equal(a, b):
        bad = (a != b).nonzero()
        raise AssertionError(f"{what}: {bad.shape[0]} mismatching elements, first at {bad[0].tolist()}: "
                             f"{a[tuple(bad[0])].item()} != {b[tuple(bad[0])].item()}")


CASES = {
    "C1": rc.c1,
    "C2": rc.c2,
    "tiny_masked": lambda: rc.small("tiny_masked", 37, 256, 16, 4, 4, seed=3, masked_ratio=0.3),
    "one_token": lambda: rc.small("one_token", 1, 128, 8, 8, 1, seed=4),
    "k1_e_eq_r": lambda: rc.small("k1", 300, 512, 8, 8, 1, seed=5),
    "ragged_chunks": lambda: rc.small("ragged", 1000, 384, 32, 4, 5, seed=6, masked_ratio=0.1),
    "r1_world": lambda: rc.small("r1", 513, 1024, 16, 1, 3, seed=7, masked_ratio=0.05),
    "k9": lambda: rc.small("k9", 200, 2048, 64, 8, 9, seed=8, masked_ratio=0.05),
    # 64 ranks x 20 chunks: too many (rank, chunk) pairs for one wavefront-wide prefix pass
    "many_ranks": lambda: rc.small("many_ranks", 5000, 256, 128, 64, 8, seed=9, masked_ratio=0.05),
    "k20": lambda: rc.small("k20", 150, 256, 64, 4, 20, seed=11, masked_ratio=0.2),
    # the limits of the interface: 1024 experts on 512 ranks
    "max_buckets": lambda: rc.small("max_buckets", 600, 128, 1024, 512, 8, seed=12, masked_ratio=0.05),
    # 36 chunks: a row of chunk totals is summed in two passes
    "many_chunks": lambda: rc.small("many_chunks", 9000, 128, 32, 8, 4, seed=10, masked_ratio=0.05),
}


@pytest.mark.parametrize("name", list(CASES))
def test_layout(name):
    case = CASES[name]()
    buf = _buffer(case)
    per_rank, per_rdma, per_expert, in_rank, _ = buf.get_dispatch_layout(case.topk_idx.cuda(), case.E)
    ref = oracle.layout(case.topk_idx, case.E, case.R)
    assert per_rdma is None
    assert_equal(per_rank, ref[0], "num_tokens_per_rank")
    assert_equal(per_expert, ref[1], "num_tokens_per_expert")
    assert_equal(in_rank, ref[2], "is_token_in_rank")


def _check_handle(handle, ref, case, do_expand):
    assert_equal(handle.psum_num_recv_tokens_per_scaleup_rank, ref.psum_num_recv_tokens_per_scaleup_rank, "psum_rank")
    assert_equal(handle.psum_num_recv_tokens_per_expert, ref.psum_num_recv_tokens_per_expert, "psum_expert")
    assert_equal(handle.num_unaligned_recv_tokens_per_expert, ref.num_unaligned_recv_tokens_per_expert, "unaligned")
    assert_equal(handle.dst_buffer_slot_idx, ref.dst_buffer_slot_idx, "dst_buffer_slot_idx")
    assert_equal(handle.recv_src_metadata[:ref.num_recv_tokens], ref.recv_src_metadata, "recv_src_metadata")
    assert_equal(handle.topk_idx, case.topk_idx, "handle.topk_idx")
    assert handle.do_expand == do_expand


@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("rank", [0, 1])
def test_dispatch_compact_bf16_and_combine(name, rank):
    case = CASES[name]()
    rank = rank % case.R
    buf = _buffer(case, rank)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    recv_x, recv_idx, recv_w, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E)
    ref = oracle.dispatch(case.x, case.topk_idx, case.topk_weights, case.E, case.R, rank, case.M)
    assert handle.num_recv_tokens == ref.num_recv_tokens
    assert handle.num_recv_tokens_per_expert_list == ref.num_recv_tokens_per_expert_list
    assert_equal(recv_x, ref.recv_x, "recv_x")
    assert_equal(recv_idx, ref.recv_topk_idx, "recv_topk_idx")
    assert_equal(recv_w, ref.recv_topk_weights, "recv_topk_weights")
    _check_handle(handle, ref, case, False)

    # combine: every received row comes back scaled by a per-row factor so that order matters
    g = torch.Generator().manual_seed(11)
    y = (ref.recv_x.float() * (0.5 + torch.rand((ref.num_recv_tokens, 1), generator=g))).to(torch.bfloat16)
    b0 = torch.randn((case.T, case.H), generator=g).to(torch.bfloat16)
    b1 = torch.randn((case.T, case.H), generator=g).to(torch.bfloat16)
    for bias_cpu in (None, b0, (b0, b1)):
        bias_gpu = None if bias_cpu is None else (bias_cpu.cuda() if torch.is_tensor(bias_cpu) else tuple(b.cuda() for b in bias_cpu))
        out, out_w, _ = buf.combine(y.cuda(), handle, topk_weights=recv_w, bias=bias_gpu)
        ref_out, ref_w = oracle.combine(y, case.topk_idx, ref.recv_src_metadata, ref.dst_buffer_slot_idx,
                                        ref.psum_num_recv_tokens_per_scaleup_rank, case.E, case.R, rank, case.M,
                                        topk_weights=ref.recv_topk_weights, bias=bias_cpu)
        # signed zeros aside, the accumulation order is identical: compare after +0.0
        assert_equal(out + 0.0, ref_out + 0.0, "combined_x")
        masked_w = case.topk_weights.masked_fill(case.topk_idx < 0, 0.0)
        assert_equal(out_w, ref_w, "combined_topk_weights")
        assert_equal(out_w, masked_w, "combined_topk_weights == topk_weights")
    buf.check_device_status()


@pytest.mark.parametrize("name", list(CASES))
def test_dispatch_fused_fp8(name):
    case = CASES[name]()
    if case.H % 128:
        pytest.skip("hidden not a multiple of 128")
    buf = _buffer(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    (recv_x, recv_sf), recv_idx, recv_w, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E, cast_to_fp8=True)
    q = oracle.per_token_cast_to_fp8(case.x)
    ref = oracle.dispatch(q, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M)
    assert_equal(recv_x, ref.recv_x, "recv_x (fp8 payload)")
    assert_equal(recv_sf, ref.recv_sf, "recv_sf (scales)")
    assert_equal(recv_idx, ref.recv_topk_idx, "recv_topk_idx")
    _check_handle(handle, ref, case, False)

    # pass-through of a pre-cast pair gives the same bytes, in row- and column-major scale layouts
    from deep_ep.utils.math import per_token_cast_to_fp8
    xq, xs = per_token_cast_to_fp8(x)
    assert_equal(xq, q[0], "stand-alone cast payload")
    assert_equal(xs, q[1], "stand-alone cast scales")
    for col_major in (False, True):
        (rx2, rsf2), _, _, h2, _ = buf.dispatch((xq, xs), idx, w, num_experts=case.E,
                                                use_tma_aligned_col_major_sf=col_major)
        assert_equal(rx2, ref.recv_x, "recv_x (pass-through)")
        assert_equal(rsf2, ref.recv_sf, "recv_sf (pass-through)")
        if col_major:
            n = rx2.shape[0]
            assert rsf2.stride() == (1, (n + 3) // 4 * 4)
    buf.check_device_status()


@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("alignment,zero_pad", [(1, False), (4, True), (128, True), (16, False)])
def test_dispatch_expanded_and_combine(name, alignment, zero_pad):
    case = CASES[name]()
    for multi_red in (True, False):
        buf = _buffer(case, allow_multiple_reduction=multi_red)
        x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
        recv_x, recv_idx, recv_w, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E, expert_alignment=alignment,
                                                           do_expand=True, do_zero_padding=zero_pad)
        ref = oracle.dispatch(case.x, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M,
                              expert_alignment=alignment, do_expand=True)
        assert recv_idx is None
        assert handle.num_expanded_tokens == ref.num_expanded_tokens == recv_x.shape[0]
        assert handle.num_recv_tokens_per_expert_list == ref.num_recv_tokens_per_expert_list
        valid = ref.expanded_row_is_valid
        if zero_pad:
            assert_equal(recv_x, ref.recv_x, "expanded recv_x incl. zero padding")
            assert_equal(recv_w, ref.recv_topk_weights, "expanded weights incl. zero padding")
        else:
            assert_equal(recv_x.cpu()[valid], ref.recv_x[valid], "expanded recv_x (valid rows)")
            assert_equal(recv_w.cpu()[valid], ref.recv_topk_weights[valid], "expanded weights (valid rows)")
        _check_handle(handle, ref, case, True)

        g = torch.Generator().manual_seed(13)
        y = (ref.recv_x.float() * (0.5 + torch.rand((ref.num_expanded_tokens, 1), generator=g))).to(torch.bfloat16)
        b0 = torch.randn((case.T, case.H), generator=g).to(torch.bfloat16)
        out, out_w, _ = buf.combine(y.cuda(), handle, topk_weights=recv_w, bias=b0.cuda())
        ref_out, ref_w = oracle.combine(y, case.topk_idx, ref.recv_src_metadata, ref.dst_buffer_slot_idx,
                                        ref.psum_num_recv_tokens_per_scaleup_rank, case.E, case.R, 0, case.M,
                                        topk_weights=ref.recv_topk_weights, bias=b0, do_expand=True,
                                        allow_multiple_reduction=multi_red)
        assert_equal(out + 0.0, ref_out + 0.0, f"combined_x (expanded, multi_red={multi_red})")
        assert_equal(out_w, case.topk_weights.masked_fill(case.topk_idx < 0, 0.0), "combined_topk_weights")
        buf.check_device_status()


@pytest.mark.parametrize("name", ["C1", "tiny_masked", "ragged_chunks"])
@pytest.mark.parametrize("do_expand", [False, True])
def test_cached_dispatch_and_no_sync(name, do_expand):
    case = CASES[name]()
    buf = _buffer(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    kw = dict(num_experts=case.E, do_expand=do_expand, expert_alignment=4 if do_expand else 1)
    recv_x, recv_idx, recv_w, handle, _ = buf.dispatch(x, idx, w, **kw)
    # no CPU sync: worst-case sized outputs, same leading rows
    rx_ns, ri_ns, rw_ns, h_ns, _ = buf.dispatch(x, idx, w, do_cpu_sync=False, **kw)
    n = recv_x.shape[0]
    assert rx_ns.shape[0] >= n and h_ns.num_recv_tokens_per_expert_list == []
    ref = oracle.dispatch(case.x, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M,
                          expert_alignment=kw["expert_alignment"], do_expand=do_expand)
    valid = ref.expanded_row_is_valid if do_expand else torch.ones(n, dtype=torch.bool)
    assert_equal(rx_ns[:n].cpu()[valid], ref.recv_x[valid], "no-sync recv_x")
    assert_equal(h_ns.dst_buffer_slot_idx, handle.dst_buffer_slot_idx, "no-sync slots")
    assert_equal(h_ns.recv_src_metadata[:handle.num_recv_tokens], handle.recv_src_metadata, "no-sync metadata")
    # cached: new payload (here FP8 instead of BF16) under the same handle
    x2 = (case.x.float() * 2 + 1).to(torch.bfloat16)
    if case.H % 128 == 0:
        (rx_c, rsf_c), ri_c, rw_c, h_c, _ = buf.dispatch(x2.cuda(), topk_weights=w, handle=handle, cast_to_fp8=True,
                                                        do_expand=do_expand)
        q2 = oracle.per_token_cast_to_fp8(x2)
        ref2 = oracle.dispatch(q2, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M,
                               expert_alignment=kw["expert_alignment"], do_expand=do_expand)
        assert_equal(rx_c.cpu()[valid], ref2.recv_x[valid], "cached recv_x")
        assert_equal(rsf_c.cpu()[valid], ref2.recv_sf[valid], "cached recv_sf")
    else:
        rx_c, ri_c, rw_c, h_c, _ = buf.dispatch(x2.cuda(), topk_weights=w, handle=handle, do_expand=do_expand)
        ref2 = oracle.dispatch(x2, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M,
                               expert_alignment=kw["expert_alignment"], do_expand=do_expand)
        assert_equal(rx_c.cpu()[valid], ref2.recv_x[valid], "cached recv_x")
    assert h_c is handle
    if not do_expand:
        assert_equal(ri_c, ref2.recv_topk_idx, "cached recv_topk_idx")
        assert_equal(rw_c, ref2.recv_topk_weights, "cached recv_topk_weights")
    else:
        assert_equal(rw_c.cpu()[valid], ref2.recv_topk_weights[valid], "cached expanded weights")
    buf.check_device_status()


@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("cast", [False, True])
def test_dispatch_without_cpu_sync(name, cast):
    """Layout and move in one call (no host round trip): worst-case sized outputs whose leading rows, and
    every handle tensor, equal the oracle's."""
    case = CASES[name]()
    if cast and case.H % 128:
        pytest.skip("hidden not a multiple of 128")
    buf = _buffer(case, rank=case.R - 1)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    stats = torch.zeros(case.E, dtype=torch.int32, device="cuda")
    for _ in range(2):   # twice: the workspace must be left clean for the next call
        recv_x, recv_idx, recv_w, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E, do_cpu_sync=False,
                                                           cast_to_fp8=cast, cumulative_local_expert_recv_stats=stats)
    payload = oracle.per_token_cast_to_fp8(case.x) if cast else case.x
    ref = oracle.dispatch(payload, case.topk_idx, case.topk_weights, case.E, case.R, case.R - 1, case.M)
    n = ref.num_recv_tokens
    assert handle.num_recv_tokens == case.M * case.R and handle.num_recv_tokens_per_expert_list == []
    if cast:
        assert_equal(recv_x[0][:n], ref.recv_x, "recv_x")
        assert_equal(recv_x[1][:n], ref.recv_sf, "recv_sf")
    else:
        assert_equal(recv_x[:n], ref.recv_x, "recv_x")
    assert_equal(recv_idx[:n], ref.recv_topk_idx, "recv_topk_idx")
    assert_equal(recv_w[:n], ref.recv_topk_weights, "recv_topk_weights")
    _check_handle(handle, ref, case, False)
    assert_equal(stats, 2 * ref.num_unaligned_recv_tokens_per_expert, "cumulative stats after two calls")
    # combine straight from the worst-case sized buffers
    y = torch.zeros((case.M * case.R, case.H), dtype=torch.bfloat16)
    y[:n] = (ref.recv_x[0] if cast else ref.recv_x).to(torch.float32).to(torch.bfloat16)
    out, out_w, _ = buf.combine(y.cuda(), handle, topk_weights=recv_w)
    ref_out, _ = oracle.combine(y[:n], case.topk_idx, ref.recv_src_metadata, ref.dst_buffer_slot_idx,
                                ref.psum_num_recv_tokens_per_scaleup_rank, case.E, case.R, case.R - 1, case.M)
    assert_equal(out + 0.0, ref_out + 0.0, "combined_x")
    buf.check_device_status()


@pytest.mark.parametrize("hidden", [192, 7232, 128, 8, 1000])
@pytest.mark.parametrize("tokens", [1, 77])
def test_standalone_cast_with_a_ragged_last_group(hidden, tokens):
    """per_token_cast_to_fp8 when hidden is not a multiple of 128 (192 = 1.5 groups, 7232 = 56.5 groups): the last
    group takes its amax over the channels that exist, and the round trip restores BF16 within FP8's resolution."""
    from deep_ep.utils.math import per_token_cast_back, per_token_cast_to_fp8
    g = torch.Generator().manual_seed(hidden + tokens)
    x = (torch.randn((tokens, hidden), generator=g) * torch.rand((tokens, 1), generator=g) * 8).to(torch.bfloat16)
    x[0, -1] = 300.0          # the largest value of its row sits in the ragged tail
    q, s = per_token_cast_to_fp8(x.cuda())
    q_ref, s_ref = oracle.per_token_cast_to_fp8(x)
    assert q.shape == (tokens, hidden) and s.shape == (tokens, (hidden + 127) // 128)
    assert_equal(q, q_ref, "fp8 payload")
    assert_equal(s, s_ref, "scales")
    back = per_token_cast_back(q, s)
    assert_equal(back, oracle.per_token_cast_back(q_ref, s_ref), "cast back")
    assert float((back.float().cpu() - x.float()).abs().max()) <= 300.0 / 16      # e4m3: 3 mantissa bits
