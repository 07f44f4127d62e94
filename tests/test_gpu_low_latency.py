"""GPU parity of the low-latency packed layout against the CPU oracle, through the Buffer API."""
import pytest
import torch

import routing_cases as rc
import routing_oracle as oracle
from test_gpu_parity import assert_equal

pytestmark = pytest.mark.gpu


def _ranges(layout_range):
    lr = layout_range.cpu()
    return lr >> 32, lr & 0xFFFFFFFF


@pytest.mark.parametrize("R,T,H,E,K,M", [(8, 128, 7168, 256, 8, 128), (2, 40, 1024, 8, 2, 64), (4, 300, 2048, 32, 6, 300),
                                         (1, 17, 512, 4, 3, 20),
                                         (2, 1500, 256, 16, 9, 1500),      # single kernel, several work items per wavefront
                                         (2, 2300, 256, 16, 9, 2300),      # too many tokens for the single-kernel path
                                         (4, 200, 512, 64, 12, 256)])
@pytest.mark.parametrize("use_fp8", [True, False])
def test_ll_stacked_sources(R, T, H, E, K, M, use_fp8):
    import deep_ep
    x, idx, w = rc.c5_sources(seed=5, R=R, T=T, H=H, E=E, K=K)
    # mask a few lanes
    g = torch.Generator().manual_seed(9)
    mask = torch.rand(idx.shape, generator=g) < 0.1
    idx = idx.masked_fill(mask, -1)
    for dst_rank in sorted({0, R - 1}):
        buf = deep_ep.Buffer(deep_ep.LogicalGroup(dst_rank, R), low_latency_mode=True)
        stats = torch.zeros(E // R, dtype=torch.int32, device="cuda")
        recv, count, handle, _, hook = buf.low_latency_dispatch(x.cuda(), idx.cuda(), M, E, use_fp8=use_fp8,
                                                                cumulative_local_expert_recv_stats=stats)
        assert hook is None
        ref_x, ref_s, ref_cnt, ref_info, ref_range = oracle.ll_dispatch(list(x), list(idx), M, E, R, dst_rank, use_fp8)
        assert_equal(count, ref_cnt, "packed_recv_count")
        assert_equal(stats, ref_cnt, "cumulative stats")
        assert_equal(handle[1], ref_range, "packed_recv_layout_range")
        px = recv[0] if use_fp8 else recv
        assert px.shape == (E // R, R * M, H)
        if use_fp8:
            assert recv[1].shape == (E // R, R * M, H // 128) and recv[1].stride(1) == 1 and recv[1].stride(2) == R * M
        for e in range(E // R):
            n = int(ref_cnt[e])
            assert_equal(px[e, :n], ref_x[e, :n], f"packed_recv_x[{e}]")
            assert_equal(handle[0][e, :n], ref_info[e, :n], f"src_info[{e}]")
            if use_fp8:
                assert_equal(recv[1][e, :n], ref_s[e, :n], f"scales[{e}]")
        # reference-test invariants (tests/legacy/test_low_latency.py:110-141)
        begin, cnt = _ranges(handle[1])
        assert torch.equal(cnt.sum(dim=1).to(torch.int32), ref_cnt)
        assert torch.equal(begin, torch.cumsum(cnt, 1) - cnt)

        # combine: expert outputs = dequantised/plain rows times (1 + local expert id / 8)
        y = torch.zeros((E // R, R * M, H), dtype=torch.bfloat16)
        for e in range(E // R):
            n = int(ref_cnt[e])
            rows = oracle.per_token_cast_back(ref_x[e, :n], ref_s[e, :n]) if use_fp8 else ref_x[e, :n]
            y[e, :n] = (rows.float() * (1 + e / 8)).to(torch.bfloat16)
        out, _, _ = buf.low_latency_combine(y.cuda(), idx.cuda(), w.cuda(), handle)
        for s in range(R):
            ref_out = oracle.ll_combine(y, idx[s], w[s], ref_info, ref_range, s, E, R, dst_rank)
            assert_equal(out[s] + 0.0, ref_out + 0.0, f"ll combined_x from source {s}")
        # single-source form gives the same rows for that source
        if R > 1:
            s = dst_rank
            recv1, count1, handle1, _, _ = buf.low_latency_dispatch(x[s].cuda(), idx[s].cuda(), M, E, use_fp8=use_fp8)
            r1 = oracle.ll_dispatch([x[i] if i == s else None for i in range(R)], list(idx), M, E, R, dst_rank, use_fp8)
            assert_equal(count1, r1[2], "single-source count")
            assert_equal(handle1[1], r1[4], "single-source layout_range")
            out1, _, _ = buf.low_latency_combine(y.cuda() * 0 + 1, idx[s].cuda(), w[s].cuda(), handle1)
            assert out1.shape == (T, H)


@pytest.mark.parametrize("R,T,H,E,K,M", [(8, 128, 7168, 256, 8, 128), (2, 40, 1024, 8, 2, 64), (2, 1500, 512, 16, 9, 1500)])
@pytest.mark.parametrize("use_ue8m0", [False, True])
def test_ll_power_of_two_scales_hooks_and_zero_copy(R, T, H, E, K, M, use_ue8m0):
    """`round_scale` / `use_ue8m0` scale formats, `return_recv_hook` and the zero-copy combine buffer
    (the mode loop of the reference's tests/legacy/test_low_latency.py:89-104,160-173)."""
    import deep_ep
    x, idx, w = rc.c5_sources(seed=6, R=R, T=T, H=H, E=E, K=K)
    x = (x.float() * torch.logspace(-3, 3, T).view(1, T, 1)).to(torch.bfloat16)      # spread the exponents
    dst_rank = R - 1
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(dst_rank, R), low_latency_mode=True)
    recv, count, handle, event, hook = buf.low_latency_dispatch(x.cuda(), idx.cuda(), M, E, use_fp8=True, round_scale=True,
                                                                use_ue8m0=use_ue8m0, return_recv_hook=True)
    assert callable(hook)
    hook()
    ref_x, ref_s, ref_cnt, ref_info, ref_range = oracle.ll_dispatch(list(x), list(idx), M, E, R, dst_rank, True, round_scale=True)
    assert_equal(count, ref_cnt, "packed_recv_count")
    assert_equal(handle[1], ref_range, "packed_recv_layout_range")
    E_l, rows = E // R, R * M
    if use_ue8m0:
        assert recv[1].dtype == torch.int32 and recv[1].shape == (E_l, rows, H // 512)
        assert recv[1].stride(1) == 1 and recv[1].stride(2) == rows
    else:
        assert recv[1].dtype == torch.float32 and recv[1].shape == (E_l, rows, H // 128)
    for e in range(E_l):
        n = int(ref_cnt[e])
        assert_equal(recv[0][e, :n].view(torch.uint8), ref_x[e, :n].view(torch.uint8), f"packed_recv_x[{e}]")
        expect = oracle.pack_ue8m0(ref_s[e, :n]) if use_ue8m0 else ref_s[e, :n]
        assert_equal(recv[1][e, :n], expect, f"scales[{e}]")
    # the reference's decode rule recovers the dispatched values to FP8 accuracy
    if use_ue8m0:
        packs = torch.empty(recv[1].shape, dtype=torch.int32)
        packs.copy_(recv[1])
        sc = (packs.view(torch.uint8).to(torch.int32) << 23).view(torch.float32)
    else:
        sc = recv[1].cpu()
    for e in range(E_l):
        n = int(ref_cnt[e])
        if n:
            back = oracle.per_token_cast_back(recv[0][e, :n].cpu(), sc[e, :n].contiguous())
            src = torch.cat([x[s][ref_info[e, (ref_range[e, s] >> 32):(ref_range[e, s] >> 32) + (ref_range[e, s] & 0xffffffff)].long()]
                             for s in range(R)])
            assert float((back.float() - src.float()).abs().max() / src.float().abs().max()) < 0.07

    # zero-copy combine: same result as passing the tensor
    y = torch.randn((E_l, rows, H), generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).cuda()
    out_a, _, hook_a = buf.low_latency_combine(y, idx.cuda(), w.cuda(), handle, return_recv_hook=True)
    hook_a()
    buf.get_next_low_latency_combine_buffer(handle)[:, :, :] = y
    out_b, _, hook_b = buf.low_latency_combine(torch.empty_like(y), idx.cuda(), w.cuda(), handle, zero_copy=True)
    assert hook_b is None
    assert_equal(out_a, out_b, "zero-copy combine")
    with pytest.raises(RuntimeError):           # the codec and zero-copy exclude each other (internode_ll.cu:1182)
        buf.low_latency_combine(y, idx.cuda(), w.cuda(), handle, use_logfmt=True, zero_copy=True)


def test_ll_empty_and_unrouted_tokens():
    import deep_ep
    R, E, K, H, M = 2, 8, 2, 512, 16
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(0, R), low_latency_mode=True)
    for T, fill in ((0, 0), (7, -1), (7, 5)):              # nothing; nothing selected; everything on the other rank
        x = torch.randn((T, H), device="cuda").to(torch.bfloat16)
        idx = torch.full((T, K), fill, dtype=torch.int64, device="cuda")
        if fill == 5:
            idx[:, 1] = 6
        w = torch.rand((T, K), device="cuda")
        recv, count, handle, _, _ = buf.low_latency_dispatch(x, idx, M, E, use_fp8=True)
        assert recv[0].shape == (E // R, R * M, H) and int(count.sum()) == 0
        assert int((handle[1] & 0xffffffff).sum()) == 0
        y = torch.ones((E // R, R * M, H), dtype=torch.bfloat16, device="cuda")
        out, _, _ = buf.low_latency_combine(y, idx, w, handle)
        assert out.shape == (T, H) and bool((out == 0).all())


def _calc_diff(a, b):
    a, b = a.double(), b.double()
    return float(1 - 2 * (a * b).sum() / ((a * a).sum() + (b * b).sum()))


@pytest.mark.parametrize("hidden", [7168, 1536])           # chunks of 1024 channels / of 512 channels
def test_low_latency_combine_with_logfmt(hidden):
    """`use_logfmt=True` (csrc/kernels/legacy/internode_ll.cu:556-712): rows pass through the LogFMT-10 codec before the
    weighted reduce.  Against the oracle's codec (exact log2 / exp2 in fp64; the kernel uses the hardware's, as the
    reference uses its hardware's): the reference's own bar calc_diff < 9e-4 against the exact result
    (tests/legacy/test_low_latency.py:178-181), near bit-equality with the oracle, and bit-equality where the codec
    must leave rows alone."""
    import deep_ep
    R, T, E, K, M = 4, 96, 32, 6, 128
    x, idx, w = rc.c5_sources(seed=91, R=R, T=T, H=hidden, E=E, K=K)
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(1, R), low_latency_mode=True)
    _, count, handle, _, _ = buf.low_latency_dispatch(x.cuda(), idx.cuda(), M, E, use_fp8=False)
    _, _, ref_cnt, ref_info, ref_range = oracle.ll_dispatch(list(x), list(idx), M, E, R, 1, False)
    g = torch.Generator().manual_seed(92)
    y = (torch.randn((E // R, R * M, hidden), generator=g) * 0.1).to(torch.bfloat16)      # expert outputs: mostly below 1
    y[0, :, :1024] = (torch.randn((R * M, 1024), generator=g) * 3).to(torch.bfloat16)      # a chunk the codec leaves alone
    y[1, :, 0:128] = 0.25                                                                  # a single-magnitude group
    out_q, _, _ = buf.low_latency_combine(y.cuda(), idx.cuda(), w.cuda(), handle, use_logfmt=True)
    out_x, _, _ = buf.low_latency_combine(y.cuda(), idx.cuda(), w.cuda(), handle, use_logfmt=False)
    assert not torch.isnan(out_q).any()
    total, same = 0, 0
    for s in range(R):
        ref_q = oracle.ll_combine(y, idx[s], w[s], ref_info, ref_range, s, E, R, 1, use_logfmt=True)
        ref_x = oracle.ll_combine(y, idx[s], w[s], ref_info, ref_range, s, E, R, 1)
        assert_equal(out_x[s] + 0.0, ref_x + 0.0, f"plain combine of source {s}")
        got = out_q[s].cpu()
        assert _calc_diff(got, ref_x) < 9e-4, "the reference's acceptance bar"
        assert _calc_diff(got, ref_q) < 1e-7, "against the oracle's codec"
        same += int((got.view(torch.int16) == ref_q.view(torch.int16)).sum())
        total += got.numel()
        # tokens whose only rows on this rank (experts [E/R, 2E/R)) come from its first expert read, in their first
        # chunk, values of magnitude >= 1: there the codec must hand the rows through unchanged
        first = E // R
        elsewhere = (idx[s] < first) | (idx[s] >= 2 * first)
        tokens = ((idx[s] == first) | elsewhere).all(dim=1)
        chunk = 1024 if hidden % 1024 == 0 else 512
        assert_equal(out_q[s].cpu()[tokens][:, :chunk] + 0.0, out_x[s].cpu()[tokens][:, :chunk] + 0.0,
                     "chunks the codec must not touch")
    assert same / total > 0.999, f"only {same / total:.5f} of the outputs equal the oracle's bit for bit"
    assert _calc_diff(out_q.cpu(), out_x.cpu()) > 1e-9, "the codec did nothing"
    with pytest.raises(RuntimeError):
        buf.low_latency_combine(y.cuda(), idx.cuda(), w.cuda(), handle, use_logfmt=True, zero_copy=True)


def test_mask_buffer_calls_of_the_reference_surface():
    """deep_ep/buffers/legacy.py:672-698: on one GPU no logical rank can stop answering, so no rank is ever masked."""
    import deep_ep
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(0, 4), low_latency_mode=True)
    status = torch.full((4,), 7, dtype=torch.int32, device="cuda")
    buf.low_latency_query_mask_buffer(status)
    assert status.tolist() == [0, 0, 0, 0]
    buf.low_latency_update_mask_buffer(2, False)
    buf.low_latency_clean_mask_buffer()
    with pytest.raises(NotImplementedError):
        buf.low_latency_update_mask_buffer(2, True)
