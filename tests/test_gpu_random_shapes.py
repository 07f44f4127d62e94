"""Seeded random sweep: shapes, routing density, layouts, payloads and call modes drawn at random, every output of
dispatch and combine compared with the CPU oracle.  The fixed cases elsewhere pin the corners; this pins the space
between them (ragged chunk counts, odd hidden sizes, rank counts that do not divide the wavefront, mixed options)."""
import os
import random

import pytest
import torch

import routing_cases as rc
import routing_oracle as oracle
from test_gpu_parity import assert_equal

pytestmark = pytest.mark.gpu


def _draw(seed):
    rnd = random.Random(seed)
    R = rnd.choice([1, 2, 3, 4, 6, 8, 16, 32])
    E = R * rnd.choice([1, 2, 3, 4, 8])
    K = rnd.randint(1, min(E, rnd.choice([2, 4, 8, 9, 12])))
    T = rnd.choice([1, 2, 63, 64, 65, 255, 256, 257, 511, 700, 1024, 1500, 2600])
    payload = rnd.choice(["bf16", "cast_fp8", "fp8_pair"])
    H = 128 * rnd.randint(1, 12) if payload != "bf16" else 8 * rnd.randint(1, 200)
    return dict(R=R, E=E, K=K, T=T, H=H, payload=payload, masked=rnd.choice([0.0, 0.1, 0.5, 0.95]),
                expand=rnd.random() < 0.5, alignment=rnd.choice([1, 1, 4, 16, 128]), zero_pad=rnd.random() < 0.5,
                cpu_sync=rnd.random() < 0.5, rank=rnd.randrange(R), launches=rnd.choice([0, 1, 2]),
                col_major=rnd.random() < 0.3, weights=rnd.random() < 0.8, biases=rnd.choice([0, 1, 2]),
                multi_red=rnd.random() < 0.5, persistent=rnd.choice([0, 0, 0, 4, 8, 15]))


@pytest.mark.parametrize("seed", range(int(os.environ.get("DEEP_EP_TEST_RANDOM_CASES", "60"))))    # more for a longer hunt
def test_random_configuration(seed, monkeypatch):
    import deep_ep
    c = _draw(1000 + seed)
    monkeypatch.setattr(deep_ep.tuning, "dispatch_launches", c["launches"])
    monkeypatch.setattr(deep_ep.tuning, "persistent_movers", c["persistent"])      # takes effect on compact fused-cast dispatches
    case = rc.small(f"rnd{seed}", c["T"], c["H"], c["E"], c["R"], c["K"], seed=seed, masked_ratio=c["masked"])
    M = case.M + (seed % 3) * 17                      # capacity above the token count on two of three cases
    buf = deep_ep.ElasticBuffer(deep_ep.LogicalGroup(c["rank"], c["R"]), num_max_tokens_per_rank=M, hidden=c["H"],
                                num_topk=c["K"], allow_multiple_reduction=c["multi_red"])
    expand = c["expand"]
    zero_pad = c["zero_pad"] and expand
    w_cpu = case.topk_weights if c["weights"] else None
    idx, w = case.topk_idx.cuda(), None if w_cpu is None else w_cpu.cuda()
    if c["payload"] == "bf16":
        src, x_arg, kw = case.x, case.x.cuda(), {}
    elif c["payload"] == "cast_fp8":
        src, x_arg, kw = oracle.per_token_cast_to_fp8(case.x), case.x.cuda(), {"cast_to_fp8": True}
    else:
        src = oracle.per_token_cast_to_fp8(case.x)
        x_arg, kw = (src[0].cuda(), src[1].cuda()), {}
    fp8 = c["payload"] != "bf16"
    recv, ridx, rw, handle, _ = buf.dispatch(x_arg, idx, w, num_experts=c["E"], expert_alignment=c["alignment"],
                                             do_expand=expand, do_zero_padding=zero_pad, do_cpu_sync=c["cpu_sync"],
                                             use_tma_aligned_col_major_sf=c["col_major"] and fp8, **kw)
    ref = oracle.dispatch(src, case.topk_idx, w_cpu, c["E"], c["R"], c["rank"], M, expert_alignment=c["alignment"],
                          do_expand=expand)
    n = ref.num_expanded_tokens if expand else ref.num_recv_tokens
    rows = slice(None) if (not expand or zero_pad) else ref.expanded_row_is_valid
    got_x, got_sf = recv if fp8 else (recv, None)
    assert got_x.shape[0] >= n and (not c["cpu_sync"] or got_x.shape[0] == n), (got_x.shape, n)
    assert_equal(got_x[:n].cpu()[rows], ref.recv_x[rows], "recv_x")
    if fp8:
        assert_equal(got_sf[:n].cpu()[rows], ref.recv_sf[rows], "recv_sf")
    if expand:
        assert ridx is None
    else:
        assert_equal(ridx[:n], ref.recv_topk_idx, "recv_topk_idx")
    if w_cpu is None:
        assert rw is None
    else:
        assert_equal(rw[:n].cpu()[rows], ref.recv_topk_weights[rows], "recv_topk_weights")
    assert_equal(handle.psum_num_recv_tokens_per_scaleup_rank, ref.psum_num_recv_tokens_per_scaleup_rank, "psum_rank")
    assert_equal(handle.psum_num_recv_tokens_per_expert, ref.psum_num_recv_tokens_per_expert, "psum_expert")
    assert_equal(handle.num_unaligned_recv_tokens_per_expert, ref.num_unaligned_recv_tokens_per_expert, "unaligned")
    assert_equal(handle.dst_buffer_slot_idx, ref.dst_buffer_slot_idx, "dst_buffer_slot_idx")
    assert_equal(handle.recv_src_metadata[:ref.num_recv_tokens], ref.recv_src_metadata, "recv_src_metadata")
    if c["cpu_sync"]:
        assert handle.num_recv_tokens_per_expert_list == ref.num_recv_tokens_per_expert_list

    # combine what was received, scaled per row so that the order of the reduction matters
    g = torch.Generator().manual_seed(seed)
    y = torch.zeros((got_x.shape[0], c["H"]), dtype=torch.bfloat16)
    y[:n] = (torch.randn((n, c["H"]), generator=g) * (0.5 + torch.rand((n, 1), generator=g))).to(torch.bfloat16)
    biases = tuple(torch.randn((case.T, c["H"]), generator=g).to(torch.bfloat16) for _ in range(c["biases"]))
    bias_cpu = None if not biases else biases[0] if len(biases) == 1 else biases
    bias_gpu = None if not biases else biases[0].cuda() if len(biases) == 1 else tuple(b.cuda() for b in biases)
    out, out_w, _ = buf.combine(y.cuda(), handle, topk_weights=rw, bias=bias_gpu)
    ref_out, ref_w = oracle.combine(y[:n], case.topk_idx, ref.recv_src_metadata, ref.dst_buffer_slot_idx,
                                    ref.psum_num_recv_tokens_per_scaleup_rank, c["E"], c["R"], c["rank"], M,
                                    topk_weights=ref.recv_topk_weights, bias=bias_cpu, do_expand=expand,
                                    allow_multiple_reduction=c["multi_red"])
    assert_equal(out + 0.0, ref_out + 0.0, "combined_x")
    if w_cpu is None:
        assert out_w is None
    else:
        assert_equal(out_w, ref_w, "combined_topk_weights")
    buf.check_device_status()


def _draw_low_latency(seed):
    rnd = random.Random(seed)
    R = rnd.choice([1, 2, 3, 4, 8])
    E = R * rnd.choice([1, 2, 4, 8, 16])
    K = rnd.randint(1, min(E, rnd.choice([2, 4, 8, 9])))
    T = rnd.choice([1, 3, 17, 64, 128, 200, 700, 2100])             # 2100 x R tokens: several work items per wavefront, or beyond the single-kernel path
    ue8m0 = rnd.random() < 0.25
    H = 512 * rnd.randint(1, 4) if ue8m0 else 128 * rnd.randint(1, 16)
    M = (T + rnd.choice([0, 5, 64]) + 3) // 4 * 4                    # rows per expert (R * M) must be a multiple of 4
    return dict(R=R, E=E, K=K, T=T, H=H, M=M, dst=rnd.randrange(R), masked=rnd.choice([0.0, 0.1, 0.6]),
                use_fp8=ue8m0 or rnd.random() < 0.6, round_scale=ue8m0 or rnd.random() < 0.3, ue8m0=ue8m0)


@pytest.mark.parametrize("seed", range(int(os.environ.get("DEEP_EP_TEST_RANDOM_CASES", "30"))))
def test_random_low_latency_configuration(seed):
    import deep_ep
    c = _draw_low_latency(5000 + seed)
    R, E, K, T, H, M, dst = c["R"], c["E"], c["K"], c["T"], c["H"], c["M"], c["dst"]
    use_fp8, round_scale = c["use_fp8"], c["round_scale"] and c["use_fp8"]
    x, idx, w = rc.c5_sources(seed=seed, R=R, T=T, H=H, E=E, K=K)
    g = torch.Generator().manual_seed(seed)
    idx = idx.masked_fill(torch.rand(idx.shape, generator=g) < c["masked"], -1)
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(dst, R), low_latency_mode=True)
    recv, count, handle, _, _ = buf.low_latency_dispatch(x.cuda(), idx.cuda(), M, E, use_fp8=use_fp8, round_scale=round_scale,
                                                         use_ue8m0=c["ue8m0"])
    ref_x, ref_s, ref_cnt, ref_info, ref_range = oracle.ll_dispatch(list(x), list(idx), M, E, R, dst, use_fp8,
                                                                    round_scale=round_scale)
    assert_equal(count, ref_cnt, "packed_recv_count")
    assert_equal(handle[1], ref_range, "packed_recv_layout_range")
    px = recv[0] if use_fp8 else recv
    for e in range(E // R):
        n = int(ref_cnt[e])
        assert_equal(px[e, :n], ref_x[e, :n], f"packed_recv_x[{e}]")
        assert_equal(handle[0][e, :n], ref_info[e, :n], f"src_info[{e}]")
        if use_fp8:
            want = oracle.pack_ue8m0(ref_s[e, :n]) if c["ue8m0"] else ref_s[e, :n]
            assert_equal(recv[1][e, :n], want, f"scales[{e}]")
    y = (torch.randn((E // R, R * M, H), generator=g) * 0.5).to(torch.bfloat16)
    out, _, _ = buf.low_latency_combine(y.cuda(), idx.cuda(), w.cuda(), handle)
    for s in range(R):
        ref_out = oracle.ll_combine(y, idx[s], w[s], ref_info, ref_range, s, E, R, dst)
        assert_equal(out[s] + 0.0, ref_out + 0.0, f"combined_x of source {s}")


def _draw_v1(seed):
    rnd = random.Random(seed)
    R = rnd.choice([1, 2, 3, 4, 8, 16])
    E = R * rnd.choice([1, 2, 4, 8])
    K = rnd.randint(1, min(E, rnd.choice([2, 4, 8, 10])))
    fp8 = rnd.random() < 0.4
    return dict(R=R, E=E, K=K, T=rnd.choice([1, 2, 65, 256, 300, 1000, 2300]), fp8=fp8,
                H=128 * rnd.randint(1, 10) if fp8 else 8 * rnd.randint(1, 160), masked=rnd.choice([0.0, 0.2, 0.7]),
                rank=rnd.randrange(R), channels=rnd.choice([1, 3, 6, 10]), alignment=rnd.choice([1, 4, 32]),
                with_topk=rnd.random() < 0.7, worst=rnd.random() < 0.4, biases=rnd.choice([0, 1, 2]))


@pytest.mark.parametrize("seed", range(int(os.environ.get("DEEP_EP_TEST_RANDOM_CASES", "30"))))
def test_random_v1_configuration(seed):
    """`Buffer.get_dispatch_layout` + `Buffer.dispatch` + `Buffer.combine` (the V1 triple) on random shapes."""
    import deep_ep
    c = _draw_v1(9000 + seed)
    R, E, rank, C, A = c["R"], c["E"], c["rank"], c["channels"], c["alignment"]
    case = rc.small(f"v1_{seed}", c["T"], c["H"], E, R, c["K"], seed=seed, masked_ratio=c["masked"])
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(rank, R))
    config = deep_ep.Config(2 * C, 6, 256)
    idx_d = case.topk_idx.cuda()
    per_rank, _, per_expert, mask_d, _ = buf.get_dispatch_layout(idx_d, E)
    want_rank, want_expert, mask = oracle.layout(case.topk_idx, E, R)
    assert_equal(per_rank, want_rank, "num_tokens_per_rank")
    assert_equal(per_expert, want_expert, "num_tokens_per_expert")
    assert_equal(mask_d, mask, "is_token_in_rank")
    if c["fp8"]:
        x_ref = oracle.per_token_cast_to_fp8(case.x)
        x_dev = (x_ref[0].cuda(), x_ref[1].cuda())
    else:
        x_ref, x_dev = case.x, case.x.cuda()
    with_topk = c["with_topk"]
    ref = oracle.intranode_dispatch(x_ref, mask, case.topk_idx if with_topk else None,
                                    case.topk_weights if with_topk else None, E, R, rank, A, C)
    kw = dict(num_tokens_per_rank=per_rank, is_token_in_rank=mask_d, num_tokens_per_expert=per_expert,
              expert_alignment=A, config=config)
    if with_topk:
        kw.update(topk_idx=idx_d, topk_weights=case.topk_weights.cuda())
    worst = case.T * R if (c["worst"] and with_topk) else 0
    recv_x, recv_idx, recv_w, _, handle, _ = buf.dispatch(x_dev, num_worst_tokens=worst, **kw)
    n = ref.recv_x.shape[0]
    got = recv_x[0] if c["fp8"] else recv_x
    assert got.shape[0] == (worst if worst else n)
    assert_equal(got[:n].view(torch.uint8), ref.recv_x.view(torch.uint8), "recv_x")
    if c["fp8"]:
        assert_equal(recv_x[1][:n], ref.recv_x_scales, "recv_x_scales")
    if with_topk:
        assert_equal(recv_idx[:n], ref.recv_topk_idx, "recv_topk_idx")
        assert_equal(recv_w[:n], ref.recv_topk_weights, "recv_topk_weights")
        assert bool((recv_idx[n:] == -1).all())
    assert_equal(handle[0], ref.rank_prefix_matrix, "rank_prefix_matrix")
    assert_equal(handle[1], ref.channel_prefix_matrix, "channel_prefix_matrix")
    assert_equal(handle[3][:n], ref.recv_src_idx, "recv_src_idx")
    assert_equal(handle[5], ref.send_head, "send_head")

    g = torch.Generator().manual_seed(seed)
    y = torch.zeros((got.shape[0], c["H"]), dtype=torch.bfloat16)
    y[:n] = torch.randn((n, c["H"]), generator=g).to(torch.bfloat16)
    biases = tuple(torch.randn((case.T, c["H"]), generator=g).to(torch.bfloat16) for _ in range(c["biases"]))
    bias_cpu = None if not biases else biases[0] if len(biases) == 1 else biases
    bias_gpu = None if not biases else biases[0].cuda() if len(biases) == 1 else tuple(b.cuda() for b in biases)
    w_in = ref.recv_topk_weights if with_topk else None
    w_dev = None
    if w_in is not None:
        w_dev = torch.zeros((got.shape[0], c["K"]), dtype=torch.float32)
        w_dev[:n] = w_in
        w_dev = w_dev.cuda()
    out, out_w, _ = buf.combine(y.cuda(), handle, topk_weights=w_dev, bias=bias_gpu, config=config)
    ref_out, ref_w = oracle.intranode_combine(y[:n], ref.send_head, w_in, bias_cpu)
    assert_equal(out + 0.0, ref_out + 0.0, "combined_x")
    if with_topk:
        assert_equal(out_w, ref_w, "combined_topk_weights")
    buf.runtime.check_device_status("intranode")
