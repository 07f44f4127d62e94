"""GPU parity of the V1 `Buffer.dispatch` / `Buffer.combine` pair against the CPU oracle, through the Buffer API
(what the reference checks in tests/legacy/test_intranode.py:90-186)."""
import pytest
import torch

import routing_cases as rc
import routing_oracle as oracle
from test_gpu_parity import assert_equal

pytestmark = pytest.mark.gpu


def _case(name, seed=0):
    if name == "C1":
        return rc.softmax_topk_case("C1", 128, 1024, 8, 2, 2, seed)
    if name == "C2":
        return rc.softmax_topk_case("C2", 4096, 2048, 64, 8, 6, seed)
    if name == "masked":
        return rc.skewed_masked_case("masked", 1000, 512, 32, 4, 5, seed, masked_ratio=0.3)
    if name == "ragged":
        return rc.uniform_topk_case("ragged", 777, 7168, 256, 8, 8, seed)
    if name == "many_lanes":
        return rc.uniform_topk_case("many_lanes", 300, 256, 64, 16, 20, seed)
    raise KeyError(name)


def _check_handle(handle, ref, num_channels):
    rank_prefix_matrix, channel_prefix_matrix, recv_channel_prefix_matrix, recv_src_idx, mask, send_head = handle
    assert_equal(rank_prefix_matrix, ref.rank_prefix_matrix, "rank_prefix_matrix")
    assert_equal(channel_prefix_matrix, ref.channel_prefix_matrix, "channel_prefix_matrix")
    assert_equal(recv_channel_prefix_matrix, ref.recv_channel_prefix_matrix, "recv_channel_prefix_matrix")
    assert_equal(recv_src_idx, ref.recv_src_idx, "recv_src_idx")
    assert_equal(send_head, ref.send_head, "send_head")
    assert channel_prefix_matrix.shape[1] == num_channels


@pytest.mark.parametrize("name", ["C1", "C2", "masked", "ragged", "many_lanes"])
@pytest.mark.parametrize("with_topk", [True, False])
@pytest.mark.parametrize("fp8", [False, True])
def test_dispatch_and_combine(name, with_topk, fp8):
    import deep_ep
    c = _case(name)
    if not with_topk and c.R > 32:
        pytest.skip("mask routing takes one lane per rank")
    rank = c.R - 1
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(rank, c.R))
    config = deep_ep.Config(12, 6, 256)
    C = 6
    A = 4 if name == "masked" else 1
    idx_d = c.topk_idx.cuda()
    per_rank, _, per_expert, mask_d, _ = buf.get_dispatch_layout(idx_d, c.E)
    mask = oracle.layout(c.topk_idx, c.E, c.R)[2]
    assert_equal(mask_d, mask, "is_token_in_rank")
    if fp8:
        q, sf = oracle.per_token_cast_to_fp8(c.x)
        x_ref = (q, sf)
        x_dev = (q.cuda(), sf.cuda().T.contiguous().T)            # column-major scales, as the reference test passes
    else:
        x_ref, x_dev = c.x, c.x.cuda()
    ref = oracle.intranode_dispatch(x_ref, mask, c.topk_idx if with_topk else None,
                                    c.topk_weights if with_topk else None, c.E, c.R, rank, A, C)
    kw = dict(num_tokens_per_rank=per_rank, is_token_in_rank=mask_d, num_tokens_per_expert=per_expert,
              expert_alignment=A, config=config)
    if with_topk:
        kw.update(topk_idx=idx_d, topk_weights=c.topk_weights.cuda())
    recv_x, recv_idx, recv_w, per_expert_list, handle, _ = buf.dispatch(x_dev, **kw)
    n = ref.recv_x.shape[0]
    if fp8:
        assert recv_x[0].shape[0] == n
        assert_equal(recv_x[0].view(torch.uint8), ref.recv_x.view(torch.uint8), "recv_x (fp8)")
        assert_equal(recv_x[1], ref.recv_x_scales, "recv_x_scales")
    else:
        assert recv_x.shape[0] == n
        assert_equal(recv_x.view(torch.int16), ref.recv_x.view(torch.int16), "recv_x")
    _check_handle(handle, ref, C)
    expect_list = ref.num_recv_tokens_per_expert_list if with_topk else \
        [(int(v) + A - 1) // A * A for v in oracle.layout(c.topk_idx, c.E, c.R)[1]]
    assert per_expert_list == expect_list
    if with_topk:
        assert_equal(recv_idx, ref.recv_topk_idx, "recv_topk_idx")
        assert_equal(recv_w, ref.recv_topk_weights, "recv_topk_weights")
        # no-CPU-sync form: worst-case rows, unused index rows read -1 (test_intranode.py:148-162)
        worst = c.T * c.R
        wx, widx, ww, empty, _, _ = buf.dispatch(x_dev, num_worst_tokens=worst, **kw)
        assert empty == [] and widx.shape[0] == worst and ww.shape[0] == worst
        wx0 = wx[0] if fp8 else wx
        assert wx0.shape[0] == worst
        assert_equal(wx0[:n].view(torch.uint8), (ref.recv_x.view(torch.uint8)), "recv_x (worst)")
        assert_equal(widx[:n], ref.recv_topk_idx, "recv_topk_idx (worst)")
        assert_equal(ww[:n], ref.recv_topk_weights, "recv_topk_weights (worst)")
        assert bool((widx[n:] == -1).all())
    else:
        assert recv_idx is None and recv_w is None
        # cached dispatch of another payload through the same handle (test_intranode.py:164-172)
        g = torch.Generator().manual_seed(3)
        x2 = torch.randn(c.x.shape, generator=g).to(torch.bfloat16)
        r2, none_idx, none_w, none_list, none_handle, _ = buf.dispatch(x2.cuda(), handle=handle, config=config)
        assert none_idx is None and none_list is None and none_handle is None
        assert_equal(r2.view(torch.int16), oracle.intranode_dispatch(x2, mask, None, None, c.E, c.R, rank, A, C).recv_x.view(torch.int16),
                     "cached recv_x")

    # combine: expert outputs = received rows (dequantised if FP8) scaled a little per row
    rows = oracle.per_token_cast_back(ref.recv_x, ref.recv_x_scales) if fp8 else ref.recv_x
    scale = 1 + (torch.arange(n) % 7).float().unsqueeze(1) / 16
    y = (rows.float() * scale).to(torch.bfloat16)
    g = torch.Generator().manual_seed(4)
    biases = (None, torch.randn(c.x.shape, generator=g).to(torch.bfloat16),
              (torch.randn(c.x.shape, generator=g).to(torch.bfloat16), torch.randn(c.x.shape, generator=g).to(torch.bfloat16)))
    for bias in biases:
        bias_d = None if bias is None else bias.cuda() if isinstance(bias, torch.Tensor) else tuple(b.cuda() for b in bias)
        w_in = ref.recv_topk_weights if with_topk else None
        out, out_w, _ = buf.combine(y.cuda(), handle, topk_weights=None if w_in is None else w_in.cuda(), bias=bias_d,
                                    config=config)
        ref_out, ref_w = oracle.intranode_combine(y, ref.send_head, w_in, bias)
        assert_equal(out + 0.0, ref_out + 0.0, "combined_x")
        if with_topk:
            assert_equal(out_w, ref_w, "combined_topk_weights")
        else:
            assert out_w is None
    buf.runtime.check_device_status("intranode")


def test_reference_round_trip_property_at_headline_shape():
    """Dispatch then combine returns x times the number of destination ranks (test_intranode.py:178-186), at
    T=8192, H=7168, 256 experts, 8 ranks, top-8."""
    import deep_ep
    c = rc.uniform_topk_case("C3", 8192, 7168, 256, 8, 8, 0)
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(0, c.R))
    idx_d, x_d, w_d = c.topk_idx.cuda(), c.x.cuda(), c.topk_weights.cuda()
    per_rank, _, per_expert, mask_d, _ = buf.get_dispatch_layout(idx_d, c.E)
    recv_x, recv_idx, recv_w, lst, handle, _ = buf.dispatch(x_d, num_tokens_per_rank=per_rank, is_token_in_rank=mask_d,
                                                           num_tokens_per_expert=per_expert, topk_idx=idx_d, topk_weights=w_d)
    assert recv_x.shape[0] == int(per_rank.sum())
    assert lst == per_expert.tolist()
    out, out_w, _ = buf.combine(recv_x, handle, topk_weights=recv_w)
    n = mask_d.sum(dim=1, keepdim=True).float()
    # n identical bf16 values summed in fp32 and rounded once
    assert torch.equal(out.float(), (x_d.float() * n).to(torch.bfloat16).float())
    assert torch.equal(out_w, w_d)
    buf.runtime.check_device_status("intranode")


def test_argument_errors():
    import deep_ep
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(0, 2))
    x = torch.zeros((4, 64), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((4, 2), dtype=torch.int64, device="cuda")
    per_rank, _, per_expert, mask, _ = buf.get_dispatch_layout(idx, 4)
    with pytest.raises(RuntimeError):
        buf.dispatch(x, num_tokens_per_rank=per_rank, is_token_in_rank=mask, num_tokens_per_expert=per_expert,
                     topk_idx=idx)                                         # weights missing
    with pytest.raises(RuntimeError):
        buf.dispatch(x, num_tokens_per_rank=per_rank, is_token_in_rank=mask[:, :1].contiguous(),
                     num_tokens_per_expert=per_expert)                      # mask of the wrong shape
    with pytest.raises(RuntimeError):
        buf.dispatch(x, num_tokens_per_rank=per_rank, is_token_in_rank=mask, num_tokens_per_expert=per_expert,
                     config=deep_ep.Config(7, 6, 256))                      # odd num_sms


def test_empty_inputs():
    """No tokens at all, and tokens that go nowhere (every top-k slot masked)."""
    import deep_ep
    R, E, K, H = 4, 16, 3, 256
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(1, R))
    for T, fill in ((0, 0), (5, -1)):
        x = torch.randn((T, H), device="cuda").to(torch.bfloat16)
        idx = torch.full((T, K), fill, dtype=torch.int64, device="cuda")
        w = torch.rand((T, K), device="cuda")
        per_rank, _, per_expert, mask, _ = buf.get_dispatch_layout(idx, E)
        assert int(per_rank.sum()) == 0 and int(per_expert.sum()) == 0 and mask.shape == (T, R) and not bool(mask.any())
        recv_x, recv_idx, recv_w, lst, handle, _ = buf.dispatch(x, num_tokens_per_rank=per_rank, is_token_in_rank=mask,
                                                               num_tokens_per_expert=per_expert, topk_idx=idx, topk_weights=w)
        assert recv_x.shape == (0, H) and recv_idx.shape == (0, K) and recv_w.shape == (0, K) and lst == [0] * E
        assert int(handle[0].abs().sum()) == 0 and handle[5].shape == (T, R) and bool((handle[5] == -1).all())
        out, out_w, _ = buf.combine(recv_x, handle, topk_weights=recv_w)
        assert out.shape == (T, H) and bool((out == 0).all()) and bool((out_w == 0).all())
    buf.runtime.check_device_status("intranode")


def test_per_source_calls_compose_into_the_world():
    """One call per logical source rank; the slices of every destination, stacked in source order, are what that
    destination holds in a real R-rank run (rows, local ids, weights, source indices, rank_prefix_matrix)."""
    import deep_ep
    R, T, H, E, K = 4, 300, 256, 32, 5
    g = torch.Generator().manual_seed(77)
    xs, idxs, ws, masks = [], [], [], []
    for r in range(R):
        n = T - 17 * r
        xs.append(torch.randn((n, H), generator=g).to(torch.bfloat16))
        scores = torch.rand((n, E), generator=g)
        idx = torch.topk(scores, K, dim=-1, sorted=False)[1].to(torch.int64)
        idxs.append(idx.masked_fill(torch.rand(idx.shape, generator=g) < 0.15, -1))
        ws.append(torch.rand((n, K), generator=g))
        masks.append(oracle.layout(idxs[-1], E, R)[2])
    world, _ = oracle.intranode_world_dispatch(xs, masks, idxs, ws, E, 1, num_channels=10)
    parts = [[] for _ in range(R)]
    prefix_sum = torch.zeros((R, R), dtype=torch.int32)
    for r in range(R):
        buf = deep_ep.Buffer(deep_ep.LogicalGroup(r, R))
        idx_d = idxs[r].cuda()
        per_rank, _, per_expert, mask_d, _ = buf.get_dispatch_layout(idx_d, E)
        recv_x, recv_idx, recv_w, _, handle, _ = buf.dispatch(
            xs[r].cuda(), num_tokens_per_rank=per_rank, is_token_in_rank=mask_d, num_tokens_per_expert=per_expert,
            topk_idx=idx_d, topk_weights=ws[r].cuda())
        counts = per_rank.cpu()
        starts = counts.cumsum(0) - counts
        for j in range(R):
            lo, hi = int(starts[j]), int(starts[j] + counts[j])
            parts[j].append((recv_x[lo:hi].cpu(), recv_idx[lo:hi].cpu(), recv_w[lo:hi].cpu(), handle[3][lo:hi].cpu()))
        prefix_sum += handle[0].cpu()
    for j in range(R):
        assert_equal(torch.cat([p[0] for p in parts[j]]), world[j].recv_x, f"recv_x of rank {j}")
        assert_equal(torch.cat([p[1] for p in parts[j]]), world[j].recv_topk_idx, f"recv_topk_idx of rank {j}")
        assert_equal(torch.cat([p[2] for p in parts[j]]), world[j].recv_topk_weights, f"recv_topk_weights of rank {j}")
        assert_equal(torch.cat([p[3] for p in parts[j]]), world[j].recv_src_idx, f"recv_src_idx of rank {j}")
    assert_equal(prefix_sum, world[0].rank_prefix_matrix, "rank_prefix_matrix summed over the calls")
