"""The reference's literal two-rank cases and known answers, through the HIP path (C ABI via deep_ep)."""
import pytest
import torch

import routing_oracle as oracle
import world
from test_gpu_parity import assert_equal
from test_oracle_routing import contribution

pytestmark = pytest.mark.gpu

G = world.load_golden()
E, R, H, M = G["num_experts"], G["num_ranks"], G["hidden"], G["capacity"]


def _buffer(multi_red=True):
    import deep_ep
    # the whole world in one call: source rank 0 with capacity R*M (see tests/world.py)
    return deep_ep.ElasticBuffer(deep_ep.LogicalGroup(0, R), num_max_tokens_per_rank=R * M, hidden=8, num_topk=2,
                                 allow_multiple_reduction=multi_red)


@pytest.mark.parametrize("name", list(G["dispatch_cases"]))
def test_literal_dispatch_cases(name):
    case = G["dispatch_cases"][name]
    K = len(case["routes"][1][0]) if case["routes"][1] else 2
    # rows must be multiples of 16 bytes: the 4 literal channels are repeated twice (hidden 8)
    x4, idx, w = world.stack_world(case["payloads"], case["routes"], case.get("weights"), M, H, K)
    x = torch.cat([x4, x4], dim=1).contiguous()
    counts = [len(r) for r in case["routes"]]
    do_expand = case.get("do_expand", False)
    A = case.get("expert_alignment", 1)
    buf = _buffer()
    recv_x, recv_idx, recv_w, handle, _ = buf.dispatch(x.cuda(), idx.cuda(), None if w is None else w.cuda(), num_experts=E,
                                                       expert_alignment=A, do_expand=do_expand,
                                                       do_zero_padding=case.get("do_zero_padding", False))
    ref = oracle.dispatch(x, idx, w, E, R, 0, R * M, expert_alignment=A, do_expand=do_expand)
    assert_equal(recv_x, ref.recv_x, "recv_x")
    assert (recv_w is None) == (w is None)
    if w is not None:
        assert_equal(recv_w, ref.recv_topk_weights, "recv_topk_weights")
    assert_equal(handle.recv_src_metadata, ref.recv_src_metadata, "recv_src_metadata")
    assert_equal(handle.dst_buffer_slot_idx, ref.dst_buffer_slot_idx, "dst_buffer_slot_idx")
    assert handle.num_recv_tokens_per_expert_list == ref.num_recv_tokens_per_expert_list
    if not do_expand:
        # per destination rank: exactly what the restated refs.dispatch says that rank receives
        xs, idxs, ws = world.per_source(x, idx, w if w is not None else torch.zeros(idx.shape), M, R, counts)
        per_dst = oracle.world_dispatch(xs, idxs, ws, M, E)
        for d, (lo, hi) in enumerate(world.bucket_bounds(handle.psum_num_recv_tokens_per_scaleup_rank.cpu())):
            rx, ridx, rw, rsrc, _ = per_dst[d]
            assert_equal(recv_x[lo:hi], rx, f"rank {d} recv_x")
            assert_equal(recv_idx[lo:hi], ridx, f"rank {d} recv_topk_idx")
            assert_equal(handle.recv_src_metadata[lo:hi, 0], rsrc, f"rank {d} source indices")
    if "expected_layout" in case:
        per = E // R
        for d in range(R):
            aligned = handle.num_recv_tokens_per_expert_list[d * per:(d + 1) * per]
            actual = handle.num_unaligned_recv_tokens_per_expert.cpu()[d * per:(d + 1) * per].tolist()
            assert sum(aligned) == case["expected_layout"][f"rank{d}"]["rows"]
            assert sum(aligned) - sum(actual) == case["expected_layout"][f"rank{d}"]["padding"]
    buf.check_device_status()


def _combine_world(routes, K, do_expand, multi_red, variant=None, weights=None, biases=None):
    buf = _buffer(multi_red)
    _, idx, w = world.stack_world(None, routes, weights, M, H, K)
    x = torch.zeros((R * M, 8), dtype=torch.bfloat16)
    _, _, recv_w, handle, _ = buf.dispatch(x.cuda(), idx.cuda(), None if w is None else w.cuda(), num_experts=E, do_expand=do_expand)
    meta = handle.recv_src_metadata.cpu()
    per = E // R
    rows = handle.num_expanded_tokens if do_expand else handle.num_recv_tokens
    y = torch.zeros((rows, 8), dtype=torch.bfloat16)
    if do_expand:
        for i in range(handle.num_recv_tokens):
            g = int(meta[i, 0])
            for k in range(K):
                row = int(meta[i, 2 + k])
                if row >= 0:
                    y[row, :4] = torch.tensor(contribution(g // M, g % M, k, variant)).to(torch.bfloat16)
    else:
        for d, (lo, hi) in enumerate(world.bucket_bounds(handle.psum_num_recv_tokens_per_scaleup_rank.cpu())):
            for i in range(lo, hi):
                g = int(meta[i, 0])
                acc = torch.zeros(4)
                for k in range(K):
                    e = int(idx[g, k])
                    if e >= 0 and e // per == d:
                        acc = acc + torch.tensor(contribution(g // M, g % M, k, variant))
                y[i, :4] = acc.to(torch.bfloat16)
    bias = None
    if biases is not None:
        bs = tuple(torch.tensor(b + b, dtype=torch.float32).to(torch.bfloat16).expand(R * M, 8).contiguous().cuda() for b in biases)
        bias = bs[0] if len(bs) == 1 else bs
    out, out_w, _ = buf.combine(y.cuda(), handle, topk_weights=recv_w, bias=bias)
    buf.check_device_status()
    return out.cpu().float()[:, :4], None if out_w is None else out_w.cpu()


def test_combine_known_answers():
    fx = G["combine"]["reference_fixture"]
    for do_expand, multi in ((False, True), (True, True), (True, False)):
        out, _ = _combine_world(fx["routes"], 2, do_expand, multi)
        assert out[0:2].tolist() == fx["expected"]["rank0"] and out[M:M + 1].tolist() == fx["expected"]["rank1"]
    fx = G["combine"]["ordering"]
    out, _ = _combine_world([[fx["route"]], []], 3, True, False, variant=fx["lane_columns"])
    assert out[0].tolist() == fx["canonical"]
    fx = G["combine"]["weight_bias"]
    out, out_w = _combine_world([fx["weight_route"], []], 2, False, True, weights=[fx["weights"], []])
    assert out[0].tolist() == fx["activation_ignores_weight"] and out_w[0].tolist() == fx["restored_weights"]
    out, _ = _combine_world([fx["bias_route"], []], 2, False, True, biases=fx["biases"])
    assert out[0].tolist() == fx["bias_once"]
    out, _ = _combine_world([[[-1, -1]], []], 2, False, True, biases=fx["biases"])
    assert out[0].tolist() == [5.0] * 4
    fx = G["combine"]["bf16_reduction"]          # 301 and 302 become bf16 (300, 302) before the fp32 sum: 602 -> 600
    import deep_ep
    buf = deep_ep.ElasticBuffer(deep_ep.LogicalGroup(0, 2), num_max_tokens_per_rank=4, hidden=8, num_topk=2)
    idx = torch.tensor([[0, 2]], dtype=torch.int64).cuda()
    _, _, _, handle, _ = buf.dispatch(torch.zeros((1, 8), dtype=torch.bfloat16).cuda(), idx, None, num_experts=4)
    y = torch.tensor(fx["contributions"]).to(torch.bfloat16).view(2, 1).expand(2, 8).contiguous()
    out, _, _ = buf.combine(y.cuda(), handle)
    assert out.cpu().float()[0].tolist() == [fx["expected"]] * 8


@pytest.mark.parametrize("name", list(G["cached_cases"]))
def test_cached_handle_moves_a_changed_payload(name):
    """The reference's cached cases: a second dispatch through the first call's handle, with every payload value
    raised by 300 and every weight negated, must route the new values exactly as the first call routed the old."""
    case = G["cached_cases"][name]
    K = len(case["routes"][0][0])
    do_expand, A = case.get("do_expand", False), case.get("expert_alignment", 1)
    zero_pad = case.get("do_zero_padding", False)
    buf = _buffer()

    def stacked(payloads, weights):
        x4, idx, w = world.stack_world(payloads, case["routes"], weights, M, H, K)
        return torch.cat([x4, x4], dim=1).contiguous(), idx, w

    x1, idx, w1 = stacked(case["payloads"], case["weights"])
    x2, _, w2 = stacked(case["second_payloads"], case["second_weights"])
    first_x, _, first_w, handle, _ = buf.dispatch(x1.cuda(), idx.cuda(), w1.cuda(), num_experts=E, expert_alignment=A,
                                                  do_expand=do_expand, do_zero_padding=zero_pad)
    recv_x, recv_idx, recv_w, same, _ = buf.dispatch(x2.cuda(), topk_weights=w2.cuda(), handle=handle, do_expand=do_expand,
                                                     do_zero_padding=zero_pad)
    assert same is handle, "the cached dispatch replaced its handle"
    for x, w, got_x, got_w in ((x1, w1, first_x, first_w), (x2, w2, recv_x, recv_w)):
        ref = oracle.dispatch(x, idx, w, E, R, 0, R * M, expert_alignment=A, do_expand=do_expand)
        n = ref.num_expanded_tokens if do_expand else ref.num_recv_tokens
        assert_equal(got_x[:n], ref.recv_x, "recv_x")                       # zero padding: padding rows are zero in both
        assert_equal(got_w[:n], ref.recv_topk_weights, "recv_topk_weights")
    assert not torch.equal(first_x.cpu(), recv_x.cpu()[:first_x.shape[0]]), "the cached dispatch ignored the new payload"
    assert not torch.equal(first_w.cpu(), recv_w.cpu()[:first_w.shape[0]]), "the cached dispatch ignored the new weights"
    if do_expand:
        # rank 0 hosts experts 0 and 1: 5 + 1 rows padded to 8 + 4; rank 1 hosts 2 and 3: 1 + 1 rows padded to 4 + 4
        assert handle.num_recv_tokens_per_expert_list == [8, 4, 4, 4]
    buf.check_device_status()
