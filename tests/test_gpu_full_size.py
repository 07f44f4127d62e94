"""The benchmark's full-size workloads (T=8192, H=7168, 256 experts, 8 logical ranks, top-8; uniform and skewed/masked
routing) checked through properties that do not need the CPU oracle at that size: counts against closed forms,
permutation / sortedness of the received rows, payload bytes against the separately verified stand-alone cast,
localisation of the expert ids, and the dispatch -> combine round trip (the reference's own acceptance property,
tests/legacy/test_intranode.py:178-186, tests/elastic/test_ep.py:371-397).  A slice of rows is also compared with the
oracle."""
import pytest
import torch

import routing_cases as rc
import routing_oracle as oracle
from test_gpu_parity import _buffer, assert_equal

pytestmark = pytest.mark.gpu


def _closed_form_counts(idx, E, R):
    """Counts straight from their definitions with library routines on the device."""
    T, K = idx.shape
    valid = idx >= 0
    per_expert = torch.bincount(idx[valid], minlength=E)
    rank_of = torch.where(valid, idx // (E // R), torch.full_like(idx, R))
    in_rank = torch.zeros((T, R + 1), dtype=torch.bool, device=idx.device)
    in_rank.scatter_(1, rank_of, True)
    return per_expert.to(torch.int32), in_rank[:, :R]


@pytest.mark.parametrize("name", ["C3", "C4"])
def test_compact_fp8_dispatch_properties(name):
    case = rc.c3() if name == "C3" else rc.c4()
    T, H, E, R, K = case.T, case.H, case.E, case.R, case.K
    buf = _buffer(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    per_expert, in_rank = _closed_form_counts(idx, E, R)

    got_rank, _, got_expert, got_in_rank, _ = buf.get_dispatch_layout(idx, E)
    assert torch.equal(got_expert, per_expert)
    assert torch.equal(got_in_rank, in_rank)
    assert torch.equal(got_rank, in_rank.sum(0).to(torch.int32))

    (recv_x, recv_sf), recv_idx, recv_w, handle, _ = buf.dispatch(x, idx, w, num_experts=E, cast_to_fp8=True)
    n = int(in_rank.sum())
    assert handle.num_recv_tokens == n == recv_x.shape[0]
    psum = handle.psum_num_recv_tokens_per_scaleup_rank
    assert torch.equal(psum, in_rank.sum(0).cumsum(0).to(torch.int32))
    assert handle.num_recv_tokens_per_expert_list == per_expert.tolist()

    meta = handle.recv_src_metadata[:n]
    src = meta[:, 0].long()                                     # rank 0 sends: source index = token index
    starts = torch.cat([psum.new_zeros(1), psum[:-1]]).long()
    row_rank = torch.bucketize(torch.arange(n, device=src.device), psum.long(), right=True)
    # each (token, destination rank) pair exactly once, buckets in rank order, tokens ascending inside a bucket
    assert bool(in_rank[src, row_rank].all())
    keys = row_rank * T + src
    assert bool((keys[1:] > keys[:-1]).all())
    # handle: dst_buffer_slot_idx of a master lane names the row that holds the token
    slot = handle.dst_buffer_slot_idx
    lanes = (slot >= 0).nonzero()
    rows = starts[(idx[lanes[:, 0], lanes[:, 1]] // (E // R))] + slot[lanes[:, 0], lanes[:, 1]].long()
    assert torch.equal(src[rows], lanes[:, 0])
    assert rows.numel() == n and rows.unique().numel() == n
    assert torch.equal(meta[:, 1].long()[rows], lanes[:, 1])       # col 1 = master lane (source rank 0)

    # payload and scales: byte-identical to the stand-alone cast of the source rows (itself oracle-checked at small sizes)
    from deep_ep.utils.math import per_token_cast_to_fp8
    xq, xs = per_token_cast_to_fp8(x)
    assert torch.equal(recv_x.view(torch.uint8), xq.view(torch.uint8)[src])
    assert torch.equal(recv_sf.view(torch.int32), xs.view(torch.int32)[src])
    # a slice against the CPU oracle
    sample = torch.arange(0, T, 97)
    q_ref, s_ref = oracle.per_token_cast_to_fp8(case.x[sample])
    assert_equal(xq[sample.cuda()], q_ref, "cast payload sample")
    assert_equal(xs[sample.cuda()], s_ref, "cast scales sample")

    # expert ids: local to the row's rank or -1; weights copied
    src_idx = idx[src]
    local = (src_idx >= 0) & (src_idx // (E // R) == row_rank.unsqueeze(1))
    expect_idx = torch.where(local, src_idx - row_rank.unsqueeze(1) * (E // R), torch.full_like(src_idx, -1))
    assert torch.equal(recv_idx, expect_idx)
    assert torch.equal(recv_w, w[src])
    buf.check_device_status()


@pytest.mark.parametrize("name", ["C3", "C4"])
@pytest.mark.parametrize("do_expand", [False, True])
@pytest.mark.parametrize("launches", [0, 1], ids=["launches_by_choice", "one_launch"])
def test_bf16_round_trip(name, do_expand, launches, monkeypatch):
    """combine(dispatch(x)) = x summed once per destination row: n equal BF16 values added in fp32, rounded once.
    At this size the library's own choice is two launches for this payload; the single launch is forced as well."""
    import deep_ep
    monkeypatch.setattr(deep_ep.tuning, "dispatch_launches", launches)
    case = rc.c3() if name == "C3" else rc.c4()
    E, R = case.E, case.R
    buf = _buffer(case, allow_multiple_reduction=False)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    per_expert, in_rank = _closed_form_counts(idx, E, R)
    recv_x, recv_idx, recv_w, handle, _ = buf.dispatch(x, idx, w, num_experts=E, do_expand=do_expand,
                                                       expert_alignment=128 if do_expand else 1)
    if do_expand:
        aligned = (per_expert + 127) // 128 * 128
        assert handle.num_recv_tokens_per_expert_list == aligned.tolist()
        assert recv_x.shape[0] == int(aligned.sum())
        # rows of expert e are x rows of the tokens that chose e, in token order
        starts = aligned.cumsum(0) - aligned
        order = torch.argsort(torch.where(idx >= 0, idx, torch.full_like(idx, E)).flatten(), stable=True)
        order = order[: int(per_expert.sum())]
        tok = order // case.K
        e_sorted = idx.flatten()[order]
        within = torch.arange(order.numel(), device=x.device) - (per_expert.cumsum(0) - per_expert)[e_sorted]
        rows = starts[e_sorted] + within
        assert torch.equal(recv_x[rows].view(torch.int16), x[tok].view(torch.int16))
        assert torch.equal(recv_w[rows], w.flatten()[order])
        n_terms = (idx >= 0).sum(1, keepdim=True)
    else:
        n_terms = in_rank.sum(1, keepdim=True)
    out, out_w, _ = buf.combine(recv_x, handle, topk_weights=recv_w)
    expect = x.float()
    acc = torch.zeros_like(expect)
    for i in range(int(n_terms.max())):
        acc = torch.where(n_terms > i, acc + expect, acc)
    assert torch.equal((out + 0.0).view(torch.int16), (acc.to(torch.bfloat16) + 0.0).view(torch.int16))
    assert torch.equal(out_w, torch.where(idx >= 0, w, torch.zeros_like(w)))
    buf.check_device_status()


@pytest.mark.parametrize("name", ["C3", "C4"])
def test_combine_against_fp32_reference_within_one_bf16_ulp(name):
    """Random expert outputs at full size: the combined rows against an fp32 scatter-add done by the library
    (different accumulation order), tolerance = 1 BF16 ulp of the fp32 result (the tolerance stated for the path) plus fp32 reordering slack."""
    case = rc.c3() if name == "C3" else rc.c4()
    buf = _buffer(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    recv_x, recv_idx, recv_w, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E)
    n = handle.num_recv_tokens
    g = torch.Generator(device="cuda").manual_seed(5)
    y = torch.randn((n, case.H), generator=g, device="cuda").to(torch.bfloat16)
    bias = torch.randn((case.T, case.H), generator=g, device="cuda").to(torch.bfloat16)
    out, _, _ = buf.combine(y, handle, bias=bias)
    ref = bias.float()
    ref.index_add_(0, handle.recv_src_metadata[:n, 0].long(), y.float())
    ref_bf16 = ref.to(torch.bfloat16).float()
    # 1 BF16 ulp of the result (8 significant bits: 2^(exponent - 8) with frexp's exponent), plus the slack a
    # different fp32 summation order can cause where the terms cancel (2^-21 of the sum of magnitudes)
    ulp = torch.ldexp(torch.ones_like(ref_bf16), torch.frexp(ref_bf16)[1] - 8)
    magnitudes = bias.float().abs()
    magnitudes.index_add_(0, handle.recv_src_metadata[:n, 0].long(), y.float().abs())
    err = (out.float() - ref_bf16).abs()
    bound = ulp + magnitudes * 2.0 ** -21
    assert bool((err <= bound).all()), f"max error {float((err / bound).max()):.2f} of the bound"
    # and the great majority of elements agree exactly
    assert float((err == 0).float().mean()) > 0.98
