"""Pins the oracle's V1 (intranode) dispatch / combine: the assertions of the reference's own test
(tests/legacy/test_intranode.py:90-186) replayed on a whole logical world built on the CPU, plus loop restatements
on small inputs and the composition of per-source shares into the world."""
import pytest
import torch

import routing_oracle as oracle


def _world(R, T, H, E, K, seed, masked=0.1):
    g = torch.Generator().manual_seed(seed)
    xs, idxs, ws, masks = [], [], [], []
    for r in range(R):
        n = max(1, T - r)                                   # ragged, like the reference's benchmark manifest
        xs.append(torch.full((n, H), float(r), dtype=torch.bfloat16))
        scores = torch.randn((n, E), generator=g).abs() + 1
        idx = torch.topk(scores, K, dim=-1, largest=True, sorted=False)[1].to(torch.int64)
        idx = idx.masked_fill(torch.rand(idx.shape, generator=g) < masked, -1)
        idxs.append(idx)
        ws.append(torch.full((n, K), float(r), dtype=torch.float32))
        masks.append(oracle.layout(idx, E, R)[2])
    return xs, idxs, ws, masks


@pytest.mark.parametrize("R,T,H,E,K,A", [(2, 9, 16, 4, 2, 1), (4, 50, 32, 16, 4, 4), (8, 130, 64, 64, 8, 1)])
def test_world_satisfies_the_reference_tests_assertions(R, T, H, E, K, A):
    xs, idxs, ws, masks = _world(R, T, H, E, K, seed=R)
    world, channel_prefix = oracle.intranode_world_dispatch(xs, masks, idxs, ws, E, A, num_channels=6)
    gbl_per_rank = torch.stack([m.sum(0) for m in masks]).sum(0)
    gbl_per_expert = torch.stack([(torch.cat([i.flatten() for i in idxs]) == e).sum() for e in range(E)])
    E_l = E // R
    for rank, recv in enumerate(world):
        # test_intranode.py:124-131 (sizes, per-expert list, constant rows per source segment)
        assert recv.recv_x.shape[0] == int(gbl_per_rank[rank])
        expect = [(int(c) + A - 1) // A * A for c in gbl_per_expert.view(R, -1)[rank]]
        assert recv.num_recv_tokens_per_expert_list == expect
        start = 0
        for i in range(R):
            end = int(recv.rank_prefix_matrix[i][rank])
            assert (recv.recv_x[start:end].float() == i).all()
            start = end
        assert start == recv.recv_x.shape[0]
        # :134-139 (local ids in range, counts per local expert)
        ids = recv.recv_topk_idx
        assert ((ids == -1) | ((ids >= 0) & (ids < E_l))).all()
        for e in range(E_l):
            assert int((ids == e).sum()) == int(gbl_per_expert[rank * E_l + e])
        # :141-146 (weights: constant per source once the -1 lanes are filled with the row maximum)
        wts = recv.recv_topk_weights.clone()
        assert (wts[ids == -1] == 0).all()
        wts[ids == -1] = wts.amax(dim=1, keepdim=True).expand_as(wts)[ids == -1]
        start = 0
        for i in range(R):
            end = int(recv.rank_prefix_matrix[i][rank])
            assert (wts[start:end] == i).all()
            start = end
        # receive-side channel starts are the senders' exclusive channel prefixes
        for i in range(R):
            assert int(recv.recv_channel_prefix_matrix[i][0]) == 0
            assert torch.equal(recv.recv_channel_prefix_matrix[i][1:], channel_prefix[i][rank][:-1])
            assert int(channel_prefix[i][rank][-1]) == int(masks[i][:, rank].sum())


@pytest.mark.parametrize("R,T,H,E,K", [(2, 7, 8, 4, 2), (4, 33, 16, 8, 3)])
def test_shares_compose_into_the_world_and_combine_restores_the_tokens(R, T, H, E, K):
    xs, idxs, ws, masks = _world(R, T, H, E, K, seed=10 + R)
    g = torch.Generator().manual_seed(1)
    xs = [torch.randn(x.shape, generator=g).to(torch.bfloat16) for x in xs]
    ws = [torch.randn(w.shape, generator=g) for w in ws]
    world, _ = oracle.intranode_world_dispatch(xs, masks, idxs, ws, E, 1, num_channels=4)
    shares = [oracle.intranode_dispatch(xs[r], masks[r], idxs[r], ws[r], E, R, r, 1, 4) for r in range(R)]
    for j in range(R):
        parts_x, parts_idx, parts_w, parts_src = [], [], [], []
        for r in range(R):
            last = shares[r].rank_prefix_matrix[-1]
            lo = int(last[:j].sum())
            hi = lo + int(last[j])
            parts_x.append(shares[r].recv_x[lo:hi])
            parts_idx.append(shares[r].recv_topk_idx[lo:hi])
            parts_w.append(shares[r].recv_topk_weights[lo:hi])
            parts_src.append(shares[r].recv_src_idx[lo:hi])
        assert torch.equal(torch.cat(parts_x), world[j].recv_x)
        assert torch.equal(torch.cat(parts_idx), world[j].recv_topk_idx)
        assert torch.equal(torch.cat(parts_w), world[j].recv_topk_weights)
        assert torch.equal(torch.cat(parts_src), world[j].recv_src_idx)
        assert torch.equal(sum(s.rank_prefix_matrix for s in shares), world[j].rank_prefix_matrix)
    # send_head restated with loops; combine of the dispatched rows = x times the number of destination ranks
    # (test_intranode.py:178-186), weights come back once per lane
    for r in range(R):
        sh = shares[r]
        row = 0
        for j in range(R):
            for t in range(xs[r].shape[0]):
                if masks[r][t, j]:
                    assert int(sh.send_head[t, j]) == row and int(sh.recv_src_idx[row]) == t
                    row += 1
                else:
                    assert int(sh.send_head[t, j]) == -1
        out, w_out = oracle.intranode_combine(sh.recv_x, sh.send_head, sh.recv_topk_weights)
        n = masks[r].sum(dim=1, keepdim=True)
        ref = torch.zeros_like(out, dtype=torch.float32)
        for t in range(xs[r].shape[0]):
            acc = torch.zeros(H)
            for _ in range(int(n[t])):
                acc = acc + xs[r][t].float()
            ref[t] = acc
        assert torch.equal(out.float() + 0.0, ref.to(torch.bfloat16).float() + 0.0)
        assert torch.equal(w_out, torch.where(idxs[r] >= 0, ws[r], torch.zeros_like(ws[r])))


def test_combine_adds_biases_first_and_ranks_in_ascending_order():
    big = float(2 ** 24)
    x = torch.tensor([[big], [-big], [1.0]], dtype=torch.bfloat16)            # rows of ranks 0, 1, 2
    head = torch.tensor([[0, 1, 2]], dtype=torch.int32)
    out, _ = oracle.intranode_combine(x, head)
    assert float(out[0, 0]) == 1.0                                            # (big - big) + 1
    head = torch.tensor([[0, 2, 1]], dtype=torch.int32)                       # rank 1 holds the 1.0, rank 2 holds -big
    out, _ = oracle.intranode_combine(x, head)
    assert float(out[0, 0]) == 0.0                                            # (big + 1) - big
    bias = (torch.tensor([[0.5]], dtype=torch.bfloat16), torch.tensor([[0.25]], dtype=torch.bfloat16))
    out, _ = oracle.intranode_combine(torch.tensor([[301.0], [302.0]], dtype=torch.bfloat16),
                                      torch.tensor([[0, 1]], dtype=torch.int32), bias=bias)
    assert float(out[0, 0]) == 604.0    # 301 is stored as 300 (tie to even); 0.75 + 300 + 302 = 602.75 -> 604 in bf16
