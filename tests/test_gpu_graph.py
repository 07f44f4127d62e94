"""The no-host-sync dispatch + combine sequence captured in a HIP graph and replayed: every replay must equal the
eager result on the same inputs (the reference advertises its worst-case-sized mode as graph compatible,
deep_ep/buffers/legacy.py:352-354, deep_ep/buffers/elastic.py:1437-1441)."""
import pytest
import torch

import routing_cases as rc
from test_gpu_parity import _buffer

pytestmark = pytest.mark.gpu


def _step(buf, x, idx, w, E, fp8):
    recv, recv_idx, recv_w, handle, _ = buf.dispatch(x, idx, w, num_experts=E, do_cpu_sync=False, cast_to_fp8=fp8)
    if fp8:
        q, sf = recv
        y = (q.float().view(q.shape[0], -1, 128) * sf.unsqueeze(2)).view(q.shape).to(torch.bfloat16)
    else:
        y = recv
    out, out_w, _ = buf.combine(y, handle, topk_weights=recv_w)
    return recv, recv_idx, handle.psum_num_recv_tokens_per_scaleup_rank, out, out_w


@pytest.mark.parametrize("fp8", [False, True])
def test_graph_replays_match_eager(fp8):
    cases = [rc.small("g0", 1500, 1024, 64, 8, 6, seed=20, masked_ratio=0.1),
             rc.small("g1", 1500, 1024, 64, 8, 6, seed=21, masked_ratio=0.3),
             rc.small("g2", 1500, 1024, 64, 8, 6, seed=22)]
    c0 = cases[0]
    buf = _buffer(c0)
    x_s, idx_s, w_s = c0.x.cuda(), c0.topk_idx.cuda(), c0.topk_weights.cuda()
    _step(buf, x_s, idx_s, w_s, c0.E, fp8)                      # warm-up: workspace allocation happens here
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_recv, g_idx, g_psum, g_out, g_w = _step(buf, x_s, idx_s, w_s, c0.E, fp8)

    for case in cases + cases[:1]:
        x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
        e_recv, e_idx, e_psum, e_out, e_w = _step(buf, x, idx, w, case.E, fp8)      # eager, its own tensors
        torch.cuda.synchronize()
        x_s.copy_(x); idx_s.copy_(idx); w_s.copy_(w)
        graph.replay()
        torch.cuda.synchronize()
        n = int(e_psum[-1])
        assert torch.equal(g_psum, e_psum)
        assert torch.equal(g_idx[:n], e_idx[:n])
        if fp8:
            assert torch.equal(g_recv[0][:n].view(torch.uint8), e_recv[0][:n].view(torch.uint8))
            assert torch.equal(g_recv[1][:n], e_recv[1][:n])
        else:
            assert torch.equal(g_recv[:n].view(torch.int16), e_recv[:n].view(torch.int16))
        assert torch.equal(g_out.view(torch.int16), e_out.view(torch.int16))
        assert torch.equal(g_w, e_w)
    buf.check_device_status()


def test_low_latency_graph_replays_match_eager():
    """The decode loop is launch bound (two ~10 us kernels per step): captured once, replayed per step."""
    import deep_ep
    R, T, H, E, K, M = 8, 128, 2048, 64, 4, 128
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(3, R), low_latency_mode=True)
    sets = [rc.c5_sources(seed=s, R=R, T=T, H=H, E=E, K=K) for s in (30, 31, 32)]
    x_s, idx_s, w_s = (t.cuda() for t in sets[0])

    def step(x, idx, w):
        recv, count, handle, _, _ = buf.low_latency_dispatch(x, idx, M, E, use_fp8=True)
        q, sf = recv
        y = (q.float().view(*q.shape[:2], -1, 128) * sf.unsqueeze(3)).view(q.shape).to(torch.bfloat16)
        out, _, _ = buf.low_latency_combine(y, idx, w, handle)
        return count, handle[1], out

    step(x_s, idx_s, w_s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_count, g_range, g_out = step(x_s, idx_s, w_s)
    for x, idx, w in sets + sets[:1]:
        x, idx, w = x.cuda(), idx.cuda(), w.cuda()
        e_count, e_range, e_out = step(x, idx, w)
        torch.cuda.synchronize()
        x_s.copy_(x); idx_s.copy_(idx); w_s.copy_(w)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_count, e_count)
        assert torch.equal(g_range, e_range)
        assert torch.equal(g_out.view(torch.int16), e_out.view(torch.int16))
