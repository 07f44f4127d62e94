"""Low-latency dispatch and combine with ragged sources through the C ABI: `num_tokens_per_src[s]` tokens of source rank
s are live, the rest of its `src_token_stride` slots hold garbage that must not reach the packed buffers.  Both kernel
paths (the single kernel for decode sizes, count + move kernels beyond) against the oracle, which takes the sources as a
list of tensors of different lengths."""
import ctypes

import pytest
import torch

import routing_cases as rc
from oracle import routing_oracle as oracle

pytestmark = pytest.mark.gpu


def _ragged_case(R, stride, counts, H, E, K, seed):
    x, idx, w = rc.c5_sources(seed=seed, R=R, T=stride, H=H, E=E, K=K)
    g = torch.Generator().manual_seed(seed + 1)
    idx = idx.masked_fill(torch.rand(idx.shape, generator=g) < 0.1, -1)
    return x, idx, w, [int(c) for c in counts]


@pytest.mark.parametrize("R,stride,counts,H,E,K,M,use_fp8", [
    (4, 128, (128, 0, 77, 1), 1024, 32, 8, 128, True),             # single kernel, even top-k
    (4, 100, (3, 100, 64, 65), 512, 16, 3, 100, False),            # single kernel, odd top-k, BF16
    (8, 250, (250, 249, 0, 0, 130, 1, 64, 200), 256, 64, 6, 252, True),   # 2000 slots: two words per source boundary
    (2, 1500, (1499, 700), 256, 16, 4, 1500, True),                # single kernel, several work items per wavefront
    (2, 2200, (2199, 900), 256, 16, 4, 2200, True),                # count + move kernels
], ids=["k8", "k3_bf16", "eight_sources", "several_items", "two_kernels"])
def test_ragged_sources_match_the_oracle(R, stride, counts, H, E, K, M, use_fp8):
    from deep_ep import _abi
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    dst = R - 1
    E_l, rows = E // R, R * M
    x, idx, w, counts = _ragged_case(R, stride, counts, H, E, K, seed=31)
    xs = [x[s, :counts[s]] for s in range(R)]           # an empty source sends nothing and still gets a (begin, 0) range
    idxs = [idx[s, :counts[s]] for s in range(R)]
    ref_x, ref_s, ref_cnt, ref_info, ref_range = oracle.ll_dispatch(xs, idxs, M, E, R, dst, use_fp8)

    xd, wd = x.to(dev), w.to(dev)
    # in two of the cases the index table sits 8 bytes off a 16-byte boundary: such a table takes the two-kernel path
    off_boundary = K in (3, 6)
    idx_store = torch.empty(idx.numel() + 2, dtype=torch.int64, device=dev)
    first = 1 if (idx_store.data_ptr() % 16 == 0) == off_boundary else 0
    idxd = idx_store[first:first + idx.numel()].view(idx.shape)
    idxd.copy_(idx)
    assert (idxd.data_ptr() % 16 != 0) == off_boundary
    n_src = torch.tensor(counts, dtype=torch.int32, device=dev)
    px = torch.full((E_l, rows, H), 0, dtype=torch.uint8 if use_fp8 else torch.bfloat16, device=dev)
    ps = torch.zeros((E_l, H // 128, rows), dtype=torch.float32, device=dev)
    cnt = torch.full((E_l,), -7, dtype=torch.int32, device=dev)
    info = torch.full((E_l, rows), -7, dtype=torch.int32, device=dev)
    rng = torch.full((E_l, R), -7, dtype=torch.int64, device=dev)
    lane_rows = torch.full((R * stride, K), -7, dtype=torch.int32, device=dev)
    ws = torch.zeros(max(_abi.lib.deep_ep_hip_ll_workspace_bytes(R, stride, K, E_l), 4096), dtype=torch.uint8, device=dev)
    d = _abi.LLDispatchArgs()
    d.use_fp8, d.num_src_ranks, d.src_rank_begin, d.src_token_stride = int(use_fp8), R, 0, stride
    d.num_tokens_per_src = n_src.data_ptr()
    d.hidden, d.num_topk, d.num_experts, d.expert_begin, d.num_local_experts = H, K, E, dst * E_l, E_l
    d.num_ranks, d.num_max_dispatch_tokens_per_rank = R, M
    d.x, d.topk_idx = xd.data_ptr(), idxd.data_ptr()
    d.packed_recv_x, d.packed_recv_x_scales, d.packed_recv_count = px.data_ptr(), ps.data_ptr() if use_fp8 else None, cnt.data_ptr()
    d.packed_recv_src_info, d.packed_recv_layout_range = info.data_ptr(), rng.data_ptr()
    d.lane_rows = lane_rows.data_ptr()
    d.workspace, d.workspace_bytes = ws.data_ptr(), ws.numel()
    stream = torch.cuda.current_stream().cuda_stream
    _abi.check(_abi.lib.deep_ep_hip_launch_ll_dispatch(ctypes.byref(d), stream), "ragged dispatch")
    torch.cuda.synchronize()
    assert int(ws[:4].view(torch.int32).item()) == 0
    assert torch.equal(cnt.cpu(), ref_cnt)
    assert torch.equal(rng.cpu(), ref_range)
    got_x = px.cpu().view(torch.float8_e4m3fn) if use_fp8 else px.cpu()
    for le in range(E_l):
        n = int(ref_cnt[le])
        assert torch.equal(info.cpu()[le, :n], ref_info[le, :n]), f"src_info of expert {le}"
        assert torch.equal(got_x[le, :n].view(torch.uint8), ref_x[le, :n].view(torch.uint8)), f"payload of expert {le}"
        if use_fp8:
            assert torch.equal(ps.cpu().transpose(1, 2)[le, :n], ref_s[le, :n]), f"scales of expert {le}"

    # combine back: expert outputs = a deterministic function of the packed rows
    y = torch.zeros((E_l, rows, H), dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(77)
    for le in range(E_l):
        n = int(ref_cnt[le])
        y[le, :n] = torch.randn((n, H), generator=g).to(torch.bfloat16)
    for use_recorded_rows in (True, False):
        out = torch.full((R * stride, H), 3.0, dtype=torch.bfloat16, device=dev)
        c = _abi.LLCombineArgs()
        c.num_src_ranks, c.src_rank_begin, c.src_token_stride, c.use_logfmt = R, 0, stride, 0
        c.num_tokens_per_src = n_src.data_ptr()
        c.hidden, c.num_topk, c.num_experts, c.expert_begin, c.num_local_experts, c.num_ranks = H, K, E, dst * E_l, E_l, R
        c.num_max_dispatch_tokens_per_rank = M
        yd = y.to(dev)
        c.x, c.topk_idx, c.topk_weights = yd.data_ptr(), idxd.data_ptr(), wd.data_ptr()
        c.packed_recv_src_info, c.packed_recv_layout_range = info.data_ptr(), rng.data_ptr()
        c.lane_rows = lane_rows.data_ptr() if use_recorded_rows else None
        c.combined_x = out.data_ptr()
        c.workspace, c.workspace_bytes = ws.data_ptr(), ws.numel()
        _abi.check(_abi.lib.deep_ep_hip_launch_ll_combine(ctypes.byref(c), stream), "ragged combine")
        torch.cuda.synchronize()
        got = out.cpu().view(R, stride, H)
        for s in range(R):
            if counts[s] == 0:
                continue
            want = oracle.ll_combine(y, idx[s, :counts[s]], w[s, :counts[s]], ref_info, ref_range, s, E, R, dst)
            assert torch.equal((got[s, :counts[s]].float() + 0.0), (want.float() + 0.0)), f"combined rows of source {s}"
            # slots past a source's count are not written
            assert bool((got[s, counts[s]:] == 3.0).all()), f"source {s}: a slot past its count was written"
