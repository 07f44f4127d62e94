"""`deep_ep_hip_launch_dispatch_static` (the dispatch whose workspace is a device array built into the library, for
callers that cannot allocate) against `deep_ep_hip_launch_dispatch` on the same inputs, through the C ABI: two calls in
a row, the second with a smaller input, bit for bit."""
import ctypes

import pytest
import torch

import routing_cases as rc

pytestmark = pytest.mark.gpu


def _dispatch(entry, case, expanded, workspace):
    from deep_ep import _abi
    dev = torch.device("cuda:0")
    T, H, K, E, R, M = case.T, case.H, case.K, case.E, case.R, case.M
    x, idx, w = case.x.to(dev), case.topk_idx.to(dev), case.topk_weights.to(dev)
    i32 = dict(dtype=torch.int32, device=dev)
    cap, ecap = M * R, M * min(K, E)
    rows = ecap if expanded else cap
    out = {
        "psum_rank": torch.zeros(R, **i32), "psum_expert": torch.zeros(E, **i32), "unaligned": torch.zeros(E, **i32),
        "slot": torch.full((T, K), -7, **i32), "meta": torch.full((cap, K + 2), -7, **i32),
        "recv_x": torch.zeros((rows, H), dtype=torch.uint8, device=dev),
        "recv_sf": torch.zeros((rows, H // 128), dtype=torch.float32, device=dev),
        "recv_idx": torch.full((cap, K), -7, dtype=torch.int64, device=dev),
        "recv_w": torch.zeros((rows,) if expanded else (cap, K), dtype=torch.float32, device=dev),
    }
    a = _abi.DispatchArgs()
    a.phases = _abi.PHASE_LAYOUT | _abi.PHASE_MOVE
    a.payload, a.do_expand = _abi.PAYLOAD_CAST_FP8, int(expanded)
    a.num_tokens, a.hidden, a.num_topk, a.num_experts, a.num_ranks = T, H, K, E, R
    a.rank_idx, a.num_max_tokens_per_rank, a.expert_alignment = 0, M, 1
    a.x, a.topk_idx, a.topk_weights = x.data_ptr(), idx.data_ptr(), w.data_ptr()
    a.num_sf_packs = H // 128
    a.psum_num_recv_tokens_per_rank = out["psum_rank"].data_ptr()
    a.psum_num_recv_tokens_per_expert = out["psum_expert"].data_ptr()
    a.num_unaligned_recv_tokens_per_expert = out["unaligned"].data_ptr()
    a.dst_buffer_slot_idx, a.recv_src_metadata = out["slot"].data_ptr(), out["meta"].data_ptr()
    a.recv_x, a.recv_sf = out["recv_x"].data_ptr(), out["recv_sf"].data_ptr()
    a.recv_sf_token_stride, a.recv_sf_hidden_stride = H // 128, 1
    a.recv_topk_idx = 0 if expanded else out["recv_idx"].data_ptr()
    a.recv_topk_weights = out["recv_w"].data_ptr()
    a.recv_capacity, a.expanded_capacity = cap, (ecap if expanded else 0)
    if workspace is not None:
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
    stream = torch.cuda.current_stream().cuda_stream
    _abi.check(entry(ctypes.byref(a), stream), "dispatch")
    torch.cuda.synchronize()
    return {k: v.cpu() for k, v in out.items()}


@pytest.mark.parametrize("expanded", [False, True], ids=["compact", "expanded"])
def test_static_workspace_dispatch_equals_the_dispatch_with_a_caller_workspace(expanded):
    from deep_ep import _abi
    torch.cuda.set_device(0)
    big = rc.small("static_big", 3000, 1024, 64, 8, 8, seed=21, masked_ratio=0.05)
    small = rc.small("static_small", 130, 512, 32, 4, 6, seed=22, masked_ratio=0.2)
    for case in (big, small):           # two calls in a row on the built-in array, the second smaller
        need = _abi.lib.deep_ep_hip_workspace_bytes(case.T, case.K, case.E, case.R)
        assert need <= _abi.STATIC_WORKSPACE_BYTES
        own = torch.zeros(need, dtype=torch.uint8, device="cuda:0")
        want = _dispatch(_abi.lib.deep_ep_hip_launch_dispatch, case, expanded, own)
        got = _dispatch(_abi.lib.deep_ep_hip_launch_dispatch_static, case, expanded, None)
        for name in want:
            assert torch.equal(got[name], want[name]), f"{case.name}: {name} differs"
        assert int(own[:4].view(torch.int32).item()) == 0


def test_static_workspace_dispatch_rejects_shapes_beyond_its_array():
    from deep_ep import _abi
    torch.cuda.set_device(0)
    a = _abi.DispatchArgs()
    a.phases = _abi.PHASE_LAYOUT
    a.num_tokens, a.hidden, a.num_topk, a.num_experts, a.num_ranks = 60000, 1024, 8, 256, 8
    a.num_max_tokens_per_rank, a.expert_alignment = 60000, 1
    assert _abi.lib.deep_ep_hip_workspace_bytes(60000, 8, 256, 8) > _abi.STATIC_WORKSPACE_BYTES
    rc_ = _abi.lib.deep_ep_hip_launch_dispatch_static(ctypes.byref(a), None)
    assert rc_ == -2 and "built-in" in _abi.last_error()
