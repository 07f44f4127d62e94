"""`deep_ep_hip_launch_dispatch_static` (the dispatch whose workspace is a device array built into the library, for
callers that cannot allocate) against `deep_ep_hip_launch_dispatch` on the same inputs, through the C ABI: two calls in
a row, the second with a smaller input, bit for bit; the call allocates nothing (device memory as the driver and as
torch's allocator see it stays where it was), its status bits land in the built-in array's own status word, and a graph
captured around it replays correctly."""
import ctypes

import pytest
import torch

import routing_cases as rc

pytestmark = pytest.mark.gpu


def _static_status(clear=True):
    """The status word of the built-in workspace, read (and cleared) through deep_ep_hip_read_status(NULL, ...)."""
    from deep_ep import _abi
    out = torch.full((1,), -1, dtype=torch.int32, device="cuda:0")
    _abi.check(_abi.lib.deep_ep_hip_read_status(None, out.data_ptr(), int(clear), torch.cuda.current_stream().cuda_stream), "status read")
    torch.cuda.synchronize()
    return int(out.item())


def _dispatch(entry, case, expanded, workspace, measure_allocations=False):
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
    torch.cuda.synchronize()
    free_before, torch_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    _abi.check(entry(ctypes.byref(a), stream), "dispatch")
    torch.cuda.synchronize()
    if measure_allocations:
        assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the free device memory"
        assert torch.cuda.memory_allocated() == torch_before
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
        got = _dispatch(_abi.lib.deep_ep_hip_launch_dispatch_static, case, expanded, None, measure_allocations=True)
        for name in want:
            assert torch.equal(got[name], want[name]), f"{case.name}: {name} differs"
        assert int(own[:4].view(torch.int32).item()) == 0
        assert _static_status() == 0


def test_static_workspace_keeps_its_own_status_word():
    """An expert id out of range is flagged in the built-in array, not in some caller's workspace; a clearing read hands
    the flag over once."""
    from deep_ep import _abi
    torch.cuda.set_device(0)
    case = rc.small("static_bad", 300, 512, 32, 4, 6, seed=23)
    assert _static_status() == 0
    case.topk_idx[7, 2] = case.E
    _dispatch(_abi.lib.deep_ep_hip_launch_dispatch_static, case, False, None)
    assert _static_status(clear=False) == _abi.STATUS_EXPERT_OUT_OF_RANGE
    assert _static_status() == _abi.STATUS_EXPERT_OUT_OF_RANGE and _static_status() == 0


def test_static_workspace_dispatch_under_graph_capture():
    """A call on a stream under capture: nothing but the dispatch's own kernels is captured (resolving the built-in array
    launches nothing that a replay would repeat), and replays with the program's own work in between stay exact."""
    from deep_ep import _abi
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    case = rc.small("static_graph", 700, 1024, 64, 8, 8, seed=24, masked_ratio=0.1)
    T, H, K, E, R, M = case.T, case.H, case.K, case.E, case.R, case.M
    own = torch.zeros(_abi.lib.deep_ep_hip_workspace_bytes(T, K, E, R), dtype=torch.uint8, device=dev)
    want = _dispatch(_abi.lib.deep_ep_hip_launch_dispatch, case, False, own)
    x, idx, w = case.x.to(dev), case.topk_idx.to(dev), case.topk_weights.to(dev)
    i32 = dict(dtype=torch.int32, device=dev)
    cap = M * R
    out = {"psum_rank": torch.zeros(R, **i32), "psum_expert": torch.zeros(E, **i32), "unaligned": torch.zeros(E, **i32),
           "slot": torch.zeros((T, K), **i32), "meta": torch.zeros((cap, K + 2), **i32),
           "recv_x": torch.zeros((cap, H), dtype=torch.uint8, device=dev),
           "recv_sf": torch.zeros((cap, H // 128), dtype=torch.float32, device=dev),
           "recv_idx": torch.zeros((cap, K), dtype=torch.int64, device=dev),
           "recv_w": torch.zeros((cap, K), dtype=torch.float32, device=dev)}
    a = _abi.DispatchArgs()
    a.phases, a.payload = _abi.PHASE_LAYOUT | _abi.PHASE_MOVE, _abi.PAYLOAD_CAST_FP8
    a.num_tokens, a.hidden, a.num_topk, a.num_experts, a.num_ranks = T, H, K, E, R
    a.rank_idx, a.num_max_tokens_per_rank, a.expert_alignment = 0, M, 1
    a.x, a.topk_idx, a.topk_weights, a.num_sf_packs = x.data_ptr(), idx.data_ptr(), w.data_ptr(), H // 128
    a.psum_num_recv_tokens_per_rank, a.psum_num_recv_tokens_per_expert = out["psum_rank"].data_ptr(), out["psum_expert"].data_ptr()
    a.num_unaligned_recv_tokens_per_expert = out["unaligned"].data_ptr()
    a.dst_buffer_slot_idx, a.recv_src_metadata = out["slot"].data_ptr(), out["meta"].data_ptr()
    a.recv_x, a.recv_sf, a.recv_sf_token_stride, a.recv_sf_hidden_stride = out["recv_x"].data_ptr(), out["recv_sf"].data_ptr(), H // 128, 1
    a.recv_topk_idx, a.recv_topk_weights, a.recv_capacity = out["recv_idx"].data_ptr(), out["recv_w"].data_ptr(), cap
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            _abi.check(_abi.lib.deep_ep_hip_launch_dispatch_static(ctypes.byref(a), side.cuda_stream), "captured dispatch")
    torch.cuda.current_stream().wait_stream(side)
    n = int(want["psum_rank"][-1])
    for replay in range(4):
        for t in out.values():
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name in ("psum_rank", "psum_expert", "unaligned", "slot"):
            assert torch.equal(out[name].cpu(), want[name]), f"replay {replay}: {name} differs"
        for name in ("recv_x", "recv_sf", "recv_idx", "recv_w", "meta"):
            assert torch.equal(out[name].cpu()[:n], want[name][:n]), f"replay {replay}: {name} differs"
        (x.float() * 2).sum().item()                     # the program's own eager work between replays
    assert _static_status() == 0


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
