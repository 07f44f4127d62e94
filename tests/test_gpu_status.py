"""Status checks for loops that never wait for the GPU: `ElasticBuffer.poll_device_status` and, underneath it, the C
ABI's `deep_ep_hip_read_status` (a small kernel that copies the workspace's status word into pinned host memory and,
in its clearing form, puts the workspace back in order), eagerly and from a replayed HIP graph."""
import ctypes
import time

import pytest
import torch

import routing_cases as rc
from test_gpu_parity import _buffer
from test_zz_no_alloc import _dispatch

pytestmark = pytest.mark.gpu


def _poll_until_done(buf, seconds=10.0):
    """Polls without ever synchronising; returns what the poll that found the read finished returned (or raises what
    it raised)."""
    deadline = time.monotonic() + seconds
    while time.monotonic() < deadline:
        if buf.poll_device_status():
            return True
        time.sleep(0.001)
    raise AssertionError("the status read did not finish")


def test_poll_is_quiet_on_clean_routing_and_loud_on_bad_routing():
    case = rc.small("status", 900, 512, 32, 4, 6, seed=31, masked_ratio=0.1)
    buf = _buffer(case)
    assert buf.poll_device_status() is True                      # nothing has run: nothing to read
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    for _ in range(3):
        buf.dispatch(x, idx, w, num_experts=case.E, do_cpu_sync=False)
    assert buf.poll_device_status() is False                     # the first call only queues the read
    assert _poll_until_done(buf) is True

    bad = idx.clone()
    bad[5, 0] = case.E + 3
    buf.dispatch(x, bad, w, num_experts=case.E, do_cpu_sync=False)
    buf.dispatch(x, idx, w, num_experts=case.E, do_cpu_sync=False)       # a clean launch does not hide the flag
    with pytest.raises(RuntimeError, match="expert id"):
        _poll_until_done(buf)
    # the read that reported the flag also cleared it: the loop goes on
    buf.dispatch(x, idx, w, num_experts=case.E, do_cpu_sync=False)
    assert _poll_until_done(buf) is True
    buf.check_device_status()


@pytest.mark.parametrize("static", [False, True], ids=["caller_workspace", "built_in_workspace"])
def test_status_read_through_the_c_abi(static):
    """The read finds what a dispatch flagged, in the caller's workspace and (workspace NULL) in the built-in one of
    deep_ep_hip_launch_dispatch_static; the plain form clears nothing, the clearing form hands the flags over once."""
    from deep_ep import _abi
    torch.cuda.set_device(0)
    case = rc.small("status_abi", 700, 512, 32, 4, 6, seed=32)
    need = _abi.lib.deep_ep_hip_workspace_bytes(case.T, case.K, case.E, case.R)
    own = None if static else torch.zeros(need, dtype=torch.uint8, device="cuda:0")
    entry = _abi.lib.deep_ep_hip_launch_dispatch_static if static else _abi.lib.deep_ep_hip_launch_dispatch
    host = torch.full((1,), -1, dtype=torch.int32, pin_memory=True)
    on_device = torch.full((1,), -1, dtype=torch.int32, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    workspace = None if static else own.data_ptr()

    def read(clear, into=host):
        _abi.check(_abi.lib.deep_ep_hip_read_status(workspace, into.data_ptr(), clear, stream), "status read")
        torch.cuda.current_stream().synchronize()
        return int(into[0])

    _dispatch(entry, case, False, own)
    assert read(0) == 0
    case.topk_idx[3, 1] = case.topk_idx[3, 0]                    # one token names an expert twice
    _dispatch(entry, case, False, own)
    assert read(0) == _abi.STATUS_DUPLICATE_EXPERT
    assert read(0, into=on_device) == _abi.STATUS_DUPLICATE_EXPERT       # device memory works too; nothing was cleared
    assert read(1) == _abi.STATUS_DUPLICATE_EXPERT
    assert read(1) == 0                                                  # the clearing read handed the flag over once
    assert _abi.lib.deep_ep_hip_read_status(workspace, None, 0, None) == -1 and "status_out" in _abi.last_error()


def test_clearing_read_repairs_the_workspace_after_a_timeout():
    """A single-launch dispatch that gave up leaves its counters, flags and tagged tables mid-protocol.  The state is forced from the
    host here (the flag set and the bookkeeping words scribbled over): the clearing read must report the flag and
    leave every bookkeeping word zero, and the next dispatch must be exact."""
    from deep_ep import _abi
    torch.cuda.set_device(0)
    case = rc.small("status_repair", 1200, 512, 32, 4, 6, seed=33)
    need = _abi.lib.deep_ep_hip_workspace_bytes(case.T, case.K, case.E, case.R)
    own = torch.zeros(need, dtype=torch.uint8, device="cuda:0")
    want = _dispatch(_abi.lib.deep_ep_hip_launch_dispatch, case, False, own)
    control = _abi.lib.deep_ep_hip_workspace_control_bytes()
    words = own[:control].view(torch.int32)
    words[4:] = -1                                                        # counters, flags, generation and tagged tables scribbled over
    words[0] = _abi.STATUS_LAYOUT_TIMEOUT
    host = torch.zeros(1, dtype=torch.int32, pin_memory=True)
    stream = torch.cuda.current_stream().cuda_stream
    _abi.check(_abi.lib.deep_ep_hip_read_status(own.data_ptr(), host.data_ptr(), 1, stream), "status read")
    torch.cuda.synchronize()
    assert int(host[0]) == _abi.STATUS_LAYOUT_TIMEOUT
    assert int(own[:control].view(torch.int32).abs().sum()) == 0
    got = _dispatch(_abi.lib.deep_ep_hip_launch_dispatch, case, False, own)
    for name in want:
        assert torch.equal(got[name], want[name]), name


def test_status_read_in_a_replayed_graph():
    """Dispatch (no host wait) + clearing status read captured once; every replay reports what that replay's routing
    input deserved, with eager work and host waits between the replays."""
    case = rc.small("status_graph", 1500, 1024, 64, 8, 6, seed=34, masked_ratio=0.1)
    from deep_ep import _abi
    buf = _buffer(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    buf.dispatch(x, idx, w, num_experts=case.E, do_cpu_sync=False)        # warm-up: the workspace is allocated here
    torch.cuda.synchronize()
    host = torch.full((1,), -1, dtype=torch.int32, pin_memory=True)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recv, _, _, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E, do_cpu_sync=False)
        buf.queue_status_read(host)
    clean = idx.clone()
    out_of_range = idx.clone()
    out_of_range[7, 2] = case.E
    twice = idx.clone()
    twice[9, 1] = twice[9, 0] = 5
    expected = [(clean, 0), (out_of_range, _abi.STATUS_EXPERT_OUT_OF_RANGE), (clean, 0), (twice, _abi.STATUS_DUPLICATE_EXPERT),
                (out_of_range, _abi.STATUS_EXPERT_OUT_OF_RANGE), (clean, 0)]
    for routes, status in expected:
        idx.copy_(routes)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert int(host[0]) == status
        (x * 2).sum().item()                                              # eager work of the program between replays
    buf.check_device_status()


def test_a_dispatch_that_gives_up_says_so_and_leaves_the_workspace_usable(monkeypatch):
    """A real LAYOUT_TIMEOUT, forced from the host: with `mover_spin_limit = 1` the mover workgroups that start before
    the layout of their own launch is there give up after one read.  Every kernel still runs to its end.  The call must
    be flagged (its outputs are invalid), the counters and flags of the workspace must be back at zero, and after the
    status has been taken the next dispatch on the same buffer must be exact again."""
    import deep_ep
    import routing_oracle as oracle
    from deep_ep import _abi
    from test_gpu_parity import assert_equal
    case = rc.small("gives_up", 6000, 1024, 64, 8, 8, seed=35, masked_ratio=0.05)
    buf = _buffer(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    ref = oracle.dispatch(case.x, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M)
    monkeypatch.setattr(deep_ep.tuning, "dispatch_launches", 1)
    buf.dispatch(x, idx, w, num_experts=case.E, do_cpu_sync=False)          # allocates the workspace
    buf.check_device_status()

    monkeypatch.setattr(deep_ep.tuning, "mover_spin_limit", 1)
    for _ in range(8):       # whether a mover starts before the layout is there is a matter of timing: a few launches at most
        buf.dispatch(x, idx, w, num_experts=case.E, do_cpu_sync=False)
        torch.cuda.synchronize()
        words = buf.runtime.workspace_control_words().clone()
        if int(words[0]) & _abi.STATUS_LAYOUT_TIMEOUT:
            break
    assert int(words[0]) & _abi.STATUS_LAYOUT_TIMEOUT, "no workgroup of eight launches was early enough to give up"
    words[0] = 0
    words[2:4] = 0
    words[32] = 0
    assert int(words.abs().sum()) == 0, "counters or flags left mid-protocol"
    with pytest.raises(RuntimeError):
        buf.check_device_status()

    monkeypatch.setattr(deep_ep.tuning, "mover_spin_limit", 0)
    recv, ridx, rw, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E, do_cpu_sync=False)
    assert_equal(recv[:ref.num_recv_tokens], ref.recv_x, "recv_x")
    assert_equal(ridx[:ref.num_recv_tokens], ref.recv_topk_idx, "recv_topk_idx")
    assert_equal(handle.dst_buffer_slot_idx, ref.dst_buffer_slot_idx, "dst_buffer_slot_idx")
    buf.check_device_status()
