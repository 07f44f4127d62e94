"""Stream and event surface on the GPU: previous_event, async_with_compute_stream, allocate_on_comm_stream,
EventOverlap hooks, determinism of repeated calls, T = 0, and argument errors raised by the host runtime."""
import pytest
import torch

import routing_cases as rc
import routing_oracle as oracle
from test_gpu_parity import assert_equal

pytestmark = pytest.mark.gpu


def _buf(case, **kw):
    import deep_ep
    return deep_ep.ElasticBuffer(deep_ep.LogicalGroup(0, case.R), num_max_tokens_per_rank=case.M, hidden=case.H,
                                 num_topk=case.K, **kw)


@pytest.mark.parametrize("with_previous_event", [False, True])
@pytest.mark.parametrize("allocate_on_comm", [False, True])
def test_async_dispatch_and_combine(with_previous_event, allocate_on_comm):
    if with_previous_event and not allocate_on_comm:
        pytest.skip("previous_event requires allocate_on_comm_stream (reference rule)")
    case = rc.c2()
    buf = _buf(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    ref = oracle.dispatch(case.x, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M)
    # some compute on the current stream that the routing must wait for
    x2 = x * 1
    prev = buf.capture() if with_previous_event else None
    recv_x, recv_idx, recv_w, handle, event = buf.dispatch(x2, idx, w, num_experts=case.E, previous_event=prev,
                                                           async_with_compute_stream=True,
                                                           allocate_on_comm_stream=allocate_on_comm)
    assert event.event is not None
    hooked = []
    event.register_hook_after_wait(lambda: hooked.append(True))
    with event:
        filler = torch.ones(1 << 20, device="cuda").sum()       # overlappable work on the compute stream
    assert hooked == [True]
    assert_equal(recv_x, ref.recv_x, "async recv_x")
    assert_equal(recv_idx, ref.recv_topk_idx, "async recv_topk_idx")
    out, out_w, ev2 = buf.combine(recv_x, handle, topk_weights=recv_w, async_with_compute_stream=True,
                                  allocate_on_comm_stream=allocate_on_comm,
                                  previous_event=buf.capture() if allocate_on_comm else None)
    ev2.current_stream_wait()
    ref_out, _ = oracle.combine(ref.recv_x, case.topk_idx, ref.recv_src_metadata, ref.dst_buffer_slot_idx,
                                ref.psum_num_recv_tokens_per_scaleup_rank, case.E, case.R, 0, case.M)
    assert_equal(out + 0.0, ref_out + 0.0, "async combined_x")
    assert torch.cuda.current_stream() != buf.get_comm_stream()
    assert float(filler) == float(1 << 20)


def test_repeated_calls_are_bitwise_identical():
    """Skewed routing with masked slots (hot experts, ragged buckets): two runs, identical bytes everywhere."""
    case = rc.skewed_masked_case("C4small", 2048, 1024, 256, 8, 8, seed=3)
    buf = _buf(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    runs = []
    for _ in range(2):
        (rx, rsf), ri, rw, h, _ = buf.dispatch(x, idx, w, num_experts=case.E, cast_to_fp8=True, do_expand=True,
                                               expert_alignment=8, do_zero_padding=True)
        y = rx.to(torch.float32).to(torch.bfloat16)
        out, ow, _ = buf.combine(y, h, topk_weights=rw)
        runs.append((rx.view(torch.uint8), rsf, rw, h.recv_src_metadata, h.dst_buffer_slot_idx, out.view(torch.int16), ow))
    for a, b in zip(*runs):
        assert torch.equal(a, b)
    ref = oracle.dispatch(oracle.per_token_cast_to_fp8(case.x), case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M,
                          expert_alignment=8, do_expand=True)
    assert_equal(runs[0][0], ref.recv_x.view(torch.uint8), "skewed expanded payload")
    assert_equal(runs[0][3], ref.recv_src_metadata, "skewed metadata")
    counts = ref.num_unaligned_recv_tokens_per_expert
    assert int(counts.max()) > 20 * max(int(counts.float().median()), 1)      # the load really is imbalanced


def test_empty_input():
    case = rc.small("empty", 4, 256, 8, 2, 2, seed=1)
    buf = _buf(case)
    x = torch.empty((0, case.H), dtype=torch.bfloat16, device="cuda")
    idx = torch.empty((0, case.K), dtype=torch.int64, device="cuda")
    w = torch.empty((0, case.K), dtype=torch.float32, device="cuda")
    for expand in (False, True):
        rx, ri, rw, h, _ = buf.dispatch(x, idx, w, num_experts=case.E, do_expand=expand)
        assert rx.shape == (0, case.H) and h.num_recv_tokens == 0 and h.num_expanded_tokens == 0
        assert h.psum_num_recv_tokens_per_scaleup_rank.tolist() == [0, 0]
        assert h.num_recv_tokens_per_expert_list == [0] * case.E
        out, ow, _ = buf.combine(rx, h, topk_weights=rw)
        assert out.shape == (0, case.H)
    a, b, c, d, _ = buf.get_dispatch_layout(idx, case.E)
    assert a.tolist() == [0, 0] and b is None and c.tolist() == [0] * case.E and d.shape == (0, 2)


def test_host_argument_errors():
    case = rc.small("err", 8, 256, 8, 2, 2, seed=2)
    buf = _buf(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    with pytest.raises(RuntimeError):
        buf.dispatch(x, idx.to(torch.int32), w, num_experts=case.E)                 # wrong index dtype
    with pytest.raises(RuntimeError):
        buf.dispatch(x, idx, w, num_experts=9)                                      # experts not divisible by ranks
    with pytest.raises(RuntimeError):
        buf.dispatch(x, idx, w, num_experts=case.E, do_zero_padding=True)           # zero padding needs expand
    with pytest.raises(RuntimeError):
        buf.dispatch(x, idx, w, num_experts=case.E, num_max_tokens_per_rank=4)      # more tokens than capacity
    with pytest.raises(RuntimeError):
        buf.dispatch((x, w), idx, w, num_experts=case.E)                            # scale factors with a 2-byte payload
    _, _, _, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E)
    with pytest.raises(AssertionError):
        buf.dispatch(x, idx, w, handle=handle)                                      # cached dispatch takes no topk_idx
    with pytest.raises(AssertionError):
        buf.dispatch(x, handle=handle, do_cpu_sync=True)
    with pytest.raises(RuntimeError):
        buf.combine(x.float(), handle)                                              # combine input must be BF16
    with pytest.raises(RuntimeError):
        buf.combine(x, handle, bias=torch.zeros((3, case.H), dtype=torch.bfloat16, device="cuda"))
    bad = idx.clone()
    bad[0, 0] = case.E + 5
    with pytest.raises(RuntimeError, match="expert id"):
        buf.dispatch(x, bad, w, num_experts=case.E)
    dup = idx.clone()
    dup[1, 1] = dup[1, 0]
    with pytest.raises(RuntimeError, match="same expert twice"):
        buf.dispatch(x, dup, w, num_experts=case.E)
    # the buffer still works after the rejected inputs
    rx, _, _, _, _ = buf.dispatch(x, idx, w, num_experts=case.E)
    assert rx.shape[0] == oracle.dispatch(case.x, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M).num_recv_tokens


def test_calls_on_two_streams_share_the_workspace_in_order():
    """An asynchronous dispatch on the communication stream that nobody has waited for yet, followed at once by plain
    calls on the compute stream with other routing: the buffer's workspace (positions, tables, counters) is shared, so the
    second call has to queue behind the first by itself.  Both results are checked against the oracle."""
    a = rc.small("two_streams_a", 3000, 1024, 64, 8, 8, seed=61, masked_ratio=0.05)
    b = rc.small("two_streams_b", 2900, 1024, 64, 8, 8, seed=62, masked_ratio=0.3)
    b.M = a.M
    buf = _buf(a)
    ref_a = oracle.dispatch(a.x, a.topk_idx, a.topk_weights, a.E, a.R, 0, a.M)
    ref_b = oracle.dispatch(b.x, b.topk_idx, b.topk_weights, b.E, b.R, 0, b.M)
    xa, ia, wa = a.x.cuda(), a.topk_idx.cuda(), a.topk_weights.cuda()
    xb, ib, wb = b.x.cuda(), b.topk_idx.cuda(), b.topk_weights.cuda()
    torch.cuda.synchronize()
    for _ in range(3):
        ra, ria, rwa, ha, ev = buf.dispatch(xa, ia, wa, num_experts=a.E, do_cpu_sync=False, async_with_compute_stream=True)
        rb, rib, rwb, hb, _ = buf.dispatch(xb, ib, wb, num_experts=b.E, do_cpu_sync=False)          # compute stream, no wait
        per_rank, _, per_expert, _, _ = buf.get_dispatch_layout(ia, a.E)                            # and a layout call on top
        ev.current_stream_wait()
        torch.cuda.synchronize()
        assert_equal(ra[:ref_a.num_recv_tokens], ref_a.recv_x, "recv_x of the asynchronous call")
        assert_equal(ha.dst_buffer_slot_idx, ref_a.dst_buffer_slot_idx, "slots of the asynchronous call")
        assert_equal(rb[:ref_b.num_recv_tokens], ref_b.recv_x, "recv_x of the call that followed")
        assert_equal(hb.dst_buffer_slot_idx, ref_b.dst_buffer_slot_idx, "slots of the call that followed")
        assert_equal(per_expert, oracle.layout(a.topk_idx, a.E, a.R)[1], "layout counts")
    buf.check_device_status()


def test_current_stream_is_restored_when_a_call_fails():
    case = rc.small("restore", 64, 256, 8, 2, 2, seed=63)
    buf = _buf(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    before = torch.cuda.current_stream()
    with pytest.raises(RuntimeError):
        buf.dispatch(x, idx, w, num_experts=case.E, num_max_tokens_per_rank=4, allocate_on_comm_stream=True,
                     previous_event=buf.capture(), async_with_compute_stream=True)
    bad = idx.clone()
    bad[0, 0] = case.E + 1
    with pytest.raises(RuntimeError, match="expert id"):
        buf.dispatch(x, bad, w, num_experts=case.E, allocate_on_comm_stream=True, previous_event=buf.capture(),
                     async_with_compute_stream=True)
    assert torch.cuda.current_stream() == before


def test_previous_event_before_epilogue_orders_the_move_phase():
    """`previous_event_before_epilogue` (csrc/elastic/buffer.hpp:528-586): the launches that write the outputs wait for
    an event recorded behind work on another stream - here the producer of the tensor a cached dispatch moves."""
    case = rc.small("before_epilogue", 2000, 2048, 32, 4, 4, seed=64)
    buf = _buf(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    _, _, _, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E)
    ref = oracle.dispatch(case.x * 2, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M)
    side = torch.cuda.Stream()
    x2 = torch.empty_like(x)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        filler = torch.ones(1 << 24, device="cuda").cumsum(0)          # keeps the side stream busy first
        torch.mul(x, 2, out=x2)
        produced = buf.capture()
    recv_x, _, _, _, event = buf.dispatch(x2, topk_weights=w, handle=handle, previous_event=buf.capture(),
                                          previous_event_before_epilogue=produced, async_with_compute_stream=True,
                                          allocate_on_comm_stream=True)
    event.current_stream_wait()
    assert_equal(recv_x, ref.recv_x, "recv_x moved after the producer finished")
    out, _, ev2 = buf.combine(recv_x, handle, previous_event=buf.capture(), previous_event_before_epilogue=produced,
                              async_with_compute_stream=True, allocate_on_comm_stream=True)
    ev2.current_stream_wait()
    ref_out, _ = oracle.combine(ref.recv_x, case.topk_idx, ref.recv_src_metadata, ref.dst_buffer_slot_idx,
                                ref.psum_num_recv_tokens_per_scaleup_rank, case.E, case.R, 0, case.M)
    assert_equal(out + 0.0, ref_out + 0.0, "combined_x")
    assert float(filler[-1]) == float(1 << 24)
