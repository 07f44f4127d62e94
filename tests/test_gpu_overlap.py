"""The case the asynchronous API exists for: single-launch dispatches and combines on the communication stream while
kernels that fill the GPU run on the compute stream (here: a chain of large matrix products standing in for the expert
GEMMs of the neighbouring micro-batch).  The counting, publishing and mover workgroups of a single-launch dispatch then
share compute units with foreign workgroups and are placed as those drain, not all at once: every result is checked
against the oracle, iteration by iteration, and the status word must stay clean (no wait of the hand-off may run out).
"""
import pytest
import torch

import routing_cases as rc
import routing_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("do_expand", [False, True])
def test_single_launch_dispatch_and_combine_under_a_gpu_filling_compute_stream(do_expand):
    import ctypes
    import deep_ep
    from deep_ep import _abi
    case = rc.skewed_masked_case("overlap", 3000, 2048, 64, 8, 8, seed=21, masked_ratio=0.05)
    T, H, K, E, R, M = case.T, case.H, case.K, case.E, case.R, case.M
    probe = _abi.DispatchArgs()
    probe.phases, probe.payload, probe.do_expand = _abi.PHASE_LAYOUT | _abi.PHASE_MOVE, _abi.PAYLOAD_CAST_FP8, int(do_expand)
    probe.num_tokens, probe.hidden, probe.num_topk, probe.num_experts, probe.num_ranks = T, H, K, E, R
    probe.num_max_tokens_per_rank, probe.expert_alignment = M, 1
    assert _abi.lib.deep_ep_hip_dispatch_kernel_launches(ctypes.byref(probe)) == 1, "this shape must take the single launch"

    buf = deep_ep.ElasticBuffer(deep_ep.LogicalGroup(0, R), num_max_tokens_per_rank=M, hidden=H, num_topk=K)
    q = oracle.per_token_cast_to_fp8(case.x)
    ref = oracle.dispatch(q, case.topk_idx, case.topk_weights, E, R, 0, M, do_expand=do_expand)
    n = ref.num_expanded_tokens if do_expand else ref.num_recv_tokens
    y = oracle.per_token_cast_back(ref.recv_x, ref.recv_sf)
    ref_out, ref_w = oracle.combine(y, case.topk_idx, ref.recv_src_metadata, ref.dst_buffer_slot_idx,
                                    ref.psum_num_recv_tokens_per_scaleup_rank, E, R, 0, M,
                                    topk_weights=ref.recv_topk_weights, do_expand=do_expand)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    ref_bytes, ref_sf = ref.recv_x.view(torch.uint8).cuda(), ref.recv_sf.cuda()
    ref_slots = ref.dst_buffer_slot_idx.cuda()
    ref_out_d, ref_w_d = (ref_out + 0.0).cuda(), ref_w.cuda()
    rows = M * min(K, E) if do_expand else M * R                  # what a dispatch without host sync allocates
    y_d = torch.zeros((rows, H), dtype=torch.bfloat16, device="cuda")
    y_d[:n] = y.cuda()

    a = torch.randn((4096, 4096), device="cuda", dtype=torch.bfloat16)
    c = torch.empty_like(a)
    for it in range(200):
        before = buf.capture()                                   # the routing input is ready here
        for _ in range(3):
            torch.mm(a, a, out=c)                                # ... and the compute stream is busy from here on
        (rx, rsf), ridx, rw, handle, ev = buf.dispatch(x, idx, w, num_experts=E, do_cpu_sync=False, cast_to_fp8=True,
                                                       do_expand=do_expand, previous_event=before,
                                                       async_with_compute_stream=True, allocate_on_comm_stream=True)
        out, out_w, ev2 = buf.combine(y_d, handle, topk_weights=rw, previous_event=ev, async_with_compute_stream=True,
                                      allocate_on_comm_stream=True)
        torch.mm(a, a, out=c)
        ev2.current_stream_wait()
        ok = (torch.equal(rx[:n].view(torch.uint8), ref_bytes) and torch.equal(rsf[:n], ref_sf) and
              torch.equal(handle.dst_buffer_slot_idx, ref_slots) and torch.equal(out + 0.0, ref_out_d) and torch.equal(out_w, ref_w_d))
        assert ok, f"iteration {it}: a result under load differs from the oracle (status {buf.runtime.device_status()})"
        if it % 50 == 49:
            assert buf.runtime.device_status() == 0, f"status word after iteration {it}"
    buf.check_device_status()
    assert torch.isfinite(c.float()).all()
