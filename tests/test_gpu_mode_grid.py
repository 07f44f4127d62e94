"""The reference's EP mode grid (tests/utils/ep_benchmark_manifest.py:34-63, driven by tests/elastic/test_ep.py:276-422):
do_handle_copy x expert_alignment {128, 1} x FP8 or BF16 x 0/1/2 bias tensors x previous event x asynchronous launch x
allocation on the communication stream (always with a previous event), 144 combinations.  Every combination runs the
reference's six calls (dispatch, expanded dispatch, cached dispatch, cached expanded dispatch with zero padding,
combine, combine of the expanded rows) on the smallest benchmark configuration and is compared with the CPU oracle.
"""
import functools
import itertools

import pytest
import torch

import routing_cases as rc
import routing_oracle as oracle
from test_gpu_parity import assert_equal

pytestmark = pytest.mark.gpu

MODES = [(copy, align, fp8, bias, prev, async_, alloc)
         for copy, align, fp8, bias, prev, async_ in itertools.product((True, False), (128, 1), (True, False), (0, 1, 2),
                                                                       (False, True), (False, True))
         for alloc in ((True,) if prev else (False, True))]


def _mode_id(m):
    return "hcopy%d-align%d-%s-bias%d-prev%d-async%d-alloc%d" % (m[0], m[1], "fp8" if m[2] else "bf16", m[3], m[4], m[5], m[6])


def test_the_grid_has_144_modes():
    assert len(MODES) == 144 and len(set(MODES)) == 144


@functools.lru_cache(maxsize=None)
def _workload():
    case = rc.c1()
    g = torch.Generator().manual_seed(21)
    biases = tuple(torch.randn((case.T, case.H), generator=g).to(torch.bfloat16) for _ in range(2))
    return case, oracle.per_token_cast_to_fp8(case.x), biases


@functools.lru_cache(maxsize=None)
def _expected(fp8, alignment, num_bias):
    """Oracle outputs for one (payload, alignment, bias count): shared by the 12 stream modes of that combination."""
    case, quantised, biases = _workload()
    payload = quantised if fp8 else case.x
    compact = oracle.dispatch(payload, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M, expert_alignment=alignment)
    expanded = oracle.dispatch(payload, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M, expert_alignment=alignment,
                               do_expand=True)
    g = torch.Generator().manual_seed(22)
    y = torch.randn((compact.num_recv_tokens, case.H), generator=g).to(torch.bfloat16)
    y_expanded = torch.randn((expanded.num_expanded_tokens, case.H), generator=g).to(torch.bfloat16)
    bias = None if num_bias == 0 else biases[0] if num_bias == 1 else biases
    common = (case.E, case.R, 0, case.M)
    out, out_w = oracle.combine(y, case.topk_idx, compact.recv_src_metadata, compact.dst_buffer_slot_idx,
                                compact.psum_num_recv_tokens_per_scaleup_rank, *common,
                                topk_weights=compact.recv_topk_weights, bias=bias)
    out_e, out_we = oracle.combine(y_expanded, case.topk_idx, expanded.recv_src_metadata, expanded.dst_buffer_slot_idx,
                                   expanded.psum_num_recv_tokens_per_scaleup_rank, *common,
                                   topk_weights=expanded.recv_topk_weights, bias=bias, do_expand=True)
    return compact, expanded, y, y_expanded, (out, out_w), (out_e, out_we)


@functools.lru_cache(maxsize=None)
def _buffer():
    import deep_ep
    case, _, _ = _workload()
    return deep_ep.ElasticBuffer(deep_ep.LogicalGroup(0, case.R), num_max_tokens_per_rank=case.M, hidden=case.H,
                                 num_topk=case.K, allow_multiple_reduction=True)


def _launch(buf, name, with_previous_event, async_, kwargs):
    """tests/elastic/test_ep.py:224-232: a captured event of the current stream goes in, the returned event is waited on
    by the current stream when the launch was asynchronous."""
    if with_previous_event:
        kwargs = dict(kwargs, previous_event=buf.capture())
    values = getattr(buf, name)(**kwargs)
    assert (values[-1].event is not None) == bool(async_)
    if async_:
        values[-1].current_stream_wait()
    return values


def _check_payload(got, ref, fp8, rows=slice(None), what="recv_x"):
    if fp8:
        assert_equal(got[0].cpu()[rows], ref.recv_x[rows], what + " (fp8 bytes)")
        assert_equal(got[1].cpu()[rows], ref.recv_sf[rows], what + " (scale factors)")
    else:
        assert_equal(got.cpu()[rows], ref.recv_x[rows], what)


@pytest.mark.parametrize("mode", MODES, ids=_mode_id)
def test_mode(mode):
    do_handle_copy, alignment, fp8, num_bias, prev, async_, alloc = mode
    case, quantised, biases = _workload()
    compact, expanded, y, y_expanded, (want, want_w), (want_e, want_we) = _expected(fp8, alignment, num_bias)
    buf = _buffer()
    idx, w = case.topk_idx.cuda(), case.topk_weights.cuda()
    x = tuple(t.cuda() for t in quantised) if fp8 else case.x.cuda()
    bias = None if num_bias == 0 else biases[0].cuda() if num_bias == 1 else tuple(b.cuda() for b in biases)
    streams = dict(async_with_compute_stream=async_, allocate_on_comm_stream=alloc)
    args = dict(x=x, topk_idx=idx, topk_weights=w, num_max_tokens_per_rank=case.M, num_experts=case.E,
                expert_alignment=alignment, do_handle_copy=do_handle_copy, do_cpu_sync=True, **streams)

    recv_x, recv_idx, recv_w, handle, _ = _launch(buf, "dispatch", prev, async_, args)
    exp_x, exp_idx, exp_w, exp_handle, _ = _launch(buf, "dispatch", prev, async_,
                                                  dict(args, do_expand=True, use_tma_aligned_col_major_sf=True))
    cached_args = dict(x=x, handle=handle, **streams)
    c_x, c_idx, c_w, c_handle, _ = _launch(buf, "dispatch", prev, async_, cached_args)
    ce_x, _, ce_w, _, _ = _launch(buf, "dispatch", prev, async_,
                                  dict(cached_args, topk_weights=w, do_expand=True, use_tma_aligned_col_major_sf=True,
                                       do_zero_padding=True, handle=exp_handle))

    _check_payload(recv_x, compact, fp8)
    assert_equal(recv_idx, compact.recv_topk_idx, "recv_topk_idx")
    assert_equal(recv_w, compact.recv_topk_weights, "recv_topk_weights")
    assert_equal(handle.recv_src_metadata, compact.recv_src_metadata, "recv_src_metadata")
    assert handle.num_recv_tokens_per_expert_list == compact.num_recv_tokens_per_expert_list
    valid = expanded.expanded_row_is_valid
    assert exp_idx is None and exp_handle.num_expanded_tokens == expanded.num_expanded_tokens
    _check_payload(exp_x, expanded, fp8, valid, "expanded recv_x")
    assert_equal(exp_w.cpu()[valid], expanded.recv_topk_weights[valid], "expanded weights")
    assert_equal(exp_handle.recv_src_metadata, expanded.recv_src_metadata, "expanded recv_src_metadata")
    if fp8:
        n = exp_x[1].shape[0]
        assert exp_x[1].stride() == (1, (n + 3) // 4 * 4) and ce_x[1].stride() == (1, (n + 3) // 4 * 4)
    _check_payload(c_x, compact, fp8, what="cached recv_x")
    assert_equal(c_idx, compact.recv_topk_idx, "cached recv_topk_idx")
    assert c_w is None and c_handle is handle
    _check_payload(ce_x, expanded, fp8, what="cached expanded recv_x incl. zero padding")
    assert_equal(ce_w, expanded.recv_topk_weights, "cached expanded weights incl. zero padding")

    # tests/elastic/test_ep.py:575-577: the handle owns a copy of topk_idx exactly when do_handle_copy is set
    assert (idx.data_ptr() != handle.topk_idx.data_ptr()) == do_handle_copy
    assert (idx.data_ptr() != c_handle.topk_idx.data_ptr()) == do_handle_copy
    assert handle.topk_idx.data_ptr() == c_handle.topk_idx.data_ptr()
    assert_equal(handle.topk_idx, case.topk_idx, "handle.topk_idx")

    out, out_w, _ = _launch(buf, "combine", prev, async_, dict(x=y.cuda(), topk_weights=recv_w, bias=bias, handle=handle, **streams))
    out_e, out_we, _ = _launch(buf, "combine", prev, async_,
                               dict(x=y_expanded.cuda(), topk_weights=exp_w, bias=bias, handle=exp_handle, **streams))
    assert_equal(out + 0.0, want + 0.0, "combined_x")
    assert_equal(out_w, want_w, "combined_topk_weights")
    assert_equal(out_e + 0.0, want_e + 0.0, "combined_x of the expanded rows")
    assert_equal(out_we, want_we, "combined_topk_weights of the expanded rows")
    buf.check_device_status()
