"""The reference's FP8 transport matrix (tests/ascend/production/run_fp8_dispatch_combine.py) through the HIP path.

Inputs and the rows every destination rank must hold come from tests/golden/fp8_transport_cases.json.  The whole
logical world runs in one call (tests/world.py): source rank s owns rows [s*4, s*4+n_s) of the input, and bucket d of
the output is what destination rank d receives.  Every case is also checked against the CPU oracle.
"""
import json
import os

import pytest
import torch

import routing_oracle as oracle
import world
from test_gpu_parity import assert_equal

pytestmark = pytest.mark.gpu

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_transport_cases.json")) as f:
    FX = json.load(f)
H, K, P, M = FX["hidden"], FX["num_topk"], FX["sf_packs"], FX["capacity"]
ROWS = FX["row_table"]
WORLDS = sorted(FX["worlds"])
CASE_NAMES = list(FX["worlds"]["2"]["cases"])


def _payload(ids, fp8):
    """Row-table indices -> [n, H] tensor of the case's payload dtype."""
    width = H if fp8 else 2 * H
    raw = torch.tensor([list(bytes.fromhex(ROWS[i])) for i in ids], dtype=torch.uint8).reshape(len(ids), width)
    return raw.view(torch.float8_e4m3fn if fp8 else torch.bfloat16)


def _stack(case, R):
    """Per-source inputs -> the world's tensors on the GPU; the packed scale factors keep the reference's transposed
    (token-minor) storage, so the kernel must honour both strides."""
    fp8 = case["fp8"]
    x = torch.zeros((R * M, H), dtype=torch.uint8 if fp8 else torch.bfloat16)
    idx = torch.full((R * M, K), -1, dtype=torch.int64)
    w = torch.zeros((R * M, K), dtype=torch.float32) if case["weighted"] else None
    sf_bits = torch.zeros((R * M, P), dtype=torch.int32)
    for s, src in enumerate(case["sources"]):
        n = len(src["routes"])
        if n == 0:
            continue
        rows = _payload(src["x"], fp8)
        x[s * M:s * M + n] = rows.view(torch.uint8) if fp8 else rows
        idx[s * M:s * M + n] = torch.tensor(src["routes"], dtype=torch.int64)
        if w is not None:
            w[s * M:s * M + n] = torch.tensor(src["weights"], dtype=torch.float32)
        if fp8:
            sf_bits[s * M:s * M + n] = torch.tensor(src["sf_bits"], dtype=torch.int32)
    if not fp8:
        return x.cuda(), None, idx.cuda(), None if w is None else w.cuda()
    x = x.view(torch.float8_e4m3fn).cuda()
    if case["packed_sf"]:
        sf = sf_bits.T.contiguous().cuda().T            # [R*M, P] with strides (1, R*M)
        assert not sf.is_contiguous() or R * M == 1
    else:
        sf = sf_bits.view(torch.float32).cuda()
    return x, sf, idx.cuda(), None if w is None else w.cuda()


def _buffer(R):
    import deep_ep
    return deep_ep.ElasticBuffer(deep_ep.LogicalGroup(0, R), num_max_tokens_per_rank=R * M, hidden=H, num_topk=K,
                                 use_fp8_dispatch=False)


def _dispatch(buf, case, R, handle=None):
    x, sf, idx, w = _stack(case, R)
    result = buf.dispatch((x, sf) if case["fp8"] else x,
                          topk_idx=None if handle is not None else idx, topk_weights=w, handle=handle,
                          num_experts=None if handle is not None else 2 * R,
                          expert_alignment=None if handle is not None else case["expert_alignment"],
                          do_cpu_sync=None if handle is not None else True,
                          do_expand=case["expanded"], do_zero_padding=case["zero_padding"],
                          use_tma_aligned_col_major_sf=case["column_major_output"] and case["fp8"])
    return result, (x, sf, idx, w)


def _verify(result, case, R, inputs, expected_handle=None):
    recv, recv_topk, recv_w, handle, event = result
    fp8, expanded = case["fp8"], case["expanded"]
    if fp8:
        assert isinstance(recv, tuple) and len(recv) == 2, "FP8 dispatch did not return payload and scales"
        recv_x, recv_sf = recv
        assert recv_x.dtype == torch.float8_e4m3fn
        assert recv_sf.dtype == (torch.int32 if case["packed_sf"] else torch.float32)
        n = recv_sf.shape[0]
        if case["column_major_output"]:
            assert recv_sf.stride() == (1, (n + 3) // 4 * 4), f"column-major SF stride {recv_sf.stride()}"
        else:
            assert recv_sf.stride() == (P, 1), f"row-major SF stride {recv_sf.stride()}"
        sf_bits = recv_sf.cpu().contiguous().view(torch.int32)
    else:
        assert not isinstance(recv, tuple), "BF16 dispatch returned scale factors"
        recv_x, sf_bits = recv, None
    assert (recv_topk is None) == expanded
    assert (recv_w is None) == (not case["weighted"])
    if expected_handle is not None:
        assert handle is expected_handle, "cached dispatch replaced its handle"
    assert event.event is None

    if expanded:
        starts = [0]
        for rows in handle.num_recv_tokens_per_expert_list:                      # aligned rows of each expert's region
            starts.append(starts[-1] + rows)
        bounds = [(starts[2 * d], starts[2 * d + 2]) for d in range(R)]
    else:
        bounds = world.bucket_bounds(handle.psum_num_recv_tokens_per_scaleup_rank.cpu())
    assert recv_x.shape[0] == bounds[-1][1]
    got_x = recv_x.cpu().view(torch.uint8)
    for d, (lo, hi) in enumerate(bounds):
        exp = case["expected"][d]
        assert hi - lo == len(exp["payload"]), f"rank {d} holds {hi - lo} rows, expected {len(exp['payload'])}"
        if hi == lo:
            continue
        keep = torch.ones(hi - lo, dtype=torch.bool)
        if expanded and not case["zero_padding"]:
            keep = torch.tensor(exp["valid"])                                    # padding rows are not written
        assert_equal(got_x[lo:hi][keep], _payload(exp["payload"], fp8).view(torch.uint8)[keep], f"rank {d} payload")
        if fp8:
            assert_equal(sf_bits[lo:hi][keep], torch.tensor(exp["sf_bits"], dtype=torch.int32)[keep], f"rank {d} SF packs")
        if not expanded:
            assert_equal(recv_topk[lo:hi], torch.tensor(exp["topk"], dtype=torch.int64).reshape(-1, K), f"rank {d} top-k")
            sources = torch.tensor([s * M + t for s, t in exp["rows"]], dtype=torch.int32)
            assert_equal(handle.recv_src_metadata[lo:hi, 0], sources, f"rank {d} source rows")
        else:
            per = handle.num_unaligned_recv_tokens_per_expert.cpu()[2 * d:2 * d + 2].tolist()
            assert per == exp["unaligned_counts"]
            assert handle.num_recv_tokens_per_expert_list[2 * d:2 * d + 2] == exp["aligned_counts"]
        if case["weighted"]:
            want = torch.tensor(exp["weights"], dtype=torch.float32)
            assert_equal(recv_w[lo:hi][keep], want[keep], f"rank {d} weights")

    # the same call against the CPU oracle, every output
    x, sf, idx, w = inputs
    pair = (x.cpu(), sf.cpu().contiguous()) if fp8 else x.cpu()
    ref = oracle.dispatch(pair, handle.topk_idx.cpu(), None if w is None else w.cpu(), 2 * R, R, 0, R * M,
                          expert_alignment=handle.expert_alignment, do_expand=expanded)
    valid = ref.expanded_row_is_valid if expanded and not case["zero_padding"] else slice(None)
    assert_equal(got_x[valid], ref.recv_x.view(torch.uint8)[valid], "payload vs oracle")
    if fp8:
        assert_equal(sf_bits[valid], ref.recv_sf.contiguous().view(torch.int32)[valid], "SF packs vs oracle")
    assert_equal(handle.recv_src_metadata, ref.recv_src_metadata, "recv_src_metadata vs oracle")
    assert_equal(handle.dst_buffer_slot_idx, ref.dst_buffer_slot_idx, "dst_buffer_slot_idx vs oracle")
    return recv, handle


@pytest.mark.parametrize("R", WORLDS)
@pytest.mark.parametrize("name", CASE_NAMES)
def test_transport_case(name, R):
    case, R = FX["worlds"][R]["cases"][name], int(R)
    buf = _buffer(R)
    result, inputs = _dispatch(buf, case, R)
    _verify(result, case, R, inputs)
    buf.check_device_status()


@pytest.mark.parametrize("R", WORLDS)
def test_cached_handle_changes_representation(R):
    """A handle made by a BF16 dispatch moves FP8 rows with packed scale factors, and the other way round."""
    steps, R = FX["worlds"][R]["cached_sequence"], int(R)
    buf = _buffer(R)
    handles = []
    for step in steps:
        reuse = None if step["reuse_handle_of"] is None else handles[step["reuse_handle_of"]]
        result, inputs = _dispatch(buf, step, R, handle=reuse)
        recv, handle = _verify(result, step, R, inputs, expected_handle=reuse)
        if step["fp8"]:
            assert isinstance(recv, tuple) and recv[1].dtype == torch.int32
        handles.append(handle)
    buf.check_device_status()


@pytest.mark.parametrize("R", WORLDS)
def test_bf16_combine_of_transported_rows(R):
    fx, R = FX["worlds"][R]["combine"], int(R)
    case = fx["dispatch"]
    buf = _buffer(R)
    result, inputs = _dispatch(buf, case, R)
    _, handle = _verify(result, case, R, inputs)
    y = torch.empty((handle.num_recv_tokens, H), dtype=torch.bfloat16)
    for d, (lo, hi) in enumerate(world.bucket_bounds(handle.psum_num_recv_tokens_per_scaleup_rank.cpu())):
        for i, fill in enumerate(fx["fill_of_row"][d]):
            y[lo + i] = fill
    combined, combined_w, event = buf.combine(y.cuda(), handle)
    assert combined_w is None and event.event is None
    for s, per_token in enumerate(fx["combined"]):
        for t, value in enumerate(per_token):
            assert combined[s * M + t].float().cpu().tolist() == [value] * H, f"source {s} token {t}"
    buf.check_device_status()


def test_generations_reuse_the_buffer():
    """100 dispatches in a row through one buffer, the payload changing with generation % 13."""
    fx = FX["worlds"]["2"]["generations_by_salt"]
    buf = _buffer(2)
    for generation in range(100):
        case = fx[generation % 13]
        result, inputs = _dispatch(buf, case, 2)
        _verify(result, case, 2, inputs)
    buf.check_device_status()


@pytest.mark.parametrize("bad", ["bf16_sf", "one_dim_sf", "short_sf", "sf_with_bf16_payload"])
def test_malformed_scale_factors_are_refused(bad):
    """A scale-factor tensor that is not [tokens, packs] of 4-byte elements raises RuntimeError before anything is
    launched, and the buffer works afterwards (run_fp8_dispatch_combine.py:432-444)."""
    case = FX["worlds"]["2"]["cases"]["normal-fp32"]
    buf = _buffer(2)
    x, sf, idx, _ = _stack(case, 2)
    if bad == "bf16_sf":
        pair = (x, sf.to(torch.bfloat16))
    elif bad == "one_dim_sf":
        pair = (x, sf.reshape(-1))
    elif bad == "short_sf":
        pair = (x, sf[:-1])
    else:
        pair = (x.to(torch.bfloat16), sf)
    with pytest.raises(RuntimeError):
        buf.dispatch(pair, topk_idx=idx, num_experts=4)
    torch.cuda.synchronize()
    result, inputs = _dispatch(buf, case, 2)
    _verify(result, case, 2, inputs)
    buf.check_device_status()
