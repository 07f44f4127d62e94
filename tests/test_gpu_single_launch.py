"""The single-launch dispatch (layout and move in one call without a host wait: counting workgroups ride at the front
of the move kernel and hand the layout to the movers through tagged words in the workspace) against the CPU oracle,
and the state it must leave behind: every launch finds and leaves the counters and flags of the workspace at zero."""
import pytest
import torch

import routing_cases as rc
import routing_oracle as oracle
from test_gpu_parity import CASES, _buffer, assert_equal

pytestmark = pytest.mark.gpu

# shapes the single launch covers (num_topk <= 8, num_ranks + num_experts <= 512, num_ranks * chunks <= 1024)
FUSED = ["C1", "C2", "tiny_masked", "one_token", "k1_e_eq_r", "ragged_chunks", "r1_world", "many_chunks"]


def _control_words(buf):
    words = buf.runtime.workspace_control_words().clone()
    words[2:4] = 0          # the two row totals a dispatch leaves for the kernels that follow it
    words[32] = 0           # the launch generation
    return words


def _check(buf, case, do_expand, payload, alignment=1):
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    if payload == "bf16":
        src, kw = case.x, {}
    else:
        src, kw = oracle.per_token_cast_to_fp8(case.x), {"cast_to_fp8": True}
    ref = oracle.dispatch(src, case.topk_idx, case.topk_weights, case.E, case.R, buf.rank_idx, case.M, do_expand=do_expand,
                          expert_alignment=alignment)
    recv, ridx, rw, handle, _ = buf.dispatch(x, idx, w, num_experts=case.E, do_cpu_sync=False, do_expand=do_expand,
                                             expert_alignment=alignment, **kw)
    n = ref.num_expanded_tokens if do_expand else ref.num_recv_tokens
    valid = ref.expanded_row_is_valid if do_expand else torch.ones(n, dtype=torch.bool)
    if payload == "bf16":
        assert_equal(recv[:n].cpu()[valid], ref.recv_x[valid], "recv_x")
    else:
        assert_equal(recv[0][:n].cpu()[valid], ref.recv_x[valid], "recv_x (fp8)")
        assert_equal(recv[1][:n].cpu()[valid], ref.recv_sf[valid], "recv_sf")
    if not do_expand:
        assert_equal(ridx[:n], ref.recv_topk_idx, "recv_topk_idx")
        assert_equal(rw[:n], ref.recv_topk_weights, "recv_topk_weights")
    else:
        assert_equal(rw[:n].cpu()[valid], ref.recv_topk_weights[valid], "recv_topk_weights")
    assert_equal(handle.psum_num_recv_tokens_per_scaleup_rank, ref.psum_num_recv_tokens_per_scaleup_rank, "psum_rank")
    assert_equal(handle.psum_num_recv_tokens_per_expert, ref.psum_num_recv_tokens_per_expert, "psum_expert")
    assert_equal(handle.num_unaligned_recv_tokens_per_expert, ref.num_unaligned_recv_tokens_per_expert, "unaligned")
    assert_equal(handle.dst_buffer_slot_idx, ref.dst_buffer_slot_idx, "dst_buffer_slot_idx")
    assert_equal(handle.recv_src_metadata[:ref.num_recv_tokens], ref.recv_src_metadata, "recv_src_metadata")
    return handle, ref


@pytest.mark.parametrize("name", FUSED)
@pytest.mark.parametrize("do_expand", [False, True], ids=["compact", "expanded"])
@pytest.mark.parametrize("payload", ["bf16", "cast_fp8"])
def test_single_launch_matches_the_oracle(name, do_expand, payload, monkeypatch):
    import deep_ep
    monkeypatch.setattr(deep_ep.tuning, "dispatch_launches", 1)
    case = CASES[name]()
    if payload == "cast_fp8" and case.H % 128 != 0:
        pytest.skip("the fused cast needs hidden % 128 == 0")
    buf = _buffer(case, rank=case.R - 1)
    _check(buf, case, do_expand, payload, alignment=4 if do_expand else 1)
    buf.check_device_status()
    assert int(_control_words(buf).abs().sum()) == 0, "the launch did not leave its bookkeeping words at zero"


def test_launches_of_changing_shape_share_one_workspace(monkeypatch):
    """Counters, flags and tables are reused by launches of different token counts, layouts and launch modes; no launch
    may take a word an earlier one left behind for its own."""
    import deep_ep
    E, R, K, H = 32, 4, 6, 512
    buf = deep_ep.ElasticBuffer(deep_ep.LogicalGroup(1, R), num_max_tokens_per_rank=4096, hidden=H, num_topk=K)
    shapes = [1, 2, 255, 256, 257, 700, 4096, 3, 1025]
    for round_ in range(2):
        for i, T in enumerate(shapes):
            case = rc.small(f"seq{T}", T, H, E, R, K, seed=100 + T, masked_ratio=0.1)
            case.M = 4096
            monkeypatch.setattr(deep_ep.tuning, "dispatch_launches", (1, 2, 0)[(i + round_) % 3])
            handle, ref = _check(buf, case, do_expand=bool((i + round_) % 2), payload=("bf16", "cast_fp8")[i % 2])
            assert int(_control_words(buf).abs().sum()) == 0, f"bookkeeping words not zero after T={T}"
    buf.check_device_status()


@pytest.mark.parametrize("T", [9000, 16384])
def test_single_launch_up_to_131072_token_lanes(T, monkeypatch):
    """Shapes between 65536 and 131072 (token, lane) pairs: the top of what the tagged position table holds.  One and
    two launches alternate on one workspace, where the position words of a dispatch in two launches share that table
    with the tagged ones; every call must be exact."""
    import deep_ep
    case = rc.small(f"lanes{T}", T, 128, 32, 8, 8, seed=60 + T % 7, masked_ratio=0.05)
    buf = _buffer(case, rank=3)
    for i, launches in enumerate((1, 2, 1, 0, 2)):
        monkeypatch.setattr(deep_ep.tuning, "dispatch_launches", launches)
        _check(buf, case, do_expand=bool(i % 2) and T <= 9000, payload=("cast_fp8", "bf16")[i % 2], alignment=4 if i % 2 else 1)
        assert int(_control_words(buf).abs().sum()) == 0
    buf.check_device_status()


@pytest.mark.parametrize("warm_rounds", [1, 0, -1])
def test_cache_warming_loads_change_nothing(warm_rounds, monkeypatch):
    """A launch with more mover workgroups than a GPU holds at a time: the first of them also load, into a piece of LDS
    nobody reads, tiles of work items further on.  Results are the oracle's whatever the distance."""
    import deep_ep
    monkeypatch.setattr(deep_ep.tuning, "dispatch_launches", 1)
    monkeypatch.setattr(deep_ep.tuning, "warm_rounds", warm_rounds)
    case = rc.small("warm", 3300, 7168, 64, 8, 8, seed=91, masked_ratio=0.05)       # 3300 mover workgroups
    buf = _buffer(case, rank=2)
    for do_expand in (False, True):
        for payload in ("cast_fp8", "bf16"):
            _check(buf, case, do_expand, payload, alignment=4 if do_expand else 1)
            assert int(_control_words(buf).abs().sum()) == 0
    buf.check_device_status()


def test_many_back_to_back_launches_without_host_sync(monkeypatch):
    """50 single-launch dispatches queued without a host wait in between: the counters of launch n must have wrapped to
    zero and its generation must have advanced before launch n + 1 starts (stream order), whatever the number of
    movers per gate."""
    import deep_ep
    monkeypatch.setattr(deep_ep.tuning, "dispatch_launches", 1)
    case = rc.small("b2b", 1500, 1024, 64, 8, 8, seed=77, masked_ratio=0.05)
    buf = _buffer(case)
    x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
    ref = oracle.dispatch(case.x, case.topk_idx, case.topk_weights, case.E, case.R, 0, case.M)
    outs = [buf.dispatch(x, idx, w, num_experts=case.E, do_cpu_sync=False) for _ in range(50)]
    torch.cuda.synchronize()
    for recv, ridx, rw, handle, _ in outs[::7] + [outs[-1]]:
        assert_equal(recv[:ref.num_recv_tokens], ref.recv_x, "recv_x")
        assert_equal(handle.dst_buffer_slot_idx, ref.dst_buffer_slot_idx, "dst_buffer_slot_idx")
    buf.check_device_status()
    assert int(_control_words(buf).abs().sum()) == 0


def test_the_launch_tag_wraps_without_taking_a_stale_word(monkeypatch):
    """The words counting workgroups hand to the movers carry the launch's tag, 1 .. 16383; the launch that uses the
    last tag clears the tagged tables and the count starts over.  More launches than there are tags, of three
    alternating shapes and both layouts (so that words of older launches lie about under every tag, beyond the token
    range of the smaller shapes too): the launches around the wrap and the last one must be exact, and the generation
    word must read launches mod 16383."""
    import deep_ep
    monkeypatch.setattr(deep_ep.tuning, "dispatch_launches", 1)
    period = 16383
    E, R, K, H = 16, 4, 4, 128
    buf = deep_ep.ElasticBuffer(deep_ep.LogicalGroup(2, R), num_max_tokens_per_rank=1024, hidden=H, num_topk=K)
    cases, refs = [], {}
    for i, T in enumerate((700, 40, 300)):           # the largest first: the buffer sizes its workspace on first use
        case = rc.small(f"wrap{T}", T, H, E, R, K, seed=500 + T, masked_ratio=0.1)
        case.M = 1024
        cases.append((case, case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()))
        for do_expand in (False, True):
            refs[i, do_expand] = oracle.dispatch(case.x, case.topk_idx, case.topk_weights, E, R, buf.rank_idx, case.M,
                                                 do_expand=do_expand, expert_alignment=2)
    assert int(buf.runtime.workspace_control_words()[32]) == 0
    launches = period + 150
    kept = {}
    for n in range(launches):
        i, do_expand = n % 3, (n // 3) % 2 == 1
        case, x, idx, w = cases[i]
        out = buf.dispatch(x, idx, w, num_experts=E, do_cpu_sync=False, do_expand=do_expand, expert_alignment=2)
        if n < 4 or abs(n - period) < 40 or n >= launches - 6:
            kept[n] = (i, do_expand, out)
    torch.cuda.synchronize()
    buf.check_device_status()
    assert int(buf.runtime.workspace_control_words()[32]) == launches % period
    for n, (i, do_expand, (recv, ridx, rw, handle, _)) in kept.items():
        ref = refs[i, do_expand]
        rows = ref.num_expanded_tokens if do_expand else ref.num_recv_tokens
        valid = ref.expanded_row_is_valid if do_expand else torch.ones(rows, dtype=torch.bool)
        assert_equal(recv[:rows].cpu()[valid], ref.recv_x[valid], f"recv_x of launch {n}")
        assert_equal(handle.dst_buffer_slot_idx, ref.dst_buffer_slot_idx, f"dst_buffer_slot_idx of launch {n}")
        assert_equal(handle.recv_src_metadata[:ref.num_recv_tokens], ref.recv_src_metadata, f"recv_src_metadata of launch {n}")
    assert int(_control_words(buf).abs().sum()) == 0
