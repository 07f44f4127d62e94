"""CPU oracle for the MoE token-routing hot path (layout / dispatch / combine / low-latency).

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this module; it exists so
that tests, the smoke check and the benchmark's CPU-baseline leg have an independent restatement
of what the reference computes.  Everything here runs on CPU torch tensors (eager mode, no
torch.compile) and favours obviousness over speed.

Each function names the reference source it restates (paths relative to the reference tree):

  layout()                  tests/legacy/test_intranode.py:37-68 (the pure-torch recipe the
                            reference checks `Buffer.get_dispatch_layout` against) and
                            csrc/kernels/legacy/layout.cu:10-122 (what is counted)
  per_token_cast_to_fp8()   deep_ep/utils/math.py:30-39 (eager semantics)
  per_token_cast_back()     deep_ep/utils/math.py:42-56
  per_token_cast_to_fp8_ll() csrc/kernels/legacy/utils.cuh:477-479,499-501 as used by internode_ll.cu:223-243: the
                            low-latency kernel's own recipe (same payload, stored scale = amax * fp32(1/448)); pinned in
                            tests/test_oracle_fp8.py by exact arithmetic (the product of two fp32 numbers is exact in
                            fp64, one rounding to fp32)
  world_dispatch()          deep_ep/utils/refs.py:10-123 with the process group replaced by an
                            explicit loop over logical source ranks
  dispatch()                one source rank's share of world_dispatch() (refs.py:55-90 send side +
                            refs.py:112-117 localisation per destination), plus the handle fields
                            of deep_ep/include/deep_ep/impls/dispatch.cuh:234-257,336-351 and
                            deep_ep/include/deep_ep/impls/dispatch_copy_epilogue.cuh:104-123,188-207
                            and the deterministic expanded placement of
                            tests/ascend/production/run_two_rank_dispatch.py:474-560
  ordered_accumulate()      deep_ep/utils/refs.py:156-174
  combine_from_lanes()      deep_ep/utils/refs.py:177-243 (grouped ordered reduction)
  combine()                 the same reduction driven from received rows + handle
                            (deep_ep/include/deep_ep/impls/combine.cuh:86-237,
                             combine_reduce_epilogue.cuh:62-142, combine_utils.cuh:111-168)
  intranode_world_dispatch() csrc/kernels/legacy/intranode.cu:20-175 (counts, prefix matrices), :320-400 (send
                            side: row order, local ids, weights zeroed off-rank), :420-545 (receive side:
                            rank offset + channel offset, recv_src_idx, -1 fill), as driven by
                            csrc/legacy/buffer.hpp:417-717; checked by tests/legacy/test_intranode.py:90-186
  intranode_dispatch()      one source rank's share of the above, destinations concatenated
  intranode_combine()       csrc/kernels/legacy/intranode.cu:940-1033 (bias_0 + bias_1, then rows in ascending
                            rank order, fp32, one rounding; top-k weights summed over the same rows)
  ll_dispatch()             csrc/legacy/buffer.hpp:1515-1541 + csrc/kernels/legacy/internode_ll.cu:361-461
  ll_combine()              csrc/kernels/legacy/internode_ll.cu:1072-1135 (BF16 branch :704-711)
  logfmt10_round_trip()     csrc/kernels/legacy/internode_ll.cu:556-637 (encode), :640-712 (decode): pinned in
                            tests/test_oracle_logfmt.py by what the grid construction fixes (a cast value decodes to
                            the nearest grid point, amax and amin survive, error bound, chunk rules, special cases)

Pinning status (which independent evidence fixes each function) is listed in tests/test_oracle_*.py:
layout -> brute force + literal cases; FP8 cast -> C software e4m3 encoder (oracle/fp8_ref.c) +
closed-form identities; dispatch -> world composition vs. the literal two-rank cases and
permutation invariants; combine -> the reference's literal known answers; low latency -> the
invariants the reference's own test asserts; V1 intranode pair -> the assertions of the reference's
tests/legacy/test_intranode.py replayed on a whole logical world + composition of per-source shares.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple, Union

import torch

TensorOrPair = Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]


def ceil_div(a: int, b: int) -> int:
    return -(-a // b)


def align(a: int, b: int) -> int:
    return ceil_div(a, b) * b


# --------------------------------------------------------------------------------------------
# Layout
# --------------------------------------------------------------------------------------------

def layout(topk_idx: torch.Tensor, num_experts: int, num_ranks: int):
    """Counts a dispatch needs: (num_tokens_per_rank[R] i32, num_tokens_per_expert[E] i32,
    is_token_in_rank[T,R] bool).  `-1` entries select nothing.  A token counts once for a rank
    however many of its experts live there; it counts once per (token, lane) for an expert.
    """
    assert topk_idx.dim() == 2 and num_experts % num_ranks == 0
    T, K = topk_idx.shape
    per_rank = num_experts // num_ranks
    idx = topk_idx.to(torch.int64)
    valid = idx >= 0
    num_tokens_per_expert = torch.bincount(idx[valid].flatten(), minlength=num_experts).to(torch.int32)
    dst = torch.where(valid, idx // per_rank, torch.full_like(idx, -1))
    is_token_in_rank = torch.zeros((T, num_ranks), dtype=torch.bool)
    for r in range(num_ranks):
        is_token_in_rank[:, r] = (dst == r).any(dim=1) if K > 0 else False
    num_tokens_per_rank = is_token_in_rank.sum(dim=0).to(torch.int32)
    return num_tokens_per_rank, num_tokens_per_expert, is_token_in_rank


# --------------------------------------------------------------------------------------------
# FP8 cast
# --------------------------------------------------------------------------------------------

def per_token_cast_to_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 [T,H] -> (e4m3fn [T,H], fp32 scales [T, ceil(H/128)]).

    Per 128-channel group: amax = max(|x|) as fp32 clamped below at 1e-4; payload =
    e4m3fn(fp32(x) * (448 / amax)) with round-to-nearest-even; scale = amax / 448.  Both
    divisions are IEEE fp32 divisions.  H is zero-padded to a multiple of 128 for the reduction.
    """
    assert x.dim() == 2
    T, H = x.shape
    Hp = align(H, 128)
    xp = torch.zeros((T, Hp), dtype=torch.float32)
    xp[:, :H] = x.to(torch.float32)
    g = xp.view(T, Hp // 128, 128)
    amax = g.abs().amax(dim=2).clamp(min=1e-4)                       # fp32
    q = (g * (torch.tensor(448.0, dtype=torch.float32) / amax).unsqueeze(2)).to(torch.float8_e4m3fn)
    scales = amax / torch.tensor(448.0, dtype=torch.float32)
    return q.view(T, Hp)[:, :H].contiguous(), scales.view(T, Hp // 128)


def _amax_dropping_nan(g: torch.Tensor) -> torch.Tensor:
    """max(|x|) over the last dimension the way the reference's low-latency kernel takes it: a running fmaxf that
    starts at the 1e-4 floor (csrc/kernels/legacy/internode_ll.cu:223-231).  C's fmaxf returns the other operand when
    one is NaN, so NaN elements do not take part; an infinity does."""
    mag = g.abs()
    mag = torch.where(torch.isnan(mag), torch.zeros_like(mag), mag)
    return mag.amax(dim=-1).clamp(min=1e-4)


def per_token_cast_to_fp8_ll(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """What the reference's low-latency kernel emits without `round_scale` (csrc/kernels/legacy/utils.cuh:477-479,
    499-501; internode_ll.cu:223-243): amax clamped below at 1e-4, payload = e4m3fn(x * (448 / amax)) as in
    per_token_cast_to_fp8, but the stored scale is the fp32 product amax * fp32(1 / 448), not the quotient amax / 448
    (the two differ in the last bit for many amax values).  The maximum is taken with fmaxf: a NaN element encodes as
    NaN but leaves its group's scale alone (the torch recipe above lets it spread over the group)."""
    assert x.dim() == 2 and x.shape[1] % 128 == 0
    T, H = x.shape
    g = x.to(torch.float32).view(T, H // 128, 128)
    amax = _amax_dropping_nan(g)
    q = (g * (torch.tensor(448.0, dtype=torch.float32) / amax).unsqueeze(2)).to(torch.float8_e4m3fn)
    scales = amax * torch.tensor(1.0 / 448.0, dtype=torch.float32)
    return q.view(T, H).contiguous(), scales


def per_token_cast_to_fp8_pow2(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """The `round_scale` variant of the low-latency kernels (csrc/kernels/legacy/utils.cuh:477-503 as used by
    internode_ll.cu:223-243): exponent = ceil(log2(amax * fp32(1/448))) with amax clamped below at 1e-4,
    payload = e4m3fn(x * 2^-exponent), scale = 2^exponent (fp32).  Scaling by a power of two is exact, so the
    only rounding is the e4m3 conversion."""
    assert x.dim() == 2
    T, H = x.shape
    assert H % 128 == 0
    g = x.to(torch.float32).view(T, H // 128, 128)
    amax = _amax_dropping_nan(g)
    ratio = amax * torch.tensor(1.0 / 448.0, dtype=torch.float32)
    mantissa, exponent = torch.frexp(ratio)                         # ratio = mantissa * 2^exponent, 0.5 <= mantissa < 1
    exponent = torch.where(mantissa == 0.5, exponent - 1, exponent)  # ceil(log2(ratio))
    scale_inv = torch.ldexp(torch.ones_like(ratio), exponent)
    q = torch.ldexp(g, (-exponent).unsqueeze(2)).to(torch.float8_e4m3fn)
    return q.view(T, H).contiguous(), scale_inv.view(T, H // 128)


def pack_ue8m0(scales: torch.Tensor) -> torch.Tensor:
    """fp32 power-of-two scales [..., G] -> int32 [..., G / 4]: byte k of pack p is the biased exponent of scale
    4p + k (csrc/kernels/legacy/utils.cuh:505-512, internode_ll.cu:440-457; decode deep_ep/utils/math.py:51-53)."""
    exps = (scales.contiguous().view(torch.int32) >> 23) & 0xff
    exps = exps.view(*scales.shape[:-1], scales.shape[-1] // 4, 4)
    return (exps[..., 0] | (exps[..., 1] << 8) | (exps[..., 2] << 16) | (exps[..., 3] << 24)).to(torch.int32)


def per_token_cast_back(x_fp8: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """Inverse of per_token_cast_to_fp8 up to quantisation: bf16(fp32(q) * scale)."""
    T, H = x_fp8.shape
    if T == 0:
        return torch.empty((0, H), dtype=torch.bfloat16)
    Hp = align(H, 128)
    xp = torch.zeros((T, Hp), dtype=torch.float32)
    xp[:, :H] = x_fp8.to(torch.float32)
    out = xp.view(T, Hp // 128, 128) * scales.to(torch.float32).reshape(T, Hp // 128, 1)
    return out.view(T, Hp)[:, :H].to(torch.bfloat16).contiguous()


# --------------------------------------------------------------------------------------------
# Dispatch
# --------------------------------------------------------------------------------------------

@dataclass
class DispatchResult:
    """Everything one source rank's dispatch produces (tensors on CPU)."""
    recv_x: torch.Tensor
    recv_sf: Optional[torch.Tensor]
    recv_topk_idx: Optional[torch.Tensor]
    recv_topk_weights: Optional[torch.Tensor]
    num_recv_tokens: int
    num_expanded_tokens: int
    num_recv_tokens_per_expert_list: List[int]
    psum_num_recv_tokens_per_scaleup_rank: torch.Tensor
    psum_num_recv_tokens_per_expert: torch.Tensor
    num_unaligned_recv_tokens_per_expert: torch.Tensor
    recv_src_metadata: torch.Tensor
    dst_buffer_slot_idx: torch.Tensor
    # which rows of an expanded recv_x are real (not alignment padding)
    expanded_row_is_valid: Optional[torch.Tensor] = None


def _unpack(x: TensorOrPair):
    return x if isinstance(x, tuple) else (x, None)


def dispatch(x: TensorOrPair, topk_idx: torch.Tensor, topk_weights: Optional[torch.Tensor],
             num_experts: int, num_ranks: int, rank_idx: int, num_max_tokens_per_rank: int,
             expert_alignment: int = 1, do_expand: bool = False,
             fill_value: float = 0.0) -> DispatchResult:
    """What source rank `rank_idx` contributes to every logical destination rank.

    Compact layout: rows grouped by destination rank d = 0..R-1, token-ascending inside a group
    (the send-side order of refs.py:62-89); recv_topk_idx is localised to d (idx - d*E_l, or -1).
    Expanded layout: one row per valid (token, lane), grouped by global expert id, each expert
    region starting at the running sum of alignment-padded counts; inside a region rows follow
    (token, lane) order.  Padding rows are filled with `fill_value` (the do_zero_padding result
    when 0); callers that do not zero-pad must ignore rows where expanded_row_is_valid is False.

    Handle fields follow the CUDA conventions: the master lane of a (token, destination) pair is
    the HIGHEST lane routed there; dst_buffer_slot_idx holds rank_idx*M + slot on master lanes
    and -1 elsewhere; recv_src_metadata[:,0] = rank_idx*M + token, [:,1] = rank_idx*K + master
    lane, [:,2+k] = expanded row of lane k (or -1; all -1 in the compact layout).
    psum_num_recv_tokens_per_expert is, per global expert, the inclusive prefix of aligned counts
    (compact) or region start + actual count (expanded).
    """
    xv, sf = _unpack(x)
    T, H = xv.shape
    K = topk_idx.shape[1]
    R, E, M, A = num_ranks, num_experts, num_max_tokens_per_rank, expert_alignment
    assert E % R == 0 and T <= M
    E_l = E // R
    idx = topk_idx.to(torch.int64)
    valid = idx >= 0
    dst = torch.where(valid, idx // E_l, torch.full_like(idx, -1))
    lane_ids = torch.arange(K, dtype=torch.int64)

    tok_parts, dst_parts, master_parts, rank_counts = [], [], [], []
    dst_slot = torch.full((T, K), -1, dtype=torch.int32)
    row_of_td = torch.full((T, R), -1, dtype=torch.int64)     # compact row of (token, destination)
    base = 0
    for d in range(R):
        hit = (dst == d)
        toks = hit.any(dim=1).nonzero(as_tuple=True)[0] if K > 0 else torch.empty(0, dtype=torch.int64)
        n = toks.numel()
        rank_counts.append(n)
        if n:
            master = torch.where(hit[toks], lane_ids, torch.full_like(lane_ids, -1)).amax(dim=1)   # highest lane
            dst_slot[toks, master] = (rank_idx * M + torch.arange(n)).to(torch.int32)
            row_of_td[toks, d] = base + torch.arange(n)
            tok_parts.append(toks)
            dst_parts.append(torch.full((n,), d, dtype=torch.int64))
            master_parts.append(master)
        base += n
    N = base
    tok = torch.cat(tok_parts) if tok_parts else torch.empty(0, dtype=torch.int64)
    dvec = torch.cat(dst_parts) if dst_parts else torch.empty(0, dtype=torch.int64)
    mvec = torch.cat(master_parts) if master_parts else torch.empty(0, dtype=torch.int64)

    psum_rank = torch.tensor(rank_counts, dtype=torch.int64).cumsum(0).to(torch.int32)

    # Per-expert counts and region starts
    counts = torch.bincount(idx[valid].flatten(), minlength=E)
    aligned = ((counts + A - 1) // A) * A
    starts = aligned.cumsum(0) - aligned
    num_expanded = int(aligned.sum().item())
    psum_expert = (starts + counts) if do_expand else aligned.cumsum(0)

    meta = torch.full((N, K + 2), -1, dtype=torch.int32)
    if N:
        meta[:, 0] = (rank_idx * M + tok).to(torch.int32)
        meta[:, 1] = (rank_idx * K + mvec).to(torch.int32)

    expanded_valid = None
    if not do_expand:
        recv_x = xv[tok]
        recv_sf = sf[tok] if sf is not None else None
        sel = idx[tok]
        lo = (dvec * E_l).unsqueeze(1)
        local = (sel >= lo) & (sel < lo + E_l)
        recv_topk_idx = torch.where(local, sel - lo, torch.full_like(sel, -1)).to(topk_idx.dtype)
        recv_w = topk_weights[tok] if topk_weights is not None else None
    else:
        # (token, lane) pairs in row-major order; stable sort by expert keeps that order inside a region
        flat_e = idx.flatten()
        flat_valid = flat_e >= 0
        pair = flat_valid.nonzero(as_tuple=True)[0]              # flattened (t*K + k), ascending
        e_of_pair = flat_e[pair]
        order = torch.sort(e_of_pair, stable=True).indices
        sorted_pair = pair[order]
        sorted_e = e_of_pair[order]
        excl = counts.cumsum(0) - counts
        within = torch.arange(sorted_e.numel()) - excl[sorted_e]
        rows = starts[sorted_e] + within                          # expanded row of each sorted pair
        t_of = sorted_pair // K if K > 0 else sorted_pair
        k_of = sorted_pair % K if K > 0 else sorted_pair

        def filled(shape, dtype):
            if dtype.is_floating_point:
                return torch.full(shape, fill_value, dtype=torch.float32).to(dtype)
            return torch.zeros(shape, dtype=dtype)

        recv_x = filled((num_expanded, H), xv.dtype)
        recv_x[rows] = xv[t_of]
        recv_sf = None
        if sf is not None:
            recv_sf = filled((num_expanded, sf.shape[1]), sf.dtype)
            recv_sf[rows] = sf[t_of]
        recv_w = None
        if topk_weights is not None:
            recv_w = filled((num_expanded,), torch.float32)
            recv_w[rows] = topk_weights[t_of, k_of]
        recv_topk_idx = None
        expanded_valid = torch.zeros((num_expanded,), dtype=torch.bool)
        expanded_valid[rows] = True
        meta[row_of_td[t_of, sorted_e // E_l], 2 + k_of] = rows.to(torch.int32)

    return DispatchResult(
        recv_x=recv_x, recv_sf=recv_sf, recv_topk_idx=recv_topk_idx, recv_topk_weights=recv_w,
        num_recv_tokens=N, num_expanded_tokens=num_expanded,
        num_recv_tokens_per_expert_list=aligned.tolist(),
        psum_num_recv_tokens_per_scaleup_rank=psum_rank,
        psum_num_recv_tokens_per_expert=psum_expert.to(torch.int32),
        num_unaligned_recv_tokens_per_expert=counts.to(torch.int32),
        recv_src_metadata=meta, dst_buffer_slot_idx=dst_slot,
        expanded_row_is_valid=expanded_valid)


def world_dispatch(xs: Sequence[TensorOrPair], topk_idxs: Sequence[torch.Tensor],
                   topk_weights: Sequence[Optional[torch.Tensor]],
                   num_max_tokens_per_rank: int, num_experts: int):
    """All logical ranks at once: what every destination rank receives from every source rank.

    This is refs.py:10-123 with `all_to_all_single` replaced by list slicing.  Returns, per
    destination rank: (recv_x or (recv_x, recv_sf), recv_topk_idx, recv_topk_weights,
    recv_src_token_idx, num_recv_tokens_per_rank).  Rows are ordered by (source rank, token).
    """
    R = len(xs)
    E_l = num_experts // R
    out = []
    for d in range(R):
        px, psf, pidx, pw, psrc, pcnt = [], [], [], [], [], []
        for s in range(R):
            xv, sf = _unpack(xs[s])
            idx = topk_idxs[s].to(torch.int64)
            lo, hi = d * E_l, (d + 1) * E_l
            inside = (idx >= lo) & (idx < hi)
            toks = inside.any(dim=1).nonzero(as_tuple=True)[0]
            pcnt.append(toks.numel())
            px.append(xv[toks])
            if sf is not None:
                psf.append(sf[toks])
            sel = idx[toks]
            pidx.append(torch.where(inside[toks], sel - lo, torch.full_like(sel, -1)).to(topk_idxs[s].dtype))
            if topk_weights[s] is not None:
                pw.append(topk_weights[s][toks])
            psrc.append((toks + s * num_max_tokens_per_rank).to(torch.int32))
        rx = torch.cat(px, 0)
        rsf = torch.cat(psf, 0) if psf else None
        out.append(((rx, rsf) if rsf is not None else rx, torch.cat(pidx, 0),
                    torch.cat(pw, 0) if pw else None, torch.cat(psrc, 0),
                    torch.tensor(pcnt, dtype=torch.int32)))
    return out


# --------------------------------------------------------------------------------------------
# Combine
# --------------------------------------------------------------------------------------------

def ordered_accumulate(data: torch.Tensor, initial: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 running sum over dim 1 in index order, a single rounding to data.dtype at the end."""
    T, K, H = data.shape
    acc = torch.zeros((T, H), dtype=torch.float32) if initial is None else initial.to(torch.float32).clone()
    for k in range(K):
        acc = acc + data[:, k, :].to(torch.float32)
    return acc.to(data.dtype)


def _bias_sum(bias):
    if bias is None:
        return None
    if isinstance(bias, (tuple, list)):
        b0, b1 = bias
        if b1 is None:
            return b0.to(torch.float32)
        return b0.to(torch.float32) + b1.to(torch.float32)
    return bias.to(torch.float32)


def combine_from_lanes(y: torch.Tensor, topk_idx: torch.Tensor, num_experts: int, num_ranks: int,
                       bias=None, reduce_in_rank: bool = True) -> torch.Tensor:
    """Reduce per-(token, lane) expert outputs y[T,K,H] (bf16; lanes with idx -1 must be zero).

    reduce_in_rank=True  (the default direct mode with multiple reduction): the lanes that share a
    destination rank are first summed in fp32 in lane order and rounded to bf16 (one row comes
    back per rank); the per-rank partials are then added in fp32, in ascending order of each
    group's last lane, on top of the fp32 bias sum, and rounded once.
    reduce_in_rank=False (expanded layout without multiple reduction): all K lanes are added in
    lane order in fp32 on top of the bias sum and rounded once.
    """
    T, K, H = y.shape
    E_l = num_experts // num_ranks
    idx = topk_idx.to(torch.int64)
    data = y
    if reduce_in_rank and K > 0:
        grp = torch.where(idx >= 0, idx // E_l, torch.full_like(idx, -1))
        lane_ids = torch.arange(K, dtype=torch.int64)
        partial = torch.zeros_like(y)
        rows = torch.arange(T)
        for g in grp.unique().tolist():          # includes -1: lanes that carry zeros
            member = (grp == g)
            has = member.any(dim=1)
            acc = torch.zeros((T, H), dtype=torch.float32)
            for k in range(K):
                acc = acc + y[:, k, :].to(torch.float32) * member[:, k].unsqueeze(1)
            last = torch.where(member, lane_ids, torch.full_like(lane_ids, -1)).amax(dim=1)
            sel = rows[has]
            partial[sel, last[has]] = acc[has].to(y.dtype)
        data = partial
    return ordered_accumulate(data, _bias_sum(bias))


def combine(x: torch.Tensor, handle_topk_idx: torch.Tensor, recv_src_metadata: torch.Tensor,
            dst_buffer_slot_idx: torch.Tensor, psum_rank: torch.Tensor,
            num_experts: int, num_ranks: int, rank_idx: int, num_max_tokens_per_rank: int,
            topk_weights: Optional[torch.Tensor] = None, bias=None,
            do_expand: bool = False, allow_multiple_reduction: bool = True):
    """Combine driven from received rows.  `x` is [N_recv, H] (compact) or [N_expanded, H].

    Returns (combined_x[T,H] bf16, combined_topk_weights[T,K] fp32 or None).  The weights are
    never multiplied into the activations; they travel back to the lane that owns them (0 for
    lanes with idx -1).
    """
    T, K = handle_topk_idx.shape
    H = x.shape[1]
    R, E, M = num_ranks, num_experts, num_max_tokens_per_rank
    E_l = E // R
    idx = handle_topk_idx.to(torch.int64)
    valid = idx >= 0
    grp = torch.where(valid, idx // E_l, torch.full_like(idx, -1))
    starts = torch.cat([torch.zeros(1, dtype=torch.int64), psum_rank.to(torch.int64)[:-1]])
    lane_ids = torch.arange(K, dtype=torch.int64)
    # master lane (highest lane of the same destination) for every valid lane
    same = (grp.unsqueeze(2) == grp.unsqueeze(1)) & valid.unsqueeze(2)        # [T, K, K]
    master = torch.where(same, lane_ids.view(1, 1, K), torch.full((1, 1, 1), -1, dtype=torch.int64)).amax(dim=2)
    master_c = master.clamp(min=0)
    slot = dst_buffer_slot_idx.to(torch.int64).gather(1, master_c) - rank_idx * M
    row = starts[grp.clamp(min=0)] + slot                                      # compact row per lane
    row = torch.where(valid, row, torch.zeros_like(row))

    y = torch.zeros((T, K, H), dtype=x.dtype)
    w_out = torch.zeros((T, K), dtype=torch.float32) if topk_weights is not None else None
    tt, kk = valid.nonzero(as_tuple=True)
    if do_expand:
        er = recv_src_metadata.to(torch.int64)[row[tt, kk], 2 + kk]
        y[tt, kk] = x[er]
        if w_out is not None:
            w_out[tt, kk] = topk_weights[er]
    else:
        is_master = valid & (master == lane_ids.view(1, K))
        mt, mk = is_master.nonzero(as_tuple=True)
        y[mt, mk] = x[row[mt, mk]]
        if w_out is not None:
            w_out[tt, kk] = topk_weights[row[tt, kk], kk]
    reduce_in_rank = (not do_expand) or allow_multiple_reduction
    out = combine_from_lanes(y, idx, E, R, bias, reduce_in_rank=reduce_in_rank)
    return out, w_out


# --------------------------------------------------------------------------------------------
# Low-latency packed layout
# --------------------------------------------------------------------------------------------

def ll_dispatch(xs: Sequence[torch.Tensor], topk_idxs: Sequence[torch.Tensor],
                num_max_dispatch_tokens_per_rank: int, num_experts: int, num_ranks: int,
                dst_rank: int, use_fp8: bool = True, round_scale: bool = False):
    """What logical destination rank `dst_rank` holds after every source rank in `xs` has sent.

    xs[s] is source rank s's bf16 [T_s, H]; entries may be None (that source sends nothing).
    Output: packed_recv_x [E_l, R*M, H] (fp8 or bf16), packed scales [E_l, R*M, H/128] fp32 whose
    last two dims are column-major in memory (returned here as a plain logical tensor),
    packed_recv_count [E_l] i32, packed_recv_src_info [E_l, R*M] i32 (token index within its
    source rank), packed_recv_layout_range [E_l, R] i64 = (begin << 32) | count.  Fill order is
    source rank ascending, then token ascending.  Rows at or beyond count[e] are unspecified
    (zero here).
    """
    R, M, E = num_ranks, num_max_dispatch_tokens_per_rank, num_experts
    E_l = E // R
    H = next(x for x in xs if x is not None).shape[1]
    px = torch.zeros((E_l, R * M, H), dtype=torch.float8_e4m3fn if use_fp8 else torch.bfloat16)
    ps = torch.zeros((E_l, R * M, H // 128), dtype=torch.float32) if use_fp8 else None
    cnt = torch.zeros((E_l,), dtype=torch.int32)
    src_info = torch.zeros((E_l, R * M), dtype=torch.int32)
    layout_range = torch.zeros((E_l, R), dtype=torch.int64)
    for s in range(R):
        if s >= len(xs) or xs[s] is None:
            continue
        x = xs[s]
        idx = topk_idxs[s].to(torch.int64)
        if use_fp8:
            q, sc = per_token_cast_to_fp8_pow2(x) if round_scale else per_token_cast_to_fp8_ll(x)
        for le in range(E_l):
            e = dst_rank * E_l + le
            toks = (idx == e).any(dim=1).nonzero(as_tuple=True)[0]
            n = toks.numel()
            b = int(cnt[le])
            layout_range[le, s] = (b << 32) | n
            if n:
                if use_fp8:
                    px[le, b:b + n] = q[toks]
                    ps[le, b:b + n] = sc[toks]
                else:
                    px[le, b:b + n] = x[toks]
                src_info[le, b:b + n] = toks.to(torch.int32)
            cnt[le] = b + n
    return px, ps, cnt, src_info, layout_range


def logfmt10_round_trip(x: torch.Tensor) -> torch.Tensor:
    """What a receiver decodes from rows sent through the LogFMT-10 codec of the reference's low-latency combine
    (csrc/kernels/legacy/internode_ll.cu:556-637 encode, :640-712 decode, chunking :754-756 and :876-885), with exact
    log2 / exp2 in fp64 where the reference uses its hardware's approximations.

    x: bf16 [..., H], H % 512 == 0.  Returns fp32 of the same shape.  Per group of 128 channels: amax, amin of |x|;
    log_amin = max(log2(amin), log_amax - 32) (amin == 0: log_amax - 32).  A chunk (1024 channels when H % 1024 == 0,
    else 512: what one warp of the send loop stages) is cast iff every group in it has log_amax < 0 and
    log_amin < log_amax; other chunks pass unchanged.  Cast value: sign and
    code = floor(max(log2|x| / step + rounding - log_amin / step, 0)) with step = (log_amax - log_amin) / 510 and
    rounding = 2 - log2((1 + 2^step) / 2) / step; decoded = 0 for code 0, else 2^((code - 1) * step + log_amin).
    """
    import numpy as np
    assert x.dtype == torch.bfloat16 and x.shape[-1] % 512 == 0
    H = x.shape[-1]
    chunk_groups = (1024 if H % 1024 == 0 else 512) // 128
    v = x.to(torch.float64).numpy().reshape(-1, H // 128, 128)
    mag = np.abs(v)
    with np.errstate(divide="ignore", invalid="ignore"):
        amax, amin = mag.max(axis=2), mag.min(axis=2)
        log_amax = np.log2(amax)
        log_amin = np.where(amin == 0, log_amax - 32.0, np.maximum(np.log2(amin), log_amax - 32.0))
        castable = (log_amax < 0) & (log_amin < log_amax)
        chunk_ok = castable.reshape(castable.shape[0], -1, chunk_groups).all(axis=2, keepdims=True)
        chunk_ok = np.broadcast_to(chunk_ok, (castable.shape[0], castable.shape[1] // chunk_groups, chunk_groups)).reshape(castable.shape)
        step = ((log_amax - log_amin) / 510.0)[:, :, None]
        step_inv = 1.0 / step
        rounding = 2.0 - np.log2((1.0 + np.exp2(step)) * 0.5) * step_inv
        fused = rounding - log_amin[:, :, None] * step_inv
        code = np.floor(np.maximum(np.log2(mag) * step_inv + fused, 0.0))
        decoded = np.where(code == 0, 0.0, np.exp2((code - 1.0) * step + log_amin[:, :, None]))
    decoded = np.where(np.signbit(v), -decoded, decoded)
    out = np.where(chunk_ok[:, :, None], decoded, v)
    return torch.from_numpy(out.reshape(x.shape).astype(np.float32))


def ll_combine(x: torch.Tensor, topk_idx: torch.Tensor, topk_weights: torch.Tensor,
               src_info: torch.Tensor, layout_range: torch.Tensor, src_rank: int,
               num_experts: int, num_ranks: int, dst_rank: int, use_logfmt: bool = False) -> torch.Tensor:
    """Weighted reduce back to source rank `src_rank`'s token order.

    x is [E_l, R*M, H] bf16 held by `dst_rank`.  out[t] = bf16( sum over lanes k in order with
    topk_idx[t,k] on dst_rank of  w[t,k] * float(x[e_local, row(t,k)]) ), accumulated with
    separate fp32 multiply and add.  Lanes routed to other ranks contribute nothing here.
    With use_logfmt every row first passes through logfmt10_round_trip.
    """
    T, K = topk_idx.shape
    E_l = num_experts // num_ranks
    H = x.shape[2]
    idx = topk_idx.to(torch.int64)
    out = torch.zeros((T, H), dtype=torch.float32)
    row_of = {}
    for le in range(E_l):
        packed = int(layout_range[le, src_rank])
        b, n = packed >> 32, packed & 0xFFFFFFFF
        for i in range(n):
            row_of[(le, int(src_info[le, b + i]))] = b + i
    for t in range(T):
        for k in range(K):
            e = int(idx[t, k])
            if e < 0 or e // E_l != dst_rank:
                continue
            le = e - dst_rank * E_l
            r = row_of[(le, t)]
            row = logfmt10_round_trip(x[le, r]) if use_logfmt else x[le, r].to(torch.float32)
            out[t] = out[t] + row * topk_weights[t, k]
    return out.to(torch.bfloat16)


# ---------------------------------------------------------------------------------------------
# V1 dispatch / combine inside one scale-up domain ("intranode")
# ---------------------------------------------------------------------------------------------
def channel_range(num_tokens: int, num_channels: int, channel: int) -> Tuple[int, int]:
    """csrc/kernels/legacy/utils.cuh:444-448."""
    per = ceil_div(num_tokens, num_channels)
    start = min(per * channel, num_tokens)
    return start, min(start + per, num_tokens)


@dataclass
class IntranodeRecv:
    """What one destination rank holds after a V1 dispatch of a whole logical world."""
    recv_x: torch.Tensor
    recv_x_scales: Optional[torch.Tensor]
    recv_topk_idx: Optional[torch.Tensor]
    recv_topk_weights: Optional[torch.Tensor]
    recv_src_idx: torch.Tensor
    num_recv_tokens_per_expert_list: List[int]
    rank_prefix_matrix: torch.Tensor           # [R, R], identical on every rank
    recv_channel_prefix_matrix: torch.Tensor   # [R, C]: start of (source, channel) inside the source's rows


def _channel_prefix(mask: torch.Tensor, num_channels: int) -> torch.Tensor:
    T, R = mask.shape
    out = torch.zeros((R, num_channels), dtype=torch.int32)
    for c in range(num_channels):
        lo, hi = channel_range(T, num_channels, c)
        out[:, c] = mask[lo:hi].sum(dim=0).to(torch.int32)
    return out.cumsum(dim=1).to(torch.int32)


def intranode_world_dispatch(xs: Sequence[TensorOrPair], masks: Sequence[torch.Tensor],
                             topk_idxs: Optional[Sequence[torch.Tensor]], topk_weights: Optional[Sequence[torch.Tensor]],
                             num_experts: int, expert_alignment: int = 1, num_channels: int = 10):
    """Returns (per-destination IntranodeRecv list, per-source channel_prefix_matrix list)."""
    R = len(xs)
    E_l = num_experts // R if num_experts else 0
    with_topk = topk_idxs is not None
    counts = torch.stack([m.sum(dim=0).to(torch.int32) for m in masks])           # [source, destination]
    rank_prefix = counts.cumsum(dim=0).to(torch.int32)
    channel_prefix = [_channel_prefix(m, num_channels) for m in masks]
    out = []
    for j in range(R):
        rows_x, rows_s, rows_idx, rows_w, rows_src = [], [], [], [], []
        for i in range(R):
            x, sf = _unpack(xs[i])
            sel = masks[i][:, j].nonzero().flatten()                               # token order
            rows_x.append(x[sel])
            if sf is not None:
                rows_s.append(sf[sel])
            rows_src.append(sel.to(torch.int32))
            if with_topk:
                idx = topk_idxs[i][sel]
                local = (idx >= j * E_l) & (idx < (j + 1) * E_l)
                rows_idx.append(torch.where(local, idx - j * E_l, torch.full_like(idx, -1)))
                rows_w.append(torch.where(local, topk_weights[i][sel], torch.zeros_like(topk_weights[i][sel])))
        per_expert = []
        if with_topk:
            stacked = torch.cat([t.flatten() for t in topk_idxs])
            for e in range(j * E_l, (j + 1) * E_l):
                per_expert.append(align(int((stacked == e).sum()), expert_alignment))
        recv_channel = torch.zeros((R, num_channels), dtype=torch.int32)
        for i in range(R):
            recv_channel[i, 1:] = channel_prefix[i][j, :-1]
        out.append(IntranodeRecv(
            recv_x=torch.cat(rows_x), recv_x_scales=torch.cat(rows_s) if rows_s else None,
            recv_topk_idx=torch.cat(rows_idx) if with_topk else None,
            recv_topk_weights=torch.cat(rows_w) if with_topk else None,
            recv_src_idx=torch.cat(rows_src), num_recv_tokens_per_expert_list=per_expert,
            rank_prefix_matrix=rank_prefix, recv_channel_prefix_matrix=recv_channel))
    return out, channel_prefix


@dataclass
class IntranodeShare:
    """One source rank's contribution, destinations concatenated in rank order (what a one-GPU call returns)."""
    recv_x: torch.Tensor
    recv_x_scales: Optional[torch.Tensor]
    recv_topk_idx: Optional[torch.Tensor]
    recv_topk_weights: Optional[torch.Tensor]
    recv_src_idx: torch.Tensor
    num_recv_tokens_per_expert_list: List[int]
    rank_prefix_matrix: torch.Tensor
    channel_prefix_matrix: torch.Tensor
    recv_channel_prefix_matrix: torch.Tensor
    send_head: torch.Tensor                    # [T, R]: row of the concatenated receive buffer, or -1


def intranode_dispatch(x: TensorOrPair, mask: torch.Tensor, topk_idx: Optional[torch.Tensor],
                       topk_weights: Optional[torch.Tensor], num_experts: int, num_ranks: int, rank: int,
                       expert_alignment: int = 1, num_channels: int = 10) -> IntranodeShare:
    R = num_ranks
    T = mask.shape[0]
    data, sf = _unpack(x)
    # A world in which only `rank` holds tokens
    empty_mask = torch.zeros((0, R), dtype=torch.bool)
    xs = [(data[:0], sf[:0]) if sf is not None else data[:0] for _ in range(R)]
    masks = [empty_mask for _ in range(R)]
    idxs = [topk_idx[:0] for _ in range(R)] if topk_idx is not None else None
    ws = [topk_weights[:0] for _ in range(R)] if topk_idx is not None else None
    xs[rank], masks[rank] = x, mask
    if topk_idx is not None:
        idxs[rank], ws[rank] = topk_idx, topk_weights
    world, channel_prefix = intranode_world_dispatch(xs, masks, idxs, ws, num_experts, expert_alignment, num_channels)
    send_head = torch.full((T, R), -1, dtype=torch.int32)
    base = 0
    for j in range(R):
        sel = mask[:, j].nonzero().flatten()
        send_head[sel, j] = base + torch.arange(sel.numel(), dtype=torch.int32)
        base += sel.numel()
    cat = lambda parts: torch.cat(parts) if parts[0] is not None else None
    return IntranodeShare(
        recv_x=torch.cat([w.recv_x for w in world]),
        recv_x_scales=cat([w.recv_x_scales for w in world]),
        recv_topk_idx=cat([w.recv_topk_idx for w in world]),
        recv_topk_weights=cat([w.recv_topk_weights for w in world]),
        recv_src_idx=torch.cat([w.recv_src_idx for w in world]),
        num_recv_tokens_per_expert_list=[c for w in world for c in w.num_recv_tokens_per_expert_list],
        rank_prefix_matrix=world[0].rank_prefix_matrix,
        channel_prefix_matrix=channel_prefix[rank],
        recv_channel_prefix_matrix=torch.stack([w.recv_channel_prefix_matrix[rank] for w in world]),
        send_head=send_head)


def intranode_combine(x: torch.Tensor, send_head: torch.Tensor, topk_weights: Optional[torch.Tensor] = None,
                      bias=None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """x: [rows, H] bf16 laid out like the dispatched rows; returns (combined_x [T, H], combined weights)."""
    T, R = send_head.shape
    H = x.shape[1]
    acc = _bias_sum(bias)
    acc = torch.zeros((T, H), dtype=torch.float32) if acc is None else acc.clone()
    w_out = None if topk_weights is None else torch.zeros((T, topk_weights.shape[1]), dtype=torch.float32)
    for j in range(R):
        rows = send_head[:, j].long()
        has = rows >= 0
        acc[has] = acc[has] + x[rows[has]].to(torch.float32)
        if w_out is not None:
            w_out[has] = w_out[has] + topk_weights[rows[has]]
    return acc.to(torch.bfloat16), w_out
