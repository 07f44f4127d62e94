"""Every BF16 bit pattern - zeros, subnormals, the whole finite range, +-Inf and all NaN patterns - through the three FP8
casts of the library (stand-alone cast, the cast fused into dispatch, the low-latency cast without and with
`round_scale`), byte for byte against the oracle.

Layout: 128-channel groups in which every pattern meets several group maxima -
  * the patterns in numeric order (neighbours share a group: groups of only zeros / subnormals, of only NaNs, with Inf),
  * two stride permutations (every group mixes all exponents; most groups hold a NaN and an Inf),
  * the finite patterns again in groups led by a fixed maximum: below the 1e-4 floor, 1, 448, the largest finite BF16
    and a subnormal (so that each finite pattern is scaled by several different factors without a NaN or Inf around).
A NaN result may carry either sign (the sign of a NaN that an fp32 multiply hands on is not fixed across processors):
NaN codes compare equal to NaN codes, NaN scales to NaN scales; everything else must match bit for bit.
"""
import pytest
import torch

import routing_oracle as oracle

pytestmark = pytest.mark.gpu

H = 1024


def _pattern_rows(allow_inf=True, allow_nan=True):
    allp = torch.arange(65536, dtype=torch.int32)
    keep = torch.ones(65536, dtype=torch.bool)
    mag = allp & 0x7fff
    if not allow_inf:
        keep &= mag != 0x7f80
    if not allow_nan:
        keep &= mag <= 0x7f80
    parts = []
    base = allp[keep]
    pad = (-base.numel()) % 128
    base = torch.cat([base, base[:pad]])
    parts.append(base)                                                    # numeric order
    n = base.numel()
    for stride in (257, 12289):                                           # odd strides: permutations of the n positions when gcd = 1
        order = (torch.arange(n, dtype=torch.int64) * stride) % n
        assert order.unique().numel() == n
        parts.append(base[order])
    finite = allp[mag < 0x7f80]
    for leader in (0x3880, 0x3f80, 0x43e0, 0x7f7f, 0x0040):               # 6.1e-5 (below the floor), 1.0, 448.0, 3.39e38, a subnormal
        f = finite[: finite.numel() // 127 * 127].view(-1, 127)
        parts.append(torch.cat([torch.full((f.shape[0], 1), leader, dtype=torch.int32), f], dim=1).reshape(-1))
    flat = torch.cat(parts)
    flat = torch.cat([flat, torch.zeros((-flat.numel()) % H, dtype=torch.int32)])
    return flat.to(torch.int16).view(torch.bfloat16).view(-1, H).contiguous()


def _assert_codes(got_q, got_s, ref_q, ref_s, what):
    g, r = got_q.cpu().view(torch.uint8), ref_q.view(torch.uint8)
    assert g.shape == r.shape, what
    g_nan, r_nan = (g & 0x7f) == 0x7f, (r & 0x7f) == 0x7f
    bad = (g_nan != r_nan) | (~r_nan & (g != r))
    assert not bad.any(), f"{what}: {int(bad.sum())} payload bytes differ, first at {bad.nonzero()[0].tolist()}: " \
                          f"{int(g[tuple(bad.nonzero()[0])])} != {int(r[tuple(bad.nonzero()[0])])}"
    gs, rs = got_s.cpu().float().contiguous(), ref_s.float().contiguous()
    assert gs.shape == rs.shape, what
    s_bad = (torch.isnan(gs) != torch.isnan(rs)) | (~torch.isnan(rs) & (gs.view(torch.int32) != rs.view(torch.int32)))
    assert not s_bad.any(), f"{what}: {int(s_bad.sum())} scales differ, first at {s_bad.nonzero()[0].tolist()}"
    return int(r_nan.sum()), int(torch.isnan(rs).sum()), int(torch.isinf(rs).sum())


def test_stand_alone_cast_on_every_bf16_pattern():
    from deep_ep.utils.math import per_token_cast_to_fp8
    x = _pattern_rows()
    q, s = per_token_cast_to_fp8(x.cuda())
    ref_q, ref_s = oracle.per_token_cast_to_fp8(x)
    nan_bytes, nan_scales, inf_scales = _assert_codes(q, s, ref_q, ref_s, "stand-alone cast")
    assert nan_scales > 100 and inf_scales >= 2 and nan_bytes > 128 * nan_scales      # the NaN groups are really in there


def test_fused_dispatch_cast_on_every_bf16_pattern():
    import deep_ep
    x = _pattern_rows()
    T = x.shape[0]
    idx = torch.zeros((T, 1), dtype=torch.int64)                          # every token to expert 0 of the only rank
    buf = deep_ep.ElasticBuffer(deep_ep.LogicalGroup(0, 1), num_max_tokens_per_rank=T, hidden=H, num_topk=1)
    for launches in (1, 2):
        deep_ep.tuning.dispatch_launches = launches
        try:
            (q, s), _, _, handle, _ = buf.dispatch(x.cuda(), idx.cuda(), None, num_experts=1, cast_to_fp8=True)
        finally:
            deep_ep.tuning.dispatch_launches = 0
        assert q.shape[0] == T
        ref_q, ref_s = oracle.per_token_cast_to_fp8(x)
        _assert_codes(q, s, ref_q, ref_s, f"fused dispatch cast ({launches} launches)")
    buf.check_device_status()


@pytest.mark.parametrize("round_scale", [False, True])
def test_low_latency_cast_on_every_bf16_pattern(round_scale):
    """The low-latency kernel's maximum drops NaNs (fmaxf, csrc/kernels/legacy/internode_ll.cu:223-231).  With
    `round_scale` an infinite maximum is outside what the reference's exponent arithmetic defines
    (csrc/kernels/legacy/utils.cuh:481-498 shifts an exponent of 128 into the sign bit), so infinities stay out of
    that input."""
    import deep_ep
    x = _pattern_rows(allow_inf=not round_scale)
    T = x.shape[0]
    M = (T + 3) // 4 * 4
    buf = deep_ep.Buffer(deep_ep.LogicalGroup(0, 1), low_latency_mode=True)
    idx = torch.zeros((T, 1), dtype=torch.int64)
    (q, s), count, handle, _, _ = buf.low_latency_dispatch(x.cuda(), idx.cuda(), M, 1, use_fp8=True, round_scale=round_scale)
    assert int(count[0]) == T
    assert torch.equal(handle[0][0, :T].cpu(), torch.arange(T, dtype=torch.int32))          # rows in token order
    ref_q, ref_s = (oracle.per_token_cast_to_fp8_pow2 if round_scale else oracle.per_token_cast_to_fp8_ll)(x)
    nan_bytes, nan_scales, inf_scales = _assert_codes(q[0, :T], s[0, :T], ref_q, ref_s, f"low-latency cast (round_scale={round_scale})")
    assert nan_scales == 0 and nan_bytes > 0 and (inf_scales > 0) == (not round_scale)
