"""Pins the FP8 cast of the oracle (CPU only).

Three independent statements of the same arithmetic must agree bit for bit:
  * oracle.per_token_cast_to_fp8 (torch eager; the conversion itself is the torch library routine),
  * oracle/fp8_ref.c (plain C: nearest-representable search, volatile fp32 arithmetic),
  * closed-form facts of the format and of the recipe.
A dropped clamp, a reciprocal-multiply instead of the division, truncation instead of round-to-nearest-even
or a wrong subnormal boundary each fail at least one test below.
"""
import ctypes
import os
import subprocess

import numpy as np
import pytest
import torch

import routing_oracle as oracle

ORACLE_DIR = os.path.dirname(os.path.abspath(oracle.__file__))


@pytest.fixture(scope="module")
def cref():
    lib = os.path.join(ORACLE_DIR, "libfp8_ref.so")
    if not os.path.exists(lib):
        subprocess.run(["make", "-C", ORACLE_DIR, lib], check=True, capture_output=True)
    h = ctypes.CDLL(lib)
    h.oracle_e4m3_from_f32.restype = ctypes.c_uint8
    h.oracle_e4m3_from_f32.argtypes = [ctypes.c_float]
    h.oracle_cast_1x128.restype = None
    h.oracle_cast_1x128.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
    h.oracle_ordered_sum_bf16.restype = None
    h.oracle_ordered_sum_bf16.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
    return h


def c_cast(cref, x_bf16):
    T, H = x_bf16.shape
    xin = x_bf16.contiguous().view(torch.int16).numpy().copy()
    out = np.zeros((T, H), dtype=np.uint8)
    scales = np.zeros((T, (H + 127) // 128), dtype=np.float32)
    cref.oracle_cast_1x128(xin.ctypes.data, T, H, out.ctypes.data, scales.ctypes.data)
    return torch.from_numpy(out), torch.from_numpy(scales)


def test_known_conversions(cref):
    # (value, expected e4m3 byte): subnormal boundary, rounding to even, saturation edge
    cases = [(2.0 ** -10, 0x00), (0.0014, 0x01), (2.0 ** -9, 0x01), (1.5 * 2.0 ** -9, 0x02), (17.0, 0x58), (19.0, 0x5a),
             (448.0, 0x7e), (448.00003, 0x7e), (464.0, 0x7e), (464.00003, 0x7f), (float("inf"), 0x7f),
             (-448.0, 0xfe), (0.0, 0x00), (1.0, 0x38), (-1.0, 0xb8), (2.0 ** -6, 0x08), (0.9375 * 2.0 ** -6, 0x08)]
    for value, byte in cases:
        t = torch.tensor([value], dtype=torch.float32)
        assert int(t.to(torch.float8_e4m3fn).view(torch.uint8)) == byte, value
        assert cref.oracle_e4m3_from_f32(float(t)) == byte, value
    # 17 -> 16 and 19 -> 20 are the two directions of round-half-to-even at spacing 2
    assert float(torch.tensor([0x58], dtype=torch.uint8).view(torch.float8_e4m3fn).float()) == 16.0
    assert float(torch.tensor([0x5a], dtype=torch.uint8).view(torch.float8_e4m3fn).float()) == 20.0


def test_c_encoder_matches_library_on_all_bf16_values(cref):
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    vals = bits.view(torch.bfloat16).to(torch.float32)
    lib = vals.to(torch.float8_e4m3fn).view(torch.uint8)
    got = torch.tensor([cref.oracle_e4m3_from_f32(float(v)) for v in vals.tolist()], dtype=torch.uint8)
    nan = vals != vals
    assert torch.equal(got[~nan], lib[~nan])
    assert ((got[nan] & 0x7f) == 0x7f).all() and ((lib[nan] & 0x7f) == 0x7f).all()


def test_c_encoder_matches_library_on_dense_fp32_sweep(cref):
    g = torch.Generator().manual_seed(0)
    mags = torch.cat([torch.rand(20000, generator=g) * 470.0, torch.rand(20000, generator=g) * 0.05,
                      2.0 ** torch.randint(-12, 9, (5000,), generator=g).float() * (1 + torch.randint(0, 17, (5000,), generator=g).float() / 16)])
    vals = mags * torch.where(torch.rand(mags.shape, generator=g) < 0.5, -1.0, 1.0)
    lib = vals.to(torch.float8_e4m3fn).view(torch.uint8)
    got = torch.tensor([cref.oracle_e4m3_from_f32(float(v)) for v in vals.tolist()], dtype=torch.uint8)
    assert torch.equal(got, lib)


@pytest.mark.parametrize("hidden", [128, 384, 7168, 200])
def test_torch_oracle_matches_c_restatement(cref, hidden):
    g = torch.Generator().manual_seed(hidden)
    x = (torch.randn((24, hidden), generator=g) * torch.logspace(-6, 4, 24).unsqueeze(1)).to(torch.bfloat16)
    x[3] = 0                      # all-zero groups: the 1e-4 clamp decides
    x[4, ::7] = 0
    q, s = oracle.per_token_cast_to_fp8(x)
    cq, cs = c_cast(cref, x)
    assert torch.equal(q.view(torch.uint8), cq)
    assert torch.equal(s.view(torch.int32), cs.view(torch.int32))


def test_every_bf16_pattern_as_payload(cref):
    # all finite bf16 magnitudes, arranged so that each 128-group has its own amax
    bits = torch.arange(0, 0x7f80, dtype=torch.int32)
    vals = bits.to(torch.int16).view(torch.bfloat16)
    x = torch.cat([vals, -vals]).view(-1, 128)
    x = x[torch.randperm(x.shape[0], generator=torch.Generator().manual_seed(1))].view(-1, 256)   # 510 groups
    q, s = oracle.per_token_cast_to_fp8(x)
    cq, cs = c_cast(cref, x)
    assert torch.equal(q.view(torch.uint8), cq)
    assert torch.equal(s.view(torch.int32), cs.view(torch.int32))


def test_recipe_identities():
    g = torch.Generator().manual_seed(2)
    x = (torch.randn((64, 1024), generator=g) * 3).to(torch.bfloat16)
    x[0] = 0
    q, s = oracle.per_token_cast_to_fp8(x)
    qb = q.view(torch.uint8).view(64, 8, 128)
    xg = x.float().view(64, 8, 128)
    amax = xg.abs().amax(dim=2)
    # the element that attains amax always encodes to +-448
    pos = xg.abs().argmax(dim=2, keepdim=True)
    enc = qb.gather(2, pos).squeeze(2) & 0x7f
    assert (enc[amax >= 1e-4] == 0x7e).all()
    # an all-zero group: payload 0, scale = 1e-4 / 448 in fp32
    assert (qb[0] == 0).all()
    expected = (torch.tensor(1e-4, dtype=torch.float32) / torch.tensor(448.0, dtype=torch.float32))
    assert (s[0] == expected).all()
    # scale is a true division, not a multiplication by the rounded reciprocal, wherever the two differ
    by_recip = amax.clamp(min=1e-4) * torch.tensor(1.0 / 448.0, dtype=torch.float32)
    differs = by_recip != s
    assert differs.any(), "sample too small to separate division from reciprocal-multiply"
    assert torch.equal(s, amax.clamp(min=1e-4) / 448.0)
    # nothing saturates: |x| * (448/amax) never reaches the NaN code
    assert ((q.view(torch.uint8) & 0x7f) != 0x7f).all()
    # dequantised values are within half an e4m3 step (relative 2^-4) of the input, or below the subnormal step
    back = oracle.per_token_cast_back(q, s).float()
    err = (back - x.float()).abs()
    tol = torch.maximum(x.float().abs() * 2.0 ** -4, (s * 2.0 ** -9).repeat_interleave(128, dim=1)) + x.float().abs() * 2.0 ** -7
    assert (err <= tol).all()


def test_ordered_sum_matches_c_restatement(cref):
    g = torch.Generator().manual_seed(3)
    rows = (torch.randn((7, 96), generator=g) * torch.tensor([1e4, 1, 1e-3, -1e4, 5, 1e-2, 3]).unsqueeze(1)).to(torch.bfloat16)
    init = torch.randn(96, generator=g)
    want = oracle.ordered_accumulate(rows.unsqueeze(0), init.unsqueeze(0))[0]
    rin = rows.view(torch.int16).numpy().copy()
    out = np.zeros(96, dtype=np.uint16)
    ini = init.numpy().copy()
    cref.oracle_ordered_sum_bf16(rin.ctypes.data, 7, 96, ini.ctypes.data, out.ctypes.data)
    assert torch.equal(want.view(torch.int16), torch.from_numpy(out.view(np.int16)))
    # the reference's bf16 known answer: contributions are bf16 first (301 -> 300, 302 -> 302), sum 602 -> bf16 600
    data = torch.tensor([[301.0], [302.0]]).to(torch.bfloat16)
    assert float(oracle.ordered_accumulate(data.unsqueeze(0))[0, 0]) == 600.0


# ---- power-of-two scales (`round_scale`) and UE8M0 packing ----
def test_pow2_scales_against_exact_arithmetic_and_the_c_encoder(cref):
    """Independent restatement with Python's exact rationals: the scale is the smallest power of two that is
    >= fp32(amax * fp32(1/448)); the payload is the nearest e4m3 code of x / scale (C nearest-code search)."""
    import math
    from fractions import Fraction
    g = torch.Generator().manual_seed(11)
    x = (torch.randn((64, 256), generator=g) * torch.logspace(-6, 4, 64).unsqueeze(1)).to(torch.bfloat16)
    x[0] = 0                                     # all-zero groups: amax clamps to 1e-4
    x[1, :128] = 448.0                           # ratio exactly 1 -> exponent 0
    x[2, :128] = 449.0                           # bf16(449) = 448 as well
    x[3, :128] = 452.0                           # just above: exponent 1
    q, s = oracle.per_token_cast_to_fp8_pow2(x)
    inv448 = np.float32(1.0) / np.float32(448.0)
    for t in range(x.shape[0]):
        for grp in range(2):
            vals = x[t, grp * 128:(grp + 1) * 128].float()
            amax = max(float(vals.abs().max()), float(np.float32(1e-4)))
            ratio = Fraction(float(np.float32(amax) * inv448))
            e = math.ceil(math.log2(ratio)) if ratio != 2 ** round(math.log2(ratio)) else round(math.log2(ratio))
            assert Fraction(2) ** (e - 1) < ratio <= Fraction(2) ** e
            assert float(s[t, grp]) == 2.0 ** e
            for c in range(0, 128, 17):
                exact = float(vals[c]) / 2.0 ** e
                code = cref.oracle_e4m3_from_f32(exact)
                assert int(q[t, grp * 128 + c].view(torch.uint8)) == code
    assert float(s[1, 0]) == 1.0 and float(s[2, 0]) == 1.0 and float(s[3, 0]) == 2.0
    assert float(s[0, 0]) == 2.0 ** -22            # 1e-4 / 448 = 2.23e-7 -> 2^-22 = 2.38e-7


def test_ue8m0_packing_round_trips_through_the_reference_decode_rule():
    s = torch.tensor([[1.0, 2.0, 0.5, 2.0 ** -22, 2.0 ** 10, 2.0 ** -3, 1.0, 4.0]])
    packed = oracle.pack_ue8m0(s)
    assert packed.shape == (1, 2) and packed.dtype == torch.int32
    assert packed[0, 0].item() == (127 | (128 << 8) | (126 << 16) | (105 << 24))
    # decode as deep_ep/utils/math.py:51-53 does
    back = (packed.view(torch.uint8).to(torch.int32) << 23).view(torch.float32)
    assert torch.equal(back.view(1, 8), s)


# ---- the low-latency kernel's stored scale: amax * fp32(1/448) ----
def test_low_latency_scale_is_the_fp32_product_with_the_reciprocal():
    """csrc/kernels/legacy/utils.cuh:477-479,499-501.  The product of two fp32 numbers is exact in fp64, so
    fp32(fp64(amax) * fp64(fp32(1/448))) is the correctly rounded fp32 product, computed without the oracle's code
    path.  The payload is the torch recipe's (pinned above).  A restatement that divided instead would be caught: the
    two rules disagree on a good share of the groups."""
    g = torch.Generator().manual_seed(23)
    x = (torch.randn((256, 512), generator=g) * torch.logspace(-5, 3, 256).unsqueeze(1)).to(torch.bfloat16)
    x[0] = 0                                      # amax clamps to 1e-4
    x[1, :128] = 448.0
    q, s = oracle.per_token_cast_to_fp8_ll(x)
    q_div, s_div = oracle.per_token_cast_to_fp8(x)
    assert torch.equal(q.view(torch.uint8), q_div.view(torch.uint8))
    amax = x.float().view(256, 4, 128).abs().amax(dim=2).clamp(min=1e-4).numpy()
    inv448 = np.float64(np.float32(1.0) / np.float32(448.0))
    exact = (amax.astype(np.float64) * inv448).astype(np.float32)
    assert np.array_equal(s.numpy().view(np.int32), exact.view(np.int32))
    differ = (s.view(torch.int32) != s_div.view(torch.int32)).float().mean().item()
    assert 0.1 < differ < 0.9, differ             # the rules differ in the last bit on many groups, agree on others
    assert abs(s.view(torch.int32) - s_div.view(torch.int32)).max().item() <= 1
    assert float(s[1, 0]) == float(np.float32(448.0) * np.float32(inv448))
    # the low-latency dispatch uses this rule, and only for the scales
    px, ps, _, _, _ = oracle.ll_dispatch([x[:8]], [torch.zeros((8, 1), dtype=torch.int64)], 8, 1, 1, 0)
    assert torch.equal(ps[0, :8], s[:8]) and torch.equal(px[0, :8].view(torch.uint8), q[:8].view(torch.uint8))


def _nonfinite_groups():
    """Four 128-channel groups: one with a NaN, one with +Inf, one with -Inf, one finite; ordinary values elsewhere."""
    g = torch.Generator().manual_seed(11)
    x = (torch.randn((1, 512), generator=g) * 2).to(torch.bfloat16)
    x[0, 5], x[0, 128 + 7], x[0, 256 + 9] = float("nan"), float("inf"), float("-inf")
    return x


def test_non_finite_inputs_of_the_torch_recipe():
    """deep_ep/utils/math.py:37-38 takes the maximum with torch's amax and clamp, which hand a NaN on (a NaN compares
    false with everything, so a maximum built from comparisons would drop it - the C restatement above does, and is
    therefore only used on finite inputs).  What follows is plain IEEE arithmetic: 448 / NaN = NaN, x * NaN = NaN;
    448 / Inf = 0, finite * 0 = +-0, Inf * 0 = NaN, Inf / 448 = Inf."""
    x = _nonfinite_groups()
    q, s = oracle.per_token_cast_to_fp8(x)
    qb = q.view(torch.uint8).view(4, 128)
    nan_code = (qb & 0x7f) == 0x7f
    assert torch.isnan(s[0, 0]) and nan_code[0].all()                         # the NaN spreads over its group
    for grp, pos in ((1, 7), (2, 9)):
        assert torch.isinf(s[0, grp]) and s[0, grp] > 0
        assert nan_code[grp, pos] and int(nan_code[grp].sum()) == 1           # only the infinity itself is NaN
        others = torch.cat([qb[grp, :pos], qb[grp, pos + 1:]])
        signs = torch.cat([x[0, grp * 128:grp * 128 + pos], x[0, grp * 128 + pos + 1:(grp + 1) * 128]]).float() < 0
        assert torch.equal(others, torch.where(signs, 0x80, 0).to(torch.uint8))      # signed zeros
    assert torch.isfinite(s[0, 3]) and not nan_code[3].any()


def test_non_finite_inputs_of_the_low_latency_recipe():
    """csrc/kernels/legacy/internode_ll.cu:223-231 takes the maximum with fmaxf, which returns the other operand when
    one is NaN (C99 7.12.12.2; numpy's fmax is that function): a NaN element leaves its group's scale alone and only
    encodes as NaN itself.  Infinities behave as in the torch recipe."""
    x = _nonfinite_groups()
    for cast in (oracle.per_token_cast_to_fp8_ll, oracle.per_token_cast_to_fp8_pow2):
        q, s = cast(x[:, :128])                                               # the group with the NaN
        qb = q.view(torch.uint8)[0]
        amax = np.fmax.reduce(np.abs(x[0, :128].float().numpy()))
        assert np.isfinite(amax) and amax >= 1e-4
        if cast is oracle.per_token_cast_to_fp8_ll:
            assert float(s[0, 0]) == float(np.float32(amax) * np.float32(1.0 / 448.0))
            finite_ref, _ = oracle.per_token_cast_to_fp8(torch.where(torch.isnan(x[:, :128]), torch.zeros_like(x[:, :128]), x[:, :128]))
            mask = torch.ones(128, dtype=torch.bool); mask[5] = False
            assert torch.equal(qb[mask], finite_ref.view(torch.uint8)[0][mask])      # the others as if the NaN were not there
        else:
            assert float(s[0, 0]) == 2.0 ** int(np.ceil(np.log2(float(np.float32(amax) * np.float32(1.0 / 448.0)))))
        assert (int(qb[5]) & 0x7f) == 0x7f and int(((qb & 0x7f) == 0x7f).sum()) == 1
    q, s = oracle.per_token_cast_to_fp8_ll(x[:, 128:384])                     # the groups with the infinities
    assert torch.isinf(s).all() and int(((q.view(torch.uint8) & 0x7f) == 0x7f).sum()) == 2
