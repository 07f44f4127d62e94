// Per-1x128 FP8 e4m3 quantisation of BF16 channels, as a wave-level building block.
//
// amax over 128 channels clamped below at 1e-4, payload = e4m3(fp32(x) * (448 / amax)) with an IEEE fp32 division;
// what is stored as the group's scale depends on which of the reference's two code paths the caller replaces.
//
// Non-finite inputs follow the same two code paths.  The torch recipe (kDivide) takes the maximum with `amax` and
// `clamp`, both of which hand a NaN on: one NaN in a group makes the group's scale and all 128 payload bytes NaN.  The
// low-latency kernel (kReciprocal, kPow2) takes it with fmaxf, which drops a NaN: only the NaN elements themselves
// encode as NaN.  An infinity makes the scale infinite and the multiplier zero in both: finite elements encode as
// (signed) zero, the infinite ones as NaN.
#pragma once

#include "device_utils.h"

namespace deep_ep_hip {

enum class ScaleRule {
    kDivide,       // stored scale = amax / 448, IEEE division: deep_ep/utils/math.py:30-39 (dispatch, stand-alone cast)
    kReciprocal,   // stored scale = amax * fp32(1 / 448): what the low-latency kernel stores,
                   // csrc/kernels/legacy/utils.cuh:477-479,499-501 (last bit differs from kDivide for many amax values)
    kPow2,         // `round_scale` of the low-latency kernel, utils.cuh:481-498: see below
};

// Each lane holds 16 consecutive BF16 channels in (a, b); 8 consecutive lanes form one group of
// 128 channels.  Writes the 16 e4m3 bytes to `out` and returns the group's stored scale.
//
// kPow2: the scale is rounded up to a power of two: exponent = ceil(log2(amax * (1/448))) read off the fp32 bit
// pattern, payload = e4m3(x * 2^-exponent), stored scale = 2^exponent.
// |f| as a bit pattern.  For non-negative floats the patterns order like the values, every NaN pattern ranks above
// infinity, and an unsigned maximum costs what fmaxf costs: the maximum of these patterns is the NaN-propagating amax.
__device__ __forceinline__ uint32_t magnitude_bits(float f) { return __float_as_uint(f) & 0x7fffffffu; }

__device__ __forceinline__ uint32_t group8_max_bits(uint32_t v) {
    v = max(v, uint32_t(dpp_read<kDppSwapNeighbours>(int(v))));
    v = max(v, uint32_t(dpp_read<kDppSwapPairs>(int(v))));
    v = max(v, uint32_t(dpp_read<kDppHalfMirror>(int(v))));
    return v;
}

constexpr uint32_t kAmaxFloorBits = 0x38d1b717u;      // 1e-4f

// The clamped group maximum of this lane's 16 values and those of the 7 neighbouring lanes.
template <bool kPropagateNan>
__device__ __forceinline__ float group_amax(const float (&f)[16]) {
    if constexpr (kPropagateNan) {
        uint32_t m = 0u;
#pragma unroll
        for (int i = 0; i < 16; ++i) m = max(m, magnitude_bits(f[i]));
        return __uint_as_float(max(group8_max_bits(m), kAmaxFloorBits));
    } else {
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i += 2) amax = fmaxf(amax, fmaxf(fabsf(f[i]), fabsf(f[i + 1])));
        return fmaxf(group8_max(amax), 1e-4f);
    }
}

template <ScaleRule kRule = ScaleRule::kDivide>
__device__ __forceinline__ float cast_16_channels(const vec16& a, const vec16& b, vec16& out) {
    const uint32_t wds[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float f[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        f[2 * i] = bf16_lo(wds[i]);
        f[2 * i + 1] = bf16_hi(wds[i]);
    }
    const float amax = group_amax<kRule == ScaleRule::kDivide>(f);
    float scale, scale_inv;
    if constexpr (kRule == ScaleRule::kPow2) {
        const uint32_t bits = __float_as_uint(amax * (1.0f / 448.0f));
        const int exponent = int((bits >> 23) & 0xffu) - 127 + ((bits & 0x7fffffu) != 0u ? 1 : 0);
        scale = __uint_as_float(uint32_t(127 - exponent) << 23);
        scale_inv = __uint_as_float(uint32_t(127 + exponent) << 23);
    } else {
        scale = 448.0f / amax;
        scale_inv = kRule == ScaleRule::kReciprocal ? amax * (1.0f / 448.0f) : amax / 448.0f;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) f[i] = f[i] * scale;
    out.x = pack_e4m3x4(f[0], f[1], f[2], f[3]);
    out.y = pack_e4m3x4(f[4], f[5], f[6], f[7]);
    out.z = pack_e4m3x4(f[8], f[9], f[10], f[11]);
    out.w = pack_e4m3x4(f[12], f[13], f[14], f[15]);
    return scale_inv;
}

}  // namespace deep_ep_hip
