// Device helpers shared by the gfx950 routing kernels: wave64 primitives, 16-byte vector
// access, bf16 / e4m3 conversion.  Everything here is written for CDNA4 (64-wide wavefronts).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace deep_ep_hip {

constexpr int kWaveSize = 64;
constexpr int kLayoutChunk = 256;   // tokens per layout workgroup (= threads per workgroup)

struct alignas(16) vec16 {
    uint32_t x, y, z, w;
};

__device__ __forceinline__ int lane_id() {
    return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

__device__ __forceinline__ uint64_t lanes_below(int lane) {
    return (lane == 0) ? 0ull : (~0ull >> (64 - lane));
}

// Broadcast the value held by `src_lane` (wave-uniform index) to every lane.
__device__ __forceinline__ int read_lane(int v, int src_lane) {
    return __builtin_amdgcn_readlane(v, src_lane);
}
__device__ __forceinline__ float read_lane(float v, int src_lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src_lane));
}

__device__ __forceinline__ vec16 load16(const void* p) {
    return *reinterpret_cast<const vec16*>(p);
}
__device__ __forceinline__ void store16(void* p, const vec16& v) {
    *reinterpret_cast<vec16*>(p) = v;
}
// Streaming (non-temporal) forms for payload that is touched exactly once.
__device__ __forceinline__ vec16 load16_stream(const void* p) {
    const uint32_t* q = reinterpret_cast<const uint32_t*>(p);
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(q));
    return vec16{t.x, t.y, t.z, t.w};
}
__device__ __forceinline__ void store16_stream(void* p, const vec16& v) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
}

// bf16 <-> fp32 on raw bits.
__device__ __forceinline__ float bf16_lo(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }

// Round-to-nearest-even fp32 -> bf16; NaN becomes the canonical quiet NaN 0x7fc0.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    uint32_t rounded = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return (f != f) ? 0x7fc0u : rounded;
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}

// fp32 -> OCP e4m3fn, round-to-nearest-even, integer arithmetic only.  Magnitudes above 464
// (the midpoint past the largest finite value 448; 464 itself ties to even = 448) and NaN give 0x7f.
__device__ __forceinline__ uint32_t f32_to_e4m3_sw(float f) {
    const uint32_t u = __float_as_uint(f);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t a = u & 0x7fffffffu;
    uint32_t r;
    if (a > 0x43e80000u) {                   // |f| > 464, inf, nan
        r = 0x7fu;
    } else if (a >= 0x3c800000u) {           // |f| >= 2^-6: normal e4m3, drop 20 mantissa bits
        const uint32_t t = a + 0x7ffffu + ((a >> 20) & 1u);
        r = (t >> 20) - (120u << 3);         // rebias 127 -> 7
    } else if (a >= 0x3a800000u) {           // 2^-10 <= |f| < 2^-6: subnormal, unit 2^-9
        const int shift = 20 + (121 - int(a >> 23));       // 21..24
        const uint32_t m = (a & 0x7fffffu) | 0x800000u;
        const uint32_t half = 1u << (shift - 1);
        r = (m + half - 1u + ((m >> shift) & 1u)) >> shift;
    } else {
        r = 0u;                              // below half the smallest subnormal (2^-10 ties to even 0)
    }
    return sign | r;
}

#ifndef DEEP_EP_HIP_SOFTWARE_FP8
#define DEEP_EP_HIP_SOFTWARE_FP8 0
#endif

// Four fp32 -> four e4m3 bytes packed little-endian (a in bits 0..7).
__device__ __forceinline__ uint32_t pack_e4m3x4(float a, float b, float c, float d) {
#if DEEP_EP_HIP_SOFTWARE_FP8
    return f32_to_e4m3_sw(a) | (f32_to_e4m3_sw(b) << 8) | (f32_to_e4m3_sw(c) << 16) | (f32_to_e4m3_sw(d) << 24);
#else
    int v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    v = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
    return uint32_t(v);
#endif
}

// Lane exchanges inside a row of 16 lanes as DPP operand modifiers (no LDS traffic, no address arithmetic).  All lanes
// of the wavefront must be active.
constexpr int kDppSwapNeighbours = 0xB1;     // quad_perm [1,0,3,2]: lane ^ 1
constexpr int kDppSwapPairs = 0x4E;          // quad_perm [2,3,0,1]: lane ^ 2
constexpr int kDppHalfMirror = 0x141;        // row_half_mirror: lane i of an aligned group of 8 reads lane 7 - i
constexpr int kDppMirror = 0x140;            // row_mirror: lane i of a row of 16 reads lane 15 - i

template <int kCtrl>
__device__ __forceinline__ int dpp_read(int v) {
    return __builtin_amdgcn_update_dpp(v, v, kCtrl, 0xf, 0xf, false);
}

// Maximum over each aligned group of 8 consecutive lanes: neighbours, pairs, then the two quads (whose lanes all hold
// their quad's maximum by then) against each other.
__device__ __forceinline__ float group8_max(float v) {
    v = fmaxf(v, __int_as_float(dpp_read<kDppSwapNeighbours>(__float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp_read<kDppSwapPairs>(__float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp_read<kDppHalfMirror>(__float_as_int(v))));
    return v;
}

// Sum over each row of 16 lanes, left in every lane of the row.
__device__ __forceinline__ int row16_sum(int v) {
    v += dpp_read<kDppSwapNeighbours>(v);
    v += dpp_read<kDppSwapPairs>(v);
    v += dpp_read<kDppHalfMirror>(v);
    v += dpp_read<kDppMirror>(v);
    return v;
}

// Inclusive prefix sum across the wave.
__device__ __forceinline__ int wave_inclusive_sum(int v) {
    const int lane = lane_id();
#pragma unroll
    for (int off = 1; off < kWaveSize; off <<= 1) {
        int o = __shfl_up(v, off, kWaveSize);
        if (lane >= off) v += o;
    }
    return v;
}

// Workgroups are handed to the 8 XCDs (each with its own L2) round-robin: workgroup i runs on XCD i % 8.
// This renumbering gives every XCD one contiguous range of logical workgroups, so that neighbouring
// work items (which write neighbouring output rows) share an L2 and their partial-line writes merge.
__device__ __forceinline__ unsigned xcd_contiguous_block(unsigned block, unsigned num_blocks) {
    constexpr unsigned kXcds = 8;
    const unsigned per = num_blocks / kXcds;
    if (block >= per * kXcds) return block;          // ragged tail keeps its index
    return (block % kXcds) * per + block / kXcds;
}

// Index of this wavefront's work item, as a wave-uniform 32-bit value (kept in scalar registers, so the
// divisions that split it into (token, tile) are short 32-bit sequences instead of per-lane 64-bit ones).
__device__ __forceinline__ unsigned wave_work_index(unsigned block, unsigned waves_per_block) {
    return block * waves_per_block + unsigned(__builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6)));
}

// x / d for 0 <= x < 2^20 and 1 <= d <= 2^16 through a float reciprocal: (x + 0.5) / d is at least 0.5 / d
// away from an integer while the float error stays below 2^-23 * x / d, so truncation is exact.
__device__ __forceinline__ int small_div(int x, float rcp_d) {
    return int((float(x) + 0.5f) * rcp_d);
}

// Agent-scope relaxed load / store (no caching that another XCD's workgroups could not see through), for words
// workgroups of one launch hand to each other.
__device__ __forceinline__ int load_agent(const int* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_agent(int* p, int v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// kThrough: an agent-scope (write-through) store; otherwise an ordinary one.
template <bool kThrough>
__device__ __forceinline__ void store_word(int* p, int v) {
    if constexpr (kThrough) store_agent(p, v);
    else *p = v;
}
template <bool kAgent>
__device__ __forceinline__ int load_word(const int* p) {
    if constexpr (kAgent) return load_agent(p);
    else return *p;
}
// 16 bytes stored at agent scope (written through), as two 8-byte atomic stores: the language offers atomics of at most
// 8 bytes, and a 16-byte store written as an instruction by hand would sit outside the compiler's hazard tracking
// (a vector store of more than 8 bytes must not have its data registers overwritten in the next cycle).
__device__ __forceinline__ void store16_agent(void* p, const vec16& v) {
    unsigned long long* q = reinterpret_cast<unsigned long long*>(p);
    __hip_atomic_store(q, (unsigned long long)(v.x) | ((unsigned long long)(v.y) << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(q + 1, (unsigned long long)(v.z) | ((unsigned long long)(v.w) << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Waits until every store this wavefront has issued is acknowledged.  After agent-scope stores this is all a
// workgroup needs before it raises a flag for another workgroup: no cache-wide write-back is involved.
__device__ __forceinline__ void wait_for_own_stores() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace deep_ep_hip
