// Counting step of the dispatch layout, shared by the stand-alone layout kernel and by the counting workgroups
// at the front of a single-launch dispatch.
//
// A workgroup of 256 threads owns a chunk of 256 consecutive tokens (one thread per token).  Each wavefront
// sets its lane bit in an LDS bitmap word per rank and per expert (ds_or_b64), so that
//   count  = popcount(bitmap)                      and
//   position of token t among chunk tokens routed to the same bucket = popcount(bitmap & lanes below t)
// with no ordering-dependent atomics: placement is a pure function of the input.  Chunk totals go to the count
// tables of the workspace.
//
// Counts what csrc/kernels/legacy/layout.cu:10-122 and the notify warps of
// deep_ep/include/deep_ep/impls/dispatch.cuh:79-199 count.
#pragma once

#include "device_utils.h"
#include "kernels.h"
#include "../../include/deep_ep_hip.h"

namespace deep_ep_hip {

static_assert(kLayoutChunk == 4 * kWaveSize, "the packed before-wave word holds three fields");

// LDS the counting step needs: the bitmap words [(R + E)][4] and one packed word per bucket (see below).
inline size_t count_lds_bytes(int R, int E) {
    return size_t(R + E) * (kLayoutChunk / kWaveSize) * sizeof(uint64_t) + size_t(R + E) * sizeof(uint32_t);
}

// bitmap: LDS of count_lds_bytes(R, E) bytes.  Must be called by all 256 threads of the workgroup.
// kThrough: positions and chunk totals are stored at agent scope (workgroups of the same launch read them); the
// position words and the copy of the rank totals in p.tagged_rank carry the launch's tag.
template <int KMAX, bool kThrough>
__device__ __forceinline__ void count_chunk(const LayoutParams& p, const int chunk, const int num_chunks, uint64_t* bitmap) {
    constexpr int kThreads = kLayoutChunk;
    constexpr int kWaves = kThreads / kWaveSize;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int t = chunk * kThreads + tid;
    const int n = p.R + p.E;
    const bool active = t < p.T;
    uint32_t tag = 0;
    if constexpr (kThrough)
        if (p.generation != nullptr) tag = (*p.generation + 1u) << kTagShift;     // constant while the launch reads it

    // The index loads go out first (they are the longest wait of the pass), before anything that could alias
    // them is stored; the bitmap is cleared while they are in flight.
    int64_t raw[KMAX];
    if (p.route_mask != nullptr) {
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
            raw[k] = (active && k < p.K && p.route_mask[int64_t(t) * p.K + k] != 0) ? int64_t(k) : int64_t(-1);
    } else if (KMAX == 8 && p.K == 8 && p.vec_idx) {
        if (active) {
            const vec16* src = reinterpret_cast<const vec16*>(p.topk_idx + int64_t(t) * 8);
            vec16 q[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) q[i] = src[i];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                raw[2 * i] = int64_t(uint64_t(q[i].x) | (uint64_t(q[i].y) << 32));
                raw[2 * i + 1] = int64_t(uint64_t(q[i].z) | (uint64_t(q[i].w) << 32));
            }
        } else {
#pragma unroll
            for (int k = 0; k < KMAX; ++k) raw[k] = -1;
        }
    } else {
#pragma unroll
        for (int k = 0; k < KMAX; ++k) raw[k] = (active && k < p.K) ? p.topk_idx[int64_t(t) * p.K + k] : int64_t(-1);
    }

    for (int i = tid; i < n * kWaves; i += kThreads) bitmap[i] = 0ull;
    __syncthreads();

    // Straight-line code from here on, no branch per routing lane: the LDS atomics of all lanes issue back to back, and
    // so do the LDS reads of the position step further down.  A lane without an expert ORs nothing into a word of its
    // own (not one word for all of them: atomics of one wavefront on one address take turns).
    // With few ranks most lanes of a wavefront would meet on the same few rank words, so the rank bitmaps are taken by
    // ballot instead: one per rank over "this token goes to rank r", no atomics.
    constexpr int kBallotRanks = 16;
    const bool ranks_by_ballot = p.R <= kBallotRanks;
    int e[KMAX], d[KMAX];
    int flags = 0;
    const float rcp_experts_per_rank = 1.0f / float(p.E_l);
    const uint64_t my_bit = 1ull << lane;
    const int idle_word = min(lane, n * kWaves - 1);
    uint64_t my_ranks = 0;                       // bit r: this token goes to rank r
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        const bool valid = raw[k] >= 0 && raw[k] < p.E;
        if (raw[k] >= p.E) flags |= DEEP_EP_HIP_STATUS_EXPERT_OUT_OF_RANGE;
        e[k] = valid ? int(raw[k]) : -1;
        d[k] = valid ? small_div(e[k], rcp_experts_per_rank) : -1;
        const uint64_t bit = valid ? my_bit : 0ull;
        atomicOr(reinterpret_cast<unsigned long long*>(&bitmap[valid ? (p.R + e[k]) * kWaves + wave : idle_word]), bit);
        if (valid) my_ranks |= 1ull << (d[k] & 63);            // used when num_ranks <= kBallotRanks
    }
    if (ranks_by_ballot) {
        uint64_t mine = 0;
        for (int r = 0; r < p.R; ++r) {
            const uint64_t members = __ballot((my_ranks >> r) & 1ull);
            if (lane == r) mine = members;
        }
        if (lane < p.R) bitmap[lane * kWaves + wave] = mine;
    } else {
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
            atomicOr(reinterpret_cast<unsigned long long*>(&bitmap[d[k] >= 0 ? d[k] * kWaves + wave : idle_word]),
                     d[k] >= 0 ? my_bit : 0ull);
    }
    if (p.copied_topk_idx != nullptr && active) {
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
            if (k < p.K) p.copied_topk_idx[int64_t(t) * p.K + k] = raw[k];
    }
    __syncthreads();

    // Per bucket: the chunk total goes out and the bits set by the wavefronts before each wavefront are packed into one LDS word (three 10-bit fields),
    // so that a position costs two independent LDS reads.
    uint32_t* before_wave = reinterpret_cast<uint32_t*>(bitmap + n * kWaves);
    for (int j = tid; j < n; j += kThreads) {
        const int c0 = __popcll(bitmap[j * kWaves]), c1 = __popcll(bitmap[j * kWaves + 1]);
        const int c2 = __popcll(bitmap[j * kWaves + 2]), c3 = __popcll(bitmap[j * kWaves + 3]);
        before_wave[j] = uint32_t(c0) | (uint32_t(c0 + c1) << 10) | (uint32_t(c0 + c1 + c2) << 20);
        int32_t* at = j < p.R ? p.tab.rank_counts + int64_t(j) * p.tab.chunks_padded + chunk
                              : p.tab.expert_counts + int64_t(chunk) * p.tab.experts_padded + (j - p.R);
        store_word<kThrough>(at, c0 + c1 + c2 + c3);
        if constexpr (kThrough) {
            if (j < p.R && p.tagged_rank != nullptr)
                store_agent(reinterpret_cast<int*>(p.tagged_rank) + j * p.tab.chunks_padded + chunk, int(uint32_t(c0 + c1 + c2 + c3) | tag));
            if (j >= p.R && p.tagged_expert_counts != nullptr)
                store_agent(reinterpret_cast<int*>(p.tagged_expert_counts) + chunk * p.tab.experts_padded + (j - p.R),
                            int(uint32_t(c0 + c1 + c2 + c3) | tag));
        }
    }
    const int pad = p.tab.chunks_padded - num_chunks;  // the padding columns of the rank table are cleared by the first workgroup
    if (chunk == 0) {
        for (int i = tid; i < p.R * pad; i += kThreads) {
            const int at = (i / pad) * p.tab.chunks_padded + num_chunks + i % pad;
            store_word<kThrough>(p.tab.rank_counts + at, 0);
            if constexpr (kThrough)
                if (p.tagged_rank != nullptr) store_agent(reinterpret_cast<int*>(p.tagged_rank) + at, int(tag));
        }
    }
    __syncthreads();

    const uint64_t below = lanes_below(lane);
    const int wave_shift = wave > 0 ? 10 * (wave - 1) : 0;
    const uint32_t earlier_mask = wave > 0 ? 0x3ffu : 0u;
    // Position inside the chunk = bits of this wavefront's word below the lane + bits of the wavefronts before it.
    auto position = [&](uint64_t word, uint32_t before) {
        return uint32_t(__popcll(word & below)) + ((before >> wave_shift) & earlier_mask);
    };

    if (active) {
        if (p.pos != nullptr) {
            // One word per (token, lane): the slot of the token inside its chunk for the lane's destination rank
            // (master lanes only) and the position of the lane inside its chunk for its expert (kernels.h).
            uint32_t packed[KMAX];
            uint64_t word_r[KMAX];
            uint32_t before_r[KMAX];
#pragma unroll
            for (int k = 0; k < KMAX; ++k) {
                const int bucket = d[k] >= 0 ? d[k] : 0;
                word_r[k] = bitmap[bucket * kWaves + wave];
                before_r[k] = before_wave[bucket];
            }
            // The master lane of a destination rank is the last lane that names it.
            bool master[KMAX];
            if (p.R <= 64) {
                // walk the lanes backwards with the set of ranks seen so far
                uint64_t later_ranks = 0;
#pragma unroll
                for (int k = KMAX - 1; k >= 0; --k) {
                    const uint64_t rank_bit = d[k] >= 0 ? 1ull << (d[k] & 63) : 0ull;
                    master[k] = (rank_bit & ~later_ranks) != 0;
                    later_ranks |= rank_bit;
                }
            } else {
#pragma unroll
                for (int k = 0; k < KMAX; ++k) {
                    master[k] = d[k] >= 0;
#pragma unroll
                    for (int j = k + 1; j < KMAX; ++j)
                        if (d[j] == d[k]) master[k] = false;
                }
            }
#pragma unroll
            for (int k = 0; k < KMAX; ++k) {
#pragma unroll
                for (int j = k + 1; j < KMAX; ++j)
                    if (e[k] >= 0 && e[j] == e[k]) flags |= DEEP_EP_HIP_STATUS_DUPLICATE_EXPERT;
                packed[k] = (master[k] ? position(word_r[k], before_r[k]) : kNoPosition) | tag;
            }
            if (p.expert_bases) {                         // only the expanded layout places rows by expert
#pragma unroll
                for (int k = 0; k < KMAX; ++k) {
                    const int bucket = e[k] >= 0 ? p.R + e[k] : 0;
                    word_r[k] = bitmap[bucket * kWaves + wave];
                    before_r[k] = before_wave[bucket];
                }
#pragma unroll
                for (int k = 0; k < KMAX; ++k)
                    packed[k] |= (e[k] >= 0 ? position(word_r[k], before_r[k]) : kNoPosition) << kExpertPositionShift;
            } else {
#pragma unroll
                for (int k = 0; k < KMAX; ++k) packed[k] |= kNoPosition << kExpertPositionShift;
            }
            if (KMAX == 8 && p.K == 8) {
                vec16* dst = reinterpret_cast<vec16*>(p.pos + int64_t(t) * 8);
                const vec16 lo{packed[0], packed[1], packed[2], packed[3]}, hi{packed[4], packed[5], packed[6], packed[7]};
                if constexpr (kThrough) {
                    store16_agent(dst, lo);
                    store16_agent(dst + 1, hi);
                } else {
                    dst[0] = lo;
                    dst[1] = hi;
                }
            } else {
#pragma unroll
                for (int k = 0; k < KMAX; ++k)
                    if (k < p.K) store_word<kThrough>(reinterpret_cast<int*>(p.pos) + int64_t(t) * p.K + k, int(packed[k]));
            }
        }
        if (p.is_token_in_rank != nullptr) {
            for (int r = 0; r < p.R; ++r)
                p.is_token_in_rank[int64_t(t) * p.R + r] = uint8_t((bitmap[r * kWaves + wave] >> lane) & 1ull);
        }
    }
    if (flags != 0) atomicOr(p.status, flags);

}

}  // namespace deep_ep_hip
