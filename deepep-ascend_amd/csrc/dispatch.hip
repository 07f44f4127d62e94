// Dispatch payload movement for gfx950: every token row is read once from HBM and written once per
// destination row (compact: one row per distinct destination rank; expanded: one row per valid
// (token, lane)), with the optional BF16 -> FP8 e4m3 per-1x128 cast fused between the load and
// the stores.
//
// Replaces the per-token warp loop of deep_ep/include/deep_ep/impls/dispatch.cuh:259-395 together
// with the receive-side copy of deep_ep/include/deep_ep/impls/dispatch_copy_epilogue.cuh:70-208:
// on one GPU the "send buffer -> peer recv buffer -> output tensor" chain collapses into a single
// scatter.  Slot numbers come from the layout pass (scan based, deterministic) instead of atomics.
//
// Work decomposition: one wavefront owns one (token, column tile).  All 16-byte loads of the tile
// are issued first, then the routing metadata is resolved while they are in flight, then the tile
// is stored to each destination with 16-byte stores.
//
// Single-launch mode ("fused"): the first workgroups of the grid are counting workgroups (one 256-token
// chunk each, the code of the layout kernel) and one publishing workgroup that writes the handle tensors.
// Mover workgroups issue their payload loads, then read the chunk totals and position words the counting
// workgroups store (again, until a word shows the tag of this launch), and work their row numbers out from
// those.  Counting workgroups have the lowest workgroup ids, wait for nothing and are therefore resident
// before any mover can wait for them; every wait is bounded.
#include <algorithm>
#include <atomic>

#include "device_utils.h"
#include "fp8_cast.h"
#include "kernels.h"
#include "layout_count.h"
#include "publish.h"
#include "../../include/deep_ep_hip.h"

namespace deep_ep_hip {

namespace {

#ifndef DEEP_EP_HIP_MOVE_THREADS
#define DEEP_EP_HIP_MOVE_THREADS 256
#endif
constexpr int kThreads = DEEP_EP_HIP_MOVE_THREADS;
constexpr int kWavesPerBlock = kThreads / kWaveSize;

// Per-lane routing state of one token, lanes [0, K) meaningful.
struct Route {
    int e;        // expert id or -1
    int d;        // destination rank or -1
    int row_c;    // compact row, on master lanes only (else -1)
    int my_row;   // compact row of this lane's destination (all valid lanes)
    int erow;     // expanded row (expanded layout), else -1
    float w;
};

// A word of the layout tables a finished layout pass (an earlier launch, or a cached handle) left in memory.
__device__ __forceinline__ int layout_word(const int32_t* at) {
    return *at;
}

// What the caller gave for one (token, lane): independent of the layout pass, so a single-launch dispatch loads
// it together with the payload, before it knows that the layout is complete.
struct RouteInputs {
    int64_t raw;         // topk_idx entry
    uint8_t mask_byte;   // is_token_in_rank entry (mask routing)
    float w;             // topk_weights entry
};

__device__ __forceinline__ RouteInputs load_route_inputs(const MoveParams& p, int t, int lane) {
    RouteInputs in{-1, 0, 0.f};
    if (lane < p.K) {
        const int64_t at = int64_t(t) * p.K + lane;
        if (p.route_mask != nullptr) in.mask_byte = p.route_mask[at];
        else if (!(p.cached && p.rank_lanes)) in.raw = p.topk_idx[at];
        if (p.topk_weights != nullptr) in.w = p.topk_weights[at];
    }
    return in;
}

// The word of the layout pass for (token, lane): the cached handle's slot, or the position word (kernels.h).
__device__ __forceinline__ uint32_t load_position_word(const MoveParams& p, int t, int lane) {
    if (lane >= p.K) return 0xffffffffu;
    const int32_t* words = p.cached ? p.cached_slot : reinterpret_cast<const int32_t*>(p.pos);
    return uint32_t(layout_word(words + int64_t(t) * p.K + lane));
}

// Single-launch dispatch: flat_bases is this workgroup's LDS copy of the exclusive prefix over the chunk totals of the
// rank buckets, expert_base the first expanded row of (the token's chunk, the lane's expert).
template <bool kFused>
__device__ __forceinline__ Route resolve_route(const MoveParams& p, const RouteInputs& in, uint32_t word, const int* flat_bases,
                                               int expert_base, int t, int lane, bool first_tile) {
    Route r{-1, -1, -1, -1, -1, in.w};
    const int chunk = t / kLayoutChunk;

    // ---- issue every load that does not depend on another one, then consume: one memory round trip ----
    int64_t raw = in.raw;
    const uint8_t mask_byte = in.mask_byte;
    const bool rank_lanes_cached = p.cached && p.rank_lanes;
    // Wave lane q < R fetches the base row of (rank q, this token's chunk) and the start of rank q's bucket; the
    // routing lanes pick theirs up by shuffle.  (More than 64 ranks: each master lane fetches its own pair below.)
    const bool bases_by_lane = !kFused && !p.cached && p.R <= kWaveSize;
    int base_of_rank = 0, start_of_rank = 0;
    if (bases_by_lane && lane < p.R) {
        base_of_rank = layout_word(p.tab.rank_bases + int64_t(lane) * p.tab.chunks_padded + chunk);
        start_of_rank = layout_word(p.tab.rank_bases + int64_t(lane) * p.tab.chunks_padded);
    }

    int slot = -1, epos = -1;
    const int cached_v = int(word);
    const uint32_t packed = word;
    if (lane < p.K) {
        if (rank_lanes_cached) {
            // V1 cached dispatch: send_head names the receive row of every (token, rank) pair
            if (cached_v >= 0) r.e = lane;
            slot = cached_v;
        } else {
            if (p.route_mask != nullptr) raw = mask_byte != 0 ? int64_t(lane) : int64_t(-1);
            if (raw >= 0 && raw < p.E) r.e = int(raw);
            if (p.cached) {
                slot = cached_v >= 0 ? cached_v - p.rank_idx * p.M : -1;
            } else {
                slot = (packed & kNoPosition) == kNoPosition ? -1 : int(packed & kNoPosition);
                epos = int((packed >> kExpertPositionShift) & kNoPosition);
            }
        }
    }
    if (r.e >= 0) r.d = small_div(r.e, p.rcp_E_l);
    else slot = -1;
    if (!p.cached) {
        int base, start;
        if constexpr (kFused) {
            const int row = (r.d >= 0 && slot >= 0 ? r.d : 0) * p.tab.chunks_padded;
            base = flat_bases[row + chunk];
            start = flat_bases[row];
        } else if (bases_by_lane) {
            const int from = r.d >= 0 ? r.d : 0;
            base = __shfl(base_of_rank, from, kWaveSize);
            start = __shfl(start_of_rank, from, kWaveSize);
        } else {
            const int64_t row = int64_t(r.d >= 0 && slot >= 0 ? r.d : 0) * p.tab.chunks_padded;
            base = layout_word(p.tab.rank_bases + row + chunk);
            start = layout_word(p.tab.rank_bases + row);
        }
        if (r.d >= 0 && slot >= 0) {
            r.row_c = base + slot;
            slot = r.row_c - start;             // slot inside the destination bucket
        }
    } else if (r.e >= 0 && slot >= 0) {
        r.row_c = p.slot_is_row ? slot : (r.d > 0 ? p.psum_rank[r.d - 1] : 0) + slot;
    }
    if (first_tile && !p.cached && lane < p.K && p.dst_buffer_slot_idx != nullptr)
        p.dst_buffer_slot_idx[int64_t(t) * p.K + lane] = (r.e >= 0 && slot >= 0) ? p.rank_idx * p.M + slot : -1;
    if (first_tile && !p.cached && p.send_head != nullptr) {
        // V1 handle: wave lane q < R reports the receive row of this token on rank q (-1: not sent there)
        int row_on_rank = -1;
        for (int j = 0; j < p.K; ++j) {
            const int dj = read_lane(r.d, j);
            const int rj = read_lane(r.row_c, j);
            if (dj == lane && rj >= 0) row_on_rank = rj;
        }
        if (lane < p.R) p.send_head[int64_t(t) * p.R + lane] = row_on_rank;
    }

    // Every valid lane learns the compact row of its destination rank from that rank's master lane.
    for (int j = 0; j < p.K; ++j) {
        const int dj = read_lane(r.d, j);
        const int rj = read_lane(r.row_c, j);
        if (r.d >= 0 && dj == r.d && rj >= 0) r.my_row = rj;
    }
    if (p.do_expand && r.e >= 0) {
        if (p.cached) {
            if (r.my_row >= 0 && r.my_row < p.recv_capacity)
                r.erow = p.recv_src_metadata[int64_t(r.my_row) * (p.K + 2) + 2 + lane];
        } else if constexpr (kFused) {
            r.erow = expert_base + epos;
        } else {
            r.erow = layout_word(p.tab.expert_bases + int64_t(chunk) * p.tab.experts_padded + r.e) + epos;
        }
    }
    return r;
}

// Token-level metadata, written once per token (by the wave that owns column tile 0).
//
// Compact layout with K <= 15: a destination row's recv_topk_idx (2 dwords per lane), recv_topk_weights and
// recv_src_metadata entries go out in ONE dword store instruction: wave lanes take the roles
//   [0, 2K) index dwords | [2K, 3K) weights | [3K, 4K + 2) metadata columns,
// each role reading the routing lane it needs through a shuffle done once per token.
__device__ __forceinline__ void write_token_metadata(const MoveParams& p, const Route& r, int t, int lane) {
    uint64_t masters = __ballot(r.row_c >= 0);
    const int K = p.K;
    if (!p.do_expand && 4 * K + 2 <= kWaveSize) {
        int src;           // routing lane this wave lane reports on
        if (lane < 2 * K) src = lane >> 1;
        else if (lane < 3 * K) src = lane - 2 * K;
        else src = lane - 3 * K - 2;                       // metadata columns 2.. (negative for columns 0 and 1)
        const int src_c = src < 0 ? 0 : (src >= K ? 0 : src);
        const int e_src = __shfl(r.e, src_c, kWaveSize);
        const int d_src = __shfl(r.d, src_c, kWaveSize);
        const uint32_t w_src = __float_as_uint(__shfl(r.w, src_c, kWaveSize));
        while (masters) {
            const int j = __builtin_ctzll(masters);
            masters &= masters - 1;
            const int row = read_lane(r.row_c, j);
            const int dj = read_lane(r.d, j);
            if (row >= p.recv_capacity) {
                if (lane == 0) atomicOr(p.status, DEEP_EP_HIP_STATUS_ROW_OVERFLOW);
                continue;
            }
            uint32_t* dst = nullptr;
            uint32_t v = 0;
            if (lane < 2 * K) {
                const int local = (d_src == dj) ? e_src - dj * p.E_l : -1;
                v = (lane & 1) ? (local < 0 ? 0xffffffffu : 0u) : uint32_t(local);
                if (p.recv_topk_idx != nullptr) dst = reinterpret_cast<uint32_t*>(p.recv_topk_idx + int64_t(row) * K) + lane;
            } else if (lane < 3 * K) {
                v = (p.zero_nonlocal_w && d_src != dj) ? 0u : w_src;
                if (p.recv_topk_weights != nullptr)
                    dst = reinterpret_cast<uint32_t*>(p.recv_topk_weights + int64_t(row) * K) + (lane - 2 * K);
            } else if (lane < 4 * K + 2) {
                const int col = lane - 3 * K;
                v = col == 0 ? uint32_t(p.rank_idx * p.M + t) : col == 1 ? uint32_t(p.rank_idx * K + j) : 0xffffffffu;
                if (!p.cached && p.recv_src_metadata != nullptr)
                    dst = reinterpret_cast<uint32_t*>(p.recv_src_metadata + int64_t(row) * (K + 2)) + col;
                if (col == 0 && p.recv_src_idx != nullptr) p.recv_src_idx[row] = t;
            }
            if (dst != nullptr) *dst = v;
        }
        return;
    }
    while (masters) {
        const int j = __builtin_ctzll(masters);
        masters &= masters - 1;
        const int row = read_lane(r.row_c, j);
        const int dj = read_lane(r.d, j);
        if (row >= p.recv_capacity) {
            if (lane == 0) atomicOr(p.status, DEEP_EP_HIP_STATUS_ROW_OVERFLOW);
            continue;
        }
        if (!p.do_expand && lane < p.K) {
            if (p.recv_topk_idx != nullptr)
                p.recv_topk_idx[int64_t(row) * p.K + lane] = (r.d == dj) ? int64_t(r.e - dj * p.E_l) : int64_t(-1);
            if (p.recv_topk_weights != nullptr)
                p.recv_topk_weights[int64_t(row) * p.K + lane] = (p.zero_nonlocal_w && r.d != dj) ? 0.f : r.w;
        }
        if (lane == 0 && p.recv_src_idx != nullptr) p.recv_src_idx[row] = t;
        if (!p.cached && p.recv_src_metadata != nullptr && lane < p.K + 2) {
            int v;
            if (lane < p.K) v = (p.do_expand && r.d == dj) ? r.erow : -1;
            else if (lane == p.K) v = p.rank_idx * p.M + t;
            else v = p.rank_idx * p.K + j;
            const int col = lane < p.K ? 2 + lane : lane - p.K;
            p.recv_src_metadata[int64_t(row) * (p.K + 2) + col] = v;
        }
    }
    if (p.do_expand && p.recv_topk_weights != nullptr && r.erow >= 0 && r.erow < p.expanded_capacity)
        p.recv_topk_weights[r.erow] = r.w;
}

// Bit mask of lanes that name a destination row, and the row each of them names.
__device__ __forceinline__ uint64_t destination_lanes(const MoveParams& p, const Route& r, int& row_of_lane) {
    if (p.do_expand) {
        row_of_lane = (r.erow >= 0 && r.erow < p.expanded_capacity) ? r.erow : -1;
        if (r.erow >= p.expanded_capacity) atomicOr(p.status, DEEP_EP_HIP_STATUS_ROW_OVERFLOW);
    } else {
        row_of_lane = (r.row_c >= 0 && r.row_c < p.recv_capacity) ? r.row_c : -1;
    }
    return __ballot(row_of_lane >= 0);
}

// ---- single-launch dispatch ----
//
// Grid: C counting workgroups (one 256-token chunk each), one publishing workgroup, then the movers.  A mover cannot
// store a row before the layout is known, and the kernel is bound by its stores, so every microsecond before the
// first store is a microsecond of the launch: the path from the counting workgroups to the movers is kept as short
// as the hardware allows.  A hand-off between workgroups of one launch costs a trip to the memory side for the
// writer's store and one for the reader's load (about a microsecond each on a busy GPU); a flag on top of the data
// would add the writer's wait for its stores, the flag's own trip and a second read.  So the data is its own flag:
//   - every word handed to the movers (chunk totals of the rank buckets, position words, expert bases) carries the
//     tag of this launch in its upper bits (kernels.h) and is stored at agent scope (written through);
//   - a mover workgroup reads what it needs - each thread four chunk totals, each wavefront the position words of
//     its token, and for the expanded layout the base of each lane's (chunk, expert) - first with ordinary loads that
//     go out before the payload loads (first_look), and, where a word does not show the tag yet, again at agent scope
//     (bounded: second_look, await_tagged_words).  It then works the rank bases out for itself (an exclusive prefix
//     sum over the R x C chunk totals, into LDS);
//   - the publisher waits for the chunk_done flags the counting workgroups raise once their stores are acknowledged,
//     clears them, and writes the per-rank and per-expert outputs of the call while the movers are already moving;
//     for the expanded layout the tagged expert bases go out first.
// The tag is generation + 1, and the generation word is advanced by whichever mover learns that every mover has read
// its words: a mover that is done reading advances its gate (mover m uses gate m % kDispatchGates, each gate a cache
// line of its own, because agent-scope atomics on one address serialise at about 11 ns each); the one that brings
// a gate to its number of movers advances gates_finished; the one that brings that to the number of gates in use
// advances the generation.  Gates and gates_finished wrap to 0 on the last increment, so nothing is reset between
// launches.  No workgroup reads the generation after it has moved: counting workgroups and the publisher read it when
// they start, and the movers' reads cannot complete before those have stored their words.  The launch that uses tag
// kTagPeriod clears the tagged tables and starts over at generation 0, so a word can never show the tag of a launch
// other than the running one.  Counting and publishing workgroups have the lowest workgroup ids and wait for nothing
// that is dispatched after them, so every wait ends; each is bounded anyway and reports
// DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT.
constexpr unsigned kLayoutSpinLimit = 1u << 22;      // polls (each with a short sleep) before giving up: seconds

// The tag of the running launch.  An ordinary (cached) load: the generation word does not change while anyone reads it -
// it is advanced only after every mover has read its tagged words, which it cannot do without the tag - and with tens of
// thousands of wavefronts asking, a read that went to memory every time would make the word's memory channel a hot spot.
__device__ __forceinline__ uint32_t launch_tag(const uint32_t* generation) {
    return (*generation + 1u) << kTagShift;
}

__device__ __forceinline__ uint64_t load_agent64(const void* p) {
    return __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ unsigned movers_of_gate(const MoveParams& p, unsigned gate) {
    return (p.num_movers + unsigned(kDispatchGates) - 1u - gate) / unsigned(kDispatchGates);
}

__device__ __forceinline__ void fused_count_block(const MoveParams& p) {
    extern __shared__ uint64_t count_lds[];
    const int c = int(blockIdx.x);
    count_chunk<8, true>(p.lay, c, p.count_blocks, count_lds);
    wait_for_own_stores();
    __syncthreads();
    if (threadIdx.x == 0) store_agent(p.chunk_done + c, 1);      // for the publisher
}

// All flags[0..n) set?  Polls (bounded), then clears them for the next launch.  Every thread must call it.
__device__ __forceinline__ void await_and_clear_flags(const MoveParams& p, int32_t* flags, int n) {
    bool complete = true;
    for (int i = threadIdx.x; i < n; i += kThreads) {
        unsigned polls = 0;
        while (load_agent(flags + i) == 0 && polls < kLayoutSpinLimit) {
            __builtin_amdgcn_s_sleep(1);
            ++polls;
        }
        if (polls == kLayoutSpinLimit) complete = false;
        store_agent(flags + i, 0);
    }
    if (!complete) atomicOr(p.status, DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT);
    __syncthreads();
}

__device__ __forceinline__ void finish_hand_off(const MoveParams& p, bool done, uint32_t tag);

// The publisher of an expanded dispatch has read the launch's tag and stored its tagged words (the expert bases): once
// every thread's stores are acknowledged it reports as a party of the hand-off.  Without this a publisher that starts
// late could read the generation after the movers - which wait only for the bases they need, none if no lane is valid -
// have advanced it, and stamp its words with the next launch's tag; and the clearing of the tables at the end of a tag
// period could overtake stores of words no mover waits for.  All threads call it.
__device__ __forceinline__ void publisher_is_done_with_the_tag(const MoveParams& p, uint32_t tag) {
    wait_for_own_stores();
    __syncthreads();
    if (threadIdx.x < kWaveSize) finish_hand_off(p, true, tag);
}

__device__ __forceinline__ void fused_publish_block(const MoveParams& p) {
    extern __shared__ uint64_t count_lds[];
    const PublishLds lds = carve_publish_lds(reinterpret_cast<int*>(count_lds), p.R, p.E);
    const LayoutTables& tab = p.lay.tab;
    const uint32_t tag = launch_tag(p.generation);
    int32_t* tagged_bases = reinterpret_cast<int32_t*>(p.tagged_expert);

    // The movers of an expanded dispatch are waiting for the expert base table, which therefore goes out before
    // anything else, from the tagged chunk totals as they arrive.
    const bool bases_first = p.do_expand && p.E <= kThreads && p.count_blocks <= 32;
    if (bases_first) {
        const bool complete = write_expert_bases_from_registers<kThreads>(tab, p.tagged_expert_counts, tagged_bases, tag, kLayoutSpinLimit,
                                                                          p.R, p.E, p.pub.A, p.count_blocks, lds);
        if (!complete && threadIdx.x == 0) atomicOr(p.status, DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT);
        publisher_is_done_with_the_tag(p, tag);
    }

    // Everything else waits until the counting workgroups have flagged that their stores are acknowledged.  The expert
    // table (a row per chunk: one writer per cache line, and this workgroup has not touched it before) is then read
    // with ordinary loads, the rank table (lines shared by the writers of 16 chunks) at agent scope.
    await_and_clear_flags(p, p.chunk_done, p.count_blocks);
    sum_expert_columns<kThreads>(tab, p.R, p.E, p.count_blocks, lds.totals);
    publish_experts<kThreads>(p.pub, lds);
    if (p.do_expand && !bases_first) {
        __syncthreads();
        write_expert_bases<kThreads, true>(tab, tagged_bases, tag, p.E, p.count_blocks, lds);
        publisher_is_done_with_the_tag(p, tag);
    }
    __syncthreads();
    scan_rank_counts<kThreads>(p.pub, tab, p.R, lds);
}

// What a mover reads of the layout before the layout is known to be there: issued ahead of the payload loads, so
// that a mover that starts after the layout is complete (most of them) has paid no extra trip for it.  Ordinary
// loads, which this XCD's L2 may answer: a word that shows the tag of this launch is this launch's word wherever it
// was cached, and one that does not is read again at agent scope.
struct FirstLook {
    uint64_t totals_lo, totals_hi;     // this thread's four chunk totals
    uint32_t position;                 // this lane's position word
};

__device__ __forceinline__ FirstLook first_look(const MoveParams& p, int t, int lane, bool has_work) {
    FirstLook f{0, 0, 0};
    const int begin = int(threadIdx.x) * 4;
    if (begin < p.R * p.tab.chunks_padded) {
        const vec16 v = load16(p.tagged_rank + begin);
        f.totals_lo = uint64_t(v.x) | (uint64_t(v.y) << 32);
        f.totals_hi = uint64_t(v.z) | (uint64_t(v.w) << 32);
    }
    if (has_work && lane < p.K) f.position = p.pos[int64_t(t) * p.K + lane];
    return f;
}

// The same words read again at agent scope, by a wavefront whose first look came back without the layout: issued before
// the wavefront turns to converting its tile, so that the answer travels while it computes.
__device__ __forceinline__ FirstLook second_look(const MoveParams& p, int t, int lane, bool has_work) {
    FirstLook f{0, 0, 0};
    const int begin = int(threadIdx.x) * 4;
    if (begin < p.R * p.tab.chunks_padded) {
        f.totals_lo = load_agent64(p.tagged_rank + begin);
        f.totals_hi = load_agent64(p.tagged_rank + begin + 2);
    }
    if (has_work && lane < p.K) f.position = uint32_t(load_agent(reinterpret_cast<const int*>(p.pos) + int64_t(t) * p.K + lane));
    return f;
}

// Has this wavefront's first look found everything it asked for?  (Wave-uniform.)
__device__ __forceinline__ bool look_is_complete(const MoveParams& p, const FirstLook& look, uint32_t tag, bool has_work, int lane) {
    bool ok = !(has_work && lane < p.K) || has_tag(look.position, tag);
    if (int(threadIdx.x) * 4 < p.R * p.tab.chunks_padded)
        ok = ok && has_tag(uint32_t(look.totals_lo), tag) && has_tag(uint32_t(look.totals_lo >> 32), tag) &&
             has_tag(uint32_t(look.totals_hi), tag) && has_tag(uint32_t(look.totals_hi >> 32), tag);
    return __all(ok);
}

__device__ __forceinline__ bool totals_tagged(uint64_t lo, uint64_t hi, uint32_t tag) {
    return has_tag(uint32_t(lo), tag) && has_tag(uint32_t(lo >> 32), tag) && has_tag(uint32_t(hi), tag) && has_tag(uint32_t(hi >> 32), tag);
}

// Every mover workgroup works the rank bases out for itself, into its LDS: the exclusive prefix sum over the flattened
// [rank][chunk] table of chunk totals, of which thread i brings entries 4i .. 4i + 3 (tags still on).  `complete`: this
// thread's waits all ended well.  All threads; ends with a barrier.  Returns whether every thread's did.
__device__ __forceinline__ bool build_rank_bases(const MoveParams& p, uint64_t lo, uint64_t hi, bool complete, const int*& bases_out) {
    extern __shared__ uint64_t count_lds[];
    int* bases = reinterpret_cast<int*>(count_lds);
    const int flat = p.R * p.tab.chunks_padded;           // a multiple of 4: a thread's entries share a row
    int* scan_tmp = bases + flat;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int begin = tid * 4;
    const int v0 = int(uint32_t(lo) & kTagValueMask), v1 = int(uint32_t(lo >> 32) & kTagValueMask);
    const int v2 = int(uint32_t(hi) & kTagValueMask), v3 = int(uint32_t(hi >> 32) & kTagValueMask);
    const int sum = v0 + v1 + v2 + v3;
    const int inc = wave_inclusive_sum(sum);
    if (lane == kWaveSize - 1) scan_tmp[wave] = inc;
    const int all_complete = __syncthreads_and(complete ? 1 : 0);
    int run = inc - sum;
    for (int w = 0; w < wave; ++w) run += scan_tmp[w];
    if (begin < flat) {
        bases[begin] = run;
        bases[begin + 1] = run + v0;
        bases[begin + 2] = run + v0 + v1;
        bases[begin + 3] = run + v0 + v1 + v2;
    }
    __syncthreads();
    bases_out = bases;
    return all_complete != 0;
}

// The mover workgroup is done reading tagged words: its first thread advances the gate.  The value the gate had is
// looked at a little later (settle_gate), after the rows have been resolved and the tile converted, so that most of
// the atomic's round trip is covered.
__device__ __forceinline__ unsigned advance_gate(const MoveParams& p, unsigned mover) {
    const unsigned gate = mover % unsigned(kDispatchGates);
    return atomicInc(p.gates + gate * kDispatchGateStride, movers_of_gate(p, gate) - 1u);
}

// Parties of a launch's hand-off: the gates in use and, for the expanded layout, the publishing workgroup, which reads
// the tag and stores tagged words (the expert bases) itself.
__device__ __forceinline__ unsigned hand_off_parties(const MoveParams& p) {
    const unsigned gates_in_use = p.num_movers < unsigned(kDispatchGates) ? p.num_movers : unsigned(kDispatchGates);
    return gates_in_use + (p.do_expand ? 1u : 0u);
}

// One party of the hand-off is done with this launch's tag (all lanes of one wavefront; `done` is looked at on the first
// lane): a gate whose movers have all read their tagged words, or the publisher of an expanded dispatch once its tagged
// stores are acknowledged.  The party that completes the count advances the generation: by then every tagged word of
// the launch has been read or acknowledged, and nobody will read the generation word for this launch again.  The launch
// that used the last tag clears the tagged tables first, all lanes together (a third of a megabyte: some 15 us once in
// 16383 launches).
__device__ __forceinline__ void finish_hand_off(const MoveParams& p, bool done, uint32_t tag) {
    const int lane = lane_id();
    int last = 0;
    if (lane == 0 && done) {
        const unsigned parties = hand_off_parties(p);
        last = atomicInc(p.gates_finished, parties - 1u) == parties - 1u ? 1 : 0;
    }
    if (__builtin_amdgcn_readfirstlane(last) == 0) return;
    uint32_t next = tag >> kTagShift;                     // generation + 1
    if (next == kTagPeriod) {
        for (int i = lane * 4; i < p.tagged_words; i += kWaveSize * 4) store16_agent(p.tagged + i, vec16{0, 0, 0, 0});
        wait_for_own_stores();
        next = 0;
    }
    if (lane == 0) store_agent(reinterpret_cast<int*>(p.generation), int(next));
}

// First wavefront of a mover workgroup (all its lanes), right before its payload stores - not after them: a wait for the
// atomic's answer behind the stores would be a wait for their acknowledgements too, with the wavefront and its workgroup's
// resources held that long (8192 x 7168 FP8, side by side on one GPU: 86.0 -> 85.7 us).  `seen` counts on its first lane.  The mover
// that was the last of its gate reports the gate.
__device__ __forceinline__ void settle_gate(const MoveParams& p, unsigned mover, unsigned seen, uint32_t tag) {
    const unsigned gate = mover % unsigned(kDispatchGates);
    finish_hand_off(p, seen == movers_of_gate(p, gate) - 1u, tag);
}

// A wavefront's wait (bounded) for the tagged words its threads want.  Returns whether this thread still misses one.
// While the layout is not there, thousands of wavefronts repeat their reads, and every request of theirs stands in
// front of the counting workgroups' stores somewhere: so a waiting wavefront first watches the one kind of word that
// comes last - the expert base of its first routing lane, else its token's position words: one 32-byte request per
// round - and only when that has arrived reads the rest again, whatever is still missing in one trip per round.
__device__ __forceinline__ bool await_tagged_words(uint32_t tag, bool wants_position, const int* position_at, uint32_t& position,
                                                   bool wants_totals, const uint32_t* totals_at, uint64_t& lo, uint64_t& hi,
                                                   bool wants_base, const int* base_at, uint32_t& base_word, unsigned spin_limit) {
    unsigned polls = 0;
    const uint64_t base_lanes = __ballot(wants_base);
    if (base_lanes != 0) {
        const bool watches = wants_base && lane_id() == __builtin_ctzll(base_lanes);
        while (__any(watches && !has_tag(base_word, tag)) && polls < spin_limit) {
            __builtin_amdgcn_s_sleep(4);
            if (watches) base_word = uint32_t(load_agent(base_at));
            ++polls;
        }
    } else {
        while (__any(wants_position && !has_tag(position, tag)) && polls < spin_limit) {
            __builtin_amdgcn_s_sleep(4);
            if (wants_position && !has_tag(position, tag)) position = uint32_t(load_agent(position_at));
            ++polls;
        }
    }
    bool missing;
    for (;;) {
        const bool no_position = wants_position && !has_tag(position, tag);
        const bool no_totals = wants_totals && !totals_tagged(lo, hi, tag);
        const bool no_base = wants_base && !has_tag(base_word, tag);
        missing = no_position || no_totals || no_base;
        if (!__any(missing) || polls >= spin_limit) break;
        if (polls != 0) __builtin_amdgcn_s_sleep(1);
        if (no_position) position = uint32_t(load_agent(position_at));
        if (no_totals) {
            lo = load_agent64(totals_at);
            hi = load_agent64(totals_at + 2);
        }
        if (no_base) base_word = uint32_t(load_agent(base_at));
        ++polls;
    }
    return missing;
}

// Mover workgroups that run beside a counting or the publishing workgroup on one CU read nothing but the layout until
// the layout is there.  A CU's vector memory pipeline takes the requests of all its wavefronts in order, and the payload
// loads of seven mover workgroups keep it busy for microseconds: stores of a counting workgroup that shares the CU
// queue up behind them (measured: positions issued 3.5 us after the launch on a quiet CU, 6 to 8 us beside prefetching
// movers), and every mover of the launch waits for those stores.  Workgroups are handed to the CUs breadth first -
// workgroup i of a launch starts on CU i % num_cus while the first seven or eight per CU are being placed (read back
// from the hardware id registers on MI355X) - so the neighbours of workgroups 0 .. count_blocks are known by index.
// Should a GPU place workgroups differently, the rule holds back other movers: slower, never wrong.
__device__ __forceinline__ bool shares_cu_with_layout_work(const MoveParams& p) {
    return blockIdx.x % unsigned(p.num_cus) <= unsigned(p.count_blocks) && blockIdx.x < unsigned(p.num_cus) * 8u;
}

// Such a workgroup's wait (bounded; await_layout reports a wait that ran out): repeats the first look until it is complete.
__device__ __forceinline__ void hold_for_layout(const MoveParams& p, uint32_t tag, FirstLook& look, int t, int lane, bool has_work) {
    uint32_t no_base = 0;
    const int begin = int(threadIdx.x) * 4;
    await_tagged_words(tag, has_work && lane < p.K, reinterpret_cast<const int*>(p.pos) + int64_t(t) * p.K + lane, look.position,
                       begin < p.R * p.tab.chunks_padded, p.tagged_rank + begin, look.totals_lo, look.totals_hi, false, nullptr, no_base,
                       p.mover_spin_limit);
}

// Everything a mover wavefront needs from the layout of its own launch.
struct FusedLayout {
    const int* flat_bases;    // LDS: exclusive prefix over the chunk totals of the rank buckets
    uint32_t position;        // this lane's position word (tag included)
    int expert_base;          // expanded layout: first row of (this token's chunk, this lane's expert)
    unsigned gate_seen;       // first thread: what advance_gate returned
    uint32_t tag;
    bool complete;            // false: a wait ran out (status already set); the wavefront stores nothing
};

__device__ __forceinline__ FusedLayout await_layout(const MoveParams& p, unsigned mover, const FirstLook& look, uint32_t tag,
                                                    const RouteInputs& in, int t, int lane, bool has_work) {
    FusedLayout f{nullptr, look.position, 0, 0u, tag, true};
    // What this thread waits for: the position word of its lane, four chunk totals, and for the expanded layout the
    // base of its lane's (chunk, expert).  Whatever is missing is read again, all of it in one trip per round.
    const bool wants_position = has_work && lane < p.K;
    const int* position_at = reinterpret_cast<const int*>(p.pos) + int64_t(t) * p.K + lane;
    const int begin = int(threadIdx.x) * 4;
    const bool wants_totals = begin < p.R * p.tab.chunks_padded;
    uint64_t lo = look.totals_lo, hi = look.totals_hi;
    bool wants_base = false;
    const int* base_at = nullptr;
    uint32_t base_word = 0;
    if (p.do_expand) {
        const int64_t e = p.route_mask != nullptr ? (in.mask_byte != 0 ? int64_t(lane) : int64_t(-1)) : in.raw;
        wants_base = wants_position && e >= 0 && e < p.E;
        base_at = reinterpret_cast<const int*>(p.tagged_expert) + int64_t(t / kLayoutChunk) * p.tab.experts_padded + (wants_base ? int(e) : 0);
        if (wants_base) base_word = uint32_t(*base_at);       // an ordinary load first, as in first_look
    }
    const bool missing = await_tagged_words(tag, wants_position, position_at, f.position, wants_totals, p.tagged_rank + begin, lo, hi,
                                            wants_base, base_at, base_word, p.mover_spin_limit);
    f.expert_base = int(base_word & kTagValueMask);
    const bool complete = build_rank_bases(p, lo, hi, !missing, f.flat_bases);      // ends with a workgroup barrier
    if (threadIdx.x == 0) {
        f.gate_seen = advance_gate(p, mover);
        if (!complete) atomicOr(p.status, DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT);
    }
    f.complete = complete;
    return f;
}

// Workgroups of a single-launch dispatch a CU holds at a time (six wavefronts per SIMD, one per SIMD and workgroup).
constexpr int kResidentWorkgroupsPerCu = 6;

// While the layout is being counted nothing can be stored, and the movers that are resident at launch can only hold so
// much payload in their registers (25 MB at 8192 x 7168): for several microseconds HBM has little to do.  Those movers
// therefore also ask for the tile of the work item two rounds of residents ahead of their own - loads that land in a
// piece of LDS nobody reads, so they cost no registers - which brings that data into the caches while memory is idle
// (a round ahead or three measured less).  Side by side at 8192 x 7168: 86.8 -> 84.9 us in a hot loop, 82.9 -> 81.4 with a
// freshly written input, 89.8 -> 90.3 after a cache flush; 4096 tokens 48.8 -> 46.2 / 49.4 -> 44.4 / 50.7 -> 50.9; 16384
// tokens 164.0 -> 162.6 / 167.7 -> 166.2 / 168.6 -> 169.2.  Movers beside the counting workgroups stay out of it.
// The loads are issued before the wavefront's own payload loads and return in order, so they have landed by the time
// the wavefront uses its payload.  Returns whether the wavefront issued any.
template <int kPairs>
__device__ __forceinline__ bool warm_next_rounds(const MoveParams& p, unsigned work, int lane) {
    if (p.warm_lds_offset == 0 || blockIdx.x >= unsigned(p.num_cus) * unsigned(kResidentWorkgroupsPerCu) ||
        shares_cu_with_layout_work(p))
        return false;
    const unsigned ahead = work + p.warm_ahead;
    if (ahead >= unsigned(p.T) * unsigned(p.tiles)) return false;
    extern __shared__ uint64_t count_lds[];
    const int t = int(ahead / unsigned(p.tiles));
    const int tile = int(ahead - unsigned(t) * unsigned(p.tiles));
    const uint8_t* src = p.x + int64_t(t) * p.row_bytes;
    uint8_t* landing = reinterpret_cast<uint8_t*>(count_lds) + p.warm_lds_offset + (threadIdx.x >> 6) * 1024;
#pragma unroll
    for (int q = 0; q < kPairs; ++q) {
        const int elem = (tile * kPairs + q) * 1024 + lane * 16;
        if (elem < p.H) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + int64_t(elem) * 2),
                                             (__attribute__((address_space(3))) void*)landing, 16, 0, 0);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + int64_t(elem) * 2 + 16),
                                             (__attribute__((address_space(3))) void*)landing, 16, 0, 0);
        }
    }
    return true;
}

// The same for the pass-through kernel, whose tile is kVecs KB of a row (BF16, 4096 x 7168: 80.3 -> 77.2 us in a hot loop,
// 75.6 -> 74.0 with a freshly written input, 83.3 -> 84.0 after a cache flush; 4600 tokens 92.9 -> 86.0 / 85.9 -> 83.5 / 95.3 -> 91.3).
template <int kVecs>
__device__ __forceinline__ bool warm_next_rounds_of_rows(const MoveParams& p, unsigned work, int lane) {
    if (p.warm_lds_offset == 0 || blockIdx.x >= unsigned(p.num_cus) * unsigned(kResidentWorkgroupsPerCu) ||
        shares_cu_with_layout_work(p))
        return false;
    const unsigned ahead = work + p.warm_ahead;
    if (ahead >= unsigned(p.T) * unsigned(p.tiles)) return false;
    extern __shared__ uint64_t count_lds[];
    const int t = int(ahead / unsigned(p.tiles));
    const int tile = int(ahead - unsigned(t) * unsigned(p.tiles));
    const uint8_t* src = p.x + int64_t(t) * p.row_bytes;
    uint8_t* landing = reinterpret_cast<uint8_t*>(count_lds) + p.warm_lds_offset + (threadIdx.x >> 6) * 1024;
#pragma unroll
    for (int i = 0; i < kVecs; ++i) {
        const int off = (tile * kVecs + i) * 1024 + lane * 16;
        if (off < p.row_bytes)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + off),
                                             (__attribute__((address_space(3))) void*)landing, 16, 0, 0);
    }
    return true;
}

// ---- pass-through payload (BF16, or FP8 with caller-provided scale packs) ----
template <int kVecs, bool kFused>
__device__ __forceinline__ void dispatch_copy(const MoveParams& p) {
    if constexpr (kFused) {
        if (blockIdx.x <= unsigned(p.count_blocks)) {
            if (blockIdx.x < unsigned(p.count_blocks)) fused_count_block(p);
            else fused_publish_block(p);
            return;
        }
    }
    const int lane = threadIdx.x & 63;
    const unsigned mover = blockIdx.x - (kFused ? unsigned(p.count_blocks) + 1u : 0u);
    const unsigned block = p.xcd_remap ? xcd_contiguous_block(mover, p.num_movers) : mover;
    const unsigned work = wave_work_index(block, kWavesPerBlock);
    const bool has_work = work < unsigned(p.T) * unsigned(p.tiles);
    if (!has_work && !kFused) return;
    const int t = has_work ? int(work / unsigned(p.tiles)) : 0;
    const int tile = has_work ? int(work - unsigned(t) * unsigned(p.tiles)) : 0;
    uint32_t tag = 0;
    FirstLook look{0, 0, 0};
    if constexpr (kFused) {
        tag = launch_tag(p.generation);
        look = first_look(p, t, lane, has_work);
        if (shares_cu_with_layout_work(p)) hold_for_layout(p, tag, look, t, lane, has_work);
    }

    bool warmed = false;
    if constexpr (kFused) warmed = warm_next_rounds_of_rows<kVecs>(p, work, lane);

    vec16 v[kVecs];
    const uint8_t* src = p.x + int64_t(t) * p.row_bytes;
#pragma unroll
    for (int i = 0; i < kVecs; ++i) {
        const int off = (tile * kVecs + i) * 1024 + lane * 16;
        v[i] = vec16{0, 0, 0, 0};
        if (has_work && off < p.row_bytes) v[i] = load16_stream(src + off);
    }

    const RouteInputs route_in = load_route_inputs(p, t, lane);
    const int* flat_bases = nullptr;
    uint32_t word;
    int expert_base = 0;
    unsigned gate_seen = 0;
    if constexpr (kFused) {
        // Payload and routing inputs are in flight; wait for this launch's layout.
        const FusedLayout f = await_layout(p, mover, look, tag, route_in, t, lane, has_work);
        gate_seen = f.gate_seen;
        if (!has_work || !f.complete) {
            if (warmed) wait_for_own_stores();       // no load may still be on its way into this workgroup's LDS
            if (threadIdx.x < kWaveSize) settle_gate(p, mover, gate_seen, tag);
            return;
        }
        word = f.position;
        flat_bases = f.flat_bases;
        expert_base = f.expert_base;
    } else {
        word = load_position_word(p, t, lane);
    }
    const Route r = resolve_route<kFused>(p, route_in, word, flat_bases, expert_base, t, lane, tile == 0);
    if (tile == 0) write_token_metadata(p, r, t, lane);
    if constexpr (kFused)
        if (threadIdx.x < kWaveSize) settle_gate(p, mover, gate_seen, tag);

    int row_of_lane;
    uint64_t dests = destination_lanes(p, r, row_of_lane);
    while (dests) {
        const int j = __builtin_ctzll(dests);
        dests &= dests - 1;
        const int row = read_lane(row_of_lane, j);
        uint8_t* dst = p.recv_x + int64_t(row) * p.row_bytes;
#pragma unroll
        for (int i = 0; i < kVecs; ++i) {
            const int off = (tile * kVecs + i) * 1024 + lane * 16;
            if (off < p.row_bytes) store16_stream(dst + off, v[i]);
        }
        if (tile == 0 && p.recv_sf != nullptr) {
            for (int g = lane; g < p.num_sf_packs; g += kWaveSize)
                p.recv_sf[int64_t(row) * p.rsf_ts + int64_t(g) * p.rsf_hs] =
                    p.sf[int64_t(t) * p.sf_ts + int64_t(g) * p.sf_hs];
        }
    }
}

// Measurement build only (-DDEEP_EP_HIP_WAVE_STAMPS, a library of its own that bench.py --wave-spans loads): every mover
// wavefront of the fused-cast kernels records when it started, when it had issued its last store and when its stores
// were acknowledged, on the 100 MHz wall clock: the span of a launch's wavefronts beside its launch-to-launch time, the
// lifetime of a wavefront, how long before the end the last one starts.
#ifdef DEEP_EP_HIP_WAVE_STAMPS
constexpr int kMaxStampedWaves = 65536;
__device__ long long wave_stamps[3 * kMaxStampedWaves];
#endif

// ---- fused BF16 -> e4m3 cast: lane owns 16 consecutive channels, 8 lanes own one 128-group ----
template <int kPairs, bool kFused>
__device__ __forceinline__ void dispatch_cast(const MoveParams& p) {
    if constexpr (kFused) {
        if (blockIdx.x <= unsigned(p.count_blocks)) {
            if (blockIdx.x < unsigned(p.count_blocks)) fused_count_block(p);
            else fused_publish_block(p);
            return;
        }
    }
    const int lane = threadIdx.x & 63;
#ifdef DEEP_EP_HIP_WAVE_STAMPS
    const long long stamp_start = wall_clock64();
#endif
    const unsigned mover = blockIdx.x - (kFused ? unsigned(p.count_blocks) + 1u : 0u);
    const unsigned block = p.xcd_remap ? xcd_contiguous_block(mover, p.num_movers) : mover;
    const unsigned work = wave_work_index(block, kWavesPerBlock);
    const bool has_work = work < unsigned(p.T) * unsigned(p.tiles);
    if (!has_work && !kFused) return;
    const int t = has_work ? int(work / unsigned(p.tiles)) : 0;
    const int tile = has_work ? int(work - unsigned(t) * unsigned(p.tiles)) : 0;
    uint32_t tag = 0;
    FirstLook look{0, 0, 0};
    if constexpr (kFused) {
        tag = launch_tag(p.generation);
        look = first_look(p, t, lane, has_work);
        if (shares_cu_with_layout_work(p)) hold_for_layout(p, tag, look, t, lane, has_work);
    }

    bool warmed = false;
    if constexpr (kFused) warmed = warm_next_rounds<kPairs>(p, work, lane);

    vec16 in[kPairs][2];
    const uint8_t* src = p.x + int64_t(t) * p.row_bytes;
#pragma unroll
    for (int q = 0; q < kPairs; ++q) {
        const int elem = (tile * kPairs + q) * 1024 + lane * 16;
        in[q][0] = vec16{0, 0, 0, 0};
        in[q][1] = vec16{0, 0, 0, 0};
        if (has_work && elem < p.H) {
            if (p.plain_loads) {
                in[q][0] = load16(src + int64_t(elem) * 2);
                in[q][1] = load16(src + int64_t(elem) * 2 + 16);
            } else {
                in[q][0] = load16_stream(src + int64_t(elem) * 2);
                in[q][1] = load16_stream(src + int64_t(elem) * 2 + 16);
            }
        }
    }

    const RouteInputs route_in = load_route_inputs(p, t, lane);

    vec16 out[kPairs];
    float my_scale = 0.f;   // lane L < 8*kPairs ends up holding the scale of group (tile*kPairs*8 + L)
    auto cast_tile = [&]() {
#pragma unroll
        for (int q = 0; q < kPairs; ++q) {
            const float scale_inv = cast_16_channels(in[q][0], in[q][1], out[q]);
            const float gathered = __shfl(scale_inv, (lane & 7) * 8, kWaveSize);
            if ((lane >> 3) == q) my_scale = gathered;
        }
    };

    const int* flat_bases = nullptr;
    uint32_t word;
    int expert_base = 0;
    unsigned gate_seen = 0;
    bool cast_done = false;
    if constexpr (kFused) {
        // Payload and routing inputs are in flight.  A wavefront whose first look found the layout (any wavefront that
        // starts after the first microseconds of the launch) resolves its rows while the payload arrives, as in a
        // launch of its own.  One that has to wait for the layout converts its tile first: when the layout appears,
        // every resident wavefront of the chip is released at once, and the conversions (a few hundred vector
        // instructions each, eight wavefronts to a SIMD) would otherwise queue up between that moment and the first
        // stores of the launch.
        if (!look_is_complete(p, look, tag, has_work, lane)) {
            look = second_look(p, t, lane, has_work);
            cast_tile();
            cast_done = true;
        }
        const FusedLayout f = await_layout(p, mover, look, tag, route_in, t, lane, has_work);
        gate_seen = f.gate_seen;
        if (!has_work || !f.complete) {
            if (warmed) wait_for_own_stores();       // no load may still be on its way into this workgroup's LDS
            if (threadIdx.x < kWaveSize) settle_gate(p, mover, gate_seen, tag);
            return;
        }
        word = f.position;
        flat_bases = f.flat_bases;
        expert_base = f.expert_base;
    } else {
        word = load_position_word(p, t, lane);
    }
    const Route r = resolve_route<kFused>(p, route_in, word, flat_bases, expert_base, t, lane, tile == 0);
    if (tile == 0) write_token_metadata(p, r, t, lane);
    if (!cast_done) cast_tile();
    if constexpr (kFused)
        if (threadIdx.x < kWaveSize) settle_gate(p, mover, gate_seen, tag);
    const int group = tile * kPairs * 8 + lane;
    const bool owns_scale = lane < kPairs * 8 && group * 128 < p.H;

    int row_of_lane;
    uint64_t dests = destination_lanes(p, r, row_of_lane);
    while (dests) {
        const int j = __builtin_ctzll(dests);
        dests &= dests - 1;
        const int row = read_lane(row_of_lane, j);
        uint8_t* dst = p.recv_x + int64_t(row) * p.H;
#pragma unroll
        for (int q = 0; q < kPairs; ++q) {
            const int elem = (tile * kPairs + q) * 1024 + lane * 16;
            if (elem < p.H) store16_stream(dst + elem, out[q]);
        }
        if (owns_scale)
            p.recv_sf[int64_t(row) * p.rsf_ts + int64_t(group) * p.rsf_hs] = __float_as_uint(my_scale);
    }
#ifdef DEEP_EP_HIP_WAVE_STAMPS
    if (lane == 0 && work < unsigned(kMaxStampedWaves)) {
        const long long issued = wall_clock64();
        wait_for_own_stores();
        long long* at = wave_stamps + size_t(work) * 3;
        at[0] = stamp_start;
        at[1] = issued;
        at[2] = wall_clock64();
    }
#endif
}

// ---- the same move as a persistent kernel with a work queue (tuning.persistent_movers) ----
// One workgroup per compute unit stays resident: a few mover wavefronts and a feeder.  Items (token, column tile) are
// handed out in chunks.  A chunk owns sixteen consecutive tickets of the workgroup's ticket counter (LDS) whatever its
// size; a mover draws a ticket, looks the chunk up in a ring of 64-bit words (chunk number, size, first item) and takes
// item `first + offset`, or draws again if the offset lies past the chunk's size.  It requests the loads of its next item
// - payload tile, top-k id, weight, position word, base row of the destination rank - before it converts and stores the
// current one.  The feeder keeps the ring one chunk ahead of the ticket counter: it asks one global counter for chunks
// (one atomic per chunk; the chunks shrink towards the end so that the workgroups run dry together) and posts them; a
// chunk of size zero ends the workgroup.  A feeder that sees the end reports to a wrapping counter at once - its workgroup
// asks for nothing after that - and the last one to report puts the global counter back to zero for the next launch.
//
// Kept as a measured alternative, not a default: on MI355X (8192 x 7168 FP8, move phase on a finished layout) it takes
// 86-95 us from launch to launch against 81 us for one short-lived wavefront per item.  With a static split of the items
// instead of the queue the same loop took 95-104 us: wavefronts get through their items at very different speeds, and
// the slowest ones set the time.  Whether a looping wavefront waits for the acknowledgement of its own stores before it
// uses the loads it issued ahead made no difference when measured (look-ahead loads issued by hand and waited for by
// count, the stores left in flight).
constexpr int kQueueSlot = 16;               // tickets per chunk
constexpr int kQueueStatic = 2;              // chunks a workgroup owns by index (no atomic)
constexpr int kQueueRing = 16;
constexpr int kQueueCounterLine = 128;       // the gate line (kernels.h) that serves as the global item counter

__device__ __forceinline__ unsigned long long queue_word(unsigned chunk, unsigned size, unsigned base) {
    return ((unsigned long long)(((chunk + 1u) << 8) | size) << 32) | base;
}

// Everything a mover needs of one item, requested together.
template <int kPairs>
struct QueuedItem {
    vec16 in[kPairs][2];
    int64_t raw;         // topk_idx entry of routing lane min(lane, K - 1)
    float w;             // its weight
    uint32_t word;       // its position word
    int base;            // base row of (rank min(lane, R - 1), the token's chunk)
};

template <int kPairs>
__device__ __forceinline__ void load_queued_item(const MoveParams& p, unsigned work, int lane, QueuedItem<kPairs>& item) {
    const int t = int(work / unsigned(p.tiles));
    const int tile = int(work - unsigned(t) * unsigned(p.tiles));
    const int64_t at = int64_t(t) * p.K + min(lane, p.K - 1);
    item.raw = p.topk_idx[at];
    item.word = p.pos[at];
    item.w = p.topk_weights != nullptr ? p.topk_weights[at] : 0.f;
    item.base = layout_word(p.tab.rank_bases + int64_t(min(lane, p.R - 1)) * p.tab.chunks_padded + t / kLayoutChunk);
    const uint8_t* src = p.x + int64_t(t) * p.row_bytes;
#pragma unroll
    for (int q = 0; q < kPairs; ++q) {
        // a segment past the end of the row reads the row's last 32 bytes instead (never stored)
        const int elem = min((tile * kPairs + q) * 1024 + lane * 16, p.H - 16);
        item.in[q][0] = load16_stream(src + int64_t(elem) * 2);
        item.in[q][1] = load16_stream(src + int64_t(elem) * 2 + 16);
    }
}

// Routes, converts and stores one item: resolve_route for the one case this kernel is launched for (compact layout, no
// cached handle, top-k routing, at most 64 ranks), with every word it needs already requested.
template <int kPairs>
__device__ __forceinline__ void finish_queued_item(const MoveParams& p, unsigned work, int lane, const QueuedItem<kPairs>& item,
                                                   int start_of_rank) {
    const int t = int(work / unsigned(p.tiles));
    const int tile = int(work - unsigned(t) * unsigned(p.tiles));
    Route r{-1, -1, -1, -1, -1, lane < p.K ? item.w : 0.f};
    int slot = -1;
    if (lane < p.K) {
        if (item.raw >= 0 && item.raw < p.E) r.e = int(item.raw);
        slot = (item.word & kNoPosition) == kNoPosition ? -1 : int(item.word & kNoPosition);
    }
    if (r.e >= 0) r.d = small_div(r.e, p.rcp_E_l);
    else slot = -1;
    {
        const int from = r.d >= 0 ? r.d : 0;
        const int base = __shfl(item.base, from, kWaveSize);
        const int start = __shfl(start_of_rank, from, kWaveSize);
        if (r.d >= 0 && slot >= 0) {
            r.row_c = base + slot;
            slot = r.row_c - start;             // slot inside the destination bucket
        }
    }
    if (tile == 0 && lane < p.K && p.dst_buffer_slot_idx != nullptr)
        p.dst_buffer_slot_idx[int64_t(t) * p.K + lane] = (r.e >= 0 && slot >= 0) ? p.rank_idx * p.M + slot : -1;
    for (int j = 0; j < p.K; ++j) {
        const int dj = read_lane(r.d, j);
        const int rj = read_lane(r.row_c, j);
        if (r.d >= 0 && dj == r.d && rj >= 0) r.my_row = rj;
    }
    if (tile == 0) write_token_metadata(p, r, t, lane);
    vec16 out[kPairs];
    float my_scale = 0.f;
#pragma unroll
    for (int q = 0; q < kPairs; ++q) {
        const float scale_inv = cast_16_channels(item.in[q][0], item.in[q][1], out[q]);
        const float gathered = __shfl(scale_inv, (lane & 7) * 8, kWaveSize);
        if ((lane >> 3) == q) my_scale = gathered;
    }
    const int group = tile * kPairs * 8 + lane;
    const bool owns_scale = lane < kPairs * 8 && group * 128 < p.H;
    int row_of_lane;
    uint64_t dests = destination_lanes(p, r, row_of_lane);
    while (dests) {
        const int j = __builtin_ctzll(dests);
        dests &= dests - 1;
        const int row = read_lane(row_of_lane, j);
        uint8_t* dst = p.recv_x + int64_t(row) * p.H;
#pragma unroll
        for (int q = 0; q < kPairs; ++q) {
            const int elem = (tile * kPairs + q) * 1024 + lane * 16;
            if (elem < p.H) store16_stream(dst + elem, out[q]);
        }
        if (owns_scale) p.recv_sf[int64_t(row) * p.rsf_ts + int64_t(group) * p.rsf_hs] = __float_as_uint(my_scale);
    }
}

template <int kPairs, int kQueueThreads>
__global__ __launch_bounds__(kQueueThreads) void dispatch_cast_queue_kernel(const MoveParams p) {
    constexpr int kQueueWaves = kQueueThreads / kWaveSize;
    __shared__ unsigned ticket;
    __shared__ unsigned long long ring[kQueueRing];
    const int lane = threadIdx.x & 63;
    const unsigned total = unsigned(p.T) * unsigned(p.tiles);
    const unsigned static_items = gridDim.x * unsigned(kQueueStatic * kQueueSlot);
    uint32_t* counter = p.gates + kQueueCounterLine * kDispatchGateStride;
    if (threadIdx.x < kQueueRing) {
        const unsigned c = threadIdx.x;
        unsigned long long word = 0ull;
        if (c < unsigned(kQueueStatic)) {
            const unsigned base = (blockIdx.x * unsigned(kQueueStatic) + c) * unsigned(kQueueSlot);
            word = queue_word(c, base < total ? min(unsigned(kQueueSlot), total - base) : 0u, base);
        }
        ring[c] = word;
        if (c == 0) ticket = 0u;
    }
    __syncthreads();

    if ((threadIdx.x >> 6) == kQueueWaves - 1) {
        // ---- the feeder (one lane) ----
        if (lane != 0) return;
        unsigned posted = kQueueStatic;
        bool ended = (blockIdx.x * unsigned(kQueueStatic) + unsigned(kQueueStatic) - 1u) * unsigned(kQueueSlot) >= total;
        unsigned size = kQueueSlot;
        unsigned polls = 0;
        while (!ended) {
            const unsigned drawing = __hip_atomic_load(&ticket, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) / unsigned(kQueueSlot);
            if (posted > drawing + 1u) {                    // the chunk being drawn and one more are there
                __builtin_amdgcn_s_sleep(8);
                if (++polls > (1u << 26)) {                 // movers that never draw again: give up, and say so
                    atomicOr(p.status, DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT);
                    break;
                }
                continue;
            }
            const unsigned base = static_items + atomicAdd(counter, size);
            if (base >= total) {
                __hip_atomic_store(&ring[posted % kQueueRing], queue_word(posted, 0u, total), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                ended = true;
            } else {
                __hip_atomic_store(&ring[posted % kQueueRing], queue_word(posted, min(size, total - base), base), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_WORKGROUP);
                ++posted;
                const unsigned left = total - base;
                size = left > total / 4u ? 16u : left > total / 16u ? 8u : 4u;
            }
        }
        if (atomicInc(p.gates_finished, gridDim.x - 1u) == gridDim.x - 1u) atomicExch(counter, 0u);
        return;
    }

    // ---- a mover ----
    // The wavefront's next item, or `total` for none.
    auto draw = [&]() {
        for (;;) {
            unsigned n = 0;
            if (lane == 0) n = __hip_atomic_fetch_add(&ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            n = unsigned(__builtin_amdgcn_readfirstlane(int(n)));
            const unsigned c = n / unsigned(kQueueSlot), o = n % unsigned(kQueueSlot);
            unsigned long long word;
            unsigned spins = 0;
            for (;;) {
                word = __hip_atomic_load(&ring[c % kQueueRing], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                if (unsigned(word >> 40) == c + 1u) break;
                __builtin_amdgcn_s_sleep(2);
                if (++spins > (1u << 24)) {                 // a feeder that makes no progress, or a slot that went on to a later chunk
                    if (lane == 0) atomicOr(p.status, DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT);
                    return total;
                }
            }
            const unsigned size = unsigned(word >> 32) & 0xffu;
            if (size == 0u) return total;
            if (o < size) return unsigned(word) + o;
        }
    };

    unsigned work = draw();
    if (work >= total) return;
    const int start_of_rank = layout_word(p.tab.rank_bases + int64_t(min(lane, p.R - 1)) * p.tab.chunks_padded);
    QueuedItem<kPairs> cur;
    load_queued_item<kPairs>(p, work, lane, cur);
    for (;;) {                                              // every mover leaves through the first branch
        const unsigned next = draw();
        if (next >= total) {
            finish_queued_item<kPairs>(p, work, lane, cur, start_of_rank);
            return;
        }
        QueuedItem<kPairs> ahead;
        load_queued_item<kPairs>(p, next, lane, ahead);
        finish_queued_item<kPairs>(p, work, lane, cur, start_of_rank);
        cur = ahead;
        work = next;
    }
}

// The kernels.  The single-launch forms also hold the counting and publishing code, whose register needs must not cost
// the movers their occupancy: they are held to six wavefronts per SIMD (80 registers) - six workgroups per CU, which
// is also where the move streams fastest (more were slower when tried with a leaner counting step, fewer are slower too).
template <int kVecs>
__global__ __launch_bounds__(kThreads) void dispatch_copy_kernel(const MoveParams p) {
    dispatch_copy<kVecs, false>(p);
}
template <int kVecs>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(6, 8))) void dispatch_copy_single_launch_kernel(const MoveParams p) {
    dispatch_copy<kVecs, true>(p);
}
template <int kPairs>
__global__ __launch_bounds__(kThreads) void dispatch_cast_kernel(const MoveParams p) {
    dispatch_cast<kPairs, false>(p);
}
template <int kPairs>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(6, 8))) void dispatch_cast_single_launch_kernel(const MoveParams p) {
    dispatch_cast<kPairs, true>(p);
}

// ---- zero the alignment padding rows of the expanded layout ----
__global__ __launch_bounds__(kThreads) void zero_padding_kernel(const PadParams p) {
    const int lane = threadIdx.x & 63;
    const int64_t work = int64_t(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
    const int pad_slots = p.A - 1;
    if (work >= int64_t(p.E) * pad_slots) return;
    const int e = int(work / pad_slots);
    const int i = int(work - int64_t(e) * pad_slots);
    const int cnt = p.num_unaligned[e];
    const int aligned = (cnt + p.A - 1) / p.A * p.A;
    if (i >= aligned - cnt) return;
    const int64_t row = int64_t(p.psum_expert[e]) + i;      // start + actual count + i
    if (row >= p.expanded_capacity) return;
    uint8_t* dst = p.recv_x + row * p.out_row_bytes;
    const vec16 zero{0, 0, 0, 0};
    for (int off = lane * 16; off < p.out_row_bytes; off += kWaveSize * 16) store16(dst + off, zero);
    if (p.recv_sf != nullptr)
        for (int g = lane; g < p.num_sf_packs; g += kWaveSize) p.recv_sf[row * p.rsf_ts + int64_t(g) * p.rsf_hs] = 0u;
    if (p.recv_topk_weights != nullptr && lane == 0) p.recv_topk_weights[row] = 0.f;
}

// ---- stand-alone per-token cast (identity routing) ----
__global__ __launch_bounds__(kThreads) void cast_kernel(const CastParams p) {
    const int lane = threadIdx.x & 63;
    const int groups = (p.H + 127) / 128;
    const int tiles = (p.H + 1023) / 1024;
    const int64_t work = int64_t(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
    if (work >= int64_t(p.T) * tiles) return;
    const int t = int(work / tiles);
    const int tile = int(work - int64_t(t) * tiles);
    const int elem = tile * 1024 + lane * 16;
    const uint16_t* src = reinterpret_cast<const uint16_t*>(p.x) + int64_t(t) * p.H;
    float f[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) f[i] = (elem + i < p.H) ? __uint_as_float(uint32_t(src[elem + i]) << 16) : 0.f;
    const float amax = group_amax<true>(f);       // a NaN in the group reaches its scale, as in the torch recipe
    const float scale = 448.0f / amax;
    const float scale_inv = amax / 448.0f;
    uint8_t* dst = p.out + int64_t(t) * p.H;
#pragma unroll
    for (int i = 0; i < 16; i += 4) {
        const uint32_t packed = pack_e4m3x4(f[i] * scale, f[i + 1] * scale, f[i + 2] * scale, f[i + 3] * scale);
#pragma unroll
        for (int b = 0; b < 4; ++b)
            if (elem + i + b < p.H) dst[elem + i + b] = uint8_t(packed >> (8 * b));
    }
    const int group = elem / 128;
    if ((lane & 7) == 0 && group < groups && elem < p.H) p.scales[int64_t(t) * groups + group] = scale_inv;
}

// ---- V1 handle bookkeeping (csrc/kernels/legacy/intranode.cu:94-125): one workgroup per destination rank
// counts the tokens of each channel (contiguous token range) that go there, then prefix-sums over channels ----
__global__ __launch_bounds__(kThreads) void intranode_prefix_kernel(const IntranodePrefixParams p) {
    extern __shared__ int channel_counts[];     // [C]
    const int d = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int per_channel = (p.T + p.C - 1) / p.C;
    for (int c = wave; c < p.C; c += kWavesPerBlock) {
        const int begin = min(per_channel * c, p.T), end = min(begin + per_channel, p.T);
        int count = 0;
        for (int t = begin + lane; t < end; t += kWaveSize) count += p.mask[int64_t(t) * p.R + d] != 0 ? 1 : 0;
        count = wave_inclusive_sum(count);
        if (lane == kWaveSize - 1) channel_counts[c] = count;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int c = 0; c < p.C; ++c) {
            if (p.recv_channel_prefix_matrix != nullptr) p.recv_channel_prefix_matrix[d * p.C + c] = run;
            run += channel_counts[c];
            if (p.channel_prefix_matrix != nullptr) p.channel_prefix_matrix[d * p.C + c] = run;
            channel_counts[c] = run;
        }
    }
    __syncthreads();
    // Only this source rank sends in a one-GPU call: the prefix over source ranks steps once, at rank_idx.
    const int total = p.C > 0 ? channel_counts[p.C - 1] : 0;
    if (p.rank_prefix_matrix != nullptr)
        for (int i = threadIdx.x; i < p.R; i += kThreads) p.rank_prefix_matrix[i * p.R + d] = i >= p.rank_idx ? total : 0;
}

// ---- rows of recv_topk_idx beyond the received ones read -1 (csrc/kernels/legacy/intranode.cu:535-545) ----
__global__ __launch_bounds__(kThreads) void fill_tail_kernel(const FillTailParams p) {
    const int64_t first = int64_t(*p.total_rows) * p.K;
    const int64_t end = p.capacity * p.K;
    for (int64_t i = first + int64_t(blockIdx.x) * kThreads + threadIdx.x; i < end; i += int64_t(gridDim.x) * kThreads)
        p.recv_topk_idx[i] = -1;
}

// An attribute of the current device, asked once per device; `fallback` when the runtime does not answer.
static int device_attribute(hipDeviceAttribute_t attribute, std::atomic<int>* cached, int fallback) {
    constexpr int kMaxDevices = 64;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fallback;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, attribute, dev) != hipSuccess || n <= 0) n = fallback;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

static int lds_bytes_per_cu() {
    static std::atomic<int> cached[64];
    return device_attribute(hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, cached, 160 * 1024);
}

// How many workgroups of a move kernel launched on a finished layout a CU should hold at a time (0: as many as fit).
// The fused cast streams fastest with fewer than the eight its registers allow - measured side by side at 8192 x 7168,
// move phase in us with 8 / 7 / 6 / 5 / 4 per CU: compact layout 82.6 / 81.6 / 81.7 / 82.0 / 83.6 (16384 tokens: 162.5 with
// eight, 156.5 with six), expanded layout 114.9 / 115.1 / 114.7 / 113.4 / 116.0 - while the BF16 copy does not care down
// to six and loses 3 us at five.  Launches that would not fill two rounds of eight per CU are left alone.
static int move_workgroups_per_cu(const MoveParams& p) {
    if (p.fused) return 0;
    if (p.move_workgroups_per_cu != 0)       // two is the least an LDS share within a workgroup's 64 KB can enforce
        return p.move_workgroups_per_cu >= 8 ? 0 : (p.move_workgroups_per_cu < 2 ? 2 : p.move_workgroups_per_cu);
    if (p.payload != DEEP_EP_HIP_PAYLOAD_CAST_FP8) return 0;
    if (int64_t(p.num_movers) < int64_t(compute_units()) * 16) return 0;
    return p.do_expand ? 5 : 6;
}

size_t move_lds_bytes(const MoveParams& p) {
    if (!p.fused) {
        // The limit is set with LDS the kernel never touches: a share that is just too large for one workgroup more,
        // whatever granule the LDS is handed out in.
        const int per_cu = move_workgroups_per_cu(p);
        if (per_cu == 0) return 0;
        return (size_t(lds_bytes_per_cu() / (per_cu + 1)) + 256) & ~size_t(255);
    }
    const size_t publish = publish_lds_bytes(p.R, p.E, kThreads);
    const size_t bitmap = count_lds_bytes(p.R, p.E);
    const size_t bases = (size_t(p.R) * p.tab.chunks_padded + kWavesPerBlock) * sizeof(int);
    const size_t bytes = std::max(bases, std::max(bitmap, publish));
    return p.warm_lds_offset != 0 ? size_t(p.warm_lds_offset) + size_t(kWavesPerBlock) * 1024 : bytes;
}

// Grid: the counting workgroups of a single-launch dispatch come first.
unsigned move_grid(MoveParams& p, int64_t waves) {
    p.num_movers = unsigned((waves + kWavesPerBlock - 1) / kWavesPerBlock);
    return p.num_movers + unsigned(p.fused ? p.count_blocks + 1 : 0);
}

// Single launch: the movers that are resident at launch warm the caches for the round after next (warm_next_rounds).
// Call after move_grid.
void plan_cache_warming(MoveParams& p) {
    p.warm_lds_offset = 0;
    if (!p.fused || p.warm_rounds < 0) return;
    const unsigned first_round = unsigned(p.num_cus) * unsigned(kResidentWorkgroupsPerCu);
    // By default two rounds ahead; launches of one and a half to two rounds warm their second round (3072 x 7168 fused
    // cast: 38.2 -> 36.1 us, 3400 tokens 43.8 -> 40.6 us), shorter ones nothing (2048 tokens: 27.9 -> 28.6 us).
    unsigned rounds = p.warm_rounds > 0 ? unsigned(p.warm_rounds) : 2u;
    if (p.warm_rounds == 0 && uint64_t(p.num_movers) <= 2ull * first_round) {
        if (2ull * p.num_movers <= 3ull * first_round) return;
        rounds = 1u;
    }
    if (uint64_t(p.num_movers) <= uint64_t(rounds) * first_round) return;
    p.warm_lds_offset = unsigned((move_lds_bytes(p) + 1023) & ~size_t(1023));
    p.warm_ahead = rounds * first_round * unsigned(kWavesPerBlock);
}

template <int kVecs>
hipError_t launch_copy(MoveParams p, hipStream_t stream) {
    p.tiles = (p.row_bytes + kVecs * 1024 - 1) / (kVecs * 1024);
    const unsigned blocks = move_grid(p, int64_t(p.T) * p.tiles);
    plan_cache_warming(p);
    if (p.fused) hipLaunchKernelGGL((dispatch_copy_single_launch_kernel<kVecs>), dim3(blocks), dim3(kThreads), move_lds_bytes(p), stream, p);
    else hipLaunchKernelGGL((dispatch_copy_kernel<kVecs>), dim3(blocks), dim3(kThreads), move_lds_bytes(p), stream, p);
    return hipGetLastError();
}

template <int kPairs>
hipError_t launch_cast(MoveParams p, hipStream_t stream) {
    p.tiles = (p.H + kPairs * 1024 - 1) / (kPairs * 1024);
    const unsigned blocks = move_grid(p, int64_t(p.T) * p.tiles);
    plan_cache_warming(p);
    if constexpr (kPairs <= 2) {
        if (p.fused) {
            hipLaunchKernelGGL((dispatch_cast_single_launch_kernel<kPairs>), dim3(blocks), dim3(kThreads), move_lds_bytes(p), stream, p);
            return hipGetLastError();
        }
    }
    if (p.fused) return hipErrorInvalidConfiguration;      // the launch plan keeps wider tiles out of the single launch
    if constexpr (kPairs <= 2) {
        if (p.persistent_movers > 0 && !p.cached && !p.do_expand && p.route_mask == nullptr && p.R <= kWaveSize &&
            p.send_head == nullptr && p.H >= 16 && p.gates != nullptr && p.gates_finished != nullptr) {
            const int64_t items = int64_t(p.T) * p.tiles;
            const int64_t wanted = (items + kQueueSlot * kQueueStatic - 1) / (kQueueSlot * kQueueStatic);
            const unsigned grid = unsigned(std::min<int64_t>(wanted, compute_units()));
            if (p.persistent_movers <= 4) hipLaunchKernelGGL((dispatch_cast_queue_kernel<kPairs, 320>), dim3(grid), dim3(320), 0, stream, p);
            else if (p.persistent_movers <= 8) hipLaunchKernelGGL((dispatch_cast_queue_kernel<kPairs, 576>), dim3(grid), dim3(576), 0, stream, p);
            else hipLaunchKernelGGL((dispatch_cast_queue_kernel<kPairs, 1024>), dim3(grid), dim3(1024), 0, stream, p);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((dispatch_cast_kernel<kPairs>), dim3(blocks), dim3(kThreads), move_lds_bytes(p), stream, p);
    return hipGetLastError();
}

}  // namespace

int compute_units() {
    static std::atomic<int> cached[64];
    return device_attribute(hipDeviceAttributeMultiprocessorCount, cached, 256);
}

// Column tile of a move launch: 1024-channel segments per wavefront for the fused cast, KB of row per wavefront for
// the pass-through payloads.
static int move_tile(const MoveParams& p) {
    if (p.payload == DEEP_EP_HIP_PAYLOAD_CAST_FP8) {
        // Two segments (2048 channels, 8 wavefronts per SIMD) measured best at hidden 7168: 92.8 us per dispatch
        // against 93.7 (4 segments) and 96.9 (7 segments, one wavefront per token).
        // The expanded layout stores eight rows per token instead of five: in a large call (64 MB of input and more)
        // one segment per wavefront is ahead there (8192 x 7168: move phase 119 us against 122 us, whole call 130
        // against 131 us).
        if (p.cast_pairs != 0) return p.cast_pairs;
        const bool large = int64_t(p.T) * p.row_bytes >= (int64_t(64) << 20);
        return (p.H <= 1024 || (p.do_expand && large)) ? 1 : 2;
    }
    // Large, bandwidth-bound calls: one 1 KB segment per wavefront measured best for this write-heavy stream (8192
    // BF16 rows of 14 KB: 143 us per dispatch against 155-159 us with 2, 4, 7 or 8 segments).  Small, latency-bound
    // calls: up to 4 KB per wavefront, so that fewer wavefronts repeat the routing work (4096 rows of 4 KB: 26 us
    // against 32 us with 1 KB segments).
    if (p.copy_vecs != 0) return p.copy_vecs;
    const int kb = (p.row_bytes + 1023) / 1024;
    const bool large = int64_t(p.T) * p.row_bytes >= (int64_t(64) << 20);
    return large ? 1 : (kb <= 1 ? 1 : kb <= 2 ? 2 : 4);
}

int64_t dispatch_move_workgroups(const MoveParams& p) {
    const int tile = move_tile(p);
    const int64_t tiles = p.payload == DEEP_EP_HIP_PAYLOAD_CAST_FP8 ? (p.H + tile * 1024 - 1) / (tile * 1024)
                                                                    : (p.row_bytes + tile * 1024 - 1) / (tile * 1024);
    return (int64_t(p.T) * tiles + kWavesPerBlock - 1) / kWavesPerBlock;
}

hipError_t launch_dispatch_move(MoveParams p, hipStream_t stream) {
    if (p.T == 0) return hipSuccess;
    p.rcp_E_l = 1.0f / float(p.E_l);
    p.num_cus = p.fused ? compute_units() : 0;
    const int tile = move_tile(p);
    if (p.payload == DEEP_EP_HIP_PAYLOAD_CAST_FP8) {
        switch (tile) {
            case 1: return launch_cast<1>(p, stream);
            case 2: return launch_cast<2>(p, stream);
            case 7: return launch_cast<7>(p, stream);
            case 8: return launch_cast<8>(p, stream);
            default: return launch_cast<4>(p, stream);
        }
    }
    switch (tile) {
        case 1: return launch_copy<1>(p, stream);
        case 2: return launch_copy<2>(p, stream);
        case 4: return launch_copy<4>(p, stream);
        case 7: return launch_copy<7>(p, stream);
        default: return launch_copy<8>(p, stream);
    }
}

hipError_t launch_zero_padding(const PadParams& p, hipStream_t stream) {
    if (p.A <= 1 || p.E == 0) return hipSuccess;
    const int64_t waves = int64_t(p.E) * (p.A - 1);
    const unsigned blocks = unsigned((waves + kWavesPerBlock - 1) / kWavesPerBlock);
    hipLaunchKernelGGL(zero_padding_kernel, dim3(blocks), dim3(kThreads), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_intranode_prefix(const IntranodePrefixParams& p, hipStream_t stream) {
    if (p.R == 0 || p.C == 0) return hipSuccess;
    hipLaunchKernelGGL(intranode_prefix_kernel, dim3(p.R), dim3(kThreads), size_t(p.C) * sizeof(int), stream, p);
    return hipGetLastError();
}

hipError_t launch_fill_tail(const FillTailParams& p, hipStream_t stream) {
    if (p.capacity == 0 || p.K == 0) return hipSuccess;
    const int64_t elems = p.capacity * p.K;
    const unsigned blocks = unsigned(elems / kThreads < 1 ? 1 : (elems / kThreads > 1024 ? 1024 : elems / kThreads));
    hipLaunchKernelGGL(fill_tail_kernel, dim3(blocks), dim3(kThreads), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_cast_kernel(const CastParams& p, hipStream_t stream) {
    if (p.T == 0) return hipSuccess;
    const int tiles = (p.H + 1023) / 1024;
    const int64_t waves = int64_t(p.T) * tiles;
    const unsigned blocks = unsigned((waves + kWavesPerBlock - 1) / kWavesPerBlock);
    hipLaunchKernelGGL(cast_kernel, dim3(blocks), dim3(kThreads), 0, stream, p);
    return hipGetLastError();
}

}  // namespace deep_ep_hip

#ifdef DEEP_EP_HIP_WAVE_STAMPS
// Copies the stamps of the first `waves` mover wavefronts of the last fused-cast launch to `out` (3 * waves values).
extern "C" int deep_ep_hip_debug_wave_stamps(long long* out, int waves) {
    if (out == nullptr || waves < 0 || waves > deep_ep_hip::kMaxStampedWaves) return 1;
    return int(hipMemcpyFromSymbol(out, HIP_SYMBOL(deep_ep_hip::wave_stamps), size_t(waves) * 3 * sizeof(long long)));
}
#endif
