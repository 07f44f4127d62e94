// Low-latency packed per-expert layout for gfx950: dispatch into [local expert][slot][hidden]
// buffers with counts, source info and per-source ranges, and the weighted combine back.
//
// Replaces csrc/kernels/legacy/internode_ll.cu:128-462 (dispatch: FP8 cast in the send phase,
// per-(expert, source) packing in the receive phase) and :714-1138 (combine: BF16 branch,
// weighted fp32 reduce :1072-1135).  Tensor contracts follow csrc/legacy/buffer.hpp:1515-1541.
// With every logical source resident in local HBM the send/receive phases and the RDMA staging
// buffers disappear; slots come from a scan, so the fill order is deterministic: source rank
// ascending, then token ascending (the reference fills in arrival order).
#include <algorithm>

#include "device_utils.h"
#include "fp8_cast.h"
#include "kernels.h"
#include "../../include/deep_ep_hip.h"

namespace deep_ep_hip {

namespace {

constexpr int kThreads = kLayoutChunk;
constexpr int kWaves = kThreads / kWaveSize;

__device__ __forceinline__ int tokens_of_source(const LLDispatchParams& p, int s) {
    const int n = p.num_tokens_per_src != nullptr ? p.num_tokens_per_src[s] : p.src_token_stride;
    return min(max(n, 0), p.src_token_stride);
}

// One workgroup per (source rank, chunk of 256 tokens).
template <int KMAX>
__global__ __launch_bounds__(kThreads) void ll_count_kernel(const LLDispatchParams p) {
    extern __shared__ uint64_t bitmap[];   // [E_l][kWaves]
    __shared__ int is_last;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int chunks_per_src = (p.src_token_stride + kThreads - 1) / kThreads;
    const int s = blockIdx.x / chunks_per_src;
    const int c = blockIdx.x - s * chunks_per_src;
    const int t = c * kThreads + tid;
    const bool active = t < tokens_of_source(p, s);
    const int64_t g = int64_t(s) * p.src_token_stride + t;

    for (int i = tid; i < p.E_l * kWaves; i += kThreads) bitmap[i] = 0ull;
    __syncthreads();

    int64_t raw[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) raw[k] = (active && k < p.K) ? p.topk_idx[g * p.K + k] : int64_t(-1);

    int le[KMAX];
    int flags = 0;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        le[k] = -1;
        if (raw[k] >= p.E) flags |= DEEP_EP_HIP_STATUS_EXPERT_OUT_OF_RANGE;
        else if (raw[k] >= p.expert_begin && raw[k] < p.expert_begin + p.E_l) le[k] = int(raw[k]) - p.expert_begin;
        if (le[k] >= 0)
            atomicOr(reinterpret_cast<unsigned long long*>(&bitmap[le[k] * kWaves + wave]), 1ull << lane);
    }
    __syncthreads();

    if (active) {
        const uint64_t below = lanes_below(lane);
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
            if (k >= p.K) break;
            int pos = -1;
            if (le[k] >= 0) {
#pragma unroll
                for (int j = 0; j < KMAX; ++j)
                    if (j != k && le[j] == le[k]) flags |= DEEP_EP_HIP_STATUS_DUPLICATE_EXPERT;
                pos = __popcll(bitmap[le[k] * kWaves + wave] & below);
                for (int w = 0; w < wave; ++w) pos += __popcll(bitmap[le[k] * kWaves + w]);
            }
            p.pos_expert[g * p.K + k] = pos;
        }
    }
    if (flags != 0) atomicOr(p.status, flags);

    for (int j = tid; j < p.E_l; j += kThreads) {
        int cnt = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) cnt += __popcll(bitmap[j * kWaves + w]);
        p.chunk_counts[int64_t(blockIdx.x) * p.E_l + j] = cnt;
    }

    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const unsigned ticket = atomicAdd(p.done_counter, 1u);
        is_last = (ticket == gridDim.x - 1) ? 1 : 0;
    }
    __syncthreads();
    if (!is_last) return;
    __threadfence();

    // Exclusive prefix over (source rank, chunk) per local expert.  Loads go in batches of 16 that are
    // all issued before the batch's stores, so a decode-sized call needs a single memory round trip.
    const int num_blocks = p.S * chunks_per_src;
    for (int j = tid; j < p.E_l; j += kThreads) {
        int running = 0, begin = 0;
        for (int b0 = 0; b0 < num_blocks; b0 += 16) {
            int v[16];
#pragma unroll
            for (int i = 0; i < 16; ++i)
                v[i] = (b0 + i < num_blocks) ? p.chunk_counts[int64_t(b0 + i) * p.E_l + j] : 0;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int b = b0 + i;
                if (b < num_blocks) {
                    if (b % chunks_per_src == 0) begin = running;
                    p.chunk_base[int64_t(b) * p.E_l + j] = running;
                    running += v[i];
                    if (b % chunks_per_src == chunks_per_src - 1)
                        p.packed_layout_range[int64_t(j) * p.R + p.src_rank_begin + b / chunks_per_src] =
                            (int64_t(begin) << 32) | int64_t(running - begin);
                }
            }
        }
        p.packed_count[j] = running;
        if (p.cumulative_stats != nullptr) p.cumulative_stats[j] += running;
        // source ranks that do not send in this call: (begin 0, count 0)
        for (int r = 0; r < p.R; ++r)
            if (r < p.src_rank_begin || r >= p.src_rank_begin + p.S) p.packed_layout_range[int64_t(j) * p.R + r] = 0;
    }
    if (tid == 0) *p.done_counter = 0u;
}

constexpr int kMoveThreads = 256;
constexpr int kMoveWaves = kMoveThreads / kWaveSize;

// Loads one column tile (kPairs * 1024 channels) of token g: lane owns 16 consecutive channels per pair.  kClamped:
// a pair past the end of the row loads the row's last 32 bytes instead of being skipped (no branch around the load;
// what it brings is never stored).
template <int kPairs, bool kClamped = false>
__device__ __forceinline__ void ll_load_tile(const uint8_t* x, int hidden, int64_t g, int tile, int lane,
                                             vec16 (&in)[kPairs][2]) {
    const uint8_t* src = x + g * (int64_t(hidden) * 2);
#pragma unroll
    for (int q = 0; q < kPairs; ++q) {
        const int elem = (tile * kPairs + q) * 1024 + lane * 16;
        if constexpr (kClamped) {
            const int at = min(elem, hidden - 16);
            in[q][0] = load16_stream(src + int64_t(at) * 2);
            in[q][1] = load16_stream(src + int64_t(at) * 2 + 16);
        } else {
            in[q][0] = vec16{0, 0, 0, 0};
            in[q][1] = vec16{0, 0, 0, 0};
            if (elem < hidden) {
                in[q][0] = load16_stream(src + int64_t(elem) * 2);
                in[q][1] = load16_stream(src + int64_t(elem) * 2 + 16);
            }
        }
    }
}

// Casts (FP8) and stores the tile to every (local expert, slot) named by lanes [0, K); t = token id within its source.
template <int kPairs, bool kFp8>
__device__ __forceinline__ void ll_store_tile(const LLDispatchParams& p, int64_t g, int tile, int lane, int t, int le, int slot,
                                              const vec16 (&in)[kPairs][2]) {
    const int rows_per_expert = p.R * p.M;
    const int row_bytes = p.H * 2;
    if (slot >= rows_per_expert) {
        atomicOr(p.status, DEEP_EP_HIP_STATUS_ROW_OVERFLOW);
        slot = -1;
    }
    if (tile == 0 && slot >= 0) p.packed_src_info[int64_t(le) * rows_per_expert + slot] = t;
    // optional shortcut for combine: the packed row of every (token, lane)
    if (tile == 0 && p.lane_slot != nullptr && lane < p.K) p.lane_slot[g * p.K + lane] = slot >= 0 ? le * rows_per_expert + slot : -1;

    uint64_t dests = __ballot(slot >= 0);
    if (dests == 0ull) return;              // nothing of this token stays on this rank: no cast either

    vec16 out[kPairs];
    float my_scale = 0.f;
    if constexpr (kFp8) {
#pragma unroll
        for (int q = 0; q < kPairs; ++q) {
            const float scale_inv = p.round_scale ? cast_16_channels<ScaleRule::kPow2>(in[q][0], in[q][1], out[q])
                                                  : cast_16_channels<ScaleRule::kReciprocal>(in[q][0], in[q][1], out[q]);
            const float gathered = __shfl(scale_inv, (lane & 7) * 8, kWaveSize);
            if ((lane >> 3) == q) my_scale = gathered;
        }
    }
    const int group = tile * kPairs * 8 + lane;
    const int num_groups = p.H / 128;
    const bool owns_scale = kFp8 && lane < kPairs * 8 && group < num_groups;

    while (dests) {
        const int j = __builtin_ctzll(dests);
        dests &= dests - 1;
        const int dle = read_lane(le, j);
        const int dslot = read_lane(slot, j);
        const int64_t row = int64_t(dle) * rows_per_expert + dslot;
        if constexpr (kFp8) {
            uint8_t* dst = p.packed_x + row * p.H;
#pragma unroll
            for (int q = 0; q < kPairs; ++q) {
                const int elem = (tile * kPairs + q) * 1024 + lane * 16;
                if (elem < p.H) store16_stream(dst + elem, out[q]);
            }
            if (owns_scale) {
                if (p.use_ue8m0) {
                    // exponent bytes, four groups to an int32 pack; packs column-major like the fp32 scales
                    // (csrc/kernels/legacy/internode_ll.cu:440-457)
                    uint8_t* bytes = reinterpret_cast<uint8_t*>(p.packed_scales);
                    const int64_t pack = (int64_t(dle) * (num_groups / 4) + (group >> 2)) * rows_per_expert + dslot;
                    bytes[pack * 4 + (group & 3)] = uint8_t(__float_as_uint(my_scale) >> 23);
                } else {
                    p.packed_scales[(int64_t(dle) * num_groups + group) * rows_per_expert + dslot] = my_scale;
                }
            }
        } else {
            uint8_t* dst = p.packed_x + row * row_bytes;
#pragma unroll
            for (int q = 0; q < kPairs; ++q) {
                const int elem = (tile * kPairs + q) * 1024 + lane * 16;
                if (elem < p.H) {
                    store16_stream(dst + int64_t(elem) * 2, in[q][0]);
                    store16_stream(dst + int64_t(elem) * 2 + 16, in[q][1]);
                }
            }
        }
    }
}

// Two-kernel path, second kernel: one wavefront per (token, column tile); slots come from the count kernel.
template <int kPairs, bool kFp8>
__global__ __launch_bounds__(kMoveThreads) void ll_move_kernel(const LLDispatchParams p, const int tiles) {
    const int lane = threadIdx.x & 63;
    const unsigned work = wave_work_index(blockIdx.x, kMoveWaves);
    const unsigned total_tokens = unsigned(p.S) * unsigned(p.src_token_stride);
    if (work >= total_tokens * unsigned(tiles)) return;
    const unsigned gu = work / unsigned(tiles);
    const int64_t g = gu;
    const int tile = int(work - gu * unsigned(tiles));
    const int s = int(gu / unsigned(p.src_token_stride));
    const int t = int(gu - unsigned(s) * unsigned(p.src_token_stride));
    if (t >= tokens_of_source(p, s)) return;

    vec16 in[kPairs][2];
    ll_load_tile<kPairs>(p.x, p.H, g, tile, lane, in);

    const int chunks_per_src = (p.src_token_stride + kLayoutChunk - 1) / kLayoutChunk;
    const int64_t chunk = int64_t(s) * chunks_per_src + t / kLayoutChunk;
    int le = -1, slot = -1;
    if (lane < p.K) {
        const int64_t raw = p.topk_idx[g * p.K + lane];
        if (raw >= p.expert_begin && raw < p.expert_begin + p.E_l && raw < p.E) {
            le = int(raw) - p.expert_begin;
            slot = p.chunk_base[chunk * p.E_l + le] + p.pos_expert[g * p.K + lane];
        }
    }
    ll_store_tile<kPairs, kFp8>(p, g, tile, lane, t, le, slot, in);
}

// Single-kernel path for decode-sized calls.  Every workgroup first rebuilds the complete routing picture in
// LDS - one bit per (local expert, token), set from its own pass over all topk_idx rows (tens of KB, L2
// resident) - so slots are prefix popcounts and no workgroup waits for another: no second launch, no ticket,
// no global scan.  Workgroup 0 only publishes counts and per-source ranges; the wavefronts of the other
// workgroups move (token, column tile) items: one each at decode sizes, several when the call has more items than
// one workgroup per compute unit can take (kSeveralItems).
//
// The kernel is bound by the chain of dependent phases of one wavefront, not by memory bandwidth: the routing pass alone
// costs every workgroup a dozen instructions per index entry.  So the index loads are the first thing on the memory
// pipeline (the pass can start as soon as they are back), the payload loads queue up behind them and land while the pass
// runs, and the pass itself is kept short: one token id per pair of entries, unpredicated 32-bit LDS atomics, range and
// duplicate checks left to the wavefront that later moves the token.
template <int kPairs, bool kFp8, int kFusedThreads, bool kSeveralItems>
__global__ __launch_bounds__(kFusedThreads) void ll_fused_kernel(const LLDispatchParams p, const int tiles) {
    constexpr int kFusedWaves = kFusedThreads / kWaveSize;
    extern __shared__ uint64_t bits[];          // [E_l][words], bit g of row le: token g selects local expert le
    // Every argument the first loads depend on is asked for in one go, up front: the wavefront starts with one trip to
    // memory for its arguments, not with one per group of them as they come into use.
    asm volatile("" ::"s"(p.topk_idx), "s"(p.x), "s"(p.num_tokens_per_src), "s"(p.S), "s"(p.src_token_stride), "s"(p.K), "s"(p.H),
                 "s"(p.E_l), "s"(tiles));
    const int tid = threadIdx.x, lane = tid & 63;
    const int total_tokens = p.S * p.src_token_stride;
    const int words = (total_tokens + 63) / 64;

    // This wavefront's first work item; a call with more items than the grid has wavefronts gives every wavefront
    // several, `item_stride` apart (the grid is held to one workgroup per compute unit, so that the routing pass below
    // is paid once per compute unit however many tokens there are).
    const unsigned num_items = unsigned(total_tokens) * unsigned(tiles);
    const unsigned item_stride = (gridDim.x - 1) * unsigned(kFusedWaves);
    unsigned work = blockIdx.x == 0 ? ~0u : wave_work_index(blockIdx.x - 1, kFusedWaves);
    bool has_work = work < num_items;
    unsigned gu = has_work ? work / unsigned(tiles) : 0u;
    int64_t g = gu;
    int tile = has_work ? int(work - gu * unsigned(tiles)) : 0;
    // token id within its source, and whether the source has that many tokens: worked out here, in the shadow of the
    // loads, not behind the routing pass
    auto place_of = [&](unsigned token, int& t_out) {
        const int src = int(token / unsigned(p.src_token_stride));
        t_out = int(token - unsigned(src) * unsigned(p.src_token_stride));
        return t_out < tokens_of_source(p, src);
    };
    int t = 0;
    bool live = place_of(gu, t) && has_work;

    // Pass over the whole index table: 16-byte loads (two entries), fully coalesced, a batch of a thread's loads in
    // flight at once.  The first batch - for decode sizes the only one - goes out here, ahead of everything else.
    // Everything up to the pass is straight-line code without a branch around any load: where control flow merges the
    // compiler can no longer tell how many loads are younger than the one it waits for and waits for all of them - the
    // pass would sit there until the payload had arrived.  So addresses are clamped instead of predicated (the launcher
    // sends only calls with an aligned table of at least two entries here), and wavefronts without a work item load
    // the tile of token 0 and drop it.
    const int total_entries = total_tokens * p.K;
    const int pairs_total = total_entries / 2;
    const vec16* idx2 = reinterpret_cast<const vec16*>(p.topk_idx);
    constexpr int kBatch = 8;
    for (int i = tid; i < p.E_l * words; i += kFusedThreads) bits[i] = 0ull;
    __syncthreads();            // here, where no wavefront is held up by the memory pipeline yet: they arrive together
    vec16 v[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) v[u] = idx2[min(tid + u * kFusedThreads, pairs_total - 1)];
    // this token's own selections: behind the routing pass they would be one more trip to the L2 on the critical path
    int64_t own_loaded = p.topk_idx[g * p.K + min(lane, p.K - 1)];
    // the payload tile: queued behind the index loads, in flight while the routing pass runs
    vec16 in[kPairs][2];
    ll_load_tile<kPairs, true>(p.x, p.H, g, tile, lane, in);
    __builtin_amdgcn_sched_barrier(0);

    // An entry sets a bit iff it names a local expert: a negative or oversized id has a non-zero upper half or a lower
    // half beyond every local id.  The atomic is not predicated: a lane without a hit ORs into a word of its own
    // behind the table, which is cheaper than branching around a handful of instructions sixteen times.  Tokens past
    // the end of a ragged source are masked out of the table afterwards.
    const uint32_t row_bytes32 = uint32_t(words) * 8u;
    const uint32_t spare = uint32_t(p.E_l) * row_bytes32 + uint32_t(lane) * 4u;     // byte offset of the lane's spare word
    auto note = [&](uint32_t word_off, uint32_t bit, uint32_t lo, uint32_t hi) {
        const uint32_t le = lo - uint32_t(p.expert_begin);
        const bool hit = le < uint32_t(p.E_l) && hi == 0u;
        const uint32_t off = hit ? __umul24(le, row_bytes32) + word_off : spare;
        atomicOr(reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(bits) + off), bit);
    };
    const float rcp_k = 1.0f / float(p.K);
    const bool even_k = (p.K & 1) == 0;
    const float rcp_half_k = 2.0f / float(p.K);
    for (int q0 = tid; q0 < pairs_total; q0 += kFusedThreads * kBatch) {
        if (q0 != tid) {
#pragma unroll
            for (int u = 0; u < kBatch; ++u) v[u] = idx2[min(q0 + u * kFusedThreads, pairs_total - 1)];
        }
        if (even_k) {
            // both entries of a pair belong to one token
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const int q = q0 + u * kFusedThreads;
                const int tok = small_div(q, rcp_half_k);
                const uint32_t word_off = (uint32_t(tok) >> 3) & ~3u;
                const uint32_t bit = q < pairs_total ? 1u << (tok & 31) : 0u;     // pairs past the end set nothing
                note(word_off, bit, v[u].x, v[u].y);
                note(word_off, bit, v[u].z, v[u].w);
            }
        } else {
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const int q = q0 + u * kFusedThreads;
                const int tok0 = small_div(2 * q, rcp_k), tok1 = small_div(2 * q + 1, rcp_k);
                const uint32_t live_pair = q < pairs_total ? 1u : 0u;
                note((uint32_t(tok0) >> 3) & ~3u, live_pair << (tok0 & 31), v[u].x, v[u].y);
                note((uint32_t(tok1) >> 3) & ~3u, live_pair << (tok1 & 31), v[u].z, v[u].w);
            }
        }
    }
    for (int f = 2 * pairs_total + tid; f < total_entries; f += kFusedThreads) {
        const uint64_t raw = uint64_t(p.topk_idx[f]);
        const int tok = small_div(f, rcp_k);
        note((uint32_t(tok) >> 3) & ~3u, 1u << (tok & 31), uint32_t(raw), uint32_t(raw >> 32));
    }
    if (p.num_tokens_per_src != nullptr) {
        // ragged sources: clear the bits of the tokens a source does not have
        __syncthreads();
        for (int i = tid; i < p.E_l * words; i += kFusedThreads) {
            const int first = (i % words) * 64, last = min(first + 64, total_tokens);
            uint64_t keep = 0ull;
            for (int ss = first / p.src_token_stride; ss * p.src_token_stride < last; ++ss) {
                const int from = max(ss * p.src_token_stride, first) - first;
                const int to = min(ss * p.src_token_stride + tokens_of_source(p, ss), last) - first;      // bits [from, to)
                if (to > from) keep |= (to == 64 ? ~0ull : (1ull << to) - 1ull) & ~((1ull << from) - 1ull);
            }
            bits[i] &= keep;
        }
    }
    __syncthreads();

    if (blockIdx.x == 0) {
        // counts and per-source ranges: one walk over each expert's words, cut at the source boundaries
        for (int le = tid; le < p.E_l; le += kFusedThreads) {
            const uint64_t* row = bits + le * words;
            int running = 0, pos = 0;
            for (int ss = 0; ss < p.S; ++ss) {
                const int begin = running, end_pos = (ss + 1) * p.src_token_stride;
                while (pos < end_pos) {
                    const int word = pos >> 6, lo = pos & 63;
                    const int take = min(64 - lo, end_pos - pos);
                    uint64_t wv = row[word] >> lo;
                    if (take < 64) wv &= (1ull << take) - 1ull;
                    running += __popcll(wv);
                    pos += take;
                }
                p.packed_layout_range[int64_t(le) * p.R + p.src_rank_begin + ss] =
                    (int64_t(begin) << 32) | int64_t(running - begin);
            }
            p.packed_count[le] = running;
            if (p.cumulative_stats != nullptr) p.cumulative_stats[le] += running;
            // source ranks that do not send in this call: (begin 0, count 0)
            for (int r = 0; r < p.R; ++r)
                if (r < p.src_rank_begin || r >= p.src_rank_begin + p.S) p.packed_layout_range[int64_t(le) * p.R + r] = 0;
        }
        return;
    }
    const int own_lane = min(lane, p.K - 1);
    while (has_work) {
        // Where this item's rows go: needs the routing table and the token's own selections, not the payload, which
        // may still be on its way.
        int le = -1, slot = -1, flags = 0;
        if (live && lane < p.K) {
            const uint32_t lo = uint32_t(own_loaded), hi = uint32_t(uint64_t(own_loaded) >> 32);
            if (int32_t(hi) > 0 || (hi == 0u && lo >= uint32_t(p.E))) flags |= DEEP_EP_HIP_STATUS_EXPERT_OUT_OF_RANGE;
            if (hi == 0u && lo - uint32_t(p.expert_begin) < uint32_t(p.E_l)) le = int(lo) - p.expert_begin;
        }
        // Slot of a selection = rows of its expert that come from tokens [0, g): a prefix popcount over the expert's
        // words, taken by the whole wavefront for one selection at a time (lane i looks at word i; at most 64 words,
        // summed in rows of 16 lanes).
        const int own_word = int(g) >> 6;
        const uint64_t own_below = lanes_below(int(g) & 63);
        uint64_t pending = __ballot(le >= 0);
        while (pending) {
            const int j = __builtin_ctzll(pending);
            pending &= pending - 1;
            const int expert = read_lane(le, j);
            const uint64_t* row = bits + expert * words;
            uint64_t wv = lane <= own_word ? row[lane] : 0ull;
            if (lane == own_word) wv &= own_below;
            const int sums = row16_sum(__popcll(wv));
            const int before = read_lane(sums, 0) + read_lane(sums, 16) + read_lane(sums, 32) + read_lane(sums, 48);
            if (lane == j) slot = before;
            if (__popcll(__ballot(le == expert)) > 1) flags |= DEEP_EP_HIP_STATUS_DUPLICATE_EXPERT;
        }
        if (tile == 0 && __ballot(flags != 0) != 0ull) {
            if (flags != 0) atomicOr(p.status, flags);
        }

        // This item's tile has to be in its registers before the next one is requested: the request below sits in a
        // branch, and behind a branch the compiler waits for every outstanding load at once - this item would wait for
        // the next item's tile.
        if constexpr (kSeveralItems) {
#pragma unroll
            for (int q = 0; q < kPairs; ++q)
                asm volatile("" : "+v"(in[q][0].x), "+v"(in[q][0].y), "+v"(in[q][0].z), "+v"(in[q][0].w),
                                  "+v"(in[q][1].x), "+v"(in[q][1].y), "+v"(in[q][1].z), "+v"(in[q][1].w));
        }
        // the next item's tile and selections are requested before this item is converted and stored
        const unsigned next_work = work + item_stride;
        const bool has_next = kSeveralItems && next_work < num_items;      // decode sizes: one item per wavefront, no loop
        const unsigned next_gu = has_next ? next_work / unsigned(tiles) : 0u;
        const int next_tile = has_next ? int(next_work - next_gu * unsigned(tiles)) : 0;
        vec16 next_in[kPairs][2];
        int64_t next_own = -1;
        int next_t = 0;
        bool next_live = false;
        if (has_next) {
            next_own = p.topk_idx[int64_t(next_gu) * p.K + own_lane];
            ll_load_tile<kPairs, true>(p.x, p.H, int64_t(next_gu), next_tile, lane, next_in);
            next_live = place_of(next_gu, next_t);
        }

        if (live) ll_store_tile<kPairs, kFp8>(p, g, tile, lane, t, le, slot, in);

        has_work = has_next;
        work = next_work;
        gu = next_gu;
        g = next_gu;
        tile = next_tile;
        own_loaded = next_own;
        t = next_t;
        live = next_live;
#pragma unroll
        for (int q = 0; q < kPairs; ++q) {
            in[q][0] = next_in[q][0];
            in[q][1] = next_in[q][1];
        }
    }
}

// ---- LogFMT-10, the codec the reference puts the rows of a low-latency combine through on the wire
// (csrc/kernels/legacy/internode_ll.cu:556-637 encode, :640-712 and :1048-1100 decode).  On one GPU nothing travels,
// so the row is encoded and decoded in registers: what is accumulated is what the receiver would have decoded.
//
// Per group of 128 channels: amax and amin of |x|; log_amin = max(log2(amin), log_amax - 32).  A chunk of rows
// (1024 channels, or 512 when hidden is not a multiple of 1024: what one warp of the reference's send loop stages)
// is cast iff every one of its groups has log_amax < 0 and log_amin < log_amax.  A cast value becomes a sign and a
// 9-bit code on a logarithmic grid with step = (log_amax - log_amin) / 510:
//   code = floor(max(log2|x| / step + rounding - log_amin / step, 0)),  rounding = 2 - log2((1 + 2^step) / 2) / step
//   decoded = code == 0 ? 0 : 2^((code - 1) * step + log_amin)
// log2 / exp2 are the hardware's (v_log_f32 / v_exp_f32), as the reference uses its hardware's approximations.

// One 16-byte vector (8 BF16 channels per lane, 64 lanes = 512 channels = 4 groups of 16 lanes) of a row.
struct LogFmtGroup {
    float log_amax, log_amin;
    bool castable;
};

__device__ __forceinline__ LogFmtGroup logfmt_group_of(const float (&mag)[8]) {
    float amax = 0.f, amin = __builtin_inff();
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        amax = fmaxf(amax, mag[c]);
        amin = fminf(amin, mag[c]);
    }
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {        // the 16 lanes of a 128-channel group
        amax = fmaxf(amax, __shfl_xor(amax, off, kWaveSize));
        amin = fminf(amin, __shfl_xor(amin, off, kWaveSize));
    }
    LogFmtGroup g;
    g.log_amax = __builtin_amdgcn_logf(amax);
    g.log_amin = amin == 0.f ? g.log_amax - 32.f : fmaxf(__builtin_amdgcn_logf(amin), g.log_amax - 32.f);
    g.castable = g.log_amax < 0.f && g.log_amin < g.log_amax;
    return g;
}

__device__ __forceinline__ void logfmt_round_trip(float (&val)[8], const float (&mag)[8], const LogFmtGroup& g) {
    const float step = (g.log_amax - g.log_amin) / 510.f;
    const float step_inv = 1.0f / step;
    const float rounding = 2.0f - __builtin_amdgcn_logf((1.0f + __builtin_amdgcn_exp2f(step)) * 0.5f) * step_inv;
    const float fused_rounding = rounding - g.log_amin * step_inv;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const uint32_t code = uint32_t(fmaxf(__builtin_amdgcn_logf(mag[c]) * step_inv + fused_rounding, 0.f));     // round down
        const float decoded = code == 0u ? 0.f : __builtin_amdgcn_exp2f(float(code - 1u) * step + g.log_amin);
        val[c] = val[c] < 0.f ? -decoded : decoded;       // a negative zero has magnitude 0: code 0 either way
    }
}

// Weighted reduce: one wavefront per (token, column tile of kVecs * 512 channels).  kLogFmt: the tile is one chunk
// of the codec (kVecs = 2 for hidden % 1024 == 0, else 1).
template <int kVecs, bool kLogFmt = false, int kBlockThreads = kMoveThreads>
__global__ __launch_bounds__(kBlockThreads) void ll_combine_kernel(const LLCombineParams p, const int tiles) {
    // all arguments the first loads depend on in one trip to memory (see ll_fused_kernel)
    asm volatile("" ::"s"(p.topk_idx), "s"(p.topk_weights), "s"(p.lane_slot), "s"(p.x), "s"(p.out), "s"(p.num_tokens_per_src),
                 "s"(p.S), "s"(p.src_token_stride), "s"(p.K), "s"(p.H), "s"(p.E_l), "s"(p.expert_begin), "s"(p.R), "s"(p.M), "s"(tiles));
    const int lane = threadIdx.x & 63;
    const unsigned work = wave_work_index(blockIdx.x, kBlockThreads / kWaveSize);
    if (work >= unsigned(p.S) * unsigned(p.src_token_stride) * unsigned(tiles)) return;
    const unsigned gu = work / unsigned(tiles);
    const int64_t g = gu;
    const int tile = int(work - gu * unsigned(tiles));
    const int s = int(gu / unsigned(p.src_token_stride));
    const int t = int(gu - unsigned(s) * unsigned(p.src_token_stride));
    const int n_s = p.num_tokens_per_src != nullptr ? min(max(p.num_tokens_per_src[s], 0), p.src_token_stride)
                                                    : p.src_token_stride;
    if (t >= n_s) return;
    const int src_rank = p.src_rank_begin + s;
    const int rows_per_expert = p.R * p.M;
    const int row_bytes = p.H * 2;

    // Every lane loads (lanes past the top-k repeat the last selection): no branch around the three loads, which go
    // out together.
    const int64_t entry = g * p.K + min(lane, p.K - 1);
    const int64_t raw = p.topk_idx[entry];
    const int recorded = p.lane_slot != nullptr ? p.lane_slot[entry] : -1;
    const float w = p.topk_weights[entry];
    int le = -1;
    if (lane < p.K && raw >= p.expert_begin && raw < p.expert_begin + p.E_l && raw < p.E) le = int(raw) - p.expert_begin;

    int row_of_lane = -1;
    if (p.lane_slot != nullptr) {
        // the dispatch that produced the handle also recorded the packed row of every (token, lane)
        if (le >= 0 && recorded >= le * rows_per_expert && recorded < (le + 1) * rows_per_expert)
            row_of_lane = recorded - le * rows_per_expert;
    } else {
        // Find the packed row of every lane: the rows this source rank put into the lane's expert are
        // [begin, begin + count); the wavefront scans their source-token ids for this token.  Ranges are loaded by
        // the lanes in parallel and, for the first 8 lanes and up to 128 rows each, all id loads are issued before
        // the first comparison: two memory round trips instead of two per lane.
        int my_begin = 0, my_count = 0;
        if (le >= 0) {
            const int64_t range = p.layout_range[int64_t(le) * p.R + src_rank];
            my_begin = int(range >> 32);
            my_count = min(int(range & 0xffffffff), rows_per_expert - my_begin);
        }
        constexpr int kFast = 8;
        int ids0[kFast], ids1[kFast];
    #pragma unroll
        for (int k = 0; k < kFast; ++k) {
            const int kle = read_lane(le, k), kb = read_lane(my_begin, k), kc = read_lane(my_count, k);
            const int32_t* ids = p.src_info + int64_t(kle < 0 ? 0 : kle) * rows_per_expert + kb;
            ids0[k] = (k < p.K && kle >= 0 && lane < kc) ? ids[lane] : -1;
            ids1[k] = (k < p.K && kle >= 0 && lane + kWaveSize < kc) ? ids[lane + kWaveSize] : -1;
        }
    #pragma unroll
        for (int k = 0; k < kFast; ++k) {
            const int kb = read_lane(my_begin, k);
            const uint64_t m0 = __ballot(ids0[k] == t), m1 = __ballot(ids1[k] == t);
            const int found = m0 ? kb + __builtin_ctzll(m0) : m1 ? kb + kWaveSize + __builtin_ctzll(m1) : -1;
            if (lane == k) row_of_lane = found;
        }
        // Lanes past the eighth, and ranges longer than 128 rows.
        for (int k = 0; k < p.K; ++k) {
            const int kle = read_lane(le, k), kb = read_lane(my_begin, k), kc = read_lane(my_count, k);
            const int have = read_lane(row_of_lane, k);
            if (kle < 0 || have >= 0) continue;
            const int first = k < kFast ? 2 * kWaveSize : 0;
            int found = -1;
            for (int base = first; base < kc; base += kWaveSize) {
                const int i = base + lane;
                const bool hit = i < kc && p.src_info[int64_t(kle) * rows_per_expert + kb + i] == t;
                const uint64_t m = __ballot(hit);
                if (m) {
                    found = kb + base + __builtin_ctzll(m);
                    break;
                }
            }
            if (lane == k) row_of_lane = found;
        }
    }

    float acc[kVecs][8];
#pragma unroll
    for (int i = 0; i < kVecs; ++i)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[i][c] = 0.f;

    uint64_t srcs = __ballot(row_of_lane >= 0);
    if constexpr (kLogFmt) {
        while (srcs) {
            const int j = __builtin_ctzll(srcs);
            srcs &= srcs - 1;
            const int64_t row = int64_t(read_lane(le, j)) * rows_per_expert + read_lane(row_of_lane, j);
            const float wj = read_lane(w, j);
            const uint8_t* src = p.x + row * row_bytes;
            // hidden % (kVecs * 512) == 0: every lane of the tile holds channels of the row
            float val[kVecs][8], mag[kVecs][8];
            LogFmtGroup group[kVecs];
            bool chunk_castable = true;
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                const vec16 v = load16_stream(src + (tile * kVecs + i) * 1024 + lane * 16);
                val[i][0] = bf16_lo(v.x); val[i][1] = bf16_hi(v.x); val[i][2] = bf16_lo(v.y); val[i][3] = bf16_hi(v.y);
                val[i][4] = bf16_lo(v.z); val[i][5] = bf16_hi(v.z); val[i][6] = bf16_lo(v.w); val[i][7] = bf16_hi(v.w);
#pragma unroll
                for (int c = 0; c < 8; ++c) mag[i][c] = fabsf(val[i][c]);
                group[i] = logfmt_group_of(mag[i]);
                chunk_castable = chunk_castable && group[i].castable;
            }
            chunk_castable = __ballot(!chunk_castable) == 0ull;          // every group of the chunk
#pragma unroll
            for (int i = 0; i < kVecs; ++i) {
                if (chunk_castable) logfmt_round_trip(val[i], mag[i], group[i]);
#pragma unroll
                for (int c = 0; c < 8; ++c) acc[i][c] += val[i][c] * wj;
            }
        }
    } else {
        // Rows go in rounds of up to four: the loads of a round are all issued before its first multiply-add, so a
        // token with many local lanes pays one trip to memory per four rows, not one per row (eight at a time would
        // need registers that cost the residency decode-sized calls depend on).  The sum keeps lane order.
        constexpr int kRound = 4;
        while (srcs) {
            int64_t row_off[kRound];
            float wj[kRound];
            bool have[kRound];
#pragma unroll
            for (int b = 0; b < kRound; ++b) {
                have[b] = srcs != 0ull;
                row_off[b] = 0;
                wj[b] = 0.f;
                if (have[b]) {
                    const int j = __builtin_ctzll(srcs);
                    srcs &= srcs - 1;
                    row_off[b] = (int64_t(read_lane(le, j)) * rows_per_expert + read_lane(row_of_lane, j)) * row_bytes;
                    wj[b] = read_lane(w, j);
                }
            }
            vec16 v[kRound][kVecs];
#pragma unroll
            for (int b = 0; b < kRound; ++b) {
                if (!have[b]) continue;                    // wave-uniform
#pragma unroll
                for (int i = 0; i < kVecs; ++i) {
                    // a column past the end of the row reads the row's last 16 bytes instead (never accumulated)
                    const int off = min((tile * kVecs + i) * 1024 + lane * 16, row_bytes - 16);
                    v[b][i] = load16_stream(p.x + row_off[b] + off);
                }
            }
#pragma unroll
            for (int b = 0; b < kRound; ++b) {
                if (!have[b]) continue;                    // an absent row adds nothing, not 0 * weight
#pragma unroll
                for (int i = 0; i < kVecs; ++i) {
                    acc[i][0] += bf16_lo(v[b][i].x) * wj[b]; acc[i][1] += bf16_hi(v[b][i].x) * wj[b];
                    acc[i][2] += bf16_lo(v[b][i].y) * wj[b]; acc[i][3] += bf16_hi(v[b][i].y) * wj[b];
                    acc[i][4] += bf16_lo(v[b][i].z) * wj[b]; acc[i][5] += bf16_hi(v[b][i].z) * wj[b];
                    acc[i][6] += bf16_lo(v[b][i].w) * wj[b]; acc[i][7] += bf16_hi(v[b][i].w) * wj[b];
                }
            }
        }
    }

    uint8_t* dst = p.out + g * row_bytes;
#pragma unroll
    for (int i = 0; i < kVecs; ++i) {
        const int off = (tile * kVecs + i) * 1024 + lane * 16;
        if (off < row_bytes) {
            vec16 o;
            o.x = pack_bf16x2(acc[i][0], acc[i][1]);
            o.y = pack_bf16x2(acc[i][2], acc[i][3]);
            o.z = pack_bf16x2(acc[i][4], acc[i][5]);
            o.w = pack_bf16x2(acc[i][6], acc[i][7]);
            store16_stream(dst + off, o);
        }
    }
}

template <int kPairs>
hipError_t launch_move(const LLDispatchParams& p, hipStream_t stream) {
    const int tiles = (p.H + kPairs * 1024 - 1) / (kPairs * 1024);
    const int64_t waves = int64_t(p.S) * p.src_token_stride * tiles;
    const unsigned blocks = unsigned((waves + kMoveWaves - 1) / kMoveWaves);
    if (p.use_fp8) hipLaunchKernelGGL((ll_move_kernel<kPairs, true>), dim3(blocks), dim3(kMoveThreads), 0, stream, p, tiles);
    else hipLaunchKernelGGL((ll_move_kernel<kPairs, false>), dim3(blocks), dim3(kMoveThreads), 0, stream, p, tiles);
    return hipGetLastError();
}

}  // namespace

template <int kPairs, int kFusedThreads>
hipError_t launch_fused(const LLDispatchParams& p, hipStream_t stream, size_t lds) {
    constexpr int kFusedWaves = kFusedThreads / kWaveSize;
    const int tiles = (p.H + kPairs * 1024 - 1) / (kPairs * 1024);
    const int64_t waves = int64_t(p.S) * p.src_token_stride * tiles;
    // one workgroup per compute unit at most (its wavefronts loop over the work items), plus workgroup 0, which publishes only
    const unsigned blocks = unsigned(std::min<int64_t>((waves + kFusedWaves - 1) / kFusedWaves, compute_units())) + 1;
    const bool several = waves > int64_t(blocks - 1) * kFusedWaves;
    if (p.use_fp8) {
        if (several) hipLaunchKernelGGL((ll_fused_kernel<kPairs, true, kFusedThreads, true>), dim3(blocks), dim3(kFusedThreads), lds, stream, p, tiles);
        else hipLaunchKernelGGL((ll_fused_kernel<kPairs, true, kFusedThreads, false>), dim3(blocks), dim3(kFusedThreads), lds, stream, p, tiles);
    } else {
        if (several) hipLaunchKernelGGL((ll_fused_kernel<kPairs, false, kFusedThreads, true>), dim3(blocks), dim3(kFusedThreads), lds, stream, p, tiles);
        else hipLaunchKernelGGL((ll_fused_kernel<kPairs, false, kFusedThreads, false>), dim3(blocks), dim3(kFusedThreads), lds, stream, p, tiles);
    }
    return hipGetLastError();
}

template <int kFusedThreads>
hipError_t launch_fused_by_width(const LLDispatchParams& p, hipStream_t stream, size_t lds) {
    // Up to 4 x 1024 channels per wavefront: fatter wavefronts spend longer in the (serial) cast than the
    // extra wavefronts cost to launch.
    const int segs = (p.H + 1023) / 1024;
    const int forced = p.pairs;
    switch (forced == 1 || forced == 2 || forced == 4 ? forced : segs <= 1 ? 1 : segs <= 2 ? 2 : 4) {
        case 1: return launch_fused<1, kFusedThreads>(p, stream, lds);
        case 2: return launch_fused<2, kFusedThreads>(p, stream, lds);
        default: return launch_fused<4, kFusedThreads>(p, stream, lds);
    }
}

hipError_t launch_ll_dispatch(const LLDispatchParams& p, hipStream_t stream) {
    if (p.S <= 0 || p.src_token_stride <= 0) return hipSuccess;
    // Decode-sized calls: one kernel, every workgroup derives the slots itself.
    const int64_t total_tokens = int64_t(p.S) * p.src_token_stride;
    // the routing table of the single-kernel path, plus one spare 32-bit word per lane
    const size_t fused_lds = size_t(p.E_l) * ((total_tokens + 63) / 64) * sizeof(uint64_t) + kWaveSize * sizeof(uint32_t);
    const bool table_fits = (reinterpret_cast<uintptr_t>(p.topk_idx) & 15) == 0 && total_tokens * p.K >= 2 && p.H >= 16;
    if (total_tokens <= 3072 && fused_lds <= 33 * 1024 && table_fits && !p.two_kernels) {      // beyond: the pair is as fast
        const int threads = p.threads != 0 ? p.threads : 512;
        if (threads == 256) return launch_fused_by_width<256>(p, stream, fused_lds);
        if (threads == 1024) return launch_fused_by_width<1024>(p, stream, fused_lds);
        return launch_fused_by_width<512>(p, stream, fused_lds);
    }

    const int chunks_per_src = (p.src_token_stride + kThreads - 1) / kThreads;
    const unsigned blocks = unsigned(p.S) * chunks_per_src;
    const size_t lds = size_t(p.E_l) * kWaves * sizeof(uint64_t);
    if (p.K <= 8) hipLaunchKernelGGL(ll_count_kernel<8>, dim3(blocks), dim3(kThreads), lds, stream, p);
    else if (p.K <= 16) hipLaunchKernelGGL(ll_count_kernel<16>, dim3(blocks), dim3(kThreads), lds, stream, p);
    else hipLaunchKernelGGL(ll_count_kernel<32>, dim3(blocks), dim3(kThreads), lds, stream, p);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
    // Small token counts: split rows finely so that more wavefronts share the work.
    return (p.H > 2048) ? launch_move<1>(p, stream) : launch_move<2>(p, stream);
}

hipError_t launch_ll_combine(const LLCombineParams& p, hipStream_t stream) {
    if (p.S <= 0 || p.src_token_stride <= 0) return hipSuccess;
    int vecs = p.vecs;
    if (vecs != 1 && vecs != 2 && vecs != 4 && vecs != 7) {
        // Decode-sized calls are over before a second round of workgroups could start: 2 KB per wavefront is the widest
        // tile whose whole grid is resident at once (measured at 1024 tokens x 7168: 1 KB 8.4 us, 2 KB 7.9, 4 KB 9.2,
        // 7 KB 9.3).  Large batches stream with 4 KB tiles.
        const int64_t tokens = int64_t(p.S) * p.src_token_stride;
        vecs = p.H * 2 <= 1024 ? 1 : tokens <= 4096 ? 2 : 4;
    }
    if (p.use_logfmt) vecs = p.H % 1024 == 0 ? 2 : 1;                                     // one codec chunk per wavefront
    const int tiles = (p.H * 2 + vecs * 1024 - 1) / (vecs * 1024);
    const int64_t waves = int64_t(p.S) * p.src_token_stride * tiles;
    const unsigned blocks = unsigned((waves + kMoveWaves - 1) / kMoveWaves);
    if (p.use_logfmt) {
        if (vecs == 2) hipLaunchKernelGGL((ll_combine_kernel<2, true>), dim3(blocks), dim3(kMoveThreads), 0, stream, p, tiles);
        else hipLaunchKernelGGL((ll_combine_kernel<1, true>), dim3(blocks), dim3(kMoveThreads), 0, stream, p, tiles);
        return hipGetLastError();
    }
    // Decode-sized calls: one wavefront per workgroup.  The wavefronts share nothing, and single-wavefront workgroups are
    // placed and retired one by one instead of in fours (1024 tokens x 7168: 7.55 against 8.1 us; large batches and the
    // routing kernels of the high-throughput path measured no difference).
    if (int64_t(p.S) * p.src_token_stride <= 4096 && (vecs == 1 || vecs == 2)) {
        if (vecs == 1) hipLaunchKernelGGL((ll_combine_kernel<1, false, kWaveSize>), dim3(unsigned(waves)), dim3(kWaveSize), 0, stream, p, tiles);
        else hipLaunchKernelGGL((ll_combine_kernel<2, false, kWaveSize>), dim3(unsigned(waves)), dim3(kWaveSize), 0, stream, p, tiles);
        return hipGetLastError();
    }
    if (vecs == 1) hipLaunchKernelGGL(ll_combine_kernel<1>, dim3(blocks), dim3(kMoveThreads), 0, stream, p, tiles);
    else if (vecs == 2) hipLaunchKernelGGL(ll_combine_kernel<2>, dim3(blocks), dim3(kMoveThreads), 0, stream, p, tiles);
    else if (vecs == 4) hipLaunchKernelGGL(ll_combine_kernel<4>, dim3(blocks), dim3(kMoveThreads), 0, stream, p, tiles);
    else hipLaunchKernelGGL(ll_combine_kernel<7>, dim3(blocks), dim3(kMoveThreads), 0, stream, p, tiles);
    return hipGetLastError();
}

}  // namespace deep_ep_hip
