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
// is stored to each destination with 16-byte stores.  No LDS, no barriers.
#include "common.cuh"
#include "cast.cuh"
#include "kernels.h"
#include "publish.cuh"
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

__device__ __forceinline__ Route resolve_route(const MoveParams& p, int t, int lane, bool first_tile) {
    Route r{-1, -1, -1, -1, -1, 0.f};
    const int chunk = t / kLayoutChunk;

    // ---- issue every load that does not depend on another one, then consume: one memory round trip ----
    int64_t raw = -1;
    uint8_t mask_byte = 0;
    uint32_t word = 0xffffffffu;     // cached: handle slot (-1 = none); otherwise the packed positions of the layout pass
    const bool rank_lanes_cached = p.cached && p.rank_lanes;
    if (lane < p.K) {
        const int64_t at = int64_t(t) * p.K + lane;
        if (p.route_mask != nullptr) mask_byte = p.route_mask[at];
        else if (!rank_lanes_cached) raw = p.topk_idx[at];
        if (p.topk_weights != nullptr) r.w = p.topk_weights[at];
        const uint32_t* words = p.cached ? reinterpret_cast<const uint32_t*>(p.cached_slot) : p.pos;
        word = words[at];
    }
    // Flat mode: per-rank chunk counts, flattened [R][chunks_padded]; lane L holds entries [L * per, (L + 1) * per).
    const int per = p.flat_per;
    vec16 counts[4];
    if (p.flat) {
        const int nflat = p.R * p.chunks_padded;
        // addresses are clamped instead of predicated (and masked only when consumed) so that the loads do not
        // wait for each other
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            counts[u] = vec16{0, 0, 0, 0};
            if (u * 4 < per) counts[u] = load16(p.chunk_counts_t + min(lane * per + u * 4, nflat - 4));   // uniform branch
        }
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
                slot = (packed & 0xffffu) == 0xffffu ? -1 : int(packed & 0xffffu);
                epos = int(packed >> 16);
            }
        }
    }
    if (r.e >= 0) r.d = small_div(r.e, p.rcp_E_l);
    else slot = -1;
    if (p.flat) {
        // Exclusive prefix of the per-rank chunk counts in (rank, chunk) order; a wave scan joins the lanes.
        // The prefix at (d, chunk) is at once the start of bucket d and the rows that earlier chunks put
        // into it, so no other table is needed.
        int ex[16];
        int sum = 0;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const bool held = u * 4 < per && lane * per + u * 4 < p.R * p.chunks_padded;
            const vec16 v = held ? counts[u] : vec16{0, 0, 0, 0};
            ex[4 * u] = sum; sum += int(v.x);
            ex[4 * u + 1] = sum; sum += int(v.y);
            ex[4 * u + 2] = sum; sum += int(v.z);
            ex[4 * u + 3] = sum; sum += int(v.w);
        }
        const int lane_base = wave_inclusive_sum(sum) - sum;
#pragma unroll
        for (int i = 0; i < 16; ++i) ex[i] += lane_base;
        // prefix at flat position f: held by lane f / per as its entry f % per (every lane takes part)
        auto prefix_at = [&](int f) {
            const int owner = f / per, off = f - owner * per;
            int got = 0;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                if (i < per) {
                    const int v = __shfl(ex[i], owner, kWaveSize);
                    if (i == off) got = v;
                }
            }
            return got;
        };
        const int fd = (r.d >= 0 ? r.d : 0) * p.chunks_padded;
        const int bucket_start = prefix_at(fd);
        const int before = prefix_at(fd + chunk);
        if (r.d >= 0 && slot >= 0) {
            r.row_c = before + slot;
            slot = r.row_c - bucket_start;      // slot inside the destination bucket
        }
    } else if (r.e >= 0 && slot >= 0) {
        if (p.slot_is_row) {
            r.row_c = slot;
        } else {
            // large R * chunks: each master lane sums its own bucket's row
            if (!p.cached) slot += row_prefix(p.chunk_counts_t, p.chunks_padded, r.d, chunk);
            r.row_c = (r.d > 0 ? p.psum_rank[r.d - 1] : 0) + slot;
        }
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
    int expert_rows_before = 0;
    if (p.do_expand && !p.cached && r.e >= 0)    // rows that earlier chunks put into this lane's expert
        expert_rows_before = row_prefix(p.chunk_counts_t, p.chunks_padded, p.R + r.e, chunk);
    if (p.do_expand && r.e >= 0) {
        if (p.cached) {
            if (r.my_row >= 0 && r.my_row < p.recv_capacity)
                r.erow = p.recv_src_metadata[int64_t(r.my_row) * (p.K + 2) + 2 + lane];
        } else {
            r.erow = p.expert_start[r.e] + expert_rows_before + epos;
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

// Layout and move in one call: workgroup 0 sums the transposed chunk counts and publishes the handle tensors.
// Every thread of the workgroup must call this before any early exit.
__device__ __forceinline__ void publish_from_chunk_counts(const MoveParams& p) {
    extern __shared__ int publish_lds[];
    publish_from_transposed_counts<kThreads>(p.pub, p.chunk_counts_t, p.chunks_padded, publish_lds);
}

// ---- pass-through payload (BF16, or FP8 with caller-provided scale packs) ----
template <int kVecs>
__global__ __launch_bounds__(kThreads) void dispatch_copy_kernel(const MoveParams p) {
    if (p.publish && blockIdx.x == 0) publish_from_chunk_counts(p);
    const int lane = threadIdx.x & 63;
    const unsigned block = p.xcd_remap ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;
    const unsigned work = wave_work_index(block, kWavesPerBlock);
    if (work >= unsigned(p.T) * unsigned(p.tiles)) return;
    const int t = int(work / unsigned(p.tiles));
    const int tile = int(work - unsigned(t) * unsigned(p.tiles));

    vec16 v[kVecs];
    const uint8_t* src = p.x + int64_t(t) * p.row_bytes;
#pragma unroll
    for (int i = 0; i < kVecs; ++i) {
        const int off = (tile * kVecs + i) * 1024 + lane * 16;
        v[i] = vec16{0, 0, 0, 0};
        if (off < p.row_bytes) v[i] = load16_stream(src + off);
    }

    const Route r = resolve_route(p, t, lane, tile == 0);
    if (tile == 0) write_token_metadata(p, r, t, lane);

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

// ---- fused BF16 -> e4m3 cast: lane owns 16 consecutive channels, 8 lanes own one 128-group ----
template <int kPairs>
__global__ __launch_bounds__(kThreads) void dispatch_cast_kernel(const MoveParams p) {
    if (p.publish && blockIdx.x == 0) publish_from_chunk_counts(p);
    const int lane = threadIdx.x & 63;
    const unsigned block = p.xcd_remap ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;
    const unsigned work = wave_work_index(block, kWavesPerBlock);
    if (work >= unsigned(p.T) * unsigned(p.tiles)) return;
    const int t = int(work / unsigned(p.tiles));
    const int tile = int(work - unsigned(t) * unsigned(p.tiles));

    vec16 in[kPairs][2];
    const uint8_t* src = p.x + int64_t(t) * p.row_bytes;
#pragma unroll
    for (int q = 0; q < kPairs; ++q) {
        const int elem = (tile * kPairs + q) * 1024 + lane * 16;
        in[q][0] = vec16{0, 0, 0, 0};
        in[q][1] = vec16{0, 0, 0, 0};
        if (elem < p.H) {
            if (p.plain_loads) {
                in[q][0] = load16(src + int64_t(elem) * 2);
                in[q][1] = load16(src + int64_t(elem) * 2 + 16);
            } else {
                in[q][0] = load16_stream(src + int64_t(elem) * 2);
                in[q][1] = load16_stream(src + int64_t(elem) * 2 + 16);
            }
        }
    }

    const Route r = resolve_route(p, t, lane, tile == 0);
    if (tile == 0) write_token_metadata(p, r, t, lane);

    vec16 out[kPairs];
    float my_scale = 0.f;   // lane L < 8*kPairs ends up holding the scale of group (tile*kPairs*8 + L)
#pragma unroll
    for (int q = 0; q < kPairs; ++q) {
        const float scale_inv = cast_16_channels(in[q][0], in[q][1], out[q]);
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
        if (owns_scale)
            p.recv_sf[int64_t(row) * p.rsf_ts + int64_t(group) * p.rsf_hs] = __float_as_uint(my_scale);
    }
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
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        f[i] = (elem + i < p.H) ? __uint_as_float(uint32_t(src[elem + i]) << 16) : 0.f;
        amax = fmaxf(amax, fabsf(f[i]));
    }
    amax = fmaxf(group8_max(amax), 1e-4f);
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

size_t move_lds_bytes(const MoveParams& p) {
    return p.publish ? publish_lds_bytes(p.R, p.E, kThreads) : 0;
}

template <int kVecs>
hipError_t launch_copy(MoveParams p, hipStream_t stream) {
    p.tiles = (p.row_bytes + kVecs * 1024 - 1) / (kVecs * 1024);
    const int64_t waves = int64_t(p.T) * p.tiles;
    const unsigned blocks = unsigned((waves + kWavesPerBlock - 1) / kWavesPerBlock);
    hipLaunchKernelGGL(dispatch_copy_kernel<kVecs>, dim3(blocks), dim3(kThreads), move_lds_bytes(p), stream, p);
    return hipGetLastError();
}

template <int kPairs>
hipError_t launch_cast(MoveParams p, hipStream_t stream) {
    p.tiles = (p.H + kPairs * 1024 - 1) / (kPairs * 1024);
    const int64_t waves = int64_t(p.T) * p.tiles;
    const unsigned blocks = unsigned((waves + kWavesPerBlock - 1) / kWavesPerBlock);
    hipLaunchKernelGGL(dispatch_cast_kernel<kPairs>, dim3(blocks), dim3(kThreads), move_lds_bytes(p), stream, p);
    return hipGetLastError();
}

int tuning_override(const char* name) {
    const char* v = getenv(name);
    return v != nullptr ? atoi(v) : 0;
}

}  // namespace

hipError_t launch_dispatch_move(MoveParams p, hipStream_t stream) {
    if (p.T == 0) return hipSuccess;
    p.rcp_E_l = 1.0f / float(p.E_l);
    {
        const char* v = getenv("DEEP_EP_HIP_XCD_REMAP");
        p.xcd_remap = v != nullptr ? atoi(v) : 0;
        const char* pl = getenv("DEEP_EP_HIP_PLAIN_LOADS");
        p.plain_loads = pl != nullptr ? atoi(pl) : 0;
    }
    if (p.payload == DEEP_EP_HIP_PAYLOAD_CAST_FP8) {
        // Column tile = kPairs * 1024 channels per wavefront.  Two pairs (2048 channels, 8 waves per SIMD)
        // measured best at hidden 7168: 92.8 us per dispatch against 93.7 (4 pairs) and 96.9 (7 pairs, one
        // wavefront per token).
        int pairs = tuning_override("DEEP_EP_HIP_CAST_PAIRS");
        if (pairs == 0) pairs = p.H <= 1024 ? 1 : 2;
        switch (pairs) {
            case 1: return launch_cast<1>(p, stream);
            case 2: return launch_cast<2>(p, stream);
            case 7: return launch_cast<7>(p, stream);
            case 8: return launch_cast<8>(p, stream);
            default: return launch_cast<4>(p, stream);
        }
    }
    // Pass-through payloads.  Large, bandwidth-bound calls: one 1 KB segment per wavefront measured best for this
    // write-heavy stream (8192 BF16 rows of 14 KB: 143 us per dispatch against 155-159 us with 2, 4, 7 or 8
    // segments).  Small, latency-bound calls: up to 4 KB per wavefront, so that fewer wavefronts repeat the routing
    // work (4096 rows of 4 KB: 26 us against 32 us with 1 KB segments).
    int vecs = tuning_override("DEEP_EP_HIP_COPY_VECS");
    if (vecs == 0) {
        const int kb = (p.row_bytes + 1023) / 1024;
        const bool large = int64_t(p.T) * p.row_bytes >= (int64_t(64) << 20);
        vecs = large ? 1 : (kb <= 1 ? 1 : kb <= 2 ? 2 : 4);
    }
    switch (vecs) {
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
