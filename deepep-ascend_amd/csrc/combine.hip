// Combine for gfx950: per origin token, gather the rows that came back, accumulate in fp32 in a
// fixed order on top of the optional biases, round once to BF16 and store.
//
// Replaces deep_ep/include/deep_ep/impls/combine.cuh:86-237 (send side, optional local reduce of
// expanded rows) and deep_ep/include/deep_ep/impls/combine_reduce_epilogue.cuh:62-142 with
// combine_utils.cuh:111-168 (ordered fp32 reduce): on one GPU the returned rows already sit in
// local HBM, so the two kernels become one gather-reduce indexed by the dispatch handle.
//
// Order of accumulation (fixed, so results are reproducible): bias_0 + bias_1 first, then one
// term per distinct destination rank in ascending order of that rank's master (highest) lane.
// Expanded layout with multiple reduction: each rank's term is the fp32 sum of that rank's rows in
// lane order rounded to BF16.  Expanded layout without multiple reduction: every valid lane is its
// own term, in lane order.
//
// One wavefront owns one (token, column tile of kVecs * 512 channels).
#include <algorithm>

#include "device_utils.h"
#include "kernels.h"
#include "../../include/deep_ep_hip.h"

namespace deep_ep_hip {

namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerBlock = kThreads / kWaveSize;
#ifndef DEEP_EP_HIP_COMBINE_BATCH
#define DEEP_EP_HIP_COMBINE_BATCH 4
#endif
constexpr int kBatch = DEEP_EP_HIP_COMBINE_BATCH;   // source rows whose loads are issued together

template <int kVecs>
__device__ __forceinline__ void add_row(float (&acc)[kVecs][8], const vec16 (&v)[kVecs]) {
#pragma unroll
    for (int i = 0; i < kVecs; ++i) {
        acc[i][0] += bf16_lo(v[i].x); acc[i][1] += bf16_hi(v[i].x);
        acc[i][2] += bf16_lo(v[i].y); acc[i][3] += bf16_hi(v[i].y);
        acc[i][4] += bf16_lo(v[i].z); acc[i][5] += bf16_hi(v[i].z);
        acc[i][6] += bf16_lo(v[i].w); acc[i][7] += bf16_hi(v[i].w);
    }
}

template <int kVecs>
__device__ __forceinline__ void load_row(vec16 (&v)[kVecs], const uint8_t* base, int64_t row, int row_bytes,
                                         int tile, int lane) {
#pragma unroll
    for (int i = 0; i < kVecs; ++i) {
        const int off = (tile * kVecs + i) * 1024 + lane * 16;
        v[i] = vec16{0, 0, 0, 0};
        if (row >= 0 && off < row_bytes) v[i] = load16_stream(base + row * row_bytes + off);
    }
}

// acc += sum of rows named by the lanes in `mask` (ascending lane order); row_of_lane < 0 adds nothing.
template <int kVecs>
__device__ __forceinline__ void accumulate_rows(float (&acc)[kVecs][8], uint64_t mask, int row_of_lane,
                                                const uint8_t* x, int row_bytes, int tile, int lane) {
    while (mask) {
        int rows[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            rows[b] = -1;
            if (mask) {
                const int j = __builtin_ctzll(mask);
                mask &= mask - 1;
                rows[b] = read_lane(row_of_lane, j);
            }
        }
        vec16 v[kBatch][kVecs];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) load_row<kVecs>(v[b], x, rows[b], row_bytes, tile, lane);
#pragma unroll
        for (int b = 0; b < kBatch; ++b)
            if (rows[b] >= 0) add_row<kVecs>(acc, v[b]);
    }
}

// kLayout: what the rows of x are.  Each gets a kernel of its own, so that the sequencing registers of the expanded
// layout do not cost the compact layout occupancy.
enum : int { kCompactRows = 0, kExpandedRows = 1, kExpandedRowsReducedPerRank = 2 };

template <int kVecs, int kLayout>
__global__ __launch_bounds__(kThreads) void combine_kernel(const CombineParams p) {
    constexpr bool kExpanded = kLayout != kCompactRows;
    const int lane = threadIdx.x & 63;
    const unsigned work = wave_work_index(blockIdx.x, kWavesPerBlock);
    if (work >= unsigned(p.T) * unsigned(p.tiles)) return;
    const int t = int(work / unsigned(p.tiles));
    const int tile = int(work - unsigned(t) * unsigned(p.tiles));
    const int row_bytes = p.H * 2;

    // Biases first: their loads do not depend on the routing metadata.
    float acc[kVecs][8];
#pragma unroll
    for (int i = 0; i < kVecs; ++i)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[i][c] = 0.f;
    if (p.bias0 != nullptr) {
        vec16 v[kVecs];
        load_row<kVecs>(v, p.bias0, t, row_bytes, tile, lane);
        add_row<kVecs>(acc, v);
    }
    if (p.bias1 != nullptr) {
        vec16 v[kVecs];
        load_row<kVecs>(v, p.bias1, t, row_bytes, tile, lane);
        add_row<kVecs>(acc, v);
    }

    // Routing of this token: lanes [0, K).
    int e = -1, d = -1, row_c = -1, my_row = -1, erow = -1;
    if (p.rank_mode) {
        // V1 handle: lane q < R reads the receive row of this token on rank q; rows are added in ascending
        // rank order and the weights of all rows are summed (csrc/kernels/legacy/intranode.cu:940-1033).
        if (lane < p.K) {
            const int v = p.slot[int64_t(t) * p.K + lane];
            if (v >= 0) {
                if (v < p.num_x_rows) row_c = v;
                else atomicOr(p.status, DEEP_EP_HIP_STATUS_ROW_OVERFLOW);
            }
        }
        const uint64_t rows_of_token = __ballot(row_c >= 0);      // taken with every lane active
        if (tile == 0 && p.out_w != nullptr && lane < p.Kw) {
            float w = 0.f;
            uint64_t rows = rows_of_token;
            while (rows) {
                const int j = __builtin_ctzll(rows);
                rows &= rows - 1;
                const int row = read_lane(row_c, j);
                if (p.topk_weights != nullptr) w += p.topk_weights[int64_t(row) * p.Kw + lane];
            }
            p.out_w[int64_t(t) * p.Kw + lane] = w;
        }
    } else if (lane < p.K) {
        const int64_t raw = p.topk_idx[int64_t(t) * p.K + lane];
        if (raw >= 0 && raw < p.E) e = int(raw);
        const int v = p.slot[int64_t(t) * p.K + lane];
        if (e >= 0) {
            d = small_div(e, 1.0f / float(p.E_l));
            if (v >= 0) {
                row_c = (d > 0 ? p.psum_rank[d - 1] : 0) + (v - p.rank_idx * p.M);
                if (!kExpanded && row_c >= p.num_x_rows) {
                    atomicOr(p.status, DEEP_EP_HIP_STATUS_ROW_OVERFLOW);
                    row_c = -1;
                }
            }
        }
    }
    for (int j = 0; j < p.K && !p.rank_mode; ++j) {
        const int dj = read_lane(d, j);
        const int rj = read_lane(row_c, j);
        if (d >= 0 && dj == d && rj >= 0) my_row = rj;
    }
    if (kExpanded && my_row >= 0 && my_row < p.num_meta_rows) {
        erow = p.meta[int64_t(my_row) * (p.K + 2) + 2 + lane];
        if (erow >= p.num_x_rows) {
            atomicOr(p.status, DEEP_EP_HIP_STATUS_ROW_OVERFLOW);
            erow = -1;
        }
    }

    // Weights travel back to the lane that owns them.
    if (tile == 0 && p.out_w != nullptr && lane < p.K && !p.rank_mode) {
        float w = 0.f;
        if (p.topk_weights != nullptr) {
            if (kExpanded) {
                if (erow >= 0) w = p.topk_weights[erow];
            } else if (my_row >= 0) {
                w = p.topk_weights[int64_t(my_row) * p.K + lane];
            }
        }
        p.out_w[int64_t(t) * p.K + lane] = w;
    }

    if constexpr (kLayout == kCompactRows) {
        accumulate_rows<kVecs>(acc, __ballot(row_c >= 0), row_c, p.x, row_bytes, tile, lane);
    } else if constexpr (kLayout == kExpandedRows) {
        accumulate_rows<kVecs>(acc, __ballot(erow >= 0), erow, p.x, row_bytes, tile, lane);
    } else {
        // One term per destination rank, in ascending order of the rank's master lane; a rank's rows are summed in
        // lane order and the sum is rounded to BF16 before it is added.  The rows are put into that order first (each
        // lane learns the place of its row in the sequence), so that their loads go out kBatch at a time across the
        // ranks: a load round per rank would cost a memory round trip for one or two rows each.
        int place = -1, ends_term = 0, alone = 0, total = 0;
        uint64_t masters = __ballot(row_c >= 0);
        while (masters) {
            const int j = __builtin_ctzll(masters);
            masters &= masters - 1;
            const int dj = read_lane(d, j);
            const uint64_t members = __ballot(d == dj && erow >= 0);
            if (d == dj && erow >= 0) {
                place = total + __popcll(members & ((uint64_t(1) << lane) - 1));
                ends_term = (members >> lane) == 1 ? 1 : 0;
                alone = __popcll(members) == 1 ? 1 : 0;         // its BF16 round trip is exact: added as it is
            }
            total += __popcll(members);
        }
        const int flags_of_lane = ends_term | (alone << 1);
        float part[kVecs][8];
#pragma unroll
        for (int i = 0; i < kVecs; ++i)
#pragma unroll
            for (int c = 0; c < 8; ++c) part[i][c] = 0.f;
        for (int first = 0; first < total; first += kBatch) {
            int rows[kBatch], flags[kBatch];
#pragma unroll
            for (int b = 0; b < kBatch; ++b) {
                rows[b] = -1;
                flags[b] = 0;
                if (first + b < total) {
                    const int j = __builtin_ctzll(__ballot(place == first + b));
                    rows[b] = read_lane(erow, j);
                    flags[b] = read_lane(flags_of_lane, j);
                }
            }
            vec16 v[kBatch][kVecs];
#pragma unroll
            for (int b = 0; b < kBatch; ++b) load_row<kVecs>(v[b], p.x, rows[b], row_bytes, tile, lane);
#pragma unroll
            for (int b = 0; b < kBatch; ++b) {
                if (rows[b] < 0) continue;
                if (flags[b] & 2) {
                    add_row<kVecs>(acc, v[b]);
                    continue;
                }
                add_row<kVecs>(part, v[b]);
                if (flags[b] & 1) {
#pragma unroll
                    for (int i = 0; i < kVecs; ++i)
#pragma unroll
                        for (int c = 0; c < 8; ++c) {
                            acc[i][c] += __uint_as_float(f32_to_bf16_bits(part[i][c]) << 16);
                            part[i][c] = 0.f;
                        }
                }
            }
        }
    }

    uint8_t* dst = p.out + int64_t(t) * row_bytes;
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

template <int kVecs, int kLayout>
hipError_t launch_layout(const CombineParams& p, unsigned blocks, hipStream_t stream) {
    hipLaunchKernelGGL((combine_kernel<kVecs, kLayout>), dim3(blocks), dim3(kThreads), 0, stream, p);
    return hipGetLastError();
}

template <int kVecs>
hipError_t launch(CombineParams p, hipStream_t stream) {
    const int row_bytes = p.H * 2;
    p.tiles = (row_bytes + kVecs * 1024 - 1) / (kVecs * 1024);
    const int64_t waves = int64_t(p.T) * p.tiles;
    const unsigned blocks = unsigned((waves + kWavesPerBlock - 1) / kWavesPerBlock);
    if (!p.do_expand || p.rank_mode) return launch_layout<kVecs, kCompactRows>(p, blocks, stream);
    if (!p.multi_red) return launch_layout<kVecs, kExpandedRows>(p, blocks, stream);
    return launch_layout<kVecs, kExpandedRowsReducedPerRank>(p, blocks, stream);
}

// ---- the token -> received-row map of a handle, rebuilt from the rows' own records ----
// A compact receive row r carries (source rank * M + token, source rank * K + master lane) in the first two columns of
// recv_src_metadata, and the rows of destination rank d are [psum[d - 1], psum[d]): so row r is slot r - psum[d - 1] of
// the master lane of its token.  Every other entry is -1.
__global__ __launch_bounds__(kThreads) void fill_slot_map_kernel(int32_t* slot, int64_t n) {
    for (int64_t i = int64_t(blockIdx.x) * kThreads + threadIdx.x; i < n; i += int64_t(gridDim.x) * kThreads) slot[i] = -1;
}

__global__ __launch_bounds__(kThreads) void scatter_slot_map_kernel(const SlotMapParams p) {
    extern __shared__ int32_t psum[];      // [R]
    for (int i = threadIdx.x; i < p.R; i += kThreads) psum[i] = p.psum_rank[i];
    __syncthreads();
    const int64_t rows = min(int64_t(psum[p.R - 1]), p.num_meta_rows);
    for (int64_t r = int64_t(blockIdx.x) * kThreads + threadIdx.x; r < rows; r += int64_t(gridDim.x) * kThreads) {
        const int token = p.meta[r * (p.K + 2)] - p.rank_idx * p.M;
        const int lane = p.meta[r * (p.K + 2) + 1] - p.rank_idx * p.K;
        if (token < 0 || token >= p.T || lane < 0 || lane >= p.K) continue;       // a row of another source rank
        int lo = 0, hi = p.R - 1;                 // first d with r < psum[d]
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (r < psum[mid]) hi = mid;
            else lo = mid + 1;
        }
        const int first = lo > 0 ? psum[lo - 1] : 0;
        p.slot[int64_t(token) * p.K + lane] = p.rank_idx * p.M + int(r - first);
    }
}

}  // namespace

hipError_t launch_rebuild_slot_map(const SlotMapParams& p, hipStream_t stream) {
    const int64_t n = int64_t(p.T) * p.K;
    if (n == 0) return hipSuccess;
    const unsigned fill_blocks = unsigned(std::min<int64_t>((n + kThreads - 1) / kThreads, 2048));
    hipLaunchKernelGGL(fill_slot_map_kernel, dim3(fill_blocks), dim3(kThreads), 0, stream, p.slot, n);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess || p.num_meta_rows == 0) return err;
    const unsigned blocks = unsigned(std::min<int64_t>((p.num_meta_rows + kThreads - 1) / kThreads, 2048));
    hipLaunchKernelGGL(scatter_slot_map_kernel, dim3(blocks), dim3(kThreads), size_t(p.R) * sizeof(int32_t), stream, p);
    return hipGetLastError();
}

hipError_t launch_combine_kernel(CombineParams p, hipStream_t stream) {
    if (p.T == 0) return hipSuccess;
    // Column tile per wavefront, in KB of a BF16 row.  Compact rows: 1 KB (512 channels, 41 registers, eight wavefronts
    // per SIMD) measured best - 8192 tokens x 7168: 117.9 us against 122.7 (2 KB) and 119.6 (4 KB); after a cache flush
    // 123.6 / 126.6 / 124.4; 4096 x 2048: 18.2 / 18.2 / 19.7.  Expanded rows are insensitive (181.7 / 181.7 / 180.5 us).
    int vecs = p.vecs;
    if (vecs == 0) vecs = (p.do_expand && !p.rank_mode && p.H * 2 > 1024) ? 2 : 1;
    switch (vecs) {
        case 1: return launch<1>(p, stream);
        case 4: return launch<4>(p, stream);
        default: return launch<2>(p, stream);
    }
}

}  // namespace deep_ep_hip
