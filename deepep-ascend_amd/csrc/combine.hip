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

template <int kVecs>
__global__ __launch_bounds__(kThreads) void combine_kernel(const CombineParams p) {
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
                if (!p.do_expand && row_c >= p.num_x_rows) {
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
    if (p.do_expand && my_row >= 0 && my_row < p.num_meta_rows) {
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
            if (p.do_expand) {
                if (erow >= 0) w = p.topk_weights[erow];
            } else if (my_row >= 0) {
                w = p.topk_weights[int64_t(my_row) * p.K + lane];
            }
        }
        p.out_w[int64_t(t) * p.K + lane] = w;
    }

    if (!p.do_expand) {
        accumulate_rows<kVecs>(acc, __ballot(row_c >= 0), row_c, p.x, row_bytes, tile, lane);
    } else if (!p.multi_red) {
        accumulate_rows<kVecs>(acc, __ballot(erow >= 0), erow, p.x, row_bytes, tile, lane);
    } else {
        uint64_t masters = __ballot(row_c >= 0);
        while (masters) {
            const int j = __builtin_ctzll(masters);
            masters &= masters - 1;
            const int dj = read_lane(d, j);
            const uint64_t members = __ballot(d == dj && erow >= 0);
            if (__popcll(members) == 1) {
                accumulate_rows<kVecs>(acc, members, erow, p.x, row_bytes, tile, lane);   // bf16 round trip is exact
            } else {
                float part[kVecs][8];
#pragma unroll
                for (int i = 0; i < kVecs; ++i)
#pragma unroll
                    for (int c = 0; c < 8; ++c) part[i][c] = 0.f;
                accumulate_rows<kVecs>(part, members, erow, p.x, row_bytes, tile, lane);
#pragma unroll
                for (int i = 0; i < kVecs; ++i)
#pragma unroll
                    for (int c = 0; c < 8; ++c)
                        acc[i][c] += __uint_as_float(f32_to_bf16_bits(part[i][c]) << 16);
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

template <int kVecs>
hipError_t launch(CombineParams p, hipStream_t stream) {
    const int row_bytes = p.H * 2;
    p.tiles = (row_bytes + kVecs * 1024 - 1) / (kVecs * 1024);
    const int64_t waves = int64_t(p.T) * p.tiles;
    const unsigned blocks = unsigned((waves + kWavesPerBlock - 1) / kWavesPerBlock);
    hipLaunchKernelGGL(combine_kernel<kVecs>, dim3(blocks), dim3(kThreads), 0, stream, p);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_combine_kernel(CombineParams p, hipStream_t stream) {
    if (p.T == 0) return hipSuccess;
    int vecs = p.vecs;
    if (vecs == 0) vecs = (p.H * 2 <= 1024) ? 1 : 2;
    switch (vecs) {
        case 1: return launch<1>(p, stream);
        case 4: return launch<4>(p, stream);
        default: return launch<2>(p, stream);
    }
}

}  // namespace deep_ep_hip
