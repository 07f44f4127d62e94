// Dispatch layout for gfx950: one pass over topk_idx produces per-rank / per-expert counts, the
// token->rank membership, and (for dispatch) the deterministic position of every (token, lane)
// inside its destination bucket.
//
// Replaces csrc/kernels/legacy/layout.cu:10-122 (get_dispatch_layout, where every block rescans
// the whole index array) and the notify warps of deep_ep/include/deep_ep/impls/dispatch.cuh:79-258
// (per-rank / per-expert counts, aligned prefix sums, host mailbox).
//
// Design: a workgroup owns a chunk of 256 consecutive tokens (one lane per token).  Each wave sets
// its lane bit in an LDS bitmap word per rank and per expert (ds_or_b64), so that
//   count  = popcount(bitmap)                      and
//   position of token t among chunk tokens routed to the same bucket = popcount(bitmap & lanes below t)
// with no ordering-dependent atomics: placement is a pure function of the input.  Chunk totals go
// to global memory (transposed, so that a consumer prefix-sums along a row); the last workgroup to finish sums
// them and publishes the public prefix sums.
#include "common.cuh"
#include "kernels.h"
#include "publish.cuh"
#include "../../include/deep_ep_hip.h"

namespace deep_ep_hip {

namespace {

constexpr int kThreads = kLayoutChunk;
constexpr int kWaves = kThreads / kWaveSize;

template <int KMAX>
__global__ __launch_bounds__(kThreads) void layout_kernel(const LayoutParams p) {
    extern __shared__ uint64_t bitmap[];   // [(R + E)][kWaves]
    __shared__ int is_last;

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int chunk = blockIdx.x;
    const int t = chunk * kThreads + tid;
    const int n = p.R + p.E;
    const bool active = t < p.T;

    for (int i = tid; i < n * kWaves; i += kThreads) bitmap[i] = 0ull;
    __syncthreads();

    // All index loads are issued before anything that could alias them is stored.
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

    int e[KMAX], d[KMAX];
    int flags = 0;
    const float rcp_experts_per_rank = 1.0f / float(p.E_l);
    const uint64_t my_bit = 1ull << lane;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        int ev = -1;
        if (raw[k] >= p.E) flags |= DEEP_EP_HIP_STATUS_EXPERT_OUT_OF_RANGE;
        else if (raw[k] >= 0) ev = int(raw[k]);
        e[k] = ev;
        d[k] = ev >= 0 ? small_div(ev, rcp_experts_per_rank) : -1;
        if (ev >= 0) {
            atomicOr(reinterpret_cast<unsigned long long*>(&bitmap[(p.R + ev) * kWaves + wave]), my_bit);
            atomicOr(reinterpret_cast<unsigned long long*>(&bitmap[d[k] * kWaves + wave]), my_bit);
        }
    }
    if (p.copied_topk_idx != nullptr && active) {
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
            if (k < p.K) p.copied_topk_idx[int64_t(t) * p.K + k] = raw[k];
    }
    __syncthreads();

    const uint64_t below = lanes_below(lane);
    auto rank_in_chunk = [&](int bucket) {
        int pos = __popcll(bitmap[bucket * kWaves + wave] & below);
        for (int w = 0; w < wave; ++w) pos += __popcll(bitmap[bucket * kWaves + w]);
        return pos;
    };

    if (active) {
        if (p.pos != nullptr) {
            // One word per (token, lane): low 16 bits = slot of the token inside its chunk for the lane's
            // destination rank (master lanes only), high 16 bits = position of the lane inside its chunk for
            // its expert; 0xffff = none.
            uint32_t packed[KMAX];
#pragma unroll
            for (int k = 0; k < KMAX; ++k) {
                uint32_t pr = 0xffffu, pe = 0xffffu;
                if (e[k] >= 0) {
                    bool master = true;
#pragma unroll
                    for (int j = 0; j < KMAX; ++j) {
                        if (j > k && d[j] == d[k]) master = false;
                        if (j != k && e[j] == e[k]) flags |= DEEP_EP_HIP_STATUS_DUPLICATE_EXPERT;
                    }
                    pe = uint32_t(rank_in_chunk(p.R + e[k]));
                    if (master) pr = uint32_t(rank_in_chunk(d[k]));
                }
                packed[k] = pr | (pe << 16);
            }
            if (KMAX == 8 && p.K == 8) {
                vec16* dst = reinterpret_cast<vec16*>(p.pos + int64_t(t) * 8);
                dst[0] = vec16{packed[0], packed[1], packed[2], packed[3]};
                dst[1] = vec16{packed[4], packed[5], packed[6], packed[7]};
            } else {
#pragma unroll
                for (int k = 0; k < KMAX; ++k)
                    if (k < p.K) p.pos[int64_t(t) * p.K + k] = packed[k];
            }
        }
        if (p.is_token_in_rank != nullptr) {
            for (int r = 0; r < p.R; ++r)
                p.is_token_in_rank[int64_t(t) * p.R + r] = uint8_t((bitmap[r * kWaves + wave] >> lane) & 1ull);
        }
    }
    if (flags != 0) atomicOr(p.status, flags);

    // Chunk totals go out transposed, [bucket][chunk], so that consumers prefix-sum along rows; the padding
    // columns up to a multiple of four are cleared by the first workgroup.
    for (int j = tid; j < n; j += kThreads) {
        int c = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) c += __popcll(bitmap[j * kWaves + w]);
        p.chunk_counts[int64_t(j) * p.chunks_padded + chunk] = c;
    }
    const int pad = p.chunks_padded - int(gridDim.x);
    if (chunk == 0)
        for (int i = tid; i < n * pad; i += kThreads)
            p.chunk_counts[int64_t(i / pad) * p.chunks_padded + gridDim.x + i % pad] = 0;
    if (p.light) return;      // the move kernel of the same call sums and publishes

    // Hand the chunk totals to whichever workgroup finishes last: release our stores, take a ticket.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __syncthreads();
    if (tid == 0) {
        const unsigned ticket = atomicAdd(p.done_counter, 1u);
        is_last = (ticket == gridDim.x - 1) ? 1 : 0;
    }
    __syncthreads();
    if (!is_last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");

    // ---- last workgroup: per-bucket totals and the public prefix sums (LDS is re-carved as int arrays) ----
    publish_from_transposed_counts<kThreads>(p.pub, p.chunk_counts, p.chunks_padded, reinterpret_cast<int*>(bitmap));
    if (tid == 0) *p.done_counter = 0u;                    // ready for the next launch
}

}  // namespace

hipError_t launch_layout_kernel(const LayoutParams& p, hipStream_t stream) {
    const int num_chunks = p.T > 0 ? (p.T + kThreads - 1) / kThreads : 1;
    const int n = p.R + p.E;
    // LDS holds the bitmap words [n][kWaves] first; the last workgroup re-carves it for the publishing step.
    const size_t bitmap_bytes = size_t(n) * kWaves * sizeof(uint64_t);
    const size_t publish_bytes = publish_lds_bytes(p.R, p.E, kThreads);
    const size_t lds = bitmap_bytes > publish_bytes ? bitmap_bytes : publish_bytes;
    LayoutParams q = p;
    q.vec_idx = (reinterpret_cast<uintptr_t>(p.topk_idx) % 16 == 0) ? 1 : 0;
    q.chunks_padded = (num_chunks + 3) / 4 * 4;
    dim3 grid(num_chunks), block(kThreads);
    if (p.K <= 8) {
        hipLaunchKernelGGL(layout_kernel<8>, grid, block, lds, stream, q);
    } else if (p.K <= 16) {
        hipLaunchKernelGGL(layout_kernel<16>, grid, block, lds, stream, q);
    } else {
        hipLaunchKernelGGL(layout_kernel<32>, grid, block, lds, stream, q);
    }
    return hipGetLastError();
}

}  // namespace deep_ep_hip
