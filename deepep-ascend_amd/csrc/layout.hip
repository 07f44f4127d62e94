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
// with no ordering-dependent atomics: placement is a pure function of the input (layout_count.h).  Chunk
// totals go to tables in the workspace; the last workgroup to finish sums them, writes the base tables the
// move kernel places rows with, and publishes the public prefix sums (publish.h).  A single-launch dispatch
// runs the same two steps inside the move kernel instead (dispatch.hip).
#include "device_utils.h"
#include "kernels.h"
#include "layout_count.h"
#include "publish.h"
#include "../../include/deep_ep_hip.h"

namespace deep_ep_hip {

namespace {

constexpr int kThreads = kLayoutChunk;
constexpr int kWaves = kThreads / kWaveSize;

template <int KMAX>
__global__ __launch_bounds__(kThreads) void layout_kernel(const LayoutParams p) {
    extern __shared__ uint64_t bitmap[];   // [(R + E)][kWaves]
    __shared__ int is_last;
    const int tid = threadIdx.x;
    count_chunk<KMAX, true>(p, int(blockIdx.x), int(gridDim.x), bitmap);

    // Hand the chunk totals to whichever workgroup finishes last: they were stored at agent scope (written through), so
    // waiting for our own stores is all the release there is - no write-back of the whole L2 - then take a ticket.
    wait_for_own_stores();
    __syncthreads();
    if (tid == 0) {
        const unsigned ticket = atomicAdd(p.done_counter, 1u);
        is_last = (ticket == gridDim.x - 1) ? 1 : 0;
    }
    __syncthreads();
    if (!is_last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");

    // ---- last workgroup: per-bucket totals, the public prefix sums and the row bases (LDS is re-carved) ----
    publish_layout<kThreads>(p.pub, p.tab, int(gridDim.x), p.expert_bases != 0, reinterpret_cast<int*>(bitmap));
    if (tid == 0) *p.done_counter = 0u;                    // ready for the next launch
}

}  // namespace

hipError_t launch_layout_kernel(const LayoutParams& p, hipStream_t stream) {
    const int num_chunks = p.T > 0 ? (p.T + kThreads - 1) / kThreads : 1;
    const int n = p.R + p.E;
    // LDS holds the bitmap words [n][kWaves] first; the last workgroup re-carves it for the publishing step.
    const size_t bitmap_bytes = count_lds_bytes(p.R, p.E);
    const size_t publish_bytes = publish_lds_bytes(p.R, p.E, kThreads);
    const size_t lds = bitmap_bytes > publish_bytes ? bitmap_bytes : publish_bytes;
    LayoutParams q = p;
    q.vec_idx = (reinterpret_cast<uintptr_t>(p.topk_idx) % 16 == 0) ? 1 : 0;
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
