// Turning per-bucket totals into the public outputs of the layout computation: per-rank and
// per-expert counts, their prefix sums (the handle tensors of dispatch) and the host mailbox.
// Mirrors what the notify warps of deep_ep/include/deep_ep/impls/dispatch.cuh:200-257 publish.
#pragma once

#include "common.cuh"
#include "kernels.h"

namespace deep_ep_hip {

// In-place inclusive scan of a[0..n) in LDS by the whole workgroup.  tmp holds one int per wavefront.
template <int kThreads>
__device__ void block_inclusive_scan(int* a, int n, int* tmp) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int per = (n + kThreads - 1) / kThreads;
    const int begin = min(tid * per, n), end = min(begin + per, n);
    int s = 0;
    for (int i = begin; i < end; ++i) s += a[i];
    const int inc = wave_inclusive_sum(s);
    if (lane == kWaveSize - 1) tmp[wave] = inc;
    __syncthreads();
    int run = inc - s;
    for (int w = 0; w < wave; ++w) run += tmp[w];
    for (int i = begin; i < end; ++i) {
        run += a[i];
        a[i] = run;
    }
    __syncthreads();
}

// totals: LDS int[R + E], rank counts then expert counts (the rank part is overwritten by its prefix sum).
// scratch: LDS int[2 * E].  Must be called by every thread of the workgroup.
template <int kThreads>
__device__ void publish_counts(const PublishParams& q, int* totals, int* scratch, int* scan_tmp) {
    const int tid = threadIdx.x;
    int* aligned = scratch;
    int* aligned_incl = scratch + q.E;
    for (int j = tid; j < q.E; j += kThreads) {
        const int cnt = totals[q.R + j];
        const int al = (cnt + q.A - 1) / q.A * q.A;
        aligned[j] = al;
        aligned_incl[j] = al;
        if (q.num_tokens_per_expert != nullptr) q.num_tokens_per_expert[j] = cnt;
        if (q.num_unaligned != nullptr) q.num_unaligned[j] = cnt;
        if (q.cumulative_stats != nullptr) q.cumulative_stats[j] += cnt;
        if (q.host_counts != nullptr) q.host_counts[q.R + j] = -al - 1;
    }
    for (int r = tid; r < q.R; r += kThreads) {
        if (q.num_tokens_per_rank != nullptr) q.num_tokens_per_rank[r] = totals[r];
        if (q.host_counts != nullptr) q.host_counts[r] = -totals[r] - 1;
    }
    __syncthreads();
    block_inclusive_scan<kThreads>(aligned_incl, q.E, scan_tmp);
    for (int j = tid; j < q.E; j += kThreads) {
        const int start = aligned_incl[j] - aligned[j];
        if (q.expert_start != nullptr) q.expert_start[j] = start;
        if (q.psum_expert != nullptr) q.psum_expert[j] = q.do_expand ? start + totals[q.R + j] : aligned_incl[j];
    }
    const int total_expanded = q.E > 0 ? aligned_incl[q.E - 1] : 0;
    __syncthreads();
    block_inclusive_scan<kThreads>(totals, q.R, scan_tmp);     // ranks: inclusive prefix in place
    for (int r = tid; r < q.R; r += kThreads)
        if (q.psum_rank != nullptr) q.psum_rank[r] = totals[r];
    if (tid == 0 && q.totals_out != nullptr) {
        q.totals_out[0] = totals[q.R - 1];
        q.totals_out[1] = total_expanded;
    }
    if (q.host_counts != nullptr) __threadfence_system();
}

}  // namespace deep_ep_hip
