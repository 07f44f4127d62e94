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

// Sums the transposed chunk counts [R + E][chunks_padded] (padding columns are zero) into per-bucket totals and
// publishes them.  lds: int[R + E] totals, int[2 * E] scratch, one int per wavefront.  Must be called by every
// thread of the workgroup.
template <int kThreads>
__device__ void publish_from_transposed_counts(const PublishParams& q, const int32_t* counts_t, int chunks_padded,
                                               int* lds) {
    const int n = q.R + q.E;
    int* totals = lds;
    int* scratch = totals + n;
    int* scan_tmp = scratch + 2 * q.E;
    for (int j = threadIdx.x; j < n; j += kThreads) {
        const int32_t* row = counts_t + int64_t(j) * chunks_padded;
        int sum = 0;
        for (int c0 = 0; c0 < chunks_padded; c0 += 32) {
            vec16 v[8];                                   // all loads of a pass in flight together
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = load16(row + min(c0 + 4 * u, chunks_padded - 4));
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (c0 + 4 * u < chunks_padded) sum += int(v[u].x) + int(v[u].y) + int(v[u].z) + int(v[u].w);
        }
        totals[j] = sum;
    }
    __syncthreads();
    publish_counts<kThreads>(q, totals, scratch, scan_tmp);
}

// Bytes of LDS publish_from_transposed_counts needs.
inline size_t publish_lds_bytes(int R, int E, int threads) {
    return size_t(R + 3 * E + threads / kWaveSize) * sizeof(int);
}

// Rows that chunks [0, chunk) put into `bucket`: a masked sum over the bucket's row of the transposed counts.
// `chunk` must be uniform over the wavefront.
__device__ __forceinline__ int row_prefix(const int32_t* counts_t, int chunks_padded, int bucket, int chunk) {
    const int32_t* row = counts_t + int64_t(bucket) * chunks_padded;
    int sum = 0;
    for (int c0 = 0; c0 < chunk; c0 += 32) {
        vec16 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = load16(row + min(c0 + 4 * u, chunks_padded - 4));
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int b = c0 + 4 * u;
            sum += (b < chunk ? int(v[u].x) : 0) + (b + 1 < chunk ? int(v[u].y) : 0) +
                   (b + 2 < chunk ? int(v[u].z) : 0) + (b + 3 < chunk ? int(v[u].w) : 0);
        }
    }
    return sum;
}

}  // namespace deep_ep_hip
