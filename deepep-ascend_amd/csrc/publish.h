// Turning per-chunk totals into the public outputs of the layout computation (per-rank and per-expert counts,
// their prefix sums - the handle tensors of dispatch - and the host mailbox) and into the base tables the move
// kernels place rows with (struct LayoutTables).  Publishes what the notify warps of
// deep_ep/include/deep_ep/impls/dispatch.cuh:200-257 publish.
#pragma once

#include "device_utils.h"
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

// LDS of the publishing workgroup: totals[R + E] | aligned[E] | aligned_incl[E] | one int per wavefront.
struct PublishLds {
    int* totals;         // rank part becomes its inclusive prefix sum in publish_ranks
    int* aligned;
    int* aligned_incl;
    int* scan_tmp;
};

__device__ __forceinline__ PublishLds carve_publish_lds(int* lds, int R, int E) {
    return PublishLds{lds, lds + R + E, lds + R + 2 * E, lds + R + 3 * E};
}

inline size_t publish_lds_bytes(int R, int E, int threads) {
    return size_t(R + 3 * E + threads / kWaveSize) * sizeof(int);
}

// ---- rank part: tables are transposed, [rank][chunk] ----

// totals[r] = sum of row r of rank_counts (padding columns are zero).  Ends with a barrier.
template <int kThreads>
__device__ void sum_rank_rows(const LayoutTables& t, int R, int* totals) {
    for (int j = threadIdx.x; j < R; j += kThreads) {
        const int32_t* row = t.rank_counts + int64_t(j) * t.chunks_padded;
        int sum = 0;
        for (int c0 = 0; c0 < t.chunks_padded; c0 += 32) {
            vec16 v[8];                                   // all loads of a pass in flight together
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = load16(row + min(c0 + 4 * u, t.chunks_padded - 4));
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (c0 + 4 * u < t.chunks_padded) sum += int(v[u].x) + int(v[u].y) + int(v[u].z) + int(v[u].w);
        }
        totals[j] = sum;
    }
    __syncthreads();
}

// Per-rank outputs; afterwards s.totals[0..R) holds the inclusive prefix sum.  Every thread must call it.
template <int kThreads>
__device__ void publish_ranks(const PublishParams& q, const PublishLds& s) {
    for (int r = threadIdx.x; r < q.R; r += kThreads) {
        if (q.num_tokens_per_rank != nullptr) q.num_tokens_per_rank[r] = s.totals[r];
        if (q.host_counts != nullptr) q.host_counts[r] = -s.totals[r] - 1;
    }
    __syncthreads();
    block_inclusive_scan<kThreads>(s.totals, q.R, s.scan_tmp);
    for (int r = threadIdx.x; r < q.R; r += kThreads)
        if (q.psum_rank != nullptr) q.psum_rank[r] = s.totals[r];
    if (threadIdx.x == 0 && q.totals_out != nullptr) q.totals_out[0] = s.totals[q.R - 1];
}

// rank_bases[r][c] = (rows of lower ranks) + sum of rank_counts[r][0..c): one thread per rank, 32 chunks per pass
// with all of a pass's loads in flight together.  s.totals[0..R) must hold the inclusive prefix sum of the ranks.
template <int kThreads>
__device__ void write_rank_bases(const LayoutTables& t, int R, const PublishLds& s) {
    for (int j = threadIdx.x; j < R; j += kThreads) {
        const int32_t* src = t.rank_counts + int64_t(j) * t.chunks_padded;
        int32_t* dst = t.rank_bases + int64_t(j) * t.chunks_padded;
        int run = j > 0 ? s.totals[j - 1] : 0;
        for (int c0 = 0; c0 < t.chunks_padded; c0 += 32) {
            vec16 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = load16(src + min(c0 + 4 * u, t.chunks_padded - 4));
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (c0 + 4 * u < t.chunks_padded) {
                    vec16 o;
                    o.x = uint32_t(run); run += int(v[u].x);
                    o.y = uint32_t(run); run += int(v[u].y);
                    o.z = uint32_t(run); run += int(v[u].z);
                    o.w = uint32_t(run); run += int(v[u].w);
                    store16(dst + c0 + 4 * u, o);
                }
            }
        }
    }
}

// The rank part as one flat pass over rank_counts ([rank][chunk], R * chunks_padded <= 4 * kThreads entries), for the
// publishing workgroup of a single-launch dispatch.  A line of that table holds the totals of up to 16 chunks, written
// through by as many counting workgroups of the same launch, some of them on this XCD: it is read at agent scope, past
// any partial copy of the line a cache may hold.  The inclusive prefix sum over the flattened table is, at the last
// entry of row r, the end of rank r's bucket.  Publishes the per-rank outputs.  Every thread of the workgroup must
// call it; s.scan_tmp: kThreads / 64 ints of LDS.
template <int kThreads>
__device__ void scan_rank_counts(const PublishParams& q, const LayoutTables& t, int R, const PublishLds& s) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int flat = R * t.chunks_padded;              // a multiple of 4: a thread's entries share a row
    const int begin = tid * 4;
    vec16 v{0, 0, 0, 0};
    if (begin < flat) {
        const unsigned long long* at = reinterpret_cast<const unsigned long long*>(t.rank_counts + begin);
        const unsigned long long lo = __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long hi = __hip_atomic_load(at + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        v = vec16{uint32_t(lo), uint32_t(lo >> 32), uint32_t(hi), uint32_t(hi >> 32)};
    }
    const int sum = int(v.x) + int(v.y) + int(v.z) + int(v.w);
    const int inc = wave_inclusive_sum(sum);
    if (lane == kWaveSize - 1) s.scan_tmp[wave] = inc;
    __syncthreads();
    int run = inc - sum;
    for (int w = 0; w < wave; ++w) run += s.scan_tmp[w];
    if (begin < flat && (begin + 4) % t.chunks_padded == 0) s.totals[begin / t.chunks_padded] = run + sum;   // inclusive prefix of the rank
    __syncthreads();
    for (int r = tid; r < R; r += kThreads) {
        const int total = s.totals[r] - (r > 0 ? s.totals[r - 1] : 0);
        if (q.num_tokens_per_rank != nullptr) q.num_tokens_per_rank[r] = total;
        if (q.host_counts != nullptr) q.host_counts[r] = -total - 1;
        if (q.psum_rank != nullptr) q.psum_rank[r] = s.totals[r];
    }
    if (tid == 0 && q.totals_out != nullptr) q.totals_out[0] = s.totals[R - 1];
}

// ---- expert part: tables are [chunk][expert], so that thread e walks column e with coalesced accesses ----

// totals[R + e] = sum over chunks of expert_counts[c][e].  Ends with a barrier.
template <int kThreads>
__device__ void sum_expert_columns(const LayoutTables& t, int R, int E, int num_chunks, int* totals) {
    for (int e = threadIdx.x; e < E; e += kThreads) {
        const int32_t* col = t.expert_counts + e;
        int sum = 0;
        for (int c0 = 0; c0 < num_chunks; c0 += 16) {
            int v[16];                                    // all loads of a pass in flight together
#pragma unroll
            for (int u = 0; u < 16; ++u) v[u] = col[int64_t(min(c0 + u, num_chunks - 1)) * t.experts_padded];
#pragma unroll
            for (int u = 0; u < 16; ++u) sum += c0 + u < num_chunks ? v[u] : 0;
        }
        totals[R + e] = sum;
    }
    __syncthreads();
}

// Per-expert outputs; afterwards the region of expert j starts at s.aligned_incl[j] - s.aligned[j].
template <int kThreads>
__device__ void publish_experts(const PublishParams& q, const PublishLds& s) {
    for (int j = threadIdx.x; j < q.E; j += kThreads) {
        const int cnt = s.totals[q.R + j];
        const int al = (cnt + q.A - 1) / q.A * q.A;
        s.aligned[j] = al;
        s.aligned_incl[j] = al;
        if (q.num_tokens_per_expert != nullptr) q.num_tokens_per_expert[j] = cnt;
        if (q.num_unaligned != nullptr) q.num_unaligned[j] = cnt;
        if (q.cumulative_stats != nullptr) q.cumulative_stats[j] += cnt;
        if (q.host_counts != nullptr) q.host_counts[q.R + j] = -al - 1;
    }
    __syncthreads();
    block_inclusive_scan<kThreads>(s.aligned_incl, q.E, s.scan_tmp);
    for (int j = threadIdx.x; j < q.E; j += kThreads) {
        const int start = s.aligned_incl[j] - s.aligned[j];
        if (q.expert_start != nullptr) q.expert_start[j] = start;
        if (q.psum_expert != nullptr) q.psum_expert[j] = q.do_expand ? start + s.totals[q.R + j] : s.aligned_incl[j];
    }
    if (threadIdx.x == 0 && q.totals_out != nullptr) q.totals_out[1] = q.E > 0 ? s.aligned_incl[q.E - 1] : 0;
    if (q.host_counts != nullptr) {
        // The status word as the counting workgroups left it (they are all done when a workgroup publishes): a host that
        // sizes its outputs from this mailbox learns about bad routing input without a second trip to the device.
        if (threadIdx.x == 0) q.host_counts[q.R + q.E] = -(q.status != nullptr ? load_agent(q.status) : 0) - 1;
        __threadfence_system();
    }
}

// table[c][e] = start of expert e's region + sum of expert_counts[0..c)[e], each word ORed with `tag`.
// kThrough: stored at agent scope.
template <int kThreads, bool kThrough>
__device__ void write_expert_bases(const LayoutTables& t, int32_t* table, uint32_t tag, int E, int num_chunks, const PublishLds& s) {
    for (int e = threadIdx.x; e < E; e += kThreads) {
        const int32_t* col = t.expert_counts + e;
        int32_t* out = table + e;
        int run = s.aligned_incl[e] - s.aligned[e];
        for (int c0 = 0; c0 < num_chunks; c0 += 16) {
            int v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) v[u] = col[int64_t(min(c0 + u, num_chunks - 1)) * t.experts_padded];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                if (c0 + u < num_chunks) {
                    store_word<kThrough>(out + int64_t(c0 + u) * t.experts_padded, int(uint32_t(run) | tag));
                    run += v[u];
                }
            }
        }
    }
}

// Does `word` carry the tag of the running single-launch dispatch (kernels.h)?
__device__ __forceinline__ bool has_tag(uint32_t word, uint32_t tag) {
    return (word & ~kTagValueMask) == tag;
}

// The expert base table in one trip, for the publishing workgroup of a single-launch expanded dispatch, whose movers
// wait for exactly this.  Thread e reads its column of the tagged chunk totals at agent scope, again (at most
// spin_limit times) until every word shows the tag - no flag of the counting workgroups is waited for, which would
// only be raised once all their stores are acknowledged - keeps the column in registers between the sum and the
// stores, and stores the bases at agent scope, each ORed with `tag`.  Needs E <= kThreads and num_chunks <= 32.
// Leaves totals / aligned / aligned_incl as publish_experts expects to recompute them.  A: expert alignment.
// Returns whether every thread got its column.
template <int kThreads>
__device__ bool write_expert_bases_from_registers(const LayoutTables& t, const uint32_t* tagged_counts, int32_t* table, uint32_t tag,
                                                  unsigned spin_limit, int R, int E, int A, int num_chunks, const PublishLds& s) {
    const int e = threadIdx.x;
    int v[32];
    int total = 0;
    bool complete = true;
    if (e < E) {
        unsigned polls = 0;
        for (;;) {
            complete = true;
#pragma unroll
            for (int u = 0; u < 32; ++u) {
                // a row start common to the workgroup plus the thread's column: one address register serves all 32 loads
                const int row_start = __builtin_amdgcn_readfirstlane(min(u, num_chunks - 1) * t.experts_padded);
                v[u] = load_agent(reinterpret_cast<const int*>(tagged_counts) + row_start + e);
            }
#pragma unroll
            for (int u = 0; u < 32; ++u) complete = complete && has_tag(uint32_t(v[u]), tag);
            if (complete || polls == spin_limit) break;
            __builtin_amdgcn_s_sleep(4);
            ++polls;
        }
#pragma unroll
        for (int u = 0; u < 32; ++u) {
            v[u] = int(uint32_t(v[u]) & kTagValueMask);
            total += u < num_chunks ? v[u] : 0;
        }
        s.totals[R + e] = total;
        const int al = (total + A - 1) / A * A;
        s.aligned[e] = al;
        s.aligned_incl[e] = al;
    }
    const int all_complete = __syncthreads_and(complete ? 1 : 0);
    block_inclusive_scan<kThreads>(s.aligned_incl, E, s.scan_tmp);
    if (e < E) {
        int run = s.aligned_incl[e] - s.aligned[e];
#pragma unroll
        for (int u = 0; u < 32; ++u) {
            if (u < num_chunks) {
                const int row_start = __builtin_amdgcn_readfirstlane(u * t.experts_padded);
                store_agent(table + row_start + e, int(uint32_t(run) | tag));
                run += v[u];
            }
        }
    }
    return all_complete != 0;
}

// publish_layout for the common sizes (at most 32 chunks, num_experts <= kThreads, R * chunks_padded <= 4 * kThreads) in one
// trip to memory instead of four: every thread first loads all it will ever need - four entries of the flattened rank
// table and its expert's column of chunk totals, kept in registers - and totals, prefix sums, public outputs and both
// base tables are worked out from those.
template <int kThreads>
__device__ void publish_layout_in_one_trip(const PublishParams& q, const LayoutTables& t, int num_chunks, bool expert_bases, int* lds) {
    const PublishLds s = carve_publish_lds(lds, q.R, q.E);
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int flat = q.R * t.chunks_padded;              // a multiple of 4: a thread's entries share a row
    const int begin = tid * 4;
    vec16 rv{0, 0, 0, 0};
    if (begin < flat) rv = load16(t.rank_counts + begin);
    int v[32];
    if (tid < q.E) {
#pragma unroll
        for (int u = 0; u < 32; ++u) {
            const int row_start = __builtin_amdgcn_readfirstlane(min(u, num_chunks - 1) * t.experts_padded);
            v[u] = t.expert_counts[row_start + tid];
        }
    }

    // rank part: exclusive prefix over the flattened table = first compact row of every (rank, chunk)
    const int sum = int(rv.x) + int(rv.y) + int(rv.z) + int(rv.w);
    const int inc = wave_inclusive_sum(sum);
    if (lane == kWaveSize - 1) s.scan_tmp[wave] = inc;
    __syncthreads();
    int run = inc - sum;
    for (int w = 0; w < wave; ++w) run += s.scan_tmp[w];
    if (begin < flat) {
        if (t.rank_bases != nullptr) {
            const uint32_t b0 = uint32_t(run), b1 = b0 + rv.x, b2 = b1 + rv.y, b3 = b2 + rv.z;
            store16(t.rank_bases + begin, vec16{b0, b1, b2, b3});
        }
        if ((begin + 4) % t.chunks_padded == 0) s.totals[begin / t.chunks_padded] = run + sum;   // inclusive prefix of the rank
    }
    if (tid < q.E) {
        int total = 0;
#pragma unroll
        for (int u = 0; u < 32; ++u) total += u < num_chunks ? v[u] : 0;
        s.totals[q.R + tid] = total;
    }
    __syncthreads();
    for (int r = tid; r < q.R; r += kThreads) {
        const int total = s.totals[r] - (r > 0 ? s.totals[r - 1] : 0);
        if (q.num_tokens_per_rank != nullptr) q.num_tokens_per_rank[r] = total;
        if (q.host_counts != nullptr) q.host_counts[r] = -total - 1;
        if (q.psum_rank != nullptr) q.psum_rank[r] = s.totals[r];
    }
    if (tid == 0 && q.totals_out != nullptr) q.totals_out[0] = s.totals[q.R - 1];

    publish_experts<kThreads>(q, s);
    if (t.expert_bases != nullptr && expert_bases && tid < q.E) {
        int at = s.aligned_incl[tid] - s.aligned[tid];
#pragma unroll
        for (int u = 0; u < 32; ++u) {
            if (u < num_chunks) {
                const int row_start = __builtin_amdgcn_readfirstlane(u * t.experts_padded);
                t.expert_bases[row_start + tid] = at;
                at += v[u];
            }
        }
    }
}

// Everything at once, for a workgroup that publishes after all counting is over (the stand-alone layout kernel):
// totals, public outputs, and - when the caller has room for them - the base tables.
template <int kThreads>
__device__ void publish_layout(const PublishParams& q, const LayoutTables& t, int num_chunks, bool expert_bases, int* lds) {
    if (num_chunks <= 32 && q.E <= kThreads && q.R * t.chunks_padded <= 4 * kThreads) {
        publish_layout_in_one_trip<kThreads>(q, t, num_chunks, expert_bases, lds);
        return;
    }
    const PublishLds s = carve_publish_lds(lds, q.R, q.E);
    sum_rank_rows<kThreads>(t, q.R, s.totals);
    sum_expert_columns<kThreads>(t, q.R, q.E, num_chunks, s.totals);
    publish_ranks<kThreads>(q, s);
    __syncthreads();
    if (t.rank_bases != nullptr) write_rank_bases<kThreads>(t, q.R, s);
    publish_experts<kThreads>(q, s);
    if (t.expert_bases != nullptr && expert_bases) {
        __syncthreads();
        write_expert_bases<kThreads, false>(t, t.expert_bases, 0u, q.E, num_chunks, s);
    }
}

}  // namespace deep_ep_hip
