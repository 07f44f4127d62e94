// Internal interface between the C-ABI entry points (api.hip) and the kernel launchers.
// Parameter blocks are plain structs passed to kernels by value.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace deep_ep_hip {

// Single-launch dispatch: number of completion counters ("gates") the movers spread over, and the distance between
// two of them in 32-bit words (one cache line each).  A persistent move kernel (never part of a single launch) keeps its
// item counter in one of these lines and counts its workgroups out on `gates_finished`; every launch leaves all of them
// at zero.
constexpr int kDispatchGates = 256;
constexpr int kDispatchGateStride = 32;
constexpr int kMaxCountBlocks = 1024;

// Single-launch dispatch: words that counting and publishing workgroups hand to the movers of the same launch carry
// the launch's tag in their upper bits, so that a reader knows a word of this launch from what an earlier launch left
// at the same place and needs no separate flag (and the writer need not wait for its store before it raises one).
// The tagged tables live in the zero-initialised bookkeeping part of the workspace, which only these kernels write:
// every word there is zero, or carries the tag of a launch since the tables were last cleared.  Tags run through
// 1 .. kTagPeriod; the launch that uses the last one clears the tables.
constexpr int kTagShift = 18;
constexpr uint32_t kTagValueMask = (1u << kTagShift) - 1u;
constexpr uint32_t kTagPeriod = (1u << (32 - kTagShift)) - 1u;      // 16383
constexpr int kTaggedRankWords = 1024;       // R x chunks (padded to a multiple of 4)
constexpr int kTaggedExpertWords = 8192;     // chunks x experts (padded to a multiple of 32)
constexpr int kTaggedPosWords = 131072;      // tokens x lanes

// A position word: bits 0-8 the slot of the token inside its chunk for the lane's destination rank (master lanes
// only), bits 9-17 the position of the lane inside its chunk for its expert, kNoPosition = none; a single-launch
// dispatch puts its tag above them.
constexpr uint32_t kNoPosition = 0x1ffu;
constexpr int kExpertPositionShift = 9;

// Byte offsets of the regions carved out of the caller's workspace.
struct WorkspaceLayout {
    size_t status;         // int32: device status bits
    size_t done_counter;   // uint32: workgroups of the layout kernel that have finished
    size_t totals;         // int32[2]: total compact rows, total expanded rows (incl. padding)
    size_t generation;     // uint32: single-launch dispatches since the tagged tables were cleared (tag = generation + 1)
    size_t gates_finished; // uint32: gates whose movers have all read the tagged tables
    size_t chunk_done;     // int32[1024]: per-chunk completion flags of a single-launch dispatch (counting workgroup -> publisher)
    size_t gates;          // uint32[kDispatchGates], one per 128-byte line: movers that have read the tagged tables
    size_t tagged;         // start of the tagged tables; everything before it reads zero between launches but for
                           // status, totals and generation
    size_t tagged_rank;    // uint32[kTaggedRankWords]: rank_counts of the running single-launch dispatch, tagged
    size_t tagged_expert;  // uint32[kTaggedExpertWords]: its expert_bases, tagged
    size_t tagged_expert_counts;   // uint32[kTaggedExpertWords]: expert_counts of an expanded single-launch dispatch, tagged
    size_t tagged_pos;     // uint32[kTaggedPosWords]: its position words, tagged
    size_t tagged_end;
    size_t expert_start;   // int32[E]: first expanded row of each expert
    size_t rank_counts;    // int32[R][C padded to a multiple of 4]: per-chunk totals of the rank buckets, transposed
    size_t rank_bases;     // int32[R][C padded]: first compact row of every (rank, chunk)
    size_t expert_counts;  // int32[C][E padded to a multiple of 32]: per-chunk totals of the expert buckets
    size_t expert_bases;   // int32[C][E padded]: first expanded row of every (chunk, expert)
    size_t pos;            // uint32[Tmax*K]: position words of a dispatch in two launches
    size_t total_bytes;
};

WorkspaceLayout make_workspace_layout(int num_max_tokens, int num_topk, int num_experts, int num_ranks);

// The tables the layout pass leaves in the workspace for the move kernels.  A chunk is 256 consecutive tokens.
//   rank_counts[r][c]    rows chunk c puts into rank r's bucket (transposed: consumers prefix-sum along a row)
//   rank_bases[r][c]     first compact row of (rank r, chunk c) = rows of lower ranks + rows of earlier chunks;
//                        rank_bases[r][0] is the start of rank r's bucket
//   expert_counts[c][e]  rows chunk c puts into expert e's region (one writer per cache line: chunk c's workgroup)
//   expert_bases[c][e]   first expanded row of (chunk c, expert e) = start of the region + rows of earlier chunks
// A row is then "base of (bucket, chunk) + position inside the chunk".
struct LayoutTables {
    int32_t* rank_counts;
    int32_t* rank_bases;
    int32_t* expert_counts;
    int32_t* expert_bases;
    int chunks_padded;    // row length of the rank tables (chunks rounded up to a multiple of 4)
    int experts_padded;   // row length of the expert tables (experts rounded up to a multiple of 32)
};

// Where the public results of the layout computation go (any pointer may be NULL).
struct PublishParams {
    int R, E;
    int A;            // expert alignment
    int do_expand;
    int32_t* num_tokens_per_rank;
    int32_t* num_tokens_per_expert;
    int32_t* psum_rank;
    int32_t* psum_expert;
    int32_t* num_unaligned;
    int32_t* cumulative_stats;
    int32_t* host_counts;            // host-mapped: [R] rank counts, [E] aligned expert counts, then the status word; v as -v-1
    const int32_t* status;           // the device status word (read for host_counts)
    int32_t* expert_start;           // workspace
    int32_t* totals_out;             // workspace: total compact rows, total expanded rows
};

struct LayoutParams {
    const int64_t* topk_idx;
    const uint8_t* route_mask;       // [T, R] bool: when set, lane r of token t is "rank r, if the mask says so" (K = E = R)
    int T, K, E, R, E_l;
    int vec_idx;          // topk_idx is 16-byte aligned (set by the launcher)
    uint8_t* is_token_in_rank;       // optional
    int64_t* copied_topk_idx;        // optional
    PublishParams pub;
    int32_t* status;
    uint32_t* done_counter;
    LayoutTables tab;                // the base tables are optional (layout-only calls have no use for them)
    int expert_bases;                // 1: also tab.expert_bases (expanded layout)
    uint32_t* pos;                   // optional (layout-only calls skip the per-lane positions)
    // Single-launch dispatch (else NULL): chunk totals of the rank buckets go to tagged_rank as well, tagged like the
    // position words, with the tag *generation names when the workgroup starts.
    uint32_t* tagged_rank;
    uint32_t* tagged_expert_counts;  // expanded layout (else NULL): likewise the chunk totals of the expert buckets, for the publisher
    const uint32_t* generation;
};

hipError_t launch_layout_kernel(const LayoutParams& p, hipStream_t stream);

struct MoveParams {
    const uint8_t* x;
    const uint32_t* sf;
    int64_t sf_ts, sf_hs;
    int num_sf_packs;
    const int64_t* topk_idx;
    const uint8_t* route_mask;       // see LayoutParams
    const float* topk_weights;
    const uint32_t* pos;
    const int32_t* expert_start;
    const int32_t* cached_slot;
    int32_t* dst_buffer_slot_idx;
    const int32_t* psum_rank;
    int32_t* recv_src_metadata;
    uint8_t* recv_x;
    uint32_t* recv_sf;
    int64_t rsf_ts, rsf_hs;
    int64_t* recv_topk_idx;
    float* recv_topk_weights;
    int64_t recv_capacity, expanded_capacity;
    int T, H, K, E, R, E_l, rank_idx, M;
    float rcp_E_l;       // 1 / E_l (set by the launcher)
    int cached, do_expand;
    int payload;         // DEEP_EP_HIP_PAYLOAD_*
    int row_bytes;       // input row bytes
    int tiles;           // column tiles per token
    unsigned warm_lds_offset;   // single-launch cast: byte offset (in the dynamic LDS) of the 4 KB landing area of the
                                // cache-warming loads, 0 = none
    unsigned warm_ahead;        // ... and how many work items ahead of its own a wavefront warms
    int xcd_remap;       // give each XCD a contiguous token range
    int plain_loads;     // payload loads without the non-temporal hint
    int cast_pairs;      // forced column tile of the fused cast, 0 = choose
    int copy_vecs;       // forced column tile of the pass-through kernels, 0 = choose
    LayoutTables tab;    // written by the layout pass
    PublishParams pub;   // single-launch dispatch: what counting workgroup 0 publishes
    int32_t* status;
    // Single-launch dispatch: the first count_blocks workgroups of the grid count (one 256-token chunk each), the
    // last of them to finish publishes; the movers wait on `sync` before they read any of it.
    int fused;
    int count_blocks;
    unsigned num_movers;     // mover workgroups (set by the launcher)
    int num_cus;             // compute units of the device (set by the launcher)
    LayoutParams lay;        // what the counting workgroups need (lay.pub is unused: `pub` above is published)
    int32_t* chunk_done;     // [kMaxCountBlocks] flags of the counting workgroups for the publisher: totals and positions stored
    uint32_t* gates;         // [kDispatchGates] wrapping counters of the movers that are done reading, kDispatchGateStride words apart
    uint32_t* gates_finished;    // wrapping counter of the gates all of whose movers are done
    unsigned mover_spin_limit;   // reads a mover repeats for a word of the layout before it gives up (set from the tuning block)
    int move_workgroups_per_cu;  // forced residency of a move kernel on a finished layout, 0 = choose (tuning block)
    int warm_rounds;             // rounds ahead the first movers of a single launch warm the caches, 0 = choose, < 0 = none (tuning block)
    int persistent_movers;       // fused-cast move kernel on a finished layout as a persistent kernel with a work queue and this many mover wavefronts per CU, 0 = off (tuning block)
    uint32_t* generation;        // see WorkspaceLayout
    uint32_t* tagged;            // the tagged tables, tagged_words long: cleared by the launch that uses the last tag
    int tagged_words;
    const uint32_t* tagged_rank;
    uint32_t* tagged_expert;
    const uint32_t* tagged_expert_counts;
    // V1 (intranode) conventions
    int rank_lanes;          // routing lanes are ranks (mask routing or a cached send_head), K == R
    int slot_is_row;         // cached_slot holds rows of the receive buffer, not rank * M + slot
    int zero_nonlocal_w;     // weights of lanes routed to another rank are delivered as 0
    int32_t* send_head;      // [T, R] out: receive row of token t on rank r, or -1
    int32_t* recv_src_idx;   // [recv_capacity] out: source token of each receive row
};

hipError_t launch_dispatch_move(MoveParams p, hipStream_t stream);
// Mover workgroups launch_dispatch_move would start for p (p.T, p.H, p.row_bytes, p.payload and the tile overrides set).
int64_t dispatch_move_workgroups(const MoveParams& p);

struct PadParams {
    uint8_t* recv_x;
    uint32_t* recv_sf;
    int64_t rsf_ts, rsf_hs;
    int num_sf_packs;
    float* recv_topk_weights;
    const int32_t* psum_expert;     // start + actual count (expanded convention)
    const int32_t* num_unaligned;
    int64_t expanded_capacity;
    int E, A, out_row_bytes;
};

hipError_t launch_zero_padding(const PadParams& p, hipStream_t stream);

// V1 (intranode) handle bookkeeping computed from is_token_in_rank, and the -1 fill of unused recv_topk_idx rows.
struct IntranodePrefixParams {
    const uint8_t* mask;             // [T, R]
    int T, R, C, rank_idx;
    int32_t* rank_prefix_matrix;         // [R, R]
    int32_t* channel_prefix_matrix;      // [R, C] inclusive over channels
    int32_t* recv_channel_prefix_matrix; // [R, C] exclusive starts
};

hipError_t launch_intranode_prefix(const IntranodePrefixParams& p, hipStream_t stream);

struct FillTailParams {
    int64_t* recv_topk_idx;          // [capacity, K]
    const int32_t* total_rows;       // device: rows in use
    int64_t capacity;
    int K;
};

hipError_t launch_fill_tail(const FillTailParams& p, hipStream_t stream);

struct CombineParams {
    const uint8_t* x;
    int64_t num_x_rows;
    const float* topk_weights;
    const uint8_t* bias0;
    const uint8_t* bias1;
    const int64_t* topk_idx;
    const int32_t* slot;
    const int32_t* meta;
    int64_t num_meta_rows;
    const int32_t* psum_rank;
    uint8_t* out;
    float* out_w;
    int T, H, K, E, R, E_l, rank_idx, M;
    int do_expand, multi_red;
    int tiles;
    int32_t* status;
    // V1 (intranode) conventions: slot is send_head [T, R] holding receive rows; terms are added in ascending
    // rank order; weights [rows, Kw] are summed over the token's rows.
    int rank_mode;
    int Kw;
    int vecs;            // forced column tile, 0 = choose
};

hipError_t launch_combine_kernel(CombineParams p, hipStream_t stream);

// dst_buffer_slot_idx of a handle rebuilt from its recv_src_metadata and per-rank prefix (see combine.hip).
struct SlotMapParams {
    const int32_t* meta;         // [num_meta_rows, K + 2]
    int64_t num_meta_rows;
    const int32_t* psum_rank;    // [R] inclusive
    int32_t* slot;               // [T, K] out
    int T, K, R, rank_idx, M;
};

hipError_t launch_rebuild_slot_map(const SlotMapParams& p, hipStream_t stream);

struct CastParams {
    const uint8_t* x;
    uint8_t* out;
    float* scales;
    int T, H;
};

hipError_t launch_cast_kernel(const CastParams& p, hipStream_t stream);

struct LLDispatchParams {
    int use_fp8;
    int round_scale, use_ue8m0;
    int S, src_rank_begin, src_token_stride;
    const int32_t* num_tokens_per_src;
    int H, K, E, expert_begin, E_l, R, M;
    const uint8_t* x;
    const int64_t* topk_idx;
    uint8_t* packed_x;
    float* packed_scales;
    int32_t* packed_count;
    int32_t* packed_src_info;
    int64_t* packed_layout_range;
    int32_t* cumulative_stats;
    int32_t* lane_slot;      // optional [S*stride, K]: packed row (le * rows + slot) of every (token, lane), -1 none
    // workspace
    int32_t* status;
    uint32_t* done_counter;
    int32_t* chunk_counts;   // [C][E_l]
    int32_t* chunk_base;     // [C][E_l]
    int32_t* pos_expert;     // [S*stride*K]
    // launch-shape overrides, 0 = choose
    int pairs, threads, two_kernels;
};

// Compute units of the current device (asked once per device).
int compute_units();

hipError_t launch_ll_dispatch(const LLDispatchParams& p, hipStream_t stream);

struct LLCombineParams {
    int S, src_rank_begin, src_token_stride;
    const int32_t* num_tokens_per_src;
    int H, K, E, expert_begin, E_l, R, M;
    const uint8_t* x;
    const int64_t* topk_idx;
    const float* topk_weights;
    const int32_t* src_info;
    const int64_t* layout_range;
    const int32_t* lane_slot;    // optional: what the dispatch recorded; replaces the search through src_info
    uint8_t* out;
    int32_t* status;
    int vecs;                    // forced column tile, 0 = choose
    int use_logfmt;              // gathered rows pass through the LogFMT-10 codec
};

hipError_t launch_ll_combine(const LLCombineParams& p, hipStream_t stream);

}  // namespace deep_ep_hip
