/*
 * C ABI of the MI355X (gfx950) MoE token-routing library: dispatch layout, dispatch
 * (BF16 / FP8 pass-through / fused BF16->FP8 e4m3 cast), combine, and the low-latency
 * packed per-expert layout.
 *
 * Conventions
 *   - Every entry point takes a pointer to a plain-old-data argument block and the HIP stream
 *     (hipStream_t passed as void*; NULL = the default stream).  All pointers inside an
 *     argument block are device pointers unless a field says otherwise.  Nothing is allocated
 *     or freed by the library; the caller owns every buffer, including the workspace.
 *   - Return value: 0 on success, a negative DEEP_EP_HIP_ERR_* for rejected arguments, or a
 *     positive hipError_t if a launch failed.  deep_ep_hip_last_error() returns the message of
 *     the last failure on the calling thread.
 *   - Launches are asynchronous on the given stream.  Calls that share one workspace must be
 *     ordered on one stream (the workspace is not re-entrant), mirroring the reference's
 *     "one workspace per buffer" rule (csrc/elastic/buffer.hpp:118-121).
 *   - num_ranks is a logical bucketing parameter: destination rank d owns experts
 *     [d*E/R, (d+1)*E/R).  All destination buckets live in the caller's own HBM.
 *
 * Reference interfaces replaced (paths relative to the reference tree):
 *   deep_ep_hip_launch_layout       csrc/kernels/legacy/layout.cu:124-150 (get_dispatch_layout)
 *   deep_ep_hip_launch_dispatch     csrc/kernels/elastic/dispatch.hpp:141,293 (launch_dispatch +
 *                                   launch_dispatch_copy_epilogue), ABI style of
 *                                   csrc/backends/ascend/elastic/kernels.hpp:274-288
 *   deep_ep_hip_launch_combine      csrc/kernels/elastic/combine.hpp:114,248 (launch_combine +
 *                                   launch_combine_reduce_epilogue)
 *   deep_ep_hip_launch_intranode_dispatch  csrc/kernels/legacy/intranode.cu:20-175 (notify_dispatch),
 *                                   :205-612 (dispatch), called from csrc/legacy/buffer.hpp:417-717
 *   deep_ep_hip_launch_intranode_combine   csrc/kernels/legacy/intranode.cu:700-1095 (combine), called from
 *                                   csrc/legacy/buffer.hpp:719-860
 *   deep_ep_hip_launch_ll_dispatch  csrc/kernels/legacy/internode_ll.cu:464-554
 *   deep_ep_hip_launch_ll_combine   csrc/kernels/legacy/internode_ll.cu:1140-1238 (LogFMT-10: :556-712, :1048-1100)
 *   deep_ep_hip_launch_cast_fp8     deep_ep/utils/math.py:30-39 (per_token_cast_to_fp8)
 */
#ifndef DEEP_EP_HIP_H_
#define DEEP_EP_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DEEP_EP_HIP_ABI_VERSION 4

#define DEEP_EP_HIP_OK 0
#define DEEP_EP_HIP_ERR_INVALID_ARGUMENT (-1)
#define DEEP_EP_HIP_ERR_WORKSPACE_TOO_SMALL (-2)
#define DEEP_EP_HIP_ERR_UNSUPPORTED (-3)

/* Limits checked by every entry point. */
#define DEEP_EP_HIP_MAX_TOPK 32
#define DEEP_EP_HIP_MAX_EXPERTS 1024
#define DEEP_EP_HIP_MAX_RANKS 512

/* Bits of the device-side status word (first int32 of the workspace, see
 * deep_ep_hip_workspace_status_offset).  Kernels OR bits in; they never trap. */
#define DEEP_EP_HIP_STATUS_EXPERT_OUT_OF_RANGE 1  /* topk_idx >= num_experts (entry ignored) */
#define DEEP_EP_HIP_STATUS_DUPLICATE_EXPERT 2     /* one token names an expert twice */
#define DEEP_EP_HIP_STATUS_ROW_OVERFLOW 4         /* a row fell outside the caller's capacity (row dropped) */
#define DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT 8       /* a single-launch dispatch gave up waiting for its own counting
                                                     workgroups (outputs of that call are invalid) */

int deep_ep_hip_abi_version(void);
const char* deep_ep_hip_last_error(void);

/* Launch-shape knobs, last member of every argument block.  All zero = the library's own choice (what the
 * measurements behind it say is best); nothing here changes results.  The library reads no environment
 * variables. */
typedef struct {
    int32_t dispatch_launches; /* dispatch with both phases in one call: 0 = a single launch (counting workgroups at
                                  the front of the move kernel) where the shape allows it (num_topk <= 8, num_ranks +
                                  num_experts <= 512, num_ranks * ceil(num_tokens / 256) <= 1024, num_tokens * num_topk
                                  <= 131072; with do_expand also ceil(num_tokens / 256) * num_experts <= 8192 and
                                  num_tokens * num_topk + num_experts * expert_alignment < 2^18) and it pays (at most
                                  16384 mover workgroups; with do_expand less than 64 MB of input); 1 = a single launch
                                  wherever the shape allows it; 2 = always layout kernel + move kernel */
    int32_t cast_pairs;        /* fused FP8 cast: 1024-channel segments per wavefront (1, 2, 4, 7, 8; above 2: two launches) */
    int32_t copy_vecs;         /* pass-through payloads: KB of row per wavefront (1, 2, 4, 7, 8) */
    int32_t plain_loads;       /* 1: payload loads allocate in the caches (for inputs known to be cache resident) */
    int32_t xcd_remap;         /* 1: consecutive workgroups of a dispatch share an XCD */
    int32_t combine_vecs;      /* combine: KB of row per wavefront (1, 2, 4) */
    int32_t ll_pairs;          /* low-latency dispatch: 1024-channel segments per wavefront (1, 2, 4) */
    int32_t ll_threads;        /* low-latency dispatch, single-kernel path: workgroup size (256, 512, 1024) */
    int32_t ll_two_kernels;    /* 1: low-latency dispatch always as count kernel + move kernel */
    int32_t ll_combine_vecs;   /* low-latency combine: KB of row per wavefront (1, 2, 4, 7) */
    int32_t mover_spin_limit;  /* single-launch dispatch: how often a mover workgroup repeats a read of the layout its own
                                  launch is still computing before it gives up, stores nothing and sets
                                  DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT (0 = 2^22, seconds; 1 makes the first workgroups of a
                                  launch give up at once: for tests of that path - every kernel still runs to its end and
                                  the workspace stays consistent) */
    int32_t move_workgroups_per_cu;  /* dispatch move kernel launched on a finished layout: workgroups a CU holds at a
                                        time (2..7; 8 and more = as many as fit; 0 = six / five for the compact / expanded
                                        layout of a large fused-cast call, no limit otherwise) */
    int32_t warm_rounds;       /* single-launch dispatch: the movers that are resident at launch also
                                  load, into the caches only, the tiles of the work items this many rounds of resident
                                  workgroups ahead of their own (0 = 2, or 1 in launches of one and a half to two rounds;
                                  negative = none) */
    int32_t persistent_movers; /* fused-cast dispatch, compact layout: > 0 = the move phase as a persistent kernel with a
                                  work queue - one resident workgroup per compute unit with this many mover wavefronts (4, 8
                                  or 15 are built; other values take the next larger) that draw their items from a counter and
                                  request the next item's loads before the current item's stores; implies layout kernel +
                                  move kernel.  Calls it does not cover (expanded layout, cached handle, mask routing) run
                                  as if it were 0.  A measured alternative (slower on MI355X), not a default */
    int32_t reserved[2];
} deep_ep_hip_tuning;

/* Bytes of workspace needed for dispatches of up to num_max_tokens tokens.  The workspace must
 * be zero-filled once before its first use; the kernels leave it ready for the next call. */
size_t deep_ep_hip_workspace_bytes(int num_max_tokens, int num_topk, int num_experts, int num_ranks);
/* Byte offset, inside the workspace, of the int32 status word. */
size_t deep_ep_hip_workspace_status_offset(void);
/* Leading bytes of the workspace that hold the status word and the launch bookkeeping of the kernels: counters and
 * flags they expect to find zero at the start of a launch (and leave zero at its end), and the tables through which the
 * workgroups of a single-launch dispatch hand each other the layout, which must never hold anything but zeros or what
 * those kernels wrote.  After DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT, zero these bytes before the workspace is used again
 * (deep_ep_hip_read_status with clear != 0 does). */
size_t deep_ep_hip_workspace_control_bytes(void);
/* The first part of those bytes: counters and flags that read zero whenever no launch is running, but for the status
 * word (offset 0), the two row totals a dispatch leaves for the kernels that follow it (offsets 8 and 12) and the
 * launch generation (offset 128).  The rest of the control bytes are the tables through which the workgroups of a
 * single-launch dispatch hand each other the layout; only the kernels write there.  (A size to look at, not to zero:
 * the generation and those tables belong together, so zero all of the control bytes or none.) */
size_t deep_ep_hip_workspace_counter_bytes(void);
/* A status read that does not synchronise the device, for loops that run without host waits (graph replays, serving
 * loops).  Enqueues on `stream` one small kernel that copies the status word of `workspace` (NULL: the built-in
 * workspace deep_ep_hip_launch_dispatch_static uses on the current device) to *status_out.  status_out must be memory
 * the GPU can write: pinned host memory from hipHostMalloc, which the host may read once an event recorded on `stream`
 * after this call has completed, or device memory.  Kernels only ever OR bits into the status word, so one read after N
 * launches reports what any of them flagged (DEEP_EP_HIP_STATUS_*).  With clear != 0 the read also puts the word back
 * to zero, and after DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT zeroes the launch bookkeeping behind it, so that the workspace is
 * ready for the next launch: *status_out then holds what was flagged since the previous clearing read.  Nothing is
 * allocated; the launch is an ordinary kernel node and may be captured into a HIP graph, every replay refreshing
 * *status_out. */
int deep_ep_hip_read_status(void* workspace, int32_t* status_out, int clear, void* stream);

/* ------------------------------------------------------------------------------------------
 * Dispatch layout (V1 `Buffer.get_dispatch_layout`): counts only.
 * ---------------------------------------------------------------------------------------- */
typedef struct {
    const int64_t* topk_idx;        /* [num_tokens, num_topk], -1 = no selection */
    int32_t num_tokens, num_topk, num_experts, num_ranks;
    int32_t* num_tokens_per_rank;   /* [num_ranks] out */
    int32_t* num_tokens_per_expert; /* [num_experts] out */
    uint8_t* is_token_in_rank;      /* [num_tokens, num_ranks] out (bool), may be NULL */
    void* workspace;
    uint64_t workspace_bytes;
} deep_ep_hip_layout_args;

int deep_ep_hip_launch_layout(const deep_ep_hip_layout_args* args, void* stream);

/* ------------------------------------------------------------------------------------------
 * Dispatch (V2 `ElasticBuffer.dispatch`), one logical source rank.
 *
 * phases: bit 0 = count/scan (fills the handle tensors psum_*, num_unaligned, host_counts and
 * the per-(token,lane) positions kept in the workspace); bit 1 = move payload and metadata.
 * A caller that needs exact output sizes runs phase 1, waits for host_counts, allocates, then
 * runs phase 2; otherwise both phases go in one call.  With cached != 0 only phase 2 is legal
 * and dst_buffer_slot_idx / psum_rank / recv_src_metadata are inputs.
 * ---------------------------------------------------------------------------------------- */
#define DEEP_EP_HIP_PHASE_LAYOUT 1
#define DEEP_EP_HIP_PHASE_MOVE 2

#define DEEP_EP_HIP_PAYLOAD_BF16 0      /* x bf16 -> recv_x bf16 */
#define DEEP_EP_HIP_PAYLOAD_FP8 1       /* x e4m3 + sf -> recv_x e4m3 + recv_sf (pass-through) */
#define DEEP_EP_HIP_PAYLOAD_CAST_FP8 2  /* x bf16 -> recv_x e4m3 + recv_sf fp32 (fused cast) */

typedef struct {
    int32_t phases;
    int32_t payload;                /* DEEP_EP_HIP_PAYLOAD_* */
    int32_t cached;                 /* reuse handle tensors instead of recomputing the layout */
    int32_t do_expand;              /* expert-major layout, one row per (token, lane) */
    int32_t do_zero_padding;        /* zero alignment padding rows (expanded layout only) */
    int32_t num_tokens, hidden, num_topk, num_experts, num_ranks;
    int32_t rank_idx;               /* logical source rank of these tokens */
    int32_t num_max_tokens_per_rank;
    int32_t expert_alignment;

    /* inputs */
    const void* x;                  /* [num_tokens, hidden] bf16 or e4m3, contiguous */
    const void* sf;                 /* payload FP8: [num_tokens, num_sf_packs] 4-byte packs */
    int64_t sf_token_stride, sf_hidden_stride;   /* in 4-byte elements */
    int32_t num_sf_packs;           /* payload FP8: packs per token; CAST_FP8: must be ceil(hidden/128) */
    const int64_t* topk_idx;        /* [num_tokens, num_topk] */
    const float* topk_weights;      /* [num_tokens, num_topk] or NULL */

    /* handle tensors: outputs of phase 1 (inputs when cached) */
    int64_t* copied_topk_idx;       /* [num_tokens, num_topk] or NULL */
    int32_t* psum_num_recv_tokens_per_rank;     /* [num_ranks] inclusive */
    int32_t* psum_num_recv_tokens_per_expert;   /* [num_experts] */
    int32_t* num_unaligned_recv_tokens_per_expert; /* [num_experts] */
    int32_t* cumulative_local_expert_recv_stats;   /* [num_experts] += actual counts, or NULL */
    int32_t* host_counts;           /* NULL, or host memory the GPU can write (hipHostMalloc), [num_ranks + num_experts + 1],
                                       zeroed by the caller before the call: per-rank counts, aligned per-expert counts,
                                       then the status word as the layout phase left it, each value v published as
                                       -v-1 (an entry is there once it reads negative: a host that polls needs no
                                       device synchronisation to size its outputs) */
    int32_t* dst_buffer_slot_idx;   /* [num_tokens, num_topk]: written by phase 2 (input when cached) */
    int32_t* recv_src_metadata;     /* [recv_capacity, num_topk + 2]: written by phase 2 (input when cached) */

    /* outputs of phase 2 */
    void* recv_x;                   /* [recv_capacity or expanded_capacity, hidden] */
    void* recv_sf;                  /* 4-byte packs, strides below; NULL for BF16 */
    int64_t recv_sf_token_stride, recv_sf_hidden_stride;
    int64_t* recv_topk_idx;         /* [recv_capacity, num_topk], compact layout only */
    float* recv_topk_weights;       /* [recv_capacity, num_topk] or [expanded_capacity]; NULL if no weights */
    int64_t recv_capacity;          /* rows the compact-indexed outputs can hold */
    int64_t expanded_capacity;      /* rows the expanded outputs can hold (do_expand) */

    void* workspace;
    uint64_t workspace_bytes;
    deep_ep_hip_tuning tuning;
} deep_ep_hip_dispatch_args;

int deep_ep_hip_launch_dispatch(const deep_ep_hip_dispatch_args* args, void* stream);

/* How many kernels deep_ep_hip_launch_dispatch would launch for the layout and move phases of these arguments (shape,
 * phases, payload, do_expand, expert_alignment and tuning are read; no pointer is dereferenced, nothing is launched): 1
 * where layout and move share a launch, else one per requested phase; 0 for a move of no tokens.  The zero-padding
 * kernel of an expanded dispatch is not counted.  Negative: an error code.  No counterpart in the reference; for callers
 * that size graphs or want to know which path a shape takes. */
int deep_ep_hip_dispatch_kernel_launches(const deep_ep_hip_dispatch_args* args);

/* The same dispatch for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  args->workspace and
 * args->workspace_bytes are ignored: the workspace is a device-resident array built into the library,
 * DEEP_EP_HIP_STATIC_WORKSPACE_BYTES long, of which every GPU the library runs on holds one copy until the process
 * ends.  Shapes with deep_ep_hip_workspace_bytes(num_tokens, num_topk, num_experts, num_ranks) beyond that are
 * rejected with DEEP_EP_HIP_ERR_WORKSPACE_TOO_SMALL.  The call allocates and frees nothing; the caller still passes
 * every input and output.  The device the stream belongs to must be current.  All calls on one GPU share that GPU's
 * array: calls that overlap on one GPU (two streams, two threads) race, and the two phases of a split call must
 * both come through this entry point.  Status bits raised by these calls are kept in the array's own status word. */
#define DEEP_EP_HIP_STATIC_WORKSPACE_BYTES (1u << 20)
int deep_ep_hip_launch_dispatch_static(const deep_ep_hip_dispatch_args* args, void* stream);

/* ------------------------------------------------------------------------------------------
 * Combine (V2 `ElasticBuffer.combine`): per origin token, fp32 sum of bias_0, bias_1 and the
 * rows that came back, in ascending master-lane order, one round-to-nearest-even BF16 store.
 * ---------------------------------------------------------------------------------------- */
typedef struct {
    int32_t do_expand;
    int32_t allow_multiple_reduction;   /* expanded layout: first reduce each rank's rows to bf16 */
    int32_t num_tokens, hidden, num_topk, num_experts, num_ranks;
    int32_t rank_idx, num_max_tokens_per_rank;
    const void* x;                      /* bf16 [num_x_rows, hidden] */
    int64_t num_x_rows;
    const float* topk_weights;          /* [num_recv, num_topk] or [num_expanded] or NULL */
    const void* bias_0;                 /* bf16 [num_tokens, hidden] or NULL */
    const void* bias_1;
    const int64_t* topk_idx;            /* handle: [num_tokens, num_topk] */
    const int32_t* dst_buffer_slot_idx; /* handle: [num_tokens, num_topk], or NULL: the call first rebuilds the map from
                                           recv_src_metadata[:, 0:2] and psum_num_recv_tokens_per_rank (two small
                                           launches) into the workspace, which must then hold
                                           deep_ep_hip_combine_workspace_bytes() bytes */
    const int32_t* recv_src_metadata;   /* handle: [num_recv_rows, num_topk + 2] (expanded layout) */
    int64_t num_recv_rows;              /* rows of recv_src_metadata */
    const int32_t* psum_num_recv_tokens_per_rank; /* handle: [num_ranks] */
    void* combined_x;                   /* bf16 [num_tokens, hidden] out */
    float* combined_topk_weights;       /* [num_tokens, num_topk] out or NULL */
    void* workspace;
    uint64_t workspace_bytes;
    deep_ep_hip_tuning tuning;
} deep_ep_hip_combine_args;

int deep_ep_hip_launch_combine(const deep_ep_hip_combine_args* args, void* stream);
/* Workspace a combine needs when it has to rebuild dst_buffer_slot_idx: the dispatch workspace of the same shape
 * (deep_ep_hip_workspace_bytes, left untouched, so that dispatch and combine can share one allocation) followed by the
 * rebuilt map.  A combine that is given dst_buffer_slot_idx needs 256 bytes (the status word). */
size_t deep_ep_hip_combine_workspace_bytes(int num_tokens, int num_topk, int num_experts, int num_ranks);

/* ------------------------------------------------------------------------------------------
 * V1 `Buffer.dispatch` / `Buffer.combine` inside one scale-up domain (the reference's "intranode" pair),
 * one logical source rank per call.
 *
 * Routing comes from topk_idx when it is given (then recv_topk_idx / recv_topk_weights are produced:
 * local expert ids or -1, weights of lanes owned by another rank delivered as 0), otherwise from
 * is_token_in_rank alone.  Receive rows are the concatenation over destination ranks d of the rows d gets
 * from this source, in token order.  Handle tensors with the reference's meaning: rank_prefix_matrix[i][d] =
 * rows rank d holds from source ranks <= i (only rank_idx sends here), channel_prefix_matrix[d][c] =
 * tokens of channels <= c sent to d (channel c = tokens [c*ceil(T/C), (c+1)*ceil(T/C))),
 * recv_channel_prefix_matrix[d][c] = the same, exclusive.  send_head[t][d] is the receive row of token t on
 * rank d, or -1 (the reference stores a queue position there; the field is opaque to callers and is what
 * cached dispatch and combine consume).
 * Limits: num_ranks <= 64; everything else as for deep_ep_hip_launch_dispatch.
 * ---------------------------------------------------------------------------------------- */
typedef struct {
    int32_t phases;                 /* DEEP_EP_HIP_PHASE_*; cached: MOVE only */
    int32_t payload;                /* DEEP_EP_HIP_PAYLOAD_* */
    int32_t cached;                 /* send_head is an input; topk_idx / is_token_in_rank are not read */
    int32_t num_tokens, hidden;
    int32_t num_topk;               /* 0 = route by is_token_in_rank alone (no top-k tensors) */
    int32_t num_experts;            /* 0 with num_topk == 0 */
    int32_t num_ranks, rank_idx;
    int32_t num_channels;           /* columns of the channel matrices (reference: config.num_sms / 2) */
    int32_t expert_alignment;
    int32_t fill_unused_topk_idx;   /* 1: rows of recv_topk_idx at and beyond the received count are set to -1
                                       (`num_worst_tokens` mode) */

    const void* x;                  /* [num_tokens, hidden] bf16 or e4m3 */
    const void* x_scales;           /* payload FP8: [num_tokens, num_scales] 4-byte elements */
    int64_t scale_token_stride, scale_hidden_stride;
    int32_t num_scales;
    const int64_t* topk_idx;        /* [num_tokens, num_topk] or NULL */
    const float* topk_weights;      /* [num_tokens, num_topk] or NULL (given iff topk_idx is) */
    const uint8_t* is_token_in_rank; /* [num_tokens, num_ranks] bool */

    /* handle and counts */
    int32_t* rank_prefix_matrix;            /* [num_ranks, num_ranks] out (phase 1), may be NULL */
    int32_t* channel_prefix_matrix;         /* [num_ranks, num_channels] out (phase 1), may be NULL */
    int32_t* recv_channel_prefix_matrix;    /* [num_ranks, num_channels] out (phase 1), may be NULL */
    int32_t* psum_num_recv_tokens_per_rank; /* [num_ranks] inclusive, out of phase 1, read by phase 2 */
    int32_t* num_recv_tokens_per_expert;    /* [num_experts] counts before alignment, out of phase 1, or NULL */
    int32_t* host_counts;                   /* host memory [num_ranks + max(num_experts, num_ranks) + 1] or NULL (see dispatch;
                                               without top-k tensors the "experts" are the ranks) */
    int32_t* send_head;                     /* [num_tokens, num_ranks]: out of phase 2 (input when cached) */
    int32_t* recv_src_idx;                  /* [recv_capacity] out of phase 2, or NULL */

    void* recv_x;                   /* [recv_capacity, hidden] */
    void* recv_x_scales;            /* [recv_capacity, num_scales], strides below */
    int64_t recv_scale_token_stride, recv_scale_hidden_stride;
    int64_t* recv_topk_idx;         /* [recv_capacity, num_topk] or NULL */
    float* recv_topk_weights;       /* [recv_capacity, num_topk] or NULL */
    int64_t recv_capacity;

    void* workspace;                /* deep_ep_hip_workspace_bytes(num_tokens, max(num_topk, num_ranks),
                                       max(num_experts, num_ranks), num_ranks) bytes */
    uint64_t workspace_bytes;
    deep_ep_hip_tuning tuning;
} deep_ep_hip_intranode_dispatch_args;

int deep_ep_hip_launch_intranode_dispatch(const deep_ep_hip_intranode_dispatch_args* args, void* stream);

/* combined_x[t] = bf16( bias_0[t] + bias_1[t] + sum over ranks d ascending with send_head[t][d] >= 0 of
 * x[send_head[t][d]] ) in fp32; combined_topk_weights[t] = sum of the same rows of topk_weights. */
typedef struct {
    int32_t num_tokens, hidden, num_ranks;
    int32_t num_topk;               /* columns of topk_weights, 0 if none */
    const void* x;                  /* bf16 [num_x_rows, hidden] */
    int64_t num_x_rows;
    const float* topk_weights;      /* [num_x_rows, num_topk] or NULL */
    const void* bias_0;             /* bf16 [num_tokens, hidden] or NULL */
    const void* bias_1;
    const int32_t* send_head;       /* handle: [num_tokens, num_ranks] */
    void* combined_x;               /* bf16 [num_tokens, hidden] out */
    float* combined_topk_weights;   /* [num_tokens, num_topk] out or NULL */
    void* workspace;                /* >= 256 bytes (status word) */
    uint64_t workspace_bytes;
    deep_ep_hip_tuning tuning;
} deep_ep_hip_intranode_combine_args;

int deep_ep_hip_launch_intranode_combine(const deep_ep_hip_intranode_combine_args* args, void* stream);

/* ------------------------------------------------------------------------------------------
 * Low-latency packed layout (V1 `Buffer.low_latency_dispatch/combine`) for one logical
 * destination rank holding experts [expert_begin, expert_begin + num_local_experts).
 * Source ranks src_rank_begin .. src_rank_begin + num_src_ranks - 1 send in one launch; the
 * tokens of the i-th source are rows [i*src_token_stride, i*src_token_stride + n_i) of x.
 * Fill order inside an expert buffer: source rank ascending, then token ascending.
 * ---------------------------------------------------------------------------------------- */
typedef struct {
    int32_t use_fp8;                    /* 1: e4m3 payload + scales; 0: bf16 payload */
    int32_t round_scale;                /* fp8: scales rounded up to powers of two */
    int32_t use_ue8m0;                  /* fp8 + round_scale: scales stored as exponent bytes, 4 per int32 pack;
                                           needs hidden % 512 == 0 */
    int32_t num_src_ranks, src_rank_begin;
    int32_t src_token_stride;           /* rows of x reserved per source rank */
    const int32_t* num_tokens_per_src;  /* [num_src_ranks] device, or NULL = src_token_stride each */
    int32_t hidden, num_topk, num_experts;
    int32_t expert_begin, num_local_experts;
    int32_t num_ranks;                  /* columns of packed_recv_layout_range */
    int32_t num_max_dispatch_tokens_per_rank;   /* slots per (expert, source rank) budget; rows per
                                                   expert buffer = num_ranks * this */
    const void* x;                      /* bf16 [num_src_ranks * src_token_stride, hidden] */
    const int64_t* topk_idx;            /* [num_src_ranks * src_token_stride, num_topk] */
    void* packed_recv_x;                /* [num_local_experts, rows, hidden] */
    float* packed_recv_x_scales;        /* fp8: element (e, row, g) at e*rows*G + g*rows + row (G = hidden/128);
                                           use_ue8m0: byte (e, row, g) at ((e*G/4 + g/4)*rows + row)*4 + g%4 */
    int32_t* packed_recv_count;         /* [num_local_experts] out */
    int32_t* packed_recv_src_info;      /* [num_local_experts, rows] out */
    int64_t* packed_recv_layout_range;  /* [num_local_experts, num_ranks] out: (begin<<32)|count; columns of ranks
                                           that do not send in this call are written as 0 */
    int32_t* cumulative_local_expert_recv_stats; /* [num_local_experts] += counts, or NULL */
    int32_t* lane_rows;                 /* optional out [num_src_ranks * src_token_stride, num_topk]: e * rows + slot of
                                           the packed row each (token, lane) went to, -1 if none.  Not part of the
                                           reference's handle; passing it to the combine saves the search through
                                           packed_recv_src_info */
    void* workspace;
    uint64_t workspace_bytes;
    deep_ep_hip_tuning tuning;
} deep_ep_hip_ll_dispatch_args;

/* Bytes of (zero-initialised, reusable) workspace a low-latency dispatch of this shape needs.  A memory of its own: it
 * must not overlap the workspace of deep_ep_hip_launch_dispatch (see deep_ep_hip_workspace_control_bytes). */
size_t deep_ep_hip_ll_workspace_bytes(int num_src_ranks, int src_token_stride, int num_topk, int num_local_experts);
int deep_ep_hip_launch_ll_dispatch(const deep_ep_hip_ll_dispatch_args* args, void* stream);

typedef struct {
    int32_t num_src_ranks, src_rank_begin;  /* source ranks whose tokens are rebuilt in this launch */
    int32_t src_token_stride;           /* rows of topk_idx / topk_weights / combined_x per source rank */
    int32_t use_logfmt;                 /* 1: every gathered row passes through the LogFMT-10 codec before it is
                                           accumulated (what the reference's rows go through on the wire): per chunk
                                           of 1024 channels (512 if hidden % 1024 != 0), if every 128-channel group has
                                           amax < 1 and amin < amax, magnitudes become 9-bit codes on a logarithmic
                                           grid between the group's amin (at most 2^32 below amax) and amax, and are
                                           decoded again; other chunks stay BF16.  Needs hidden % 512 == 0. */
    const int32_t* num_tokens_per_src;  /* [num_src_ranks] device, or NULL = src_token_stride each */
    int32_t hidden, num_topk, num_experts;
    int32_t expert_begin, num_local_experts, num_ranks;
    int32_t num_max_dispatch_tokens_per_rank;
    const void* x;                      /* bf16 [num_local_experts, rows, hidden] */
    const int64_t* topk_idx;            /* [num_src_ranks * src_token_stride, num_topk] */
    const float* topk_weights;          /* [num_src_ranks * src_token_stride, num_topk] */
    const int32_t* packed_recv_src_info;
    const int64_t* packed_recv_layout_range;
    const int32_t* lane_rows;           /* optional: lane_rows of the dispatch that made the handle */
    void* combined_x;                   /* bf16 [num_src_ranks * src_token_stride, hidden] out; rows past a
                                           source's token count are left untouched */
    void* workspace;
    uint64_t workspace_bytes;
    deep_ep_hip_tuning tuning;
} deep_ep_hip_ll_combine_args;

int deep_ep_hip_launch_ll_combine(const deep_ep_hip_ll_combine_args* args, void* stream);

/* ------------------------------------------------------------------------------------------
 * Stand-alone per-token 1x128 FP8 cast: bf16 [num_tokens, hidden] -> e4m3 + fp32 scales
 * (row-major [num_tokens, ceil(hidden/128)]).
 * ---------------------------------------------------------------------------------------- */
typedef struct {
    const void* x;
    void* out;
    float* scales;
    int32_t num_tokens, hidden;
} deep_ep_hip_cast_args;

int deep_ep_hip_launch_cast_fp8(const deep_ep_hip_cast_args* args, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DEEP_EP_HIP_H_ */
