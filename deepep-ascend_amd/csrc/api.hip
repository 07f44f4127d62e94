// extern "C" entry points: argument validation, workspace carving, kernel sequencing.
// The declarations (and the reference interfaces they stand in for) are in include/deep_ep_hip.h.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "../../include/deep_ep_hip.h"
#include "device_utils.h"
#include "kernels.h"

namespace deep_ep_hip {

namespace {

thread_local char g_last_error[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t err, const char* what) {
    snprintf(g_last_error, sizeof(g_last_error), "%s: %s", what, hipGetErrorString(err));
    return int(err) > 0 ? int(err) : DEEP_EP_HIP_ERR_INVALID_ARGUMENT;
}

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

#define REQUIRE(cond, ...)                                                     \
    do {                                                                       \
        if (!(cond)) return fail(DEEP_EP_HIP_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
    } while (0)

int check_routing_shape(int T, int K, int E, int R) {
    REQUIRE(T >= 0, "num_tokens must be >= 0 (got %d)", T);
    REQUIRE(K >= 1 && K <= DEEP_EP_HIP_MAX_TOPK, "num_topk must be in [1, %d] (got %d)", DEEP_EP_HIP_MAX_TOPK, K);
    REQUIRE(R >= 1 && R <= DEEP_EP_HIP_MAX_RANKS, "num_ranks must be in [1, %d] (got %d)", DEEP_EP_HIP_MAX_RANKS, R);
    REQUIRE(E >= 1 && E <= DEEP_EP_HIP_MAX_EXPERTS, "num_experts must be in [1, %d] (got %d)", DEEP_EP_HIP_MAX_EXPERTS, E);
    REQUIRE(E % R == 0, "num_experts (%d) must be divisible by num_ranks (%d)", E, R);
    return DEEP_EP_HIP_OK;
}

// How a dispatch call is cut into launches.
struct LaunchPlan {
    int chunks, chunks_padded;
    bool fused;       // one launch: counting workgroups at the front of the move kernel
};

// Past this many mover workgroups the per-workgroup cost of the single-launch protocol (a look at the layout, one
// atomic, two workgroup barriers) outweighs the launch it saves: 28 672 workgroups of 8192 BF16 rows of 14 KB take
// 180 us in one launch against 140 us in two; 8 192 workgroups of the same rows cast to FP8 take 92 us against 97 us.
constexpr int64_t kMaxFusedMovers = 16384;

LaunchPlan plan_launches(int T, int K, int E, int R, bool do_layout, bool do_move, bool do_expand, int alignment, int payload, int H,
                         int row_bytes, const deep_ep_hip_tuning& tuning) {
    LaunchPlan q{};
    q.chunks = T > 0 ? (T + kLayoutChunk - 1) / kLayoutChunk : 1;
    q.chunks_padded = (q.chunks + 3) / 4 * 4;
    q.fused = do_layout && do_move && T > 0 && K <= 8 && (R + E) <= 512 && R * q.chunks_padded <= kTaggedRankWords &&
              int64_t(T) * K <= kTaggedPosWords && tuning.dispatch_launches != 2 &&
              !(tuning.persistent_movers > 0 && payload == DEEP_EP_HIP_PAYLOAD_CAST_FP8);      // the persistent move runs on a finished layout
    if (q.fused && do_expand) {
        // the tagged expert bases: the table must fit, and a row number must fit under the tag
        const int64_t experts_padded = (int64_t(E) + 31) / 32 * 32;
        q.fused = q.chunks * experts_padded <= kTaggedExpertWords &&
                  int64_t(T) * K + int64_t(E) * alignment <= int64_t(kTagValueMask);
    }
    // The single-launch cast kernels exist for tiles of one and two segments (wider ones would spill registers under
    // the occupancy the counting code is held to): a forced wider tile takes two launches.
    if (payload == DEEP_EP_HIP_PAYLOAD_CAST_FP8 && tuning.cast_pairs > 2) q.fused = false;
    // The expanded layout of a large call (64 MB of input and more) is faster in two launches: every mover of a single
    // launch waits for the publisher's expert bases, a second hand-off, while a move kernel of its own streams from its
    // first microsecond (8192 x 7168: 123-128 us against 130-134 us; from 4096 tokens down the single launch is ahead,
    // 66.5 against 72.8 us).
    if (q.fused && do_expand && tuning.dispatch_launches != 1 && int64_t(T) * row_bytes >= (int64_t(64) << 20)) q.fused = false;
    if (q.fused && tuning.dispatch_launches != 1) {
        MoveParams probe{};
        probe.T = T; probe.H = H; probe.row_bytes = row_bytes; probe.payload = payload; probe.do_expand = do_expand ? 1 : 0;
        probe.cast_pairs = tuning.cast_pairs; probe.copy_vecs = tuning.copy_vecs;
        q.fused = dispatch_move_workgroups(probe) <= kMaxFusedMovers;
    }
    return q;
}

LayoutTables carve_tables(uint8_t* ws, const WorkspaceLayout& w, int num_tokens, int num_experts) {
    LayoutTables t{};
    t.rank_counts = reinterpret_cast<int32_t*>(ws + w.rank_counts);
    t.rank_bases = reinterpret_cast<int32_t*>(ws + w.rank_bases);
    t.expert_counts = reinterpret_cast<int32_t*>(ws + w.expert_counts);
    t.expert_bases = reinterpret_cast<int32_t*>(ws + w.expert_bases);
    const int chunks = num_tokens > 0 ? (num_tokens + kLayoutChunk - 1) / kLayoutChunk : 1;
    t.chunks_padded = (chunks + 3) / 4 * 4;
    t.experts_padded = (num_experts + 31) / 32 * 32;
    return t;
}

void fill_fused(MoveParams& m, const LayoutParams& lay, const LaunchPlan& plan, uint8_t* ws, const WorkspaceLayout& w) {
    m.fused = 1;
    m.count_blocks = plan.chunks;
    m.lay = lay;
    m.lay.vec_idx = (reinterpret_cast<uintptr_t>(lay.topk_idx) % 16 == 0) ? 1 : 0;
    m.chunk_done = reinterpret_cast<int32_t*>(ws + w.chunk_done);
    m.gates = reinterpret_cast<uint32_t*>(ws + w.gates);
    m.gates_finished = reinterpret_cast<uint32_t*>(ws + w.gates_finished);
    m.generation = reinterpret_cast<uint32_t*>(ws + w.generation);
    m.tagged = reinterpret_cast<uint32_t*>(ws + w.tagged);
    m.tagged_words = int((w.tagged_end - w.tagged) / 4);
    m.tagged_rank = reinterpret_cast<const uint32_t*>(ws + w.tagged_rank);
    m.tagged_expert = reinterpret_cast<uint32_t*>(ws + w.tagged_expert);
    // positions of this launch are read by its own movers: they go to the tagged table
    m.pos = reinterpret_cast<const uint32_t*>(ws + w.tagged_pos);
    m.lay.pos = reinterpret_cast<uint32_t*>(ws + w.tagged_pos);
    m.lay.tagged_rank = reinterpret_cast<uint32_t*>(ws + w.tagged_rank);
    m.tagged_expert_counts = reinterpret_cast<const uint32_t*>(ws + w.tagged_expert_counts);
    m.lay.tagged_expert_counts = m.do_expand ? reinterpret_cast<uint32_t*>(ws + w.tagged_expert_counts) : nullptr;
    m.lay.generation = m.generation;
}

}  // namespace

WorkspaceLayout make_workspace_layout(int num_max_tokens, int num_topk, int num_experts, int num_ranks) {
    WorkspaceLayout w{};
    const size_t n = size_t(num_ranks) + num_experts;
    const size_t chunks = num_max_tokens > 0 ? (size_t(num_max_tokens) + kLayoutChunk - 1) / kLayoutChunk : 1;
    const size_t chunks_padded = (chunks + 3) / 4 * 4;
    const size_t lanes = size_t(num_max_tokens > 0 ? num_max_tokens : 1) * num_topk;
    size_t off = 0;
    w.status = off;
    w.done_counter = off + 4;
    w.totals = off + 8;
    // A line of their own for the two words only agent-scope stores and atomics write: the line of the status word also
    // takes ordinary stores (the row totals), and a cache that writes such a line back whole would undo them.
    w.generation = off + 128;
    w.gates_finished = off + 132;
    off = 256;
    w.chunk_done = off;    off = align_up(off + size_t(kMaxCountBlocks) * 4, 256);
    w.gates = off;         off = align_up(off + size_t(kDispatchGates) * kDispatchGateStride * 4, 256);
    w.tagged = off;
    w.tagged_rank = off;   off += size_t(kTaggedRankWords) * 4;
    w.tagged_expert = off; off += size_t(kTaggedExpertWords) * 4;
    w.tagged_pos = off;    off += size_t(kTaggedPosWords) * 4;
    w.tagged_expert_counts = off; off += size_t(kTaggedExpertWords) * 4;
    w.tagged_end = off;
    w.expert_start = off;  off = align_up(off + size_t(num_experts) * 4, 256);
    const size_t experts_padded = (size_t(num_experts) + 31) / 32 * 32;
    w.rank_counts = off;   off = align_up(off + chunks_padded * num_ranks * 4, 256);
    w.rank_bases = off;    off = align_up(off + chunks_padded * num_ranks * 4, 256);
    w.expert_counts = off; off = align_up(off + chunks * experts_padded * 4, 256);
    w.expert_bases = off;  off = align_up(off + chunks * experts_padded * 4, 256);
    // Position words of a dispatch in two launches (tag 0).  Shapes the tagged table holds use that table: its words are
    // rewritten by whichever layout pass runs next, and a single-launch dispatch takes no word without its own tag.
    if (lanes <= size_t(kTaggedPosWords)) {
        w.pos = w.tagged_pos;
    } else {
        w.pos = off;       off = align_up(off + lanes * 4, 256);
    }
    w.total_bytes = off;
    return w;
}

}  // namespace deep_ep_hip

using namespace deep_ep_hip;

// ---- the workspace of deep_ep_hip_launch_dispatch_static: device memory that exists without any allocation ----
constexpr size_t kStaticWorkspaceBytes = DEEP_EP_HIP_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticWorkspaceBytes];

namespace {

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];          // address of `scratch` on each device (every GPU holds its own copy)
bool g_scratch_ready[kMaxDevices];
std::mutex g_scratch_mutex;

// The status word as memory has it (past every cache between the kernels that OR into it and this read), stored so
// that a host polling pinned memory sees it.  A clearing read swaps the word with zero and, if a single-launch dispatch
// had given up, zeroes the bookkeeping words that launch left mid-protocol.
__global__ void read_status_kernel(int32_t* status, int32_t* out, int clear, uint32_t* control, int control_words) {
    __shared__ int32_t seen;
    if (threadIdx.x == 0) {
        const int32_t v = clear ? __hip_atomic_exchange(status, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                : __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(out, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        seen = v;
    }
    __syncthreads();
    if (clear && (seen & DEEP_EP_HIP_STATUS_LAYOUT_TIMEOUT))
        for (int i = threadIdx.x; i < control_words; i += blockDim.x) store_agent(reinterpret_cast<int*>(control) + i, 0);
}

// Device address of `scratch` on the current device, resolved on first use.  The array needs no clearing: a `__device__`
// array without an initialiser reads zero when its code object is loaded, which is the state a fresh workspace must
// have, and nothing is launched here (the first call may be under graph capture: a clearing kernel captured with it
// would run again on every replay).
int static_workspace(void** out) {
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return hip_fail(err, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(DEEP_EP_HIP_ERR_UNSUPPORTED, "device index %d is beyond %d", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ready[dev]) {
        void* ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess || ptr == nullptr) return hip_fail(err, "hipGetSymbolAddress(scratch)");
        g_scratch_ptr[dev] = ptr;
        g_scratch_ready[dev] = true;
    }
    *out = g_scratch_ptr[dev];
    return DEEP_EP_HIP_OK;
}

int dispatch_with_workspace(const deep_ep_hip_dispatch_args* a, void* workspace, uint64_t workspace_bytes, hipStream_t stream) {
    if (int rc = check_routing_shape(a->num_tokens, a->num_topk, a->num_experts, a->num_ranks)) return rc;
    const int T = a->num_tokens, H = a->hidden, K = a->num_topk, E = a->num_experts, R = a->num_ranks;
    const bool do_layout = (a->phases & DEEP_EP_HIP_PHASE_LAYOUT) != 0;
    const bool do_move = (a->phases & DEEP_EP_HIP_PHASE_MOVE) != 0;
    REQUIRE(do_layout || do_move, "phases selects nothing");
    REQUIRE(!(a->cached && do_layout), "a cached dispatch has no layout phase");
    REQUIRE(a->rank_idx >= 0 && a->rank_idx < R, "rank_idx %d outside [0, %d)", a->rank_idx, R);
    REQUIRE(T <= a->num_max_tokens_per_rank, "num_tokens (%d) exceeds num_max_tokens_per_rank (%d)", T,
            a->num_max_tokens_per_rank);
    REQUIRE(int64_t(a->num_max_tokens_per_rank) * R < (int64_t(1) << 31), "num_max_tokens_per_rank * num_ranks overflows int32");
    REQUIRE(a->expert_alignment >= 1, "expert_alignment must be >= 1");
    REQUIRE(!a->do_zero_padding || a->do_expand, "do_zero_padding requires do_expand");
    REQUIRE(T == 0 || a->topk_idx != nullptr, "topk_idx is NULL");
    REQUIRE(workspace != nullptr, "workspace is NULL");
    REQUIRE(a->psum_num_recv_tokens_per_rank != nullptr && a->psum_num_recv_tokens_per_expert != nullptr &&
            a->num_unaligned_recv_tokens_per_expert != nullptr, "handle prefix-sum tensors are NULL");
    const WorkspaceLayout w = make_workspace_layout(T, K, E, R);
    if (workspace_bytes < w.total_bytes)
        return fail(DEEP_EP_HIP_ERR_WORKSPACE_TOO_SMALL, "workspace has %llu bytes, %zu needed",
                    (unsigned long long)workspace_bytes, w.total_bytes);
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    int32_t* status = reinterpret_cast<int32_t*>(ws + w.status);

    int elem_in = 2, elem_out = 2;
    switch (a->payload) {
        case DEEP_EP_HIP_PAYLOAD_BF16: break;
        case DEEP_EP_HIP_PAYLOAD_FP8: elem_in = elem_out = 1; break;
        case DEEP_EP_HIP_PAYLOAD_CAST_FP8: elem_out = 1; break;
        default: return fail(DEEP_EP_HIP_ERR_INVALID_ARGUMENT, "unknown payload kind %d", a->payload);
    }

    if (do_move) {
        REQUIRE(H >= 1, "hidden must be positive");
        REQUIRE((int64_t(H) * elem_in) % 16 == 0, "a row of x must be a multiple of 16 bytes (hidden %d, %d-byte elements)", H, elem_in);
        REQUIRE(int64_t(H) * elem_in < (int64_t(1) << 30), "row too large");
        REQUIRE(T == 0 || a->x != nullptr, "x is NULL");
        const bool no_rows = a->recv_capacity == 0 && a->expanded_capacity == 0;     // empty outputs have no storage
        REQUIRE(a->recv_x != nullptr || no_rows, "recv_x is NULL");
        REQUIRE(a->recv_src_metadata != nullptr || a->recv_capacity == 0, "recv_src_metadata is NULL");
        REQUIRE(a->dst_buffer_slot_idx != nullptr || T == 0, "dst_buffer_slot_idx is NULL");
        REQUIRE(a->recv_capacity >= 0 && a->expanded_capacity >= 0, "negative capacity");
        REQUIRE(a->recv_capacity < (int64_t(1) << 31) && a->expanded_capacity < (int64_t(1) << 31), "capacity overflows int32 rows");
        if (a->payload == DEEP_EP_HIP_PAYLOAD_BF16)
            REQUIRE(a->num_sf_packs == 0 && a->sf == nullptr && a->recv_sf == nullptr, "a BF16 payload carries no scale factors");
        if (a->payload == DEEP_EP_HIP_PAYLOAD_FP8) {
            REQUIRE(a->num_sf_packs >= 0, "num_sf_packs must be >= 0");
            REQUIRE(a->num_sf_packs == 0 || a->sf != nullptr || T == 0, "sf is NULL");
            REQUIRE(a->num_sf_packs == 0 || a->recv_sf != nullptr || no_rows, "recv_sf is NULL");
        }
        if (a->payload == DEEP_EP_HIP_PAYLOAD_CAST_FP8) {
            REQUIRE(H % 128 == 0, "the fused FP8 cast needs hidden %% 128 == 0 (got %d)", H);
            REQUIRE(a->num_sf_packs == H / 128, "num_sf_packs must be hidden / 128 for the fused cast");
            REQUIRE(a->recv_sf != nullptr || no_rows, "recv_sf is NULL");
        }
        REQUIRE(!(a->do_expand == 0 && a->recv_topk_idx == nullptr && a->recv_capacity > 0), "recv_topk_idx is NULL");
    }

    // Publishing targets of the layout results (the layout kernel's last workgroup, or the publishing workgroup of a
    // single-launch dispatch).
    PublishParams pub{};
    pub.R = R; pub.E = E; pub.A = a->expert_alignment; pub.do_expand = a->do_expand ? 1 : 0;
    pub.psum_rank = a->psum_num_recv_tokens_per_rank;
    pub.psum_expert = a->psum_num_recv_tokens_per_expert;
    pub.num_unaligned = a->num_unaligned_recv_tokens_per_expert;
    pub.cumulative_stats = a->cumulative_local_expert_recv_stats;
    pub.host_counts = a->host_counts;
    pub.status = status;
    pub.expert_start = reinterpret_cast<int32_t*>(ws + w.expert_start);
    pub.totals_out = reinterpret_cast<int32_t*>(ws + w.totals);

    // The layout pass leaves, per (token, lane), a position inside the token's 256-token chunk and, per (bucket,
    // chunk), the first row of that chunk's share of the bucket; the move kernel adds the two.  Layout and move in
    // one call: the counting workgroups ride at the front of the move kernel (one launch); shapes that does not
    // cover run the layout kernel first.
    const LaunchPlan plan = plan_launches(T, K, E, R, do_layout, do_move, a->do_expand != 0, a->expert_alignment, a->payload, H,
                                          H * elem_in, a->tuning);
    LayoutParams lay{};
    lay.topk_idx = a->topk_idx;
    lay.T = T; lay.K = K; lay.E = E; lay.R = R; lay.E_l = E / R;
    lay.copied_topk_idx = a->copied_topk_idx;
    lay.pub = pub;
    lay.status = status;
    lay.done_counter = reinterpret_cast<uint32_t*>(ws + w.done_counter);
    lay.tab = carve_tables(ws, w, T, E);
    lay.expert_bases = a->do_expand ? 1 : 0;
    lay.pos = reinterpret_cast<uint32_t*>(ws + w.pos);

    if (do_layout && !plan.fused) {
        hipError_t err = launch_layout_kernel(lay, stream);
        if (err != hipSuccess) return hip_fail(err, "dispatch layout launch");
    }

    if (do_move) {
        MoveParams m{};
        m.x = static_cast<const uint8_t*>(a->x);
        m.sf = static_cast<const uint32_t*>(a->sf);
        m.sf_ts = a->sf_token_stride; m.sf_hs = a->sf_hidden_stride;
        m.num_sf_packs = a->num_sf_packs;
        m.topk_idx = a->topk_idx;
        m.topk_weights = a->topk_weights;
        m.pos = reinterpret_cast<const uint32_t*>(ws + w.pos);
        m.expert_start = reinterpret_cast<const int32_t*>(ws + w.expert_start);
        m.cached_slot = a->dst_buffer_slot_idx;
        m.dst_buffer_slot_idx = a->dst_buffer_slot_idx;
        m.psum_rank = a->psum_num_recv_tokens_per_rank;
        m.recv_src_metadata = a->recv_src_metadata;
        m.recv_x = static_cast<uint8_t*>(a->recv_x);
        m.recv_sf = static_cast<uint32_t*>(a->recv_sf);
        m.rsf_ts = a->recv_sf_token_stride; m.rsf_hs = a->recv_sf_hidden_stride;
        m.recv_topk_idx = a->recv_topk_idx;
        m.recv_topk_weights = a->topk_weights != nullptr ? a->recv_topk_weights : nullptr;
        m.recv_capacity = a->recv_capacity;
        m.expanded_capacity = a->expanded_capacity;
        m.T = T; m.H = H; m.K = K; m.E = E; m.R = R; m.E_l = E / R;
        m.rank_idx = a->rank_idx; m.M = a->num_max_tokens_per_rank;
        m.cached = a->cached ? 1 : 0;
        m.do_expand = a->do_expand ? 1 : 0;
        m.payload = a->payload;
        m.row_bytes = H * elem_in;
        m.tab = lay.tab;
        m.pub = pub;
        m.status = status;
        m.cast_pairs = a->tuning.cast_pairs; m.copy_vecs = a->tuning.copy_vecs;
        m.mover_spin_limit = a->tuning.mover_spin_limit > 0 ? unsigned(a->tuning.mover_spin_limit) : (1u << 22);   // seconds
        m.move_workgroups_per_cu = a->tuning.move_workgroups_per_cu;
        m.warm_rounds = a->tuning.warm_rounds;
        m.persistent_movers = a->tuning.persistent_movers;
        m.plain_loads = a->tuning.plain_loads; m.xcd_remap = a->tuning.xcd_remap;
        m.gates = reinterpret_cast<uint32_t*>(ws + w.gates);               // a persistent move kernel keeps its item counter there
        m.gates_finished = reinterpret_cast<uint32_t*>(ws + w.gates_finished);
        if (plan.fused) fill_fused(m, lay, plan, ws, w);

        hipError_t err = launch_dispatch_move(m, stream);
        if (err != hipSuccess) return hip_fail(err, "dispatch move launch");

        if (a->do_zero_padding && a->expert_alignment > 1) {
            PadParams z{};
            z.recv_x = static_cast<uint8_t*>(a->recv_x);
            z.recv_sf = (a->payload != DEEP_EP_HIP_PAYLOAD_BF16) ? static_cast<uint32_t*>(a->recv_sf) : nullptr;
            z.rsf_ts = a->recv_sf_token_stride; z.rsf_hs = a->recv_sf_hidden_stride;
            z.num_sf_packs = a->num_sf_packs;
            z.recv_topk_weights = a->topk_weights != nullptr ? a->recv_topk_weights : nullptr;
            z.psum_expert = a->psum_num_recv_tokens_per_expert;
            z.num_unaligned = a->num_unaligned_recv_tokens_per_expert;
            z.expanded_capacity = a->expanded_capacity;
            z.E = E; z.A = a->expert_alignment;
            z.out_row_bytes = H * elem_out;
            err = launch_zero_padding(z, stream);
            if (err != hipSuccess) return hip_fail(err, "zero padding launch");
        }
    }
    return DEEP_EP_HIP_OK;
}

}  // namespace


extern "C" {

int deep_ep_hip_abi_version(void) { return DEEP_EP_HIP_ABI_VERSION; }

const char* deep_ep_hip_last_error(void) { return g_last_error; }

size_t deep_ep_hip_workspace_bytes(int num_max_tokens, int num_topk, int num_experts, int num_ranks) {
    if (num_max_tokens < 0 || num_topk < 1 || num_experts < 1 || num_ranks < 1) return 0;
    return make_workspace_layout(num_max_tokens, num_topk, num_experts, num_ranks).total_bytes;
}

size_t deep_ep_hip_combine_workspace_bytes(int num_tokens, int num_topk, int num_experts, int num_ranks) {
    if (num_tokens < 0 || num_topk < 1 || num_experts < 1 || num_ranks < 1) return 0;
    const size_t tables = make_workspace_layout(num_tokens, num_topk, num_experts, num_ranks).total_bytes;
    return tables + align_up(size_t(num_tokens > 0 ? num_tokens : 1) * num_topk * 4, 256);
}

size_t deep_ep_hip_workspace_status_offset(void) { return 0; }

size_t deep_ep_hip_workspace_control_bytes(void) { return make_workspace_layout(1, 1, 1, 1).expert_start; }

size_t deep_ep_hip_workspace_counter_bytes(void) { return make_workspace_layout(1, 1, 1, 1).tagged; }

int deep_ep_hip_read_status(void* workspace, int32_t* status_out, int clear, void* stream) {
    REQUIRE(status_out != nullptr, "status_out is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (workspace == nullptr)
        if (int rc = static_workspace(&workspace)) return rc;
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    const WorkspaceLayout w = make_workspace_layout(1, 1, 1, 1);
    hipLaunchKernelGGL(read_status_kernel, dim3(1), dim3(256), 0, s, reinterpret_cast<int32_t*>(ws + w.status), status_out,
                       clear, reinterpret_cast<uint32_t*>(ws), static_cast<int>(w.expert_start / 4));
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return hip_fail(err, "launching the status read");
    return DEEP_EP_HIP_OK;
}

int deep_ep_hip_launch_layout(const deep_ep_hip_layout_args* a, void* stream) {
    REQUIRE(a != nullptr, "args is NULL");
    if (int rc = check_routing_shape(a->num_tokens, a->num_topk, a->num_experts, a->num_ranks)) return rc;
    REQUIRE(a->num_tokens == 0 || a->topk_idx != nullptr, "topk_idx is NULL");
    REQUIRE(a->num_tokens_per_rank != nullptr && a->num_tokens_per_expert != nullptr, "count outputs are NULL");
    REQUIRE(a->workspace != nullptr, "workspace is NULL");
    const WorkspaceLayout w = make_workspace_layout(a->num_tokens, a->num_topk, a->num_experts, a->num_ranks);
    if (a->workspace_bytes < w.total_bytes)
        return fail(DEEP_EP_HIP_ERR_WORKSPACE_TOO_SMALL, "workspace has %llu bytes, %zu needed",
                    (unsigned long long)a->workspace_bytes, w.total_bytes);
    uint8_t* ws = static_cast<uint8_t*>(a->workspace);
    LayoutParams p{};
    p.topk_idx = a->topk_idx;
    p.T = a->num_tokens; p.K = a->num_topk; p.E = a->num_experts; p.R = a->num_ranks;
    p.E_l = p.E / p.R;
    p.is_token_in_rank = a->is_token_in_rank;
    p.pub.R = p.R; p.pub.E = p.E; p.pub.A = 1;
    p.pub.num_tokens_per_rank = a->num_tokens_per_rank;
    p.pub.num_tokens_per_expert = a->num_tokens_per_expert;
    p.pub.expert_start = reinterpret_cast<int32_t*>(ws + w.expert_start);
    p.pub.totals_out = reinterpret_cast<int32_t*>(ws + w.totals);
    p.status = reinterpret_cast<int32_t*>(ws + w.status);
    p.done_counter = reinterpret_cast<uint32_t*>(ws + w.done_counter);
    p.tab = carve_tables(ws, w, p.T, p.E);
    p.tab.rank_bases = nullptr;       // a layout-only call publishes counts, not row bases
    p.tab.expert_bases = nullptr;
    hipError_t err = launch_layout_kernel(p, static_cast<hipStream_t>(stream));
    if (err != hipSuccess) return hip_fail(err, "layout launch");
    return DEEP_EP_HIP_OK;
}

int deep_ep_hip_launch_dispatch(const deep_ep_hip_dispatch_args* a, void* stream) {
    REQUIRE(a != nullptr, "args is NULL");
    return dispatch_with_workspace(a, a->workspace, a->workspace_bytes, static_cast<hipStream_t>(stream));
}

int deep_ep_hip_dispatch_kernel_launches(const deep_ep_hip_dispatch_args* a) {
    REQUIRE(a != nullptr, "args is NULL");
    if (int rc = check_routing_shape(a->num_tokens, a->num_topk, a->num_experts, a->num_ranks)) return rc;
    const bool do_layout = (a->phases & DEEP_EP_HIP_PHASE_LAYOUT) != 0;
    const bool do_move = (a->phases & DEEP_EP_HIP_PHASE_MOVE) != 0;
    REQUIRE(do_layout || do_move, "phases selects nothing");
    REQUIRE(a->payload == DEEP_EP_HIP_PAYLOAD_BF16 || a->payload == DEEP_EP_HIP_PAYLOAD_FP8 ||
            a->payload == DEEP_EP_HIP_PAYLOAD_CAST_FP8, "unknown payload kind %d", a->payload);
    if (a->num_tokens == 0) return do_layout ? 1 : 0;      // an empty move launches nothing
    const int elem_in = a->payload == DEEP_EP_HIP_PAYLOAD_FP8 ? 1 : 2;
    const LaunchPlan plan = plan_launches(a->num_tokens, a->num_topk, a->num_experts, a->num_ranks, do_layout, do_move,
                                          a->do_expand != 0, a->expert_alignment, a->payload, a->hidden, a->hidden * elem_in,
                                          a->tuning);
    return plan.fused ? 1 : int(do_layout) + int(do_move);
}

int deep_ep_hip_launch_dispatch_static(const deep_ep_hip_dispatch_args* a, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    REQUIRE(a != nullptr, "args is NULL");
    if (int rc = check_routing_shape(a->num_tokens, a->num_topk, a->num_experts, a->num_ranks)) return rc;
    const size_t need = make_workspace_layout(a->num_tokens, a->num_topk, a->num_experts, a->num_ranks).total_bytes;
    if (need > kStaticWorkspaceBytes)
        return fail(DEEP_EP_HIP_ERR_WORKSPACE_TOO_SMALL,
                    "this shape needs %zu bytes of workspace, the built-in one has %zu: pass a workspace of your own to "
                    "deep_ep_hip_launch_dispatch", need, kStaticWorkspaceBytes);
    void* ws = nullptr;
    if (int rc = static_workspace(&ws)) return rc;
    return dispatch_with_workspace(a, ws, kStaticWorkspaceBytes, stream);
}

int deep_ep_hip_launch_combine(const deep_ep_hip_combine_args* a, void* stream) {
    REQUIRE(a != nullptr, "args is NULL");
    if (int rc = check_routing_shape(a->num_tokens, a->num_topk, a->num_experts, a->num_ranks)) return rc;
    REQUIRE(a->hidden >= 1 && (int64_t(a->hidden) * 2) % 16 == 0, "hidden (%d) must give rows that are multiples of 16 bytes", a->hidden);
    REQUIRE(a->rank_idx >= 0 && a->rank_idx < a->num_ranks, "rank_idx %d outside [0, %d)", a->rank_idx, a->num_ranks);
    REQUIRE(a->num_x_rows >= 0 && a->num_x_rows < (int64_t(1) << 31), "num_x_rows out of range");
    const bool any = a->num_tokens > 0;
    REQUIRE(!any || (a->topk_idx != nullptr && a->psum_num_recv_tokens_per_rank != nullptr), "handle tensors are NULL");
    REQUIRE(!any || a->combined_x != nullptr, "combined_x is NULL");
    REQUIRE(!any || a->x != nullptr || a->num_x_rows == 0, "x is NULL");
    REQUIRE(a->num_recv_rows >= 0, "num_recv_rows must be >= 0");
    REQUIRE(!(a->do_expand && any && a->num_recv_rows > 0 && a->recv_src_metadata == nullptr),
            "the expanded layout needs recv_src_metadata");
    REQUIRE(a->workspace != nullptr && a->workspace_bytes >= 256, "workspace is NULL or smaller than 256 bytes");
    const int32_t* slot = a->dst_buffer_slot_idx;
    if (slot == nullptr && any) {
        // The handle came without its token -> row map: rebuild it behind the dispatch tables of the workspace.
        REQUIRE(a->recv_src_metadata != nullptr || a->num_recv_rows == 0, "without dst_buffer_slot_idx the map is rebuilt from recv_src_metadata, which is NULL");
        const size_t need = deep_ep_hip_combine_workspace_bytes(a->num_tokens, a->num_topk, a->num_experts, a->num_ranks);
        if (a->workspace_bytes < need)
            return fail(DEEP_EP_HIP_ERR_WORKSPACE_TOO_SMALL, "workspace has %llu bytes, %zu needed to rebuild dst_buffer_slot_idx",
                        (unsigned long long)a->workspace_bytes, need);
        SlotMapParams q{};
        q.meta = a->recv_src_metadata;
        q.num_meta_rows = a->num_recv_rows;
        q.psum_rank = a->psum_num_recv_tokens_per_rank;
        q.slot = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(a->workspace) +
                                            make_workspace_layout(a->num_tokens, a->num_topk, a->num_experts, a->num_ranks).total_bytes);
        q.T = a->num_tokens; q.K = a->num_topk; q.R = a->num_ranks; q.rank_idx = a->rank_idx; q.M = a->num_max_tokens_per_rank;
        const hipError_t err = launch_rebuild_slot_map(q, static_cast<hipStream_t>(stream));
        if (err != hipSuccess) return hip_fail(err, "slot map launch");
        slot = q.slot;
    }
    CombineParams p{};
    p.x = static_cast<const uint8_t*>(a->x);
    p.num_x_rows = a->num_x_rows;
    p.topk_weights = a->topk_weights;
    p.bias0 = static_cast<const uint8_t*>(a->bias_0);
    p.bias1 = static_cast<const uint8_t*>(a->bias_1);
    p.topk_idx = a->topk_idx;
    p.slot = slot;
    p.meta = a->recv_src_metadata;
    p.num_meta_rows = a->num_recv_rows;
    p.psum_rank = a->psum_num_recv_tokens_per_rank;
    p.out = static_cast<uint8_t*>(a->combined_x);
    p.out_w = a->combined_topk_weights;
    p.T = a->num_tokens; p.H = a->hidden; p.K = a->num_topk; p.E = a->num_experts; p.R = a->num_ranks;
    p.E_l = p.E / p.R;
    p.rank_idx = a->rank_idx; p.M = a->num_max_tokens_per_rank;
    p.do_expand = a->do_expand ? 1 : 0;
    p.multi_red = a->allow_multiple_reduction ? 1 : 0;
    p.status = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(a->workspace));
    p.vecs = a->tuning.combine_vecs;
    hipError_t err = launch_combine_kernel(p, static_cast<hipStream_t>(stream));
    if (err != hipSuccess) return hip_fail(err, "combine launch");
    return DEEP_EP_HIP_OK;
}

int deep_ep_hip_launch_intranode_dispatch(const deep_ep_hip_intranode_dispatch_args* a, void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    REQUIRE(a != nullptr, "args is NULL");
    // An empty batch has NULL tensors: the routing mode follows num_topk, not the pointers.
    const bool with_topk = a->num_topk > 0 || a->topk_idx != nullptr;
    const int T = a->num_tokens, H = a->hidden, R = a->num_ranks;
    REQUIRE(R >= 1 && R <= 64, "num_ranks must be in [1, 64] (got %d)", R);
    REQUIRE(!a->cached || !with_topk, "a cached dispatch takes no topk_idx");
    REQUIRE((a->topk_idx != nullptr) == (a->topk_weights != nullptr), "topk_idx and topk_weights go together");
    REQUIRE(!with_topk || T == 0 || a->topk_idx != nullptr, "topk_idx is NULL");
    // Routing lanes: the top-k lanes, or one lane per rank.
    const int K = with_topk ? a->num_topk : R;
    const int E = with_topk ? a->num_experts : R;
    REQUIRE(with_topk || R <= DEEP_EP_HIP_MAX_TOPK, "routing by is_token_in_rank alone supports up to %d ranks", DEEP_EP_HIP_MAX_TOPK);
    if (int rc = check_routing_shape(T, K, E, R)) return rc;
    const bool do_layout = (a->phases & DEEP_EP_HIP_PHASE_LAYOUT) != 0;
    const bool do_move = (a->phases & DEEP_EP_HIP_PHASE_MOVE) != 0;
    REQUIRE(do_layout || do_move, "phases selects nothing");
    REQUIRE(!(a->cached && do_layout), "a cached dispatch has no layout phase");
    REQUIRE(a->rank_idx >= 0 && a->rank_idx < R, "rank_idx %d outside [0, %d)", a->rank_idx, R);
    REQUIRE(a->expert_alignment >= 1, "expert_alignment must be >= 1");
    REQUIRE(a->num_channels >= 0 && a->num_channels <= 8192, "num_channels must be in [0, 8192]");
    REQUIRE(a->num_channels >= 1 || (a->rank_prefix_matrix == nullptr && a->channel_prefix_matrix == nullptr &&
                                     a->recv_channel_prefix_matrix == nullptr),
            "num_channels must be >= 1 when the prefix matrices are requested");
    REQUIRE(a->cached || T == 0 || with_topk || a->is_token_in_rank != nullptr, "is_token_in_rank is NULL");
    REQUIRE(a->workspace != nullptr, "workspace is NULL");
    REQUIRE(a->cached || a->psum_num_recv_tokens_per_rank != nullptr, "psum_num_recv_tokens_per_rank is NULL");
    const WorkspaceLayout w = make_workspace_layout(T, K, E, R);
    if (a->workspace_bytes < w.total_bytes)
        return fail(DEEP_EP_HIP_ERR_WORKSPACE_TOO_SMALL, "workspace has %llu bytes, %zu needed",
                    (unsigned long long)a->workspace_bytes, w.total_bytes);
    uint8_t* ws = static_cast<uint8_t*>(a->workspace);
    int32_t* status = reinterpret_cast<int32_t*>(ws + w.status);

    int elem_in = 2;
    switch (a->payload) {
        case DEEP_EP_HIP_PAYLOAD_BF16: break;
        case DEEP_EP_HIP_PAYLOAD_FP8: elem_in = 1; break;
        case DEEP_EP_HIP_PAYLOAD_CAST_FP8: break;
        default: return fail(DEEP_EP_HIP_ERR_INVALID_ARGUMENT, "unknown payload kind %d", a->payload);
    }
    if (do_move) {
        REQUIRE(H >= 1 && (int64_t(H) * elem_in) % 16 == 0 && int64_t(H) * elem_in < (int64_t(1) << 30),
                "a row of x must be a multiple of 16 bytes (hidden %d, %d-byte elements)", H, elem_in);
        REQUIRE(T == 0 || a->x != nullptr, "x is NULL");
        REQUIRE(a->recv_capacity >= 0 && a->recv_capacity < (int64_t(1) << 31), "recv_capacity out of range");
        REQUIRE(a->recv_x != nullptr || a->recv_capacity == 0, "recv_x is NULL");
        REQUIRE(a->send_head != nullptr || T == 0, "send_head is NULL");
        if (a->payload == DEEP_EP_HIP_PAYLOAD_BF16)
            REQUIRE(a->num_scales == 0 && a->x_scales == nullptr && a->recv_x_scales == nullptr,
                    "a BF16 payload carries no scales");
        const bool no_rows = a->recv_capacity == 0;                       // empty outputs have no storage
        if (a->payload == DEEP_EP_HIP_PAYLOAD_FP8) {
            REQUIRE(a->num_scales >= 0, "num_scales must be >= 0");
            REQUIRE(a->num_scales == 0 || T == 0 || a->x_scales != nullptr, "x_scales is NULL");
            REQUIRE(a->num_scales == 0 || no_rows || a->recv_x_scales != nullptr, "recv_x_scales is NULL");
        }
        if (a->payload == DEEP_EP_HIP_PAYLOAD_CAST_FP8)
            REQUIRE(H % 128 == 0 && a->num_scales == H / 128 && (a->recv_x_scales != nullptr || no_rows),
                    "the fused FP8 cast needs hidden %% 128 == 0, num_scales == hidden / 128 and recv_x_scales");
        REQUIRE(!with_topk || a->recv_capacity == 0 || (a->recv_topk_idx != nullptr && a->recv_topk_weights != nullptr),
                "recv_topk_idx / recv_topk_weights is NULL");
    }

    PublishParams pub{};
    pub.R = R; pub.E = E; pub.A = a->expert_alignment; pub.do_expand = 0;
    pub.psum_rank = a->psum_num_recv_tokens_per_rank;
    pub.num_unaligned = with_topk ? a->num_recv_tokens_per_expert : nullptr;
    pub.host_counts = a->host_counts;
    pub.status = status;
    pub.expert_start = reinterpret_cast<int32_t*>(ws + w.expert_start);
    pub.totals_out = reinterpret_cast<int32_t*>(ws + w.totals);

    const LaunchPlan plan = plan_launches(T, K, E, R, do_layout, do_move, false, 1, a->payload, H, H * elem_in, a->tuning);
    LayoutParams lay{};
    lay.topk_idx = a->topk_idx;
    lay.route_mask = with_topk ? nullptr : a->is_token_in_rank;
    lay.T = T; lay.K = K; lay.E = E; lay.R = R; lay.E_l = E / R;
    lay.pub = pub;
    lay.status = status;
    lay.done_counter = reinterpret_cast<uint32_t*>(ws + w.done_counter);
    lay.tab = carve_tables(ws, w, T, E);
    lay.pos = reinterpret_cast<uint32_t*>(ws + w.pos);

    if (do_layout) {
        hipError_t err = hipSuccess;
        if (!plan.fused) {
            err = launch_layout_kernel(lay, stream);
            if (err != hipSuccess) return hip_fail(err, "intranode dispatch layout launch");
        }

        if (a->rank_prefix_matrix != nullptr || a->channel_prefix_matrix != nullptr ||
            a->recv_channel_prefix_matrix != nullptr) {
            REQUIRE(a->is_token_in_rank != nullptr || T == 0, "the prefix matrices are computed from is_token_in_rank");
            IntranodePrefixParams q{};
            q.mask = a->is_token_in_rank;
            q.T = T; q.R = R; q.C = a->num_channels; q.rank_idx = a->rank_idx;
            q.rank_prefix_matrix = a->rank_prefix_matrix;
            q.channel_prefix_matrix = a->channel_prefix_matrix;
            q.recv_channel_prefix_matrix = a->recv_channel_prefix_matrix;
            err = launch_intranode_prefix(q, stream);
            if (err != hipSuccess) return hip_fail(err, "intranode prefix launch");
        }
    }

    if (do_move) {
        MoveParams m{};
        m.x = static_cast<const uint8_t*>(a->x);
        m.sf = static_cast<const uint32_t*>(a->x_scales);
        m.sf_ts = a->scale_token_stride; m.sf_hs = a->scale_hidden_stride;
        m.num_sf_packs = a->num_scales;
        m.topk_idx = a->topk_idx;
        m.route_mask = (with_topk || a->cached) ? nullptr : a->is_token_in_rank;
        m.topk_weights = a->topk_weights;
        m.pos = reinterpret_cast<const uint32_t*>(ws + w.pos);
        m.expert_start = reinterpret_cast<const int32_t*>(ws + w.expert_start);
        m.cached_slot = a->send_head;
        m.dst_buffer_slot_idx = nullptr;
        m.psum_rank = a->psum_num_recv_tokens_per_rank;
        m.recv_src_metadata = nullptr;
        m.recv_x = static_cast<uint8_t*>(a->recv_x);
        m.recv_sf = static_cast<uint32_t*>(a->recv_x_scales);
        m.rsf_ts = a->recv_scale_token_stride; m.rsf_hs = a->recv_scale_hidden_stride;
        m.recv_topk_idx = with_topk ? a->recv_topk_idx : nullptr;
        m.recv_topk_weights = with_topk ? a->recv_topk_weights : nullptr;
        m.recv_capacity = a->recv_capacity;
        m.expanded_capacity = 0;
        m.T = T; m.H = H; m.K = K; m.E = E; m.R = R; m.E_l = E / R;
        m.rank_idx = a->rank_idx; m.M = T > 0 ? T : 1;
        m.cached = a->cached ? 1 : 0;
        m.do_expand = 0;
        m.payload = a->payload;
        m.row_bytes = H * elem_in;
        m.tab = lay.tab;
        m.pub = pub;
        m.status = status;
        m.cast_pairs = a->tuning.cast_pairs; m.copy_vecs = a->tuning.copy_vecs;
        m.mover_spin_limit = a->tuning.mover_spin_limit > 0 ? unsigned(a->tuning.mover_spin_limit) : (1u << 22);   // seconds
        m.move_workgroups_per_cu = a->tuning.move_workgroups_per_cu;
        m.warm_rounds = a->tuning.warm_rounds;
        m.persistent_movers = a->tuning.persistent_movers;
        m.plain_loads = a->tuning.plain_loads; m.xcd_remap = a->tuning.xcd_remap;
        m.gates = reinterpret_cast<uint32_t*>(ws + w.gates);               // a persistent move kernel keeps its item counter there
        m.gates_finished = reinterpret_cast<uint32_t*>(ws + w.gates_finished);
        if (plan.fused) fill_fused(m, lay, plan, ws, w);

        m.rank_lanes = with_topk ? 0 : 1;
        m.slot_is_row = a->cached ? 1 : 0;
        m.zero_nonlocal_w = 1;
        m.send_head = a->cached ? nullptr : a->send_head;
        m.recv_src_idx = a->cached ? nullptr : a->recv_src_idx;
        hipError_t err = launch_dispatch_move(m, stream);
        if (err != hipSuccess) return hip_fail(err, "intranode dispatch move launch");

        if (a->fill_unused_topk_idx && with_topk && !a->cached) {
            FillTailParams f{};
            f.recv_topk_idx = a->recv_topk_idx;
            f.total_rows = reinterpret_cast<const int32_t*>(ws + w.totals);
            f.capacity = a->recv_capacity;
            f.K = K;
            err = launch_fill_tail(f, stream);
            if (err != hipSuccess) return hip_fail(err, "intranode fill launch");
        }
    }
    return DEEP_EP_HIP_OK;
}

int deep_ep_hip_launch_intranode_combine(const deep_ep_hip_intranode_combine_args* a, void* stream) {
    REQUIRE(a != nullptr, "args is NULL");
    REQUIRE(a->num_tokens >= 0, "num_tokens must be >= 0");
    REQUIRE(a->num_ranks >= 1 && a->num_ranks <= 64, "num_ranks must be in [1, 64] (got %d)", a->num_ranks);
    REQUIRE(a->num_topk >= 0 && a->num_topk <= DEEP_EP_HIP_MAX_TOPK, "num_topk must be in [0, %d]", DEEP_EP_HIP_MAX_TOPK);
    REQUIRE(a->hidden >= 1 && (int64_t(a->hidden) * 2) % 16 == 0, "hidden (%d) must give rows that are multiples of 16 bytes", a->hidden);
    REQUIRE(a->num_x_rows >= 0 && a->num_x_rows < (int64_t(1) << 31), "num_x_rows out of range");
    const bool any = a->num_tokens > 0;
    REQUIRE(!any || (a->send_head != nullptr && a->combined_x != nullptr), "send_head / combined_x is NULL");
    REQUIRE(!any || a->x != nullptr || a->num_x_rows == 0, "x is NULL");
    REQUIRE(a->num_topk == 0 || a->topk_weights == nullptr || a->combined_topk_weights != nullptr, "combined_topk_weights is NULL");
    REQUIRE(a->workspace != nullptr && a->workspace_bytes >= 256, "workspace is NULL or smaller than 256 bytes");
    CombineParams p{};
    p.x = static_cast<const uint8_t*>(a->x);
    p.num_x_rows = a->num_x_rows;
    p.topk_weights = a->topk_weights;
    p.bias0 = static_cast<const uint8_t*>(a->bias_0);
    p.bias1 = static_cast<const uint8_t*>(a->bias_1);
    p.slot = a->send_head;
    p.out = static_cast<uint8_t*>(a->combined_x);
    p.out_w = a->num_topk > 0 ? a->combined_topk_weights : nullptr;
    p.T = a->num_tokens; p.H = a->hidden; p.K = a->num_ranks; p.E = a->num_ranks; p.R = a->num_ranks; p.E_l = 1;
    p.rank_mode = 1;
    p.Kw = a->num_topk;
    p.status = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(a->workspace));
    p.vecs = a->tuning.combine_vecs;
    hipError_t err = launch_combine_kernel(p, static_cast<hipStream_t>(stream));
    if (err != hipSuccess) return hip_fail(err, "intranode combine launch");
    return DEEP_EP_HIP_OK;
}

size_t deep_ep_hip_ll_workspace_bytes(int num_src_ranks, int src_token_stride, int num_topk, int num_local_experts) {
    if (num_src_ranks < 1 || src_token_stride < 1 || num_topk < 1 || num_local_experts < 1) return 0;
    const size_t chunks = size_t(num_src_ranks) * ((size_t(src_token_stride) + kLayoutChunk - 1) / kLayoutChunk);
    size_t off = 256;
    off = align_up(off + chunks * num_local_experts * 4, 256) ;
    off = align_up(off + chunks * num_local_experts * 4, 256);
    off = align_up(off + size_t(num_src_ranks) * src_token_stride * num_topk * 4, 256);
    return off;
}

int deep_ep_hip_launch_ll_dispatch(const deep_ep_hip_ll_dispatch_args* a, void* stream) {
    REQUIRE(a != nullptr, "args is NULL");
    REQUIRE(a->num_src_ranks >= 1 && a->src_token_stride >= 1, "need at least one source rank and one token slot");
    REQUIRE(a->num_topk >= 1 && a->num_topk <= DEEP_EP_HIP_MAX_TOPK, "num_topk must be in [1, %d]", DEEP_EP_HIP_MAX_TOPK);
    REQUIRE(a->num_experts >= 1 && a->num_local_experts >= 1 && a->num_local_experts <= DEEP_EP_HIP_MAX_EXPERTS,
            "bad expert counts");
    REQUIRE(a->expert_begin >= 0 && a->expert_begin + a->num_local_experts <= a->num_experts, "local expert range outside [0, num_experts)");
    REQUIRE(a->num_ranks >= 1 && a->src_rank_begin >= 0 && a->src_rank_begin + a->num_src_ranks <= a->num_ranks,
            "source ranks outside [0, num_ranks)");
    REQUIRE(a->num_max_dispatch_tokens_per_rank >= 1, "num_max_dispatch_tokens_per_rank must be positive");
    REQUIRE(int64_t(a->num_ranks) * a->num_max_dispatch_tokens_per_rank < (int64_t(1) << 31), "rows per expert overflow int32");
    REQUIRE(a->src_token_stride <= a->num_max_dispatch_tokens_per_rank, "src_token_stride exceeds num_max_dispatch_tokens_per_rank");
    REQUIRE(a->lane_rows == nullptr || int64_t(a->num_local_experts) * a->num_ranks * a->num_max_dispatch_tokens_per_rank < (int64_t(1) << 31),
            "lane_rows needs num_local_experts * rows per expert below 2^31");
    REQUIRE(a->hidden >= 16 && a->hidden % 16 == 0, "hidden must be a multiple of 16");
    REQUIRE(!a->use_fp8 || a->hidden % 128 == 0, "FP8 needs hidden %% 128 == 0");
    REQUIRE(!a->use_fp8 || a->packed_recv_x_scales != nullptr, "packed_recv_x_scales is NULL");
    REQUIRE(!a->round_scale || a->use_fp8, "round_scale needs use_fp8");
    REQUIRE(!a->use_ue8m0 || (a->round_scale && a->hidden % 512 == 0), "use_ue8m0 needs round_scale and hidden %% 512 == 0");
    REQUIRE(a->x != nullptr && a->topk_idx != nullptr && a->packed_recv_x != nullptr && a->packed_recv_count != nullptr &&
            a->packed_recv_src_info != nullptr && a->packed_recv_layout_range != nullptr, "NULL tensor");
    const size_t need = deep_ep_hip_ll_workspace_bytes(a->num_src_ranks, a->src_token_stride, a->num_topk, a->num_local_experts);
    REQUIRE(a->workspace != nullptr, "workspace is NULL");
    if (a->workspace_bytes < need)
        return fail(DEEP_EP_HIP_ERR_WORKSPACE_TOO_SMALL, "workspace has %llu bytes, %zu needed",
                    (unsigned long long)a->workspace_bytes, need);
    uint8_t* ws = static_cast<uint8_t*>(a->workspace);
    const size_t chunks = size_t(a->num_src_ranks) * ((size_t(a->src_token_stride) + kLayoutChunk - 1) / kLayoutChunk);
    LLDispatchParams p{};
    p.use_fp8 = a->use_fp8 ? 1 : 0;
    p.round_scale = a->round_scale ? 1 : 0;
    p.use_ue8m0 = a->use_ue8m0 ? 1 : 0;
    p.S = a->num_src_ranks; p.src_rank_begin = a->src_rank_begin; p.src_token_stride = a->src_token_stride;
    p.num_tokens_per_src = a->num_tokens_per_src;
    p.H = a->hidden; p.K = a->num_topk; p.E = a->num_experts; p.expert_begin = a->expert_begin;
    p.E_l = a->num_local_experts; p.R = a->num_ranks; p.M = a->num_max_dispatch_tokens_per_rank;
    p.x = static_cast<const uint8_t*>(a->x);
    p.topk_idx = a->topk_idx;
    p.packed_x = static_cast<uint8_t*>(a->packed_recv_x);
    p.packed_scales = a->packed_recv_x_scales;
    p.packed_count = a->packed_recv_count;
    p.packed_src_info = a->packed_recv_src_info;
    p.packed_layout_range = a->packed_recv_layout_range;
    p.cumulative_stats = a->cumulative_local_expert_recv_stats;
    p.lane_slot = a->lane_rows;
    size_t off = 256;
    p.status = reinterpret_cast<int32_t*>(ws);
    p.done_counter = reinterpret_cast<uint32_t*>(ws + 4);
    p.chunk_counts = reinterpret_cast<int32_t*>(ws + off); off = align_up(off + chunks * p.E_l * 4, 256);
    p.chunk_base = reinterpret_cast<int32_t*>(ws + off);   off = align_up(off + chunks * p.E_l * 4, 256);
    p.pos_expert = reinterpret_cast<int32_t*>(ws + off);
    p.pairs = a->tuning.ll_pairs; p.threads = a->tuning.ll_threads; p.two_kernels = a->tuning.ll_two_kernels;
    hipError_t err = launch_ll_dispatch(p, static_cast<hipStream_t>(stream));
    if (err != hipSuccess) return hip_fail(err, "low-latency dispatch launch");
    return DEEP_EP_HIP_OK;
}

int deep_ep_hip_launch_ll_combine(const deep_ep_hip_ll_combine_args* a, void* stream) {
    REQUIRE(a != nullptr, "args is NULL");
    REQUIRE(a->num_src_ranks >= 1 && a->src_token_stride >= 1, "need at least one source rank and one token slot");
    REQUIRE(a->num_topk >= 1 && a->num_topk <= DEEP_EP_HIP_MAX_TOPK, "num_topk must be in [1, %d]", DEEP_EP_HIP_MAX_TOPK);
    REQUIRE(a->hidden >= 8 && (int64_t(a->hidden) * 2) % 16 == 0, "hidden must give rows that are multiples of 16 bytes");
    REQUIRE(a->num_local_experts >= 1 && a->expert_begin >= 0 && a->expert_begin + a->num_local_experts <= a->num_experts,
            "local expert range outside [0, num_experts)");
    REQUIRE(a->num_ranks >= 1 && a->src_rank_begin >= 0 && a->src_rank_begin + a->num_src_ranks <= a->num_ranks,
            "source ranks outside [0, num_ranks)");
    REQUIRE(a->num_max_dispatch_tokens_per_rank >= 1, "num_max_dispatch_tokens_per_rank must be positive");
    REQUIRE(a->x != nullptr && a->topk_idx != nullptr && a->topk_weights != nullptr &&
            a->packed_recv_src_info != nullptr && a->packed_recv_layout_range != nullptr && a->combined_x != nullptr, "NULL tensor");
    REQUIRE(a->workspace != nullptr && a->workspace_bytes >= 256, "workspace is NULL or smaller than 256 bytes");
    REQUIRE(!a->use_logfmt || a->hidden % 512 == 0, "use_logfmt needs hidden %% 512 == 0 (got %d)", a->hidden);
    LLCombineParams p{};
    p.S = a->num_src_ranks; p.src_rank_begin = a->src_rank_begin; p.src_token_stride = a->src_token_stride;
    p.num_tokens_per_src = a->num_tokens_per_src;
    p.H = a->hidden; p.K = a->num_topk; p.E = a->num_experts;
    p.expert_begin = a->expert_begin; p.E_l = a->num_local_experts; p.R = a->num_ranks;
    p.M = a->num_max_dispatch_tokens_per_rank;
    p.x = static_cast<const uint8_t*>(a->x);
    p.topk_idx = a->topk_idx;
    p.topk_weights = a->topk_weights;
    p.src_info = a->packed_recv_src_info;
    p.layout_range = a->packed_recv_layout_range;
    p.lane_slot = a->lane_rows;
    p.out = static_cast<uint8_t*>(a->combined_x);
    p.status = reinterpret_cast<int32_t*>(a->workspace);
    p.vecs = a->tuning.ll_combine_vecs;
    p.use_logfmt = a->use_logfmt ? 1 : 0;
    hipError_t err = launch_ll_combine(p, static_cast<hipStream_t>(stream));
    if (err != hipSuccess) return hip_fail(err, "low-latency combine launch");
    return DEEP_EP_HIP_OK;
}

int deep_ep_hip_launch_cast_fp8(const deep_ep_hip_cast_args* a, void* stream) {
    REQUIRE(a != nullptr, "args is NULL");
    REQUIRE(a->num_tokens >= 0 && a->hidden >= 1, "bad shape");
    REQUIRE(a->num_tokens == 0 || (a->x != nullptr && a->out != nullptr && a->scales != nullptr), "NULL tensor");
    CastParams p{static_cast<const uint8_t*>(a->x), static_cast<uint8_t*>(a->out), a->scales, a->num_tokens, a->hidden};
    hipError_t err = launch_cast_kernel(p, static_cast<hipStream_t>(stream));
    if (err != hipSuccess) return hip_fail(err, "cast launch");
    return DEEP_EP_HIP_OK;
}

}  // extern "C"
