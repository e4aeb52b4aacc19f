// Host side of libmoe355: handle, workspace carving, stage sequencing.  No device memory is allocated here;
// the caller owns every buffer (the reference carves one stream-ordered arena per driver, mma.cuh:385-391,
// combine.cuh:214-224 -- the same idea, made the caller's).
#include <algorithm>
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "moe_internal.hpp"

namespace moe355 {

// per-dtype pieces defined next to their kernels
int bf16_tile(int64_t pairs, int experts, int H, int I, int swiglu, int opt_block_rows, int opt_tile);
int bf16_block_m(int tile);
int bf16_block_n0(int tile);
int bf16_block_n1(int tile);
int f32_block_m();
int f32_block_n();
hipError_t launch_ffn_tiled_bf16(const FfnArgs&, int tile, int max_mtiles, int nnt0, int nnt1, hipStream_t, bool f16);
hipError_t launch_ffn_persistent_bf16(const FfnArgs&, int tile, int blocks, bool early, hipStream_t, bool f16);
int ffn_persistent_occupancy_bf16(int tile);
hipError_t launch_gemm_dense_bf16(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t, int,
                                  int opt_tile, hipStream_t, bool f16);
hipError_t launch_ffn_tiled_f32(const FfnArgs&, int max_mtiles, int nnt0, int nnt1, hipStream_t);
hipError_t launch_ffn_persistent_f32(const FfnArgs&, int blocks, hipStream_t);
hipError_t launch_gemm_dense_f32(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t, int,
                                 hipStream_t);
hipError_t launch_ffn_fp8(const FfnArgs&, int max_mtiles, int nnt0, int nnt1, int blocks, hipStream_t);
int fp8_block_m();
int fp8_block_n0(int swiglu);
int fp8_block_n1();
int ffn_persistent_occupancy_fp8();
hipError_t launch_ffn_fp8_tile(const FfnArgs&, int max_mtiles, int nnt0, int nnt1, int blocks, hipStream_t);
hipError_t launch_ffn_fp8_mfma(const FfnArgs&, int S, int64_t A, int max_mtiles, int nnt0, int nnt1, hipStream_t);
int fp8_tile_block_m();
int fp8_tile_block_n0(int swiglu);
int fp8_tile_block_n1();
int ffn_persistent_occupancy_fp8_tile();
hipError_t launch_ffn_f32_tile(const FfnArgs&, int max_mtiles, int nnt0, int nnt1, int blocks, hipStream_t);
bool gemm_dense_f32_takes_tile(int64_t M, int64_t N, int64_t K);
hipError_t launch_gemm_dense_f32_tile(const void*, const void*, const void*, void*, int64_t, int64_t, int64_t, int,
                                      hipStream_t);
int f32_tile_block_m();
int f32_tile_block_n0(int swiglu);
int f32_tile_block_n1();
int ffn_persistent_occupancy_f32_tile();

namespace {

constexpr size_t kAlign = 256;
constexpr int kSplitWorkgroups = 256;   // resident workgroups the partial-sum tail is sized for (one per compute unit of a whole MI355X)
size_t align_up(size_t v) { return (v + kAlign - 1) / kAlign * kAlign; }
int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

struct Derived {
    bool wide_in_workspace;   // the widened weight copies live in the workspace (false: the caller brings prepared ones)
    int S, H, I, E, k, A;
    int act_dtype;     // MOE_DTYPE_F32, MOE_DTYPE_BF16 or MOE_DTYPE_FP16
    size_t act_bytes;
    int64_t capacity;
    FfnPlan plan;
    int nblk;          // workgroups of the slot-assignment kernels
    int wide_mats;     // weight matrices per expert (3 with SwiGLU, else 2)
    int max_mtiles;
};

struct WsLayout {
    size_t logits, topk_idx, topk_w, slot, pair_row, token_indices, expert_count, expert_offset, rank_local,
        block_hist, mtiles, seg0, seg1, segq, qstate, cstate, done0, done1, pair_mt, wg_clock, arrive, stats_prob, stats_cnt, h, y,
        wide, xq, sx, hq, sh, split_cnt, split_part, total;
};

// Storage type of activations (x, biases, h, y, out): the layer's own, except that tf32 -- fp32 storage with
// reduced-precision multiplies in the reference (processor/tiling.cuh:131-143) -- is stored and computed as fp32 here
// (gfx950 has no tf32 matrix instruction; full fp32 is the superset), and e4m3 layers keep bf16 activations.
int act_dtype_of(int torch_dtype) {
    if (torch_dtype == MOE_DTYPE_F32 || torch_dtype == MOE_DTYPE_TF32) return MOE_DTYPE_F32;
    return torch_dtype == MOE_DTYPE_FP16 ? MOE_DTYPE_FP16 : MOE_DTYPE_BF16;
}

int check_supported(const moe_config& c) {
    if (c.num_experts > kMaxExperts || c.expert_top_k > kMaxTopK) return MOE_ERR_UNSUPPORTED;
    if (c.torch_dtype == MOE_DTYPE_FP8_E4M3_B128 && (c.hidden_size % 128 || c.intermediate_size % 128))
        return MOE_ERR_UNSUPPORTED;     // one scale per 128 x 128 block of a weight matrix
    if (c.hidden_size > 16384) return MOE_ERR_UNSUPPORTED;   // the router keeps a token row in registers
    return MOE_OK;
}

int derive(const moe_config& c, const moe_options& o, Derived* d) {
    int rc = moe_config_validate(&c, nullptr, 0);
    if (rc) return rc;
    rc = check_supported(c);
    if (rc) return rc;
    d->S = (int)moe_config_tokens(&c);
    d->H = c.hidden_size;
    d->I = c.intermediate_size;
    d->E = c.num_experts;
    d->k = c.expert_top_k;
    d->A = d->S * d->k;
    d->act_dtype = act_dtype_of(c.torch_dtype);
    d->act_bytes = d->act_dtype == MOE_DTYPE_F32 ? 4 : 2;
    moe_config_capacity(&c, &d->capacity);
    if (d->capacity > d->A) d->capacity = d->A;
    d->plan = ffn_plan(c.torch_dtype, c.hidden_act, d->H, d->I, d->A, d->E, o);
    d->wide_mats = c.hidden_act == MOE_ACT_SWIGLU ? 3 : 2;
    d->wide_in_workspace = d->plan.widen && o.prepared_weights != 1;
    d->nblk = ceil_div(d->A, kRouteBlock);
    d->max_mtiles = ceil_div(d->A, d->plan.block_m) + d->E;
    return MOE_OK;
}

WsLayout layout(const Derived& d) {
    WsLayout w;
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes); return o; };
    w.logits = take((size_t)d.S * d.E * 4);
    w.topk_idx = take((size_t)d.A * 4);
    w.topk_w = take((size_t)d.A * 4);
    w.slot = take((size_t)d.A * 4);
    w.pair_row = take((size_t)d.A * 4);
    w.token_indices = take((size_t)d.A * 4);
    w.expert_count = take((size_t)d.E * 4);
    w.expert_offset = take((size_t)(d.E + 1) * 4);
    w.rank_local = take((size_t)d.A * 4);
    w.block_hist = take((size_t)d.nblk * d.E * 4);
    w.mtiles = take((size_t)d.max_mtiles * sizeof(MTile));
    w.seg0 = take((size_t)d.E * sizeof(Segment));
    w.seg1 = take((size_t)(d.E + 1) * sizeof(Segment));       // one more: split_tail cuts a segment in two
    w.segq = take((size_t)(2 * d.E + 1) * sizeof(Segment));   // one more: round_tail or split_tail cuts a segment in two
    w.qstate = take(sizeof(QueueState));
    w.cstate = take(sizeof(CombineState));
    w.done0 = take((size_t)d.max_mtiles * 4);
    w.done1 = take((size_t)d.max_mtiles * 4);
    w.pair_mt = take((size_t)d.A * 4);
    w.wg_clock = take((size_t)kMaxQueueWorkgroups * 2 * sizeof(int64_t));
    w.arrive = take((size_t)d.S * d.plan.nnt1 * 4);
    w.stats_prob = take((size_t)kStatsBlocks * d.E * 8);
    w.stats_cnt = take((size_t)kStatsBlocks * d.E * 4);
    w.h = take((size_t)d.A * d.I * d.act_bytes);
    w.y = take((size_t)d.A * d.H * d.act_bytes);
    // bf16 copies of an e4m3 layer's expert weights (up, down, gate), rewritten by every call of such a plan
    w.wide = take(d.wide_in_workspace ? (size_t)d.wide_mats * d.E * d.I * d.H * 2 : 0);
    // e4m3 x e4m3 plan: token rows and intermediate rows as e4m3 codes + one fp32 scale per (row, 128 columns)
    const bool m8 = d.plan.mfma8;
    w.xq = take(m8 ? (size_t)d.S * d.H : 0);
    w.sx = take(m8 ? (size_t)d.S * (d.H / 128) * 4 : 0);
    w.hq = take(m8 ? (size_t)d.A * d.I : 0);
    w.sh = take(m8 ? (size_t)d.A * (d.I / 128) * 4 : 0);
    // down-projection tiles computed as partial sums: a counter and ksplit fp32 copies of the tile for each
    const size_t split_tiles = d.plan.ksplit > 1 ? (size_t)d.plan.tail_blocks * d.plan.nnt1 : 0;
    w.split_cnt = take(split_tiles * 4);
    w.split_part = take(split_tiles * d.plan.ksplit * ((size_t)d.plan.block_m * bf16_block_n1(d.plan.tile)) * 4);
    w.total = off;
    return w;
}

}  // namespace

FfnPlan ffn_plan(int dtype, int act, int H, int I, int64_t A, int E, const moe_options& o) {
    FfnPlan p;
    p.tile = 0;
    p.kernel_dtype = dtype;
    p.widen = false;
    p.mfma8 = false;
    p.ksplit = 1;
    p.tail_blocks = 0;
    const bool sw = act == MOE_ACT_SWIGLU;
    if (dtype == MOE_DTYPE_FP8_E4M3_B128) {
        // With this many rows per expert one more pass over the weights (e4m3 -> bf16 into the workspace) costs less
        // than the e4m3 tile GEMM loses to the bf16 one.
        p.widen = A / (E > 0 ? E : 1) >= kFp8WidenRowsPerExpert;
        if (o.fp8_widen != MOE_OPT_AUTO) p.widen = o.fp8_widen != 0;
        if (o.fp8_mfma == 1) p.widen = false;             // asked for the e4m3 x e4m3 tile GEMM: the weights stay as stored
        if (p.widen) p.kernel_dtype = dtype = MOE_DTYPE_BF16;
    }
    if (dtype == MOE_DTYPE_F32 || dtype == MOE_DTYPE_TF32) {
        // 0: 64 x 64 tiles on the vector ALUs (small and ragged layers); 1: 128 x 128 tiles on the matrix cores
        // (from a full row block per expert on average, and enough 128 x 128 tiles to occupy the compute units twice over:
        // below that the smaller tiles of the vector kernel spread the same work over more of the chip)
        const int64_t tiles = (A / f32_tile_block_m()) * (ceil_div(I, f32_tile_block_n0(sw)) + ceil_div(H, f32_tile_block_n1()));
        p.tile = H % 128 == 0 && I % 128 == 0 && A / (E > 0 ? E : 1) >= kF32TileRowsPerExpert && tiles >= kF32TileMinTiles ? 1 : 0;
        if (o.f32_tile == 0 || (o.f32_tile == 1 && H % 128 == 0 && I % 128 == 0)) p.tile = o.f32_tile;
        if (p.tile) {
            p.block_m = f32_tile_block_m();
            p.nnt0 = ceil_div(I, f32_tile_block_n0(sw));
            p.nnt1 = ceil_div(H, f32_tile_block_n1());
        } else {
            p.block_m = f32_block_m();
            p.nnt0 = sw ? ceil_div(I, f32_block_n() / 2) : ceil_div(I, f32_block_n());
            p.nnt1 = ceil_div(H, f32_block_n());
        }
    } else if (dtype == MOE_DTYPE_FP8_E4M3_B128) {
        // 0: weight streamer over 16-token row blocks (decode); 1: 128 x 128 tile GEMM once the experts see enough
        // rows for a weight tile to be reused from LDS instead of being fetched again per 16 rows
        p.tile = A / (E > 0 ? E : 1) >= kFp8TileRowsPerExpert ? 1 : 0;
        if (o.fp8_tile != MOE_OPT_AUTO) p.tile = o.fp8_tile;
        if (o.fp8_mfma == 1) p.tile = 1, p.mfma8 = true;   // tokens quantised per (row, 128 columns), fp8 matrix instructions
        p.block_m = p.tile ? fp8_tile_block_m() : fp8_block_m();
        p.nnt0 = ceil_div(I, p.tile ? fp8_tile_block_n0(sw) : fp8_block_n0(sw));
        p.nnt1 = ceil_div(H, p.tile ? fp8_tile_block_n1() : fp8_block_n1());
    } else {
        p.tile = bf16_tile(A, E, H, I, sw, o.block_rows, o.tile16);
        p.block_m = bf16_block_m(p.tile);
        p.nnt0 = sw ? ceil_div(I, bf16_block_n0(p.tile) / 2) : ceil_div(I, bf16_block_n0(p.tile));
        p.nnt1 = ceil_div(H, bf16_block_n1(p.tile));
        // Partial sums for the down-projection tiles of the last row blocks: F tasks of a 1/F of the contraction
        // dimension each (the hand-ordered slab loop takes multiples of 128).  How many row blocks: the workgroups reach
        // the short tasks spread over the length of a long one, F short ones; F / 2 rounds of short tasks absorb that
        // spread on average, one more round is the tail proper.  Sized for kSplitWorkgroups resident workgroups whatever
        // the device has (the workspace size must not depend on the device).
        const int F = o.tail_split == 2 || o.tail_split == 4 ? o.tail_split : 1;
        if (F > 1 && p.tile != 0 && I % (128 * F) == 0 && o.combine <= 0 && o.queue_early != 1) {
            p.ksplit = F;
            p.tail_blocks = ceil_div((int64_t)(F / 2 + 1) * kSplitWorkgroups, (int64_t)p.nnt1 * F);
        }
    }
    return p;
}

}  // namespace moe355

using namespace moe355;

constexpr int kTimedCalls = 64;
constexpr int kDefaultSpinLimit = 1 << 24;   // polls (with a short sleep each) of a dependency wait: many seconds

struct moe_handle {
    moe_config cfg;
    Derived d;
    WsLayout ws;
    moe_arch arch;
    moe_options opt;       // the options in force, every AUTO resolved (moe_get_options)
    int ffn_mode;
    int queue_groups;      // task queues of the FFN stage: one per XCD, or 1
    int queue_lag;         // experts of up-projection work between an expert's two projections in the queue
    int row_chunk;         // task order inside a queue segment (FfnArgs::row_chunk)
    int64_t* task_trace;   // the caller's device buffer for per-task records of the queue kernel, or null
    int task_trace_cap;    // records it holds
    int combine_mode;      // 0: a launch of its own, 1: arrival counters inside the FFN kernels, 2: tasks of the FFN queue
    int wall_clock_khz;    // rate of the constant clock the queue kernels stamp their entry and exit with
    int spin_limit;        // polls a dependency wait of the queue kernel makes before it gives up
    int32_t* stall_host;   // pinned host word the queue kernel sets when such a wait expired (never cleared by a kernel)
    int timing;
    // stage timing: a ring of kTimedCalls x (MOE_STAGE_COUNT + 1) events, one row per moe_forward call
    hipEvent_t ev[kTimedCalls][MOE_STAGE_COUNT + 1];
    bool ev_valid;
    int64_t ev_calls;      // calls recorded since timing was enabled
    int last_hip;
};

// ---- the workspace of moe_forward_static: one array per GPU, owned by the code object, never allocated or freed ----
// In host code the array's name is only a handle for hipGetSymbolAddress; the address the kernels need is looked up
// once per device (with that device current) and kept in g_scratch_ptr.
constexpr size_t kStaticScratchBytes = MOE355_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];
static hipError_t g_scratch_err[kMaxDevices];
static bool g_scratch_done[kMaxDevices];
static std::mutex g_scratch_mutex;

// Looks up this device's copy of `scratch` (the device must be current).  Called from moe_create.
static void resolve_static_scratch(int dev) {
    if (dev < 0 || dev >= kMaxDevices) return;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_done[dev]) return;
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    g_scratch_err[dev] = e;
    g_scratch_ptr[dev] = e == hipSuccess ? ptr : nullptr;
    g_scratch_done[dev] = true;
}

namespace {

int hip_fail(moe_handle* h, hipError_t e) {
    if (h) h->last_hip = (int)e;
    return MOE_ERR_HIP;
}

int check_ws(const moe_handle* h, const void* ws, size_t bytes) {
    if (!ws || ((uintptr_t)ws % kAlign) || bytes < h->ws.total) return MOE_ERR_WORKSPACE;
    return MOE_OK;
}

template <typename T>
T* at(void* ws, size_t off) { return reinterpret_cast<T*>(static_cast<char*>(ws) + off); }

int resolved_ffn_mode(const moe_handle* h);

RouteArgs route_args(const moe_handle* h, void* ws) {
    const Derived& d = h->d;
    const WsLayout& w = h->ws;
    RouteArgs a{};
    a.topk_idx = at<int32_t>(ws, w.topk_idx);
    a.rank_local = at<int32_t>(ws, w.rank_local);
    a.block_hist = at<int32_t>(ws, w.block_hist);
    a.slot = at<int32_t>(ws, w.slot);
    a.pair_row = at<int32_t>(ws, w.pair_row);
    a.token_indices = at<int32_t>(ws, w.token_indices);
    a.expert_count = at<int32_t>(ws, w.expert_count);
    a.expert_offset = at<int32_t>(ws, w.expert_offset);
    a.mtiles = at<MTile>(ws, w.mtiles);
    a.seg_phase0 = at<Segment>(ws, w.seg0);
    a.seg_phase1 = at<Segment>(ws, w.seg1);
    a.seg_queue = at<Segment>(ws, w.segq);
    a.q = at<QueueState>(ws, w.qstate);
    a.done0 = at<int32_t>(ws, w.done0);
    // arrival counters [S, nnt1] of the combine inside the FFN kernels, or the flags [S * slices] of the combine tasks of
    // the queue (a slice is at least 1024 columns, a column tile at most 256: the flags fit the same array); the latter
    // exist in task-queue mode only
    const bool queue_combine = h->combine_mode == 2 && resolved_ffn_mode(h) == MOE_FFN_PERSISTENT;
    a.arrive = (h->combine_mode == 1 || queue_combine) ? at<int32_t>(ws, w.arrive) : nullptr;
    a.arrive_n = d.S * d.plan.nnt1;
    a.done1 = queue_combine ? at<int32_t>(ws, w.done1) : nullptr;
    a.pair_mt = queue_combine ? at<int32_t>(ws, w.pair_mt) : nullptr;
    a.cs = queue_combine ? at<CombineState>(ws, w.cstate) : nullptr;
    a.task_trace = h->task_trace;
    a.S = d.S; a.k = d.k; a.E = d.E; a.A = d.A; a.nblk = d.nblk;
    a.drop = h->cfg.drop_tokens;
    a.capacity = (int)d.capacity;
    a.block_m = d.plan.block_m;
    a.nnt0 = d.plan.nnt0;
    a.nnt1 = d.plan.nnt1;
    a.max_mtiles = d.max_mtiles;
    a.lag = h->queue_lag;
    a.groups = h->queue_groups;
    a.tail_workgroups = h->opt.tail_round == 0 ? 0 : h->arch.persistent_blocks;
    if (d.plan.ksplit > 1) {
        a.tail_split = d.plan.ksplit;
        a.tail_blocks = d.plan.tail_blocks;
        a.split_cnt = at<int32_t>(ws, w.split_cnt);
    }
    return a;
}

// The mode a forward call runs in.  The queue pays off once there are more tasks than resident workgroups; tiny
// layers launch once per projection.  Row blocks are estimated on the host as the larger of kept rows / block rows
// and the experts that can be hit at all (every hit expert owns at least one row block).
int resolved_ffn_mode(const moe_handle* h) {
    // the e4m3 x e4m3 plan quantises the intermediate rows between the projections: always one launch per projection
    if (h->d.plan.mfma8) return MOE_FFN_TILED;
    if (h->ffn_mode != MOE_FFN_AUTO) return h->ffn_mode;
    const Derived& d = h->d;
    int64_t row_blocks = d.A / d.plan.block_m + 1;
    const int64_t hit = d.A < d.E ? d.A : d.E;
    if (row_blocks < hit) row_blocks = hit;
    const int64_t est_tasks = row_blocks * (d.plan.nnt0 + d.plan.nnt1);
    // The queue pays off from a couple of tasks per resident workgroup on.  The fp32 matrix-core tile has long tasks
    // (a down-projection tile of the reference's knob file takes half a millisecond) and needs twice that to balance:
    // 4096 tokens of that file, 2.6 tasks per workgroup, take 0.79 ms on the queue and 0.60 ms as two launches.
    const bool f32_tile = (d.plan.kernel_dtype == MOE_DTYPE_F32 || d.plan.kernel_dtype == MOE_DTYPE_TF32) && d.plan.tile;
    // With a single expert the queue has no second expert's up projection to run beside the down projection: it is the
    // two launches plus dependency waits and written-through intermediate rows (the reference's knob file: 1.13 ms
    // against 1.03-1.10 ms as two launches; the same file in bf16 0.183 against 0.170 ms; the Mixtral dimensions with one
    // expert: no difference).
    const bool tile16 = d.plan.kernel_dtype == MOE_DTYPE_BF16 || d.plan.kernel_dtype == MOE_DTYPE_FP16;
    if ((f32_tile || tile16) && d.E == 1) return MOE_FFN_TILED;
    return est_tasks >= (f32_tile ? 4 : 2) * (int64_t)h->arch.persistent_blocks ? MOE_FFN_PERSISTENT : MOE_FFN_TILED;
}

}  // namespace

extern "C" {

// ---- options ----
namespace {
struct OptField {
    const char* name;            // field name; the environment variable is MOE355_ + upper case
    int32_t moe_options::*ptr;
    int lo, hi;                  // domain (besides MOE_OPT_AUTO)
    bool pow2;                   // only powers of two
};
const OptField kOptFields[] = {
    {"tile16", &moe_options::tile16, 0, 3, false},
    {"block_rows", &moe_options::block_rows, 128, 256, true},
    {"f32_tile", &moe_options::f32_tile, 0, 1, false},
    {"fp8_tile", &moe_options::fp8_tile, 0, 1, false},
    {"fp8_widen", &moe_options::fp8_widen, 0, 1, false},
    {"queue_groups", &moe_options::queue_groups, 1, kMaxQueueGroups, true},
    {"queue_lag", &moe_options::queue_lag, 1, kMaxExperts, false},
    {"queue_early", &moe_options::queue_early, 0, 1, false},
    {"row_chunk", &moe_options::row_chunk, 0, 4096, false},
    {"blocks_per_cu", &moe_options::blocks_per_cu, 1, 16, false},
    {"combine", &moe_options::combine, 0, 2, false},
    {"gate_kernel", &moe_options::gate_kernel, 0, 1, false},
    {"gate_mfma", &moe_options::gate_mfma, 0, 1, false},
    {"gate_tile", &moe_options::gate_tile, 0, 2, false},
    {"gate_fused_topk", &moe_options::gate_fused_topk, 0, 1, false},
    {"grouped_tile", &moe_options::grouped_tile, 0, 2, false},
    {"tail_round", &moe_options::tail_round, 0, 1, false},
    {"fp8_mfma", &moe_options::fp8_mfma, 0, 1, false},
    {"prepared_weights", &moe_options::prepared_weights, 0, 1, false},
    {"tail_split", &moe_options::tail_split, 1, 4, true},
};
bool opt_in_domain(const OptField& f, int v) {
    if (v == MOE_OPT_AUTO) return true;
    if (v < f.lo || v > f.hi) return false;
    return !f.pow2 || (v & (v - 1)) == 0;
}
int check_options(const moe_options& o) {
    for (const OptField& f : kOptFields)
        if (!opt_in_domain(f, o.*(f.ptr))) return MOE_ERR_BAD_ARGUMENT;
    for (int32_t r : o.reserved)
        if (r != MOE_OPT_AUTO) return MOE_ERR_BAD_ARGUMENT;
    return MOE_OK;
}
// The options of the entry points that take none: defaults, then the environment.
moe_options ambient_options() {
    moe_options o;
    moe_options_default(&o);
    moe_options_from_env(&o);
    return o;
}
}  // namespace

int moe_options_default(moe_options* opt) {
    if (!opt) return MOE_ERR_BAD_ARGUMENT;
    for (const OptField& f : kOptFields) opt->*(f.ptr) = MOE_OPT_AUTO;
    for (int32_t& r : opt->reserved) r = MOE_OPT_AUTO;
    return MOE_OK;
}

int moe_options_from_env(moe_options* opt) {
    if (!opt) return MOE_ERR_BAD_ARGUMENT;
    for (const OptField& f : kOptFields) {
        char var[64] = "MOE355_";
        size_t n = strlen(var);
        for (const char* c = f.name; *c && n + 1 < sizeof var; ++c) var[n++] = (char)(*c >= 'a' && *c <= 'z' ? *c - 32 : *c);
        var[n] = 0;
        const char* env = getenv(var);
        if (!env || !*env) continue;
        char* endp = nullptr;
        const long v = strtol(env, &endp, 10);
        if (endp == env || *endp) continue;                       // not a number: ignored
        if (v >= INT32_MIN && v <= INT32_MAX && opt_in_domain(f, (int)v)) opt->*(f.ptr) = (int32_t)v;
    }
    return MOE_OK;
}

int moe_workspace_bytes_with_options(const moe_config* cfg, const moe_options* opt, size_t* bytes) {
    if (!cfg || !bytes || !opt) return MOE_ERR_BAD_ARGUMENT;
    int rc = check_options(*opt);
    if (rc) return rc;
    Derived d;
    rc = derive(*cfg, *opt, &d);
    if (rc) return rc;
    *bytes = layout(d).total;
    return MOE_OK;
}

int moe_workspace_bytes(const moe_config* cfg, size_t* bytes) {
    const moe_options o = ambient_options();
    return moe_workspace_bytes_with_options(cfg, &o, bytes);
}

int moe_create(const moe_config* cfg, moe_handle** out) {
    const moe_options o = ambient_options();
    return moe_create_with_options(cfg, &o, out);
}

int moe_create_with_options(const moe_config* cfg, const moe_options* opt, moe_handle** out) {
    if (!cfg || !out || !opt) return MOE_ERR_BAD_ARGUMENT;
    *out = nullptr;
    int rc = check_options(*opt);
    if (rc) return rc;
    Derived d;
    rc = derive(*cfg, *opt, &d);
    if (rc) return rc;
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) return MOE_ERR_NO_DEVICE;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return MOE_ERR_NO_DEVICE;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return MOE_ERR_NO_DEVICE;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return MOE_ERR_NO_DEVICE;   // the only code object we carry
    moe_handle* h = new (std::nothrow) moe_handle();
    if (!h) return MOE_ERR_BAD_ARGUMENT;
    h->cfg = *cfg;
    h->d = d;
    h->ws = layout(d);
    h->opt = *opt;
    h->ffn_mode = MOE_FFN_AUTO;
    h->timing = 0;
    h->ev_valid = false;
    h->ev_calls = 0;
    h->last_hip = 0;
    memset(&h->arch, 0, sizeof h->arch);
    h->arch.device = dev;
    h->arch.compute_units = prop.multiProcessorCount;
    // A gfx950 XCD has 32 active compute units; a partitioned device (CPX / DPX / QPX modes) shows fewer CUs and
    // fewer XCDs.  Queues are built per XCD, and a queue nobody calls home would starve (ffn_common.hpp), so the
    // count follows what this device really has: 8 on a whole MI355X, 1 on a single-XCD partition.
    {
        int x = prop.multiProcessorCount / 32, p2 = 1;
        while (p2 * 2 <= x && p2 < kMaxQueueGroups) p2 *= 2;
        h->arch.xcds = p2;
    }
    h->arch.wavefront_size = prop.warpSize;
    h->arch.lds_bytes_per_cu = (int)prop.maxSharedMemoryPerMultiProcessor;
    h->arch.max_clock_khz = prop.clockRate;
    if (hipDeviceGetAttribute(&h->wall_clock_khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || h->wall_clock_khz <= 0)
        h->wall_clock_khz = 100000;   // 100 MHz on gfx950
    snprintf(h->arch.name, sizeof h->arch.name, "%s", prop.gcnArchName);
    const int kdt = d.plan.kernel_dtype;
    const bool tile16 = kdt == MOE_DTYPE_BF16 || kdt == MOE_DTYPE_FP16;
    int per_cu = ffn_persistent_blocks(kdt, d.plan.tile, 1);
    if (opt->blocks_per_cu != MOE_OPT_AUTO) per_cu = opt->blocks_per_cu;    // resident workgroups per CU
    h->arch.persistent_blocks = prop.multiProcessorCount * per_cu;
    // One task queue per XCD for the MFMA-bound bf16 tiles, whose operand tiles are then shared in that XCD's L2;
    // so does the e4m3 tile GEMM; the fp32 kernels (the matrix-core tile measured 5 % faster on one queue than on eight)
    // and the e4m3 weight streamer keep a single queue.
    h->queue_groups = (tile16 || (kdt == MOE_DTYPE_FP8_E4M3_B128 && d.plan.tile)) ? h->arch.xcds : 1;
    if (opt->queue_groups != MOE_OPT_AUTO && opt->queue_groups <= h->arch.xcds) h->queue_groups = opt->queue_groups;   // never more queues than XCDs
    if (h->queue_groups > h->arch.persistent_blocks) h->queue_groups = 1;   // every queue needs a home workgroup
    // The e4m3 tile GEMM holds 64 workgroups per XCD on 128 x 128 tiles whose token rows (bf16) take twice the L2 space
    // of their weight rows (e4m3): two row blocks at a time, all of a queue's column tiles of those (measured on the
    // Mixtral shape with e4m3 weights: 6.57 ms against 6.96 with all row blocks of the expert at a time; 1: 6.62,
    // 4: 6.76, 8: 6.89).  The bf16 tiles are indifferent (within 1 %) and keep the plain order.
    h->row_chunk = (kdt == MOE_DTYPE_FP8_E4M3_B128 && d.plan.tile) ? 2 : 0;
    if (opt->row_chunk != MOE_OPT_AUTO) h->row_chunk = opt->row_chunk;
    {   // phase-0 tasks an average expert contributes; enough experts of them to cover four tasks per workgroup
        const int64_t avg_mt = d.A / ((int64_t)d.E * d.plan.block_m) > 0 ? d.A / ((int64_t)d.E * d.plan.block_m) : 1;
        const int64_t per_expert = avg_mt * d.plan.nnt0;
        int64_t lag = (4 * (int64_t)h->arch.persistent_blocks + per_expert - 1) / per_expert;
        if (lag < 1) lag = 1;
        if (opt->queue_lag != MOE_OPT_AUTO) lag = opt->queue_lag;
        if (lag > d.E) lag = d.E;
        h->queue_lag = (int)lag;
    }
    // Combine: a launch of its own unless asked otherwise.  Inside the FFN kernels by arrival counters it is bit-identical
    // and measured slower on every shape (Mixtral shape +2.9 % per step, 16 experts of 512 rows +14 %, 64 small experts
    // +18 %, decode +0.9 %): the workgroup that completes a token holds a whole compute unit while it gathers k rows
    // at memory latency, where the separate launch does the same gather with the whole chip's occupancy in 8-38 us.
    h->combine_mode = opt->combine == MOE_OPT_AUTO ? 0 : opt->combine;
    if (d.plan.mfma8) h->combine_mode = 0;                // that plan's kernels leave the combine to its own launch
    h->spin_limit = kDefaultSpinLimit;
    h->task_trace = nullptr;
    h->task_trace_cap = 0;
    h->stall_host = nullptr;
    {   // host memory, allocated once per handle; the hot path never allocates
        void* p = nullptr;
        const hipError_t e = hipHostMalloc(&p, sizeof(int32_t), hipHostMallocDefault);
        if (e != hipSuccess) { delete h; return MOE_ERR_HIP; }
        h->stall_host = static_cast<int32_t*>(p);
        *h->stall_host = 0;
    }
    // what moe_get_options reports: the values in force
    h->opt.tile16 = tile16 ? d.plan.tile : MOE_OPT_AUTO;
    h->opt.block_rows = tile16 ? d.plan.block_m : MOE_OPT_AUTO;
    h->opt.f32_tile = (kdt == MOE_DTYPE_F32 || kdt == MOE_DTYPE_TF32) ? d.plan.tile : MOE_OPT_AUTO;
    h->opt.fp8_tile = kdt == MOE_DTYPE_FP8_E4M3_B128 ? d.plan.tile : MOE_OPT_AUTO;
    h->opt.fp8_widen = cfg->torch_dtype == MOE_DTYPE_FP8_E4M3_B128 ? (int)d.plan.widen : MOE_OPT_AUTO;
    h->opt.queue_groups = h->queue_groups;
    h->opt.queue_lag = h->queue_lag;
    h->opt.queue_early = opt->queue_early == 1 && tile16 && d.plan.tile == 1 ? 1 : 0;
    h->opt.row_chunk = h->row_chunk;
    h->opt.blocks_per_cu = per_cu;
    h->opt.combine = h->combine_mode;
    h->opt.prepared_weights = d.plan.widen && !d.wide_in_workspace ? 1 : 0;
    h->opt.fp8_mfma = cfg->torch_dtype == MOE_DTYPE_FP8_E4M3_B128 ? (int)d.plan.mfma8 : MOE_OPT_AUTO;
    h->opt.tail_split = tile16 ? d.plan.ksplit : MOE_OPT_AUTO;
    resolve_static_scratch(dev);
    *out = h;
    return MOE_OK;
}

int moe_get_options(const moe_handle* h, moe_options* opt) {
    if (!h || !opt) return MOE_ERR_BAD_ARGUMENT;
    *opt = h->opt;
    return MOE_OK;
}

int moe_get_workspace_bytes(const moe_handle* h, size_t* bytes) {
    if (!h || !bytes) return MOE_ERR_BAD_ARGUMENT;
    *bytes = h->ws.total;
    return MOE_OK;
}

int moe_destroy(moe_handle* h) {
    if (!h) return MOE_OK;
    if (h->ev_valid)
        for (auto& row : h->ev)
            for (auto& e : row) (void)hipEventDestroy(e);
    if (h->stall_host) (void)hipHostFree(h->stall_host);
    delete h;
    return MOE_OK;
}

int moe_get_arch(const moe_handle* h, moe_arch* out) {
    if (!h || !out) return MOE_ERR_BAD_ARGUMENT;
    *out = h->arch;
    return MOE_OK;
}

int moe_get_plan(const moe_handle* h, int32_t* block_rows, int32_t* col_tiles_up, int32_t* col_tiles_down) {
    if (!h) return MOE_ERR_BAD_ARGUMENT;
    if (block_rows) *block_rows = h->d.plan.block_m;
    if (col_tiles_up) *col_tiles_up = h->d.plan.nnt0;
    if (col_tiles_down) *col_tiles_down = h->d.plan.nnt1;
    return MOE_OK;
}

int moe_get_kernel_dtype(const moe_handle* h, int32_t* dtype) {
    if (!h || !dtype) return MOE_ERR_BAD_ARGUMENT;
    *dtype = h->d.plan.kernel_dtype;
    return MOE_OK;
}

int moe_set_ffn_mode(moe_handle* h, int mode) {
    if (!h || mode < MOE_FFN_AUTO || mode > MOE_FFN_PERSISTENT) return MOE_ERR_BAD_ARGUMENT;
    h->ffn_mode = mode;
    return MOE_OK;
}

int moe_get_ffn_mode(const moe_handle* h, int32_t* mode) {
    if (!h || !mode) return MOE_ERR_BAD_ARGUMENT;
    *mode = resolved_ffn_mode(h);
    return MOE_OK;
}

int moe_set_stage_timing(moe_handle* h, int enable) {
    if (!h) return MOE_ERR_BAD_ARGUMENT;
    if (enable && !h->ev_valid) {
        for (auto& row : h->ev)
            for (auto& e : row) {
                hipError_t rc = hipEventCreate(&e);
                if (rc != hipSuccess) return hip_fail(h, rc);
            }
        h->ev_valid = true;
    }
    h->timing = enable ? 1 : 0;
    h->ev_calls = 0;
    return MOE_OK;
}

int moe_get_stage_ms(moe_handle* h, int stage, float* ms, int32_t* calls) {
    if (!h || !ms || stage < 0 || stage >= MOE_STAGE_COUNT) return MOE_ERR_BAD_ARGUMENT;
    if (!h->ev_valid || h->ev_calls < 1) return MOE_ERR_BAD_ARGUMENT;
    const int n = (int)(h->ev_calls < kTimedCalls ? h->ev_calls : kTimedCalls);
    double sum = 0.0;
    for (int i = 0; i < n; ++i) {
        const int row = (int)((h->ev_calls - 1 - i) % kTimedCalls);
        hipError_t rc = hipEventSynchronize(h->ev[row][MOE_STAGE_COUNT]);
        if (rc != hipSuccess) return hip_fail(h, rc);
        float t = 0.0f;
        rc = hipEventElapsedTime(&t, h->ev[row][stage], h->ev[row][stage + 1]);
        if (rc != hipSuccess) return hip_fail(h, rc);
        sum += t;
    }
    *ms = (float)(sum / n);
    if (calls) *calls = n;
    return MOE_OK;
}

int moe_get_stage_samples(moe_handle* h, int stage, float* ms, int32_t capacity, int32_t* count) {
    if (!h || !ms || !count || capacity < 1 || stage < 0 || stage > MOE_STAGE_COUNT) return MOE_ERR_BAD_ARGUMENT;
    if (!h->ev_valid || h->ev_calls < 1) return MOE_ERR_BAD_ARGUMENT;
    int n = (int)(h->ev_calls < kTimedCalls ? h->ev_calls : kTimedCalls);
    if (n > capacity) n = capacity;
    for (int i = 0; i < n; ++i) {   // oldest of the n most recent calls first
        const int row = (int)((h->ev_calls - n + i) % kTimedCalls);
        hipError_t rc = hipEventSynchronize(h->ev[row][MOE_STAGE_COUNT]);
        if (rc != hipSuccess) return hip_fail(h, rc);
        const int a = stage == MOE_STAGE_COUNT ? 0 : stage, b = stage == MOE_STAGE_COUNT ? MOE_STAGE_COUNT : stage + 1;
        rc = hipEventElapsedTime(&ms[i], h->ev[row][a], h->ev[row][b]);
        if (rc != hipSuccess) return hip_fail(h, rc);
    }
    *count = n;
    return MOE_OK;
}

int moe_last_hip_error(const moe_handle* h) { return h ? h->last_hip : 0; }

int moe_gate(moe_handle* h, const void* x, const void* gate_w, const float* gate_bias, float* logits,
             int32_t* topk_idx, float* topk_w, void* workspace, size_t workspace_bytes, void* stream) {
    if (!h || !x || !gate_w || !topk_idx || !topk_w) return MOE_ERR_BAD_ARGUMENT;
    int rc = check_ws(h, workspace, workspace_bytes);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    const Derived& d = h->d;
    float* lg = logits ? logits : at<float>(workspace, h->ws.logits);
    const hipError_t e = launch_gate(x, gate_w, gate_bias, lg, logits != nullptr, d.S, d.H, d.E, d.k, h->cfg.gate_fn,
                                     h->cfg.norm_topk_prob, topk_idx, topk_w, d.act_dtype, h->opt, st);
    if (e != hipSuccess) return hip_fail(h, e);
    return MOE_OK;
}

int moe_router_stats(moe_handle* h, const float* logits, const int32_t* topk_idx, float* load, float* mean_prob,
                     float* aux_loss, void* workspace, size_t workspace_bytes, void* stream) {
    if (!h || !logits || !topk_idx || (!load && !mean_prob && !aux_loss)) return MOE_ERR_BAD_ARGUMENT;
    int rc = check_ws(h, workspace, workspace_bytes);
    if (rc) return rc;
    const Derived& d = h->d;
    const hipError_t e = launch_router_stats(logits, topk_idx, d.S, d.E, d.k, h->cfg.gate_fn,
                                             at<double>(workspace, h->ws.stats_prob),
                                             at<int32_t>(workspace, h->ws.stats_cnt), load, mean_prob, aux_loss,
                                             (hipStream_t)stream);
    return e == hipSuccess ? MOE_OK : hip_fail(h, e);
}

int moe_route(moe_handle* h, const int32_t* topk_idx, int32_t* slot, int32_t* expert_count, int32_t* expert_offset,
              int32_t* token_indices, int32_t* pair_row, void* workspace, size_t workspace_bytes, void* stream) {
    if (!h || !topk_idx || !slot || !expert_count || !expert_offset || !token_indices) return MOE_ERR_BAD_ARGUMENT;
    int rc = check_ws(h, workspace, workspace_bytes);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    RouteArgs a = route_args(h, workspace);
    a.topk_idx = topk_idx;
    hipError_t e = launch_route(a, st);
    if (e != hipSuccess) return hip_fail(h, e);
    const Derived& d = h->d;
    struct Copy { void* dst; const void* src; size_t n; };
    const Copy copies[] = {
        {slot, a.slot, (size_t)d.A * 4},
        {expert_count, a.expert_count, (size_t)d.E * 4},
        {expert_offset, a.expert_offset, (size_t)d.E * 4},
        {token_indices, a.token_indices, (size_t)d.A * 4},
        {pair_row, a.pair_row, (size_t)d.A * 4},
    };
    for (const Copy& c : copies) {
        if (!c.dst) continue;
        e = hipMemcpyAsync(c.dst, c.src, c.n, hipMemcpyDeviceToDevice, st);
        if (e != hipSuccess) return hip_fail(h, e);
    }
    return MOE_OK;
}

}  // extern "C"

namespace {

// The bf16 copies of an e4m3 layer's expert weights: [up | down | gate], each [E, N, K].
hipError_t widen_weights(const Derived& d, const moe_weights* w, char* wide, hipStream_t st) {
    const int64_t mat = (int64_t)d.I * d.H;
    const void* src[3] = {w->w_up, w->w_down, w->w_gate};
    const float* scl[3] = {w->s_up, w->s_down, w->s_gate};
    for (int i = 0; i < d.wide_mats; ++i) {
        // w_up and w_gate are [E, I, H], w_down is [E, H, I]
        const hipError_t e = launch_widen_block128(src[i], scl[i], wide + (size_t)i * d.E * mat * 2, d.E, i == 1 ? d.H : d.I,
                                                   i == 1 ? d.I : d.H, st);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// The whole layer on a workspace that has passed check_ws (the caller's, or this device's static array).
int forward_on(moe_handle* h, const void* x, const moe_weights* w, void* out, const moe_routing_out* routing,
               void* workspace, size_t workspace_bytes, void* stream) {
    if (!h || !x || !w || !out) return MOE_ERR_BAD_ARGUMENT;
    // a dependency wait of an earlier call expired: that call's output was poisoned; say so until the caller clears it
    if (*(volatile int32_t*)h->stall_host) return MOE_ERR_QUEUE_STALL;
    {   // the handle's grid size, queue count and (static) workspace belong to the device it was created on
        int dev = -1;
        if (hipGetDevice(&dev) != hipSuccess || dev != h->arch.device) return MOE_ERR_BAD_ARGUMENT;
    }
    const moe_config& c = h->cfg;
    const bool sw = c.hidden_act == MOE_ACT_SWIGLU;
    const bool fp8 = c.torch_dtype == MOE_DTYPE_FP8_E4M3_B128;
    if (!w->gate_w || !w->w_up || !w->w_down) return MOE_ERR_BAD_ARGUMENT;
    if (sw != (w->w_gate != nullptr)) return MOE_ERR_BAD_ARGUMENT;
    if (!sw && w->b_gate) return MOE_ERR_BAD_ARGUMENT;
    if (fp8 && (!w->s_up || !w->s_down || sw != (w->s_gate != nullptr))) return MOE_ERR_BAD_ARGUMENT;
    if (!fp8 && (w->s_up || w->s_down || w->s_gate)) return MOE_ERR_BAD_ARGUMENT;
    if (w->prepared && (!h->d.plan.widen || ((uintptr_t)w->prepared % kAlign))) return MOE_ERR_BAD_ARGUMENT;   // nothing to prepare on this plan
    if (!w->prepared && h->d.plan.widen && !h->d.wide_in_workspace) return MOE_ERR_BAD_ARGUMENT;   // promised at moe_create
    int rc = check_ws(h, workspace, workspace_bytes);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    const Derived& d = h->d;
    const WsLayout& L = h->ws;
    hipError_t e;
    const bool timing = h->timing && h->ev_valid;
    const int ev_row = (int)(h->ev_calls % kTimedCalls);
    auto mark = [&](int i) -> hipError_t { return timing ? hipEventRecord(h->ev[ev_row][i], st) : hipSuccess; };

    if ((e = mark(0)) != hipSuccess) return hip_fail(h, e);
    // ---- gate ----
    float* logits = at<float>(workspace, L.logits);
    int32_t* topk_idx = at<int32_t>(workspace, L.topk_idx);
    float* topk_w = at<float>(workspace, L.topk_w);
    e = launch_gate(x, w->gate_w, w->gate_bias, logits, false, d.S, d.H, d.E, d.k, c.gate_fn, c.norm_topk_prob, topk_idx,
                    topk_w, d.act_dtype, h->opt, st);
    if (e != hipSuccess) return hip_fail(h, e);
    if ((e = mark(1)) != hipSuccess) return hip_fail(h, e);
    // ---- slots, capacity, task tables ----
    const RouteArgs ra = route_args(h, workspace);
    e = launch_route(ra, st);
    if (e != hipSuccess) return hip_fail(h, e);
    if ((e = mark(2)) != hipSuccess) return hip_fail(h, e);
    // ---- expert FFN ----
    FfnArgs fa{};        // every field starts null / zero: a member nobody sets must not reach a kernel as stack garbage
    fa.x = x;
    fa.token_indices = ra.token_indices;
    fa.w_up = w->w_up; fa.w_gate = w->w_gate; fa.w_down = w->w_down;
    fa.b_up = w->b_up; fa.b_gate = w->b_gate; fa.b_down = w->b_down;
    fa.s_up = w->s_up; fa.s_gate = w->s_gate; fa.s_down = w->s_down;
    fa.h = at<char>(workspace, L.h);
    fa.y = at<char>(workspace, L.y);
    fa.mtiles = ra.mtiles;
    fa.groups = ra.groups;
    fa.seg_phase0 = ra.seg_phase0; fa.seg_phase1 = ra.seg_phase1; fa.seg_queue = ra.seg_queue;
    fa.q = ra.q;
    fa.done0 = ra.done0;
    fa.H = d.H; fa.I = d.I; fa.E = d.E;
    fa.act = c.hidden_act;
    fa.spin_limit = h->spin_limit;
    fa.host_stall = h->stall_host;
    fa.wg_clock = at<int64_t>(workspace, L.wg_clock);
    fa.row_chunk = h->row_chunk;
    fa.arrive = ra.done1 ? nullptr : ra.arrive;
    fa.done1 = ra.done1;
    fa.pair_mt = ra.pair_mt;
    fa.combined = ra.done1 ? ra.arrive : nullptr;
    fa.cs = ra.cs;
    if (d.plan.ksplit > 1) {
        fa.split_cnt = ra.split_cnt;
        fa.split_part = at<float>(workspace, L.split_part);
        fa.split_extra_blocks = (d.plan.ksplit - 1) * d.plan.tail_blocks;
    }
    if (d.plan.mfma8) {
        fa.xq = at<uint8_t>(workspace, L.xq);
        fa.sx = at<float>(workspace, L.sx);
        fa.hq = at<uint8_t>(workspace, L.hq);
        fa.sh = at<float>(workspace, L.sh);
    }
    fa.task_trace = h->task_trace;
    fa.task_trace_cap = h->task_trace_cap;
    fa.pair_row = ra.pair_row;
    fa.topk_w = topk_w;
    fa.out = out;
    fa.S = d.S; fa.k = d.k; fa.nnt1 = d.plan.nnt1;
    fa.drop = c.drop_tokens;
    {   // operand extents for the buffer descriptors of the 256-row bf16 tile (chosen only when they fit 32 bits)
        const int64_t es = d.act_bytes;
        fa.x_bytes = (uint32_t)((int64_t)d.S * d.H * es);
        fa.h_bytes = (uint32_t)((int64_t)d.A * d.I * es);
        fa.w_bytes = (uint32_t)((int64_t)d.I * d.H * es);
    }
    const int mode = resolved_ffn_mode(h);
    const int kdt = d.plan.kernel_dtype;
    if (d.plan.widen) {   // the layer's e4m3 weights become bf16 ones; from here on it is a bf16 layer
        // made once by moe_prepare_weights, or by this call in the workspace
        char* wide = w->prepared ? static_cast<char*>(const_cast<void*>(w->prepared)) : at<char>(workspace, L.wide);
        if (!w->prepared) {
            e = widen_weights(d, w, wide, st);
            if (e != hipSuccess) return hip_fail(h, e);
        }
        const void** dst[3] = {&fa.w_up, &fa.w_down, &fa.w_gate};
        for (int i = 0; i < d.wide_mats; ++i) *dst[i] = wide + (size_t)i * d.E * d.I * d.H * 2;
        fa.s_up = fa.s_gate = fa.s_down = nullptr;
    }
    if (d.plan.mfma8) {
        e = launch_ffn_fp8_mfma(fa, d.S, d.A, d.max_mtiles, d.plan.nnt0, d.plan.nnt1, st);
    } else if (kdt == MOE_DTYPE_FP8_E4M3_B128) {
        e = (d.plan.tile ? launch_ffn_fp8_tile : launch_ffn_fp8)(fa, d.max_mtiles, d.plan.nnt0, d.plan.nnt1,
                                                                 mode == MOE_FFN_PERSISTENT ? h->arch.persistent_blocks : 0, st);
    } else if (mode == MOE_FFN_PERSISTENT) {
        e = launch_ffn_persistent(fa, kdt, d.plan, h->arch.persistent_blocks, h->opt.queue_early == 1, st);
    } else {
        e = launch_ffn_tiled(fa, kdt, d.plan, d.max_mtiles, st);
    }
    if (e != hipSuccess) return hip_fail(h, e);
    if ((e = mark(3)) != hipSuccess) return hip_fail(h, e);
    // ---- combine (already done inside the FFN kernels unless that is switched off) ----
    if (!fa.arrive) {   // everything, or what the combine tasks of the queue kernel have left
        e = launch_combine(fa.y, ra.pair_row, topk_w, d.S, d.k, d.H, d.act_dtype, out, fa.combined, st);
        if (e != hipSuccess) return hip_fail(h, e);
    }
    if ((e = mark(4)) != hipSuccess) return hip_fail(h, e);
    if (timing) h->ev_calls += 1;

    if (routing) {
        struct Copy { void* dst; const void* src; size_t n; };
        const Copy copies[] = {
            {routing->topk_idx, topk_idx, (size_t)d.A * 4},
            {routing->topk_w, topk_w, (size_t)d.A * 4},
            {routing->slot, ra.slot, (size_t)d.A * 4},
            {routing->expert_count, ra.expert_count, (size_t)d.E * 4},
            {routing->expert_offset, ra.expert_offset, (size_t)d.E * 4},
            {routing->token_indices, ra.token_indices, (size_t)d.A * 4},
        };
        for (const Copy& cp : copies) {
            if (!cp.dst) continue;
            e = hipMemcpyAsync(cp.dst, cp.src, cp.n, hipMemcpyDeviceToDevice, st);
            if (e != hipSuccess) return hip_fail(h, e);
        }
    }
    return MOE_OK;
}

}  // namespace

extern "C" {

int moe_forward(moe_handle* h, const void* x, const moe_weights* w, void* out, const moe_routing_out* routing,
                void* workspace, size_t workspace_bytes, void* stream) {
    return forward_on(h, x, w, out, routing, workspace, workspace_bytes, stream);
}

int moe_forward_static(moe_handle* h, const void* x, const moe_weights* w, void* out, const moe_routing_out* routing,
                       void* stream) {
    if (!h) return MOE_ERR_BAD_ARGUMENT;
    if (h->ws.total > kStaticScratchBytes) return MOE_ERR_WORKSPACE;   // the layer needs more than the array holds
    const int dev = h->arch.device;
    if (dev < 0 || dev >= kMaxDevices || !g_scratch_done[dev]) return MOE_ERR_NO_DEVICE;
    if (!g_scratch_ptr[dev]) return hip_fail(h, g_scratch_err[dev]);
    return forward_on(h, x, w, out, routing, g_scratch_ptr[dev], kStaticScratchBytes, stream);
}

int moe_prepared_bytes(const moe_handle* h, size_t* bytes) {
    if (!h || !bytes) return MOE_ERR_BAD_ARGUMENT;
    *bytes = h->d.plan.widen ? (size_t)h->d.wide_mats * h->d.E * h->d.I * h->d.H * 2 : 0;
    return MOE_OK;
}

int moe_prepare_weights(moe_handle* h, const moe_weights* w, void* prepared, size_t prepared_bytes, void* stream) {
    if (!h || !w) return MOE_ERR_BAD_ARGUMENT;
    size_t need = 0;
    moe_prepared_bytes(h, &need);
    if (need == 0) return MOE_OK;                       // this plan reads the weights as they are
    if (!prepared || ((uintptr_t)prepared % kAlign) || prepared_bytes < need) return MOE_ERR_WORKSPACE;
    const bool sw = h->cfg.hidden_act == MOE_ACT_SWIGLU;
    if (!w->w_up || !w->w_down || !w->s_up || !w->s_down || sw != (w->w_gate != nullptr) || sw != (w->s_gate != nullptr))
        return MOE_ERR_BAD_ARGUMENT;
    const hipError_t e = widen_weights(h->d, w, static_cast<char*>(prepared), (hipStream_t)stream);
    return e == hipSuccess ? MOE_OK : hip_fail(h, e);
}

int moe_set_spin_limit(moe_handle* h, int32_t polls) {
    if (!h) return MOE_ERR_BAD_ARGUMENT;
    h->spin_limit = polls == 0 ? kDefaultSpinLimit : polls;
    return MOE_OK;
}

int moe_clear_stall(moe_handle* h) {
    if (!h) return MOE_ERR_BAD_ARGUMENT;
    *(volatile int32_t*)h->stall_host = 0;
    return MOE_OK;
}

int moe_get_stall(const moe_handle* h, int32_t* stalled) {
    if (!h || !stalled) return MOE_ERR_BAD_ARGUMENT;
    *stalled = *(volatile int32_t*)h->stall_host != 0;
    return MOE_OK;
}

namespace {
// The workspace a getter reads: the caller's, or (null) this device's static array, as moe_forward_static used it.
const char* getter_workspace(const moe_handle* h, const void* workspace) {
    if (workspace) return static_cast<const char*>(workspace);
    const int dev = h->arch.device;
    if (dev < 0 || dev >= kMaxDevices || !g_scratch_done[dev]) return nullptr;
    return static_cast<const char*>(g_scratch_ptr[dev]);
}
}  // namespace

int moe_get_task_counts(moe_handle* h, const void* workspace, void* stream, int64_t* gemm0_tasks,
                        int64_t* gemm1_tasks) {
    if (!h) return MOE_ERR_BAD_ARGUMENT;
    const char* ws = getter_workspace(h, workspace);
    if (!ws) return MOE_ERR_WORKSPACE;
    QueueState q;
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = hipMemcpyAsync(&q, ws + h->ws.qstate, sizeof q,
                                  hipMemcpyDeviceToHost, st);
    if (e != hipSuccess) return hip_fail(h, e);
    e = hipStreamSynchronize(st);
    if (e != hipSuccess) return hip_fail(h, e);
    if (gemm0_tasks) *gemm0_tasks = q.tasks_phase0;
    if (gemm1_tasks) *gemm1_tasks = q.tasks_phase1;
    // the handle's word is the one that is sticky and that moe_clear_stall clears; the workspace word only says what the
    // last call on that workspace did
    return *(volatile int32_t*)h->stall_host ? MOE_ERR_QUEUE_STALL : MOE_OK;
}

int moe_get_queue_balance(moe_handle* h, const void* workspace, void* stream, int32_t* workgroups, float* span_us,
                          float* mean_active_us, float* mean_tail_idle_us) {
    if (!h) return MOE_ERR_BAD_ARGUMENT;
    const char* ws = getter_workspace(h, workspace);
    if (!ws) return MOE_ERR_WORKSPACE;
    if (resolved_ffn_mode(h) != MOE_FFN_PERSISTENT) return MOE_ERR_UNSUPPORTED;
    const int n = std::min(h->arch.persistent_blocks, kMaxQueueWorkgroups);
    std::vector<int64_t> t((size_t)2 * n);
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = hipMemcpyAsync(t.data(), ws + h->ws.wg_clock, t.size() * 8,
                                  hipMemcpyDeviceToHost, st);
    if (e != hipSuccess) return hip_fail(h, e);
    e = hipStreamSynchronize(st);
    if (e != hipSuccess) return hip_fail(h, e);
    int64_t first = INT64_MAX, last = INT64_MIN;
    double active = 0;
    for (int i = 0; i < n; ++i) {
        first = std::min(first, t[2 * i]);
        last = std::max(last, t[2 * i + 1]);
        active += (double)(t[2 * i + 1] - t[2 * i]);
    }
    double tail = 0;
    for (int i = 0; i < n; ++i) tail += (double)(last - t[2 * i + 1]);
    const double tick_us = 1000.0 / h->wall_clock_khz;
    if (workgroups) *workgroups = n;
    if (span_us) *span_us = (float)((double)(last - first) * tick_us);
    if (mean_active_us) *mean_active_us = (float)(active / n * tick_us);
    if (mean_tail_idle_us) *mean_tail_idle_us = (float)(tail / n * tick_us);
    return MOE_OK;
}

size_t moe_task_trace_bytes(int64_t max_tasks) { return 16 + 32 * (size_t)(max_tasks > 0 ? max_tasks : 0); }

int moe_set_task_trace(moe_handle* h, void* device_buffer, size_t bytes) {
    if (!h) return MOE_ERR_BAD_ARGUMENT;
    if (!device_buffer || bytes < moe_task_trace_bytes(1)) {
        h->task_trace = nullptr;
        h->task_trace_cap = 0;
        return device_buffer ? MOE_ERR_BAD_ARGUMENT : MOE_OK;
    }
    if ((uintptr_t)device_buffer % 8) return MOE_ERR_BAD_ARGUMENT;
    const int64_t zero[2] = {0, 0};
    const hipError_t e = hipMemcpy(device_buffer, zero, sizeof zero, hipMemcpyHostToDevice);   // not on the hot path
    if (e != hipSuccess) return hip_fail(h, e);
    h->task_trace = static_cast<int64_t*>(device_buffer);
    h->task_trace_cap = (int)std::min<size_t>((bytes - 16) / 32, (size_t)INT32_MAX);
    return MOE_OK;
}

int moe_get_task_trace(moe_handle* h, void* stream, moe_task_record* out, int64_t capacity, int64_t* count) {
    if (!h || !count || capacity < 0 || (capacity > 0 && !out)) return MOE_ERR_BAD_ARGUMENT;
    if (!h->task_trace) return MOE_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    int64_t head[2];
    hipError_t e = hipMemcpyAsync(head, h->task_trace, sizeof head, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return hip_fail(h, e);
    const int64_t written = std::min<int64_t>((int64_t)(head[0] & 0xFFFFFFFF), h->task_trace_cap);
    const int64_t n = std::min(written, capacity);
    *count = written;
    if (n == 0) return MOE_OK;
    std::vector<int64_t> raw((size_t)written * 4);
    e = hipMemcpyAsync(raw.data(), h->task_trace + 2, raw.size() * 8, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return hip_fail(h, e);
    int64_t first = INT64_MAX;
    for (int64_t i = 0; i < written; ++i) first = std::min(first, raw[4 * i + 2]);
    const double tick_us = 1000.0 / h->wall_clock_khz;
    for (int64_t i = 0; i < n; ++i) {
        const int64_t w0 = raw[4 * i], w1 = raw[4 * i + 1];
        moe_task_record& r = out[i];
        r.phase = (int32_t)(w0 >> 56);
        r.expert = (int32_t)((w0 >> 40) & 0xFFFF);
        r.row_block = (int32_t)((w0 >> 20) & 0xFFFFF);
        r.col_tile = (int32_t)(w0 & 0xFFFFF);
        r.workgroup = (int32_t)(w1 >> 32);
        r.rows = (int32_t)(w1 & 0xFFFFFFFF);
        r.start_us = (float)((double)(raw[4 * i + 2] - first) * tick_us);
        r.end_us = (float)((double)(raw[4 * i + 3] - first) * tick_us);
    }
    return MOE_OK;
}

int moe_gemm_bias_act_tile(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N, int64_t K,
                           int32_t dtype, int32_t act, int32_t tile, void* stream) {
    if (!A || !B || !C || M < 1 || N < 1 || K < 1) return MOE_ERR_BAD_ARGUMENT;
    if (act != MOE_ACT_RELU && act != MOE_ACT_GELU && act != MOE_ACT_NONE) return MOE_ERR_BAD_ARGUMENT;
    if (tile != MOE_OPT_AUTO && (tile < 0 || tile > 2)) return MOE_ERR_BAD_ARGUMENT;
    if (M > INT32_MAX / 2 || N > INT32_MAX / 2 || K > INT32_MAX / 2) return MOE_ERR_UNSUPPORTED;
    hipError_t e;
    if (dtype == MOE_DTYPE_F32 || dtype == MOE_DTYPE_TF32) {
        if (K % 16 || N % 2 || tile == 2) return MOE_ERR_UNSUPPORTED;
        e = launch_gemm_bias_act(A, B, bias, C, M, N, K, dtype, act, tile, (hipStream_t)stream);
    } else if (dtype == MOE_DTYPE_BF16 || dtype == MOE_DTYPE_FP16) {
        if (K % 64 || N % 4) return MOE_ERR_UNSUPPORTED;
        e = launch_gemm_dense_bf16(A, B, bias, C, M, N, K, act, tile, (hipStream_t)stream, dtype == MOE_DTYPE_FP16);
    } else {
        return MOE_ERR_UNSUPPORTED;
    }
    return e == hipSuccess ? MOE_OK : MOE_ERR_HIP;
}

int moe_gemm_bias_act(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N, int64_t K,
                      int32_t dtype, int32_t act, void* stream) {
    return moe_gemm_bias_act_tile(A, B, bias, C, M, N, K, dtype, act, MOE_OPT_AUTO, stream);
}

int moe_backward_scratch_bytes(const moe_config* cfg, size_t* bytes) {
    if (!cfg || !bytes) return MOE_ERR_BAD_ARGUMENT;
    Derived d;
    moe_options o;
    moe_options_default(&o);                    // the scratch depends on the shape only
    const int rc = derive(*cfg, o, &d);
    if (rc) return rc;
    if (cfg->torch_dtype == MOE_DTYPE_FP8_E4M3_B128) return MOE_ERR_UNSUPPORTED;
    *bytes = backward_scratch_bytes(d.A, d.E, d.H, d.I, (int)d.act_bytes);
    return MOE_OK;
}

int moe_transpose(const void* src, void* dst, int64_t batch, int64_t rows, int64_t cols, int32_t elem_bytes, void* stream) {
    if (!src || !dst || batch < 0 || rows < 0 || cols < 0) return MOE_ERR_BAD_ARGUMENT;
    if (elem_bytes != 2 && elem_bytes != 4) return MOE_ERR_UNSUPPORTED;
    if (batch > 65535 || rows > INT32_MAX || cols > INT32_MAX) return MOE_ERR_UNSUPPORTED;
    const hipError_t e = launch_transpose(src, dst, batch, rows, cols, elem_bytes, (hipStream_t)stream);
    return e == hipSuccess ? MOE_OK : MOE_ERR_HIP;
}

namespace {
int check_backward_call(const moe_handle* h, int32_t N, int32_t K, const void* scratch, size_t scratch_bytes) {
    if (h->cfg.torch_dtype == MOE_DTYPE_FP8_E4M3_B128) return MOE_ERR_UNSUPPORTED;
    const bool dims_ok = (N == h->d.H && K == h->d.I) || (N == h->d.I && K == h->d.H);
    if (!dims_ok) return MOE_ERR_BAD_ARGUMENT;      // (N, K) is a projection of this layer, one way or the other
    if (!scratch || ((uintptr_t)scratch % kAlign) || scratch_bytes < backward_scratch_bytes(h->d.A, h->d.E, h->d.H, h->d.I, (int)h->d.act_bytes))
        return MOE_ERR_WORKSPACE;
    return MOE_OK;
}
}  // namespace

int moe_expert_gemm(moe_handle* h, const void* a_rows, const void* w, const void* bias, const int32_t* expert_count,
                    const int32_t* expert_offset, int32_t N, int32_t K, int32_t act, void* out_rows, void* scratch,
                    size_t scratch_bytes, void* stream) {
    if (!h || !a_rows || !w || !expert_count || !expert_offset || !out_rows) return MOE_ERR_BAD_ARGUMENT;
    if (act != MOE_ACT_RELU && act != MOE_ACT_GELU && act != MOE_ACT_NONE) return MOE_ERR_BAD_ARGUMENT;
    const int rc = check_backward_call(h, N, K, scratch, scratch_bytes);
    if (rc) return rc;
    const hipError_t e = launch_expert_gemm(a_rows, w, bias, expert_count, expert_offset, h->d.A, h->d.E, N, K, act,
                                            h->d.act_dtype, h->opt, out_rows, scratch, (hipStream_t)stream);
    return e == hipSuccess ? MOE_OK : hip_fail(h, e);
}

int moe_expert_gemm_act_backward(moe_handle* h, const void* dy_rows, const void* w, const void* u_rows, const void* g_rows,
                                 const int32_t* expert_count, const int32_t* expert_offset, int32_t N, int32_t K,
                                 void* du_rows, void* dg_rows, void* scratch, size_t scratch_bytes, void* stream) {
    if (!h || !dy_rows || !w || !u_rows || !expert_count || !expert_offset || !du_rows) return MOE_ERR_BAD_ARGUMENT;
    const bool gated = h->cfg.hidden_act == MOE_ACT_SWIGLU;
    if (gated != (g_rows != nullptr) || gated != (dg_rows != nullptr)) return MOE_ERR_BAD_ARGUMENT;
    const int rc = check_backward_call(h, N, K, scratch, scratch_bytes);
    if (rc) return rc;
    if (N != h->d.I || K != h->d.H) return MOE_ERR_BAD_ARGUMENT;      // the data gradient of the down projection: [rows, H] -> [rows, I]
    if (expert_gemm_dact_tile(h->d.A, h->d.E, N, K, h->d.act_dtype, h->opt) == 0) return MOE_ERR_UNSUPPORTED;
    const hipError_t e = launch_expert_gemm_dact(dy_rows, w, u_rows, g_rows, expert_count, expert_offset, h->d.A, h->d.E, N, K,
                                                 h->cfg.hidden_act, h->d.act_dtype, h->opt, du_rows, dg_rows, scratch,
                                                 (hipStream_t)stream);
    return e == hipSuccess ? MOE_OK : hip_fail(h, e);
}

int moe_expert_gemm_act_backward_supported(const moe_handle* h, int32_t* supported) {
    if (!h || !supported) return MOE_ERR_BAD_ARGUMENT;
    *supported = h->cfg.torch_dtype != MOE_DTYPE_FP8_E4M3_B128 &&
                 expert_gemm_dact_tile(h->d.A, h->d.E, h->d.I, h->d.H, h->d.act_dtype, h->opt) != 0;
    return MOE_OK;
}

int moe_expert_wgrad(moe_handle* h, const void* dy_rows, const void* a_rows, const int32_t* expert_count,
                     const int32_t* expert_offset, int32_t N, int32_t K, void* dw, void* scratch, size_t scratch_bytes,
                     void* stream) {
    if (!h || !dy_rows || !a_rows || !expert_count || !expert_offset || !dw) return MOE_ERR_BAD_ARGUMENT;
    const int rc = check_backward_call(h, N, K, scratch, scratch_bytes);
    if (rc) return rc;
    const hipError_t e = launch_expert_wgrad(dy_rows, a_rows, expert_count, expert_offset, h->d.A, h->d.E, N, K,
                                             h->d.act_dtype, h->opt, dw, scratch, (hipStream_t)stream);
    return e == hipSuccess ? MOE_OK : hip_fail(h, e);
}

namespace {
bool backward_dtype(const moe_handle* h) {
    return h->cfg.torch_dtype != MOE_DTYPE_FP8_E4M3_B128;
}
}  // namespace

int moe_act_backward(moe_handle* h, const void* dh_rows, const void* u_rows, const void* g_rows, int64_t rows,
                     void* du_rows, void* dg_rows, void* stream) {
    if (!h || !dh_rows || !u_rows || !du_rows || rows < 0) return MOE_ERR_BAD_ARGUMENT;
    if (!backward_dtype(h)) return MOE_ERR_UNSUPPORTED;
    const bool sw = h->cfg.hidden_act == MOE_ACT_SWIGLU;
    if (sw != (g_rows != nullptr) || sw != (dg_rows != nullptr)) return MOE_ERR_BAD_ARGUMENT;
    if (rows > h->d.A) return MOE_ERR_BAD_ARGUMENT;
    const hipError_t e = launch_act_backward(dh_rows, u_rows, g_rows, rows * h->d.I, h->cfg.hidden_act,
                                             h->d.act_dtype, du_rows, dg_rows, (hipStream_t)stream);
    return e == hipSuccess ? MOE_OK : hip_fail(h, e);
}

int moe_bias_grad(moe_handle* h, const void* dy_rows, const int32_t* expert_count, const int32_t* expert_offset, int32_t N,
                  void* db, void* stream) {
    if (!h || !dy_rows || !expert_count || !expert_offset || !db) return MOE_ERR_BAD_ARGUMENT;
    if (!backward_dtype(h)) return MOE_ERR_UNSUPPORTED;
    if (N != h->d.H && N != h->d.I) return MOE_ERR_BAD_ARGUMENT;
    const hipError_t e = launch_bias_grad(dy_rows, expert_count, expert_offset, h->d.E, N,
                                          h->d.act_dtype, db, (hipStream_t)stream);
    return e == hipSuccess ? MOE_OK : hip_fail(h, e);
}

int moe_combine_backward(moe_handle* h, const void* dout, const void* y_rows, const int32_t* pair_row, const float* topk_w,
                         void* dy_rows, float* dw, void* stream) {
    if (!h || !dout || !y_rows || !pair_row || !topk_w || !dy_rows || !dw) return MOE_ERR_BAD_ARGUMENT;
    if (!backward_dtype(h)) return MOE_ERR_UNSUPPORTED;
    const hipError_t e = launch_combine_backward(dout, y_rows, pair_row, topk_w, h->d.S, h->d.k, h->d.H,
                                                 h->d.act_dtype, dy_rows, dw, (hipStream_t)stream);
    return e == hipSuccess ? MOE_OK : hip_fail(h, e);
}

int moe_combine(const void* y_rows, const int32_t* pair_row, const float* topk_w, int32_t S, int32_t k, int32_t H,
                int32_t act_dtype, void* out, void* stream) {
    if (!y_rows || !pair_row || !topk_w || !out || S < 0 || k < 1 || H < 1) return MOE_ERR_BAD_ARGUMENT;
    if (act_dtype != MOE_DTYPE_F32 && act_dtype != MOE_DTYPE_BF16 && act_dtype != MOE_DTYPE_FP16) return MOE_ERR_UNSUPPORTED;
    if (H % (act_dtype == MOE_DTYPE_F32 ? 4 : 8)) return MOE_ERR_UNSUPPORTED;
    const hipError_t e = launch_combine(y_rows, pair_row, topk_w, S, k, H, act_dtype, out, nullptr, (hipStream_t)stream);
    return e == hipSuccess ? MOE_OK : MOE_ERR_HIP;
}

}  // extern "C"

namespace moe355 {

hipError_t launch_ffn_tiled(const FfnArgs& a, int dtype, const FfnPlan& p, int max_mtiles, hipStream_t st) {
    if (dtype == MOE_DTYPE_F32 || dtype == MOE_DTYPE_TF32)
        return p.tile ? launch_ffn_f32_tile(a, max_mtiles, p.nnt0, p.nnt1, 0, st)
                      : launch_ffn_tiled_f32(a, max_mtiles, p.nnt0, p.nnt1, st);
    return launch_ffn_tiled_bf16(a, p.tile, max_mtiles, p.nnt0, p.nnt1, st, dtype == MOE_DTYPE_FP16);
}

hipError_t launch_ffn_persistent(const FfnArgs& a, int dtype, const FfnPlan& p, int blocks, bool early, hipStream_t st) {
    if (dtype == MOE_DTYPE_F32 || dtype == MOE_DTYPE_TF32)
        return p.tile ? launch_ffn_f32_tile(a, 0, p.nnt0, p.nnt1, blocks, st) : launch_ffn_persistent_f32(a, blocks, st);
    return launch_ffn_persistent_bf16(a, p.tile, blocks, early, st, dtype == MOE_DTYPE_FP16);
}

int ffn_persistent_blocks(int dtype, int tile, int compute_units) {
    if (dtype == MOE_DTYPE_F32 || dtype == MOE_DTYPE_TF32)
        return compute_units * (tile ? ffn_persistent_occupancy_f32_tile() : 4);
    if (dtype == MOE_DTYPE_FP8_E4M3_B128)
        return compute_units * (tile ? ffn_persistent_occupancy_fp8_tile() : ffn_persistent_occupancy_fp8());
    return compute_units * ffn_persistent_occupancy_bf16(tile);
}

hipError_t launch_gemm_bias_act(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N,
                                int64_t K, int dtype, int act, int opt_tile, hipStream_t st) {
    if (dtype == MOE_DTYPE_F32 || dtype == MOE_DTYPE_TF32) {
        bool tile = gemm_dense_f32_takes_tile(M, N, K);
        if (opt_tile == 0) tile = false;     // asked to keep the vector-ALU kernel
        return tile ? launch_gemm_dense_f32_tile(A, B, bias, C, M, N, K, act, st)
                    : launch_gemm_dense_f32(A, B, bias, C, M, N, K, act, st);
    }
    return launch_gemm_dense_bf16(A, B, bias, C, M, N, K, act, opt_tile, st, dtype == MOE_DTYPE_FP16);
}

}  // namespace moe355
