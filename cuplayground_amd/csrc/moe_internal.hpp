// Internal declarations shared by the host side of libmoe355 and its gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/moe355.h"
#include "queue_order.hpp"

namespace moe355 {

constexpr int kWave = 64;          // gfx950 wavefront

// 16-bit storage types as the kernels see them: raw bit patterns with a tag that selects the conversion.
struct bf16_s { uint16_t bits; };
struct f16_s { uint16_t bits; };
constexpr int kMaxExperts = 512;   // top-k keeps E/64 logits per lane in registers, 8 at most
constexpr int kMaxTopK = 16;
constexpr int kRouteBlock = 256;   // pairs per workgroup in the slot-assignment kernels

// One row block of an expert: rows [row0, row0 + rows) of the packed (expert-major) row space.
struct MTile {
    int32_t expert;
    int32_t row0;
    int32_t rows;
    int32_t pad;
};

// Words at the start of the queue-state block of the workspace (carved out of the workspace in api.hip).
constexpr int kMaxQueueGroups = 8;   // XCDs of a gfx950
// e4m3 layers: average rows per expert from which the tile GEMM replaces the weight streamer.  Measured on two shapes
// (H 4096, I 14336, 8 experts and H 7168, I 2048, 64 experts): at 16 rows per expert the streamer is 18 % faster, at 32
// the tile GEMM 13-17 %, at 128 it is 2.5 times and from 1024 on 3.3 times as fast.
constexpr int kFp8TileRowsPerExpert = 32;
// ... and from which widening the weights to bf16 in the workspace (one pass over them per call, 4.9 TB/s) and running
// the bf16 tile GEMM replaces the e4m3 tile GEMM.  Measured, e4m3 tile time / this: H 4096, I 14336, 8 experts 1.01 at
// 512 rows per expert, 1.08 at 768, 1.18 at 1024, 1.34 at 2048; H 7168, I 2048, 64 experts 0.95 at 512, 1.17 at 1024,
// 1.30 at 2048; H = I = 2048, 16 experts 1.23 at 1024, 1.36 at 2048.
constexpr int kFp8WidenRowsPerExpert = 768;
// fp32 layers: average rows per expert and number of 128 x 128 tiles from which the matrix-core tile replaces the 64 x 64
// vector-ALU one.  Measured FFN stage, vector / matrix: the reference's knob file (8192 rows, one expert, H 1024, I 4096)
// 2.13 / 1.13 ms; 512 rows per expert, 16 experts, H 1024, I 2048, SwiGLU 1.81 / 1.00 ms; 64 rows per expert, 8 experts,
// H 1024, I 4096 (320 tiles) 0.387 / 0.384 ms; 128 rows per expert, 8 experts, H 256, I 512 (48 tiles) 0.059 / 0.077 ms.
constexpr int kF32TileRowsPerExpert = 128;
// (H 1024, I 4096: one expert x 1024 rows, 320 tiles, 0.391 / 0.348 ms; one expert x 2048 rows 0.644 / 0.398; four experts,
// top-2, SwiGLU, 2048 tokens 1.705 / 1.119 ms.)
constexpr int kF32TileMinTiles = 320;
struct QueueState {
    int32_t groups;        // queue groups (1 or the number of XCDs)
    int32_t total_tasks;   // tasks of both phases (holes not counted)
    int32_t tasks_phase0;
    int32_t tasks_phase1;
    int32_t num_mtiles;
    int32_t kept_rows;
    int32_t stall;         // set when a bounded dependency wait expired
    int32_t nseg;          // segments in the merged queue
    int32_t heads[kMaxQueueGroups];   // next id to pop, per group (persistent mode)
    int32_t ids_queue;     // ids per group in the merged queue (holes included)
    int32_t ids_phase0;    // ids per group in the phase-0 table / the phase-1 table (tiled mode)
    int32_t ids_phase1;
    int32_t split_mt0;     // first row block whose down-projection tiles run as partial sums (num_mtiles: none)
    int32_t nseg_phase1;   // segments of the phase-1 table (the experts, plus one when a run was cut at split_mt0)
    int32_t pad[3];
};
// State of the combine tasks of the queue kernels, in a cache line of its own: the workgroups that have run out of GEMM
// tasks poll it, and must not stand in the way of the queue heads that the busy ones pop.
struct CombineState {
    int32_t down_done;         // down-projection tiles finished so far (the combine tasks stop when all are)
    int32_t pad[63];
};

// Everything the FFN kernels need; passed by value.
struct FfnArgs {
    const void* x;              // [S,H]
    const int32_t* token_indices;
    const void* w_up;           // [E,I,H]
    const void* w_gate;         // [E,I,H] or null
    const void* w_down;         // [E,H,I]
    const void* b_up;
    const void* b_gate;
    const void* b_down;
    const float* s_up;
    const float* s_gate;
    const float* s_down;
    void* h;                    // [A,I] intermediate, activation dtype
    void* y;                    // [A,H] expert outputs, activation dtype
    const MTile* mtiles;
    const Segment* seg_phase0;  // E segments, task ids local to phase 0
    const Segment* seg_phase1;  // QueueState::nseg_phase1 segments, task ids local to phase 1
    const Segment* seg_queue;   // 2E segments in queue order
    QueueState* q;
    int32_t* done0;             // per MTile: finished phase-0 column tiles
    int32_t* host_stall;        // pinned host word of the handle, set (system scope) when a dependency wait expires
    int32_t H, I, E;
    int32_t act;
    int32_t spin_limit;
    int32_t groups;             // queue groups the schedule was built for
    int32_t row_chunk;          // order of a segment's tasks: 0 = row blocks fastest; R > 0 = R row blocks at a time, all column tiles of those, row blocks fastest inside
    uint32_t x_bytes, h_bytes, w_bytes;   // extents of x, h and one weight matrix (meaningful below 4 GiB)
    int64_t* wg_clock;          // queue kernels: [2 * workgroup] constant-rate clock at entry, [2 * workgroup + 1] at exit
    int64_t* task_trace;        // null, or the caller's trace buffer: [0] records written, [2 + 4 i ..] record i (trace_task)
    int32_t task_trace_cap;     // records the buffer holds
    // Combine inside the FFN kernels (null `arrive`: the separate combine launch is used instead).
    int32_t* arrive;            // [S, nnt1]: finished down-projection tiles per (token, column tile)
    const int32_t* pair_row;    // [S, k] packed row of every (token, rank), -1 when dropped
    const float* topk_w;        // [S, k]
    void* out;                  // [S, H] in the activation type
    int32_t S, k, nnt1;
    int32_t drop;               // tokens may have lost every pair: their output rows are zeroed at kernel entry
    // Combine as tasks of the queue kernel (null `combined`: not used).  A unit is (token, slice of 256 x 16 bytes of
    // its row); combined[unit] is set by the workgroup that takes the unit.
    int32_t* done1;             // per MTile: finished phase-1 column tiles
    const int32_t* pair_mt;     // [S, k] row block (MTile index) of every (token, rank), -1 when dropped
    int32_t* combined;          // [slices, S]: 1 once the unit has been taken
    CombineState* cs;
    // Down-projection tiles of the queue's tail as partial sums over the contraction dimension (null split_cnt: not used)
    int32_t* split_cnt;         // [tiles]: parts of the tile that have been stored
    float* split_part;          // [tiles][parts][block rows x block columns] fp32, in the accumulator layout of the tile
    int32_t split_extra_blocks; // (parts - 1) x the most row blocks that can run so: what the down projection's id space grows by
    // e4m3 x e4m3 plan (null xq: not used): the token rows and the intermediate rows as e4m3 codes with one scale per
    // (row, 128 columns), written by quant_rows128 passes in front of the two projections
    uint8_t* xq;                // [S, H]
    float* sx;                  // [S, H / 128]
    uint8_t* hq;                // [A, I]
    float* sh;                  // [A, I / 128]
};
constexpr int kMaxQueueWorkgroups = 4096;   // workgroups of a queue kernel that get a slot in wg_clock

struct RouteArgs {
    const int32_t* topk_idx;    // [A]
    int32_t* rank_local;        // [A]
    int32_t* block_hist;        // [nblk, E] counts, then exclusive prefix over blocks
    int32_t* slot;              // [A]
    int32_t* pair_row;          // [A]
    int32_t* token_indices;     // [A]
    int32_t* expert_count;      // [E]
    int32_t* expert_offset;     // [E+1]
    MTile* mtiles;
    Segment* seg_phase0;
    Segment* seg_phase1;
    Segment* seg_queue;
    QueueState* q;
    int32_t* done0;
    int32_t* arrive;            // null, or counters of the combine inside the FFN kernels, cleared here: arrive_n of them
    int32_t arrive_n;
    int32_t* done1;             // null, or per MTile the finished phase-1 column tiles (combine as queue tasks), cleared here
    int32_t* pair_mt;           // [A] row block of every pair (-1: dropped)
    CombineState* cs;           // null, or the state of the combine tasks, cleared here
    int32_t S, k, E, A, nblk;
    int32_t drop;
    int32_t capacity;
    int32_t block_m;            // rows per MTile
    int32_t nnt0, nnt1;         // column tiles of phase 0 / phase 1
    int32_t max_mtiles;
    int32_t lag;                // experts of phase-0 work queued between an expert's two phases
    int32_t groups;             // queue groups: 1, or one per XCD
    int32_t tail_workgroups;    // 0, or the workgroups of the queue kernel: the tail of the queue is rounded to them (route.hip: round_tail)
    int32_t tail_split;         // 0 / 1: whole tiles everywhere; F: the down-projection tiles of the last row blocks run as F partial sums
    int32_t tail_blocks;        // ... how many row blocks (what the partial-sum buffers were sized for)
    int32_t* split_cnt;         // [tail_blocks * nnt1] arrival counters of those tiles, cleared here
    int64_t* task_trace;        // null, or the FFN stage's trace buffer: its record count starts every call at zero
};

// ---- launchers (defined next to their kernels) ----
// Router: logits, top-k, weights (gate.hip).  opt: the handle's options gate_kernel / gate_mfma / gate_tile /
// gate_fused_topk (MOE_OPT_AUTO: chosen from the shape).
hipError_t launch_gate(const void* x, const void* gate_w, const float* gate_bias, float* logits, bool keep_logits, int S,
                       int H, int E, int k, int gate_fn, int norm, int32_t* topk_idx, float* topk_w, int act_dtype,
                       const moe_options& opt, hipStream_t st);
constexpr int kStatsBlocks = 64;   // per-block partials of the router statistics kept in the workspace
hipError_t launch_router_stats(const float* logits, const int32_t* topk_idx, int S, int E, int k, int gate_fn,
                               double* part_prob, int32_t* part_cnt, float* load, float* mean_prob, float* aux_loss,
                               hipStream_t st);
hipError_t launch_route(const RouteArgs& a, hipStream_t st);
// taken: null, or [slices, S] flags of the (token, slice of 256 x 16 bytes) units that are already combined and are skipped
hipError_t launch_combine(const void* y_rows, const int32_t* pair_row, const float* topk_w, int S, int k, int H,
                          int act_dtype, void* out, const int32_t* taken, hipStream_t st);

// FFN stage.  block_m / block_n are the tile sizes the routing stage must be told about.
struct FfnPlan {
    int kernel_dtype;   // the dtype whose kernels run: the layer's, or bf16 for an e4m3 layer whose weights are widened
    bool widen;         // e4m3 layer run as a bf16 layer on weights widened into the workspace by every call
    int ksplit;         // 16-bit layers on the hand-ordered tiles: parts a down-projection tile of the last row blocks is summed in (1: whole tiles)
    int tail_blocks;    // ... and how many row blocks those are
    bool mfma8;         // e4m3 layer on the tile GEMM with both operands e4m3 (tokens quantised per row and 128 columns)
    int tile;        // 16-bit layers: which tile the kernels are instantiated with (ffn_bf16.hip: bf16_tile)
    int block_m;
    int nnt0;        // column tiles of phase 0
    int nnt1;        // column tiles of phase 1
};
FfnPlan ffn_plan(int dtype, int act, int H, int I, int64_t A, int E, const moe_options& o);
hipError_t launch_widen_block128(const void* q, const float* scales, void* out, int64_t matrices, int64_t N, int64_t K,
                                 hipStream_t st);
// bf16 rows -> e4m3 codes + one fp32 scale per (row, 128 columns); limit: null, or a device word with the rows that matter
hipError_t launch_quant_rows128(const void* x, void* q, float* scales, int64_t rows, int64_t K, const int32_t* limit,
                                hipStream_t st);
hipError_t launch_ffn_tiled(const FfnArgs& a, int dtype, const FfnPlan& p, int max_mtiles, hipStream_t st);
hipError_t launch_ffn_persistent(const FfnArgs& a, int dtype, const FfnPlan& p, int blocks, bool early, hipStream_t st);
int ffn_persistent_blocks(int dtype, int tile, int compute_units);

// ---- backward building blocks (csrc/backward.hip) ----
size_t backward_scratch_bytes(int64_t A, int E, int H, int I, int elem_bytes);
hipError_t launch_transpose(const void* src, void* dst, int64_t batch, int64_t rows, int64_t cols, int elem_bytes,
                            hipStream_t st);
int expert_gemm_dact_tile(int64_t A, int E, int N, int K, int dtype, const moe_options& opt);
hipError_t launch_expert_gemm_dact(const void* dy_rows, const void* w, const void* u_rows, const void* g_rows,
                                   const int32_t* count, const int32_t* offset, int64_t A, int E, int N, int K, int hidden_act,
                                   int dtype, const moe_options& opt, void* du_rows, void* dg_rows, void* scratch,
                                   hipStream_t st);
hipError_t launch_expert_gemm(const void* a_rows, const void* w, const void* bias, const int32_t* count,
                              const int32_t* offset, int64_t A, int E, int N, int K, int act, int dtype,
                              const moe_options& opt, void* out_rows, void* scratch, hipStream_t st);
hipError_t launch_expert_wgrad(const void* dy_rows, const void* a_rows, const int32_t* count, const int32_t* offset,
                               int64_t A, int E, int N, int K, int dtype, const moe_options& opt, void* dw, void* scratch,
                               hipStream_t st);

hipError_t launch_act_backward(const void* dh, const void* u, const void* g, int64_t n, int act, int dtype, void* du,
                               void* dg, hipStream_t st);
hipError_t launch_bias_grad(const void* dy, const int32_t* count, const int32_t* offset, int E, int N, int dtype, void* db,
                            hipStream_t st);
hipError_t launch_combine_backward(const void* dout, const void* y, const int32_t* pair_row, const float* topk_w, int S,
                                   int k, int H, int dtype, void* dy, float* dw, hipStream_t st);

// tile: MOE_OPT_AUTO, or the tile asked for (moe_gemm_bias_act_tile)
hipError_t launch_gemm_bias_act(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N,
                                int64_t K, int dtype, int act, int tile, hipStream_t st);

}  // namespace moe355
