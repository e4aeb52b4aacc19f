/*
 * moe355 -- C ABI of the MI355X (gfx950) fused MoE forward: gate -> slot assignment -> expert FFN -> combine,
 * all experts resident on one GPU.
 *
 * The reference (osayamenja/cuPlayground) has no FFI: its operator surface is the JSON knob file
 * (aristos_config.json, aristos_config.schema.json:5-71) turned into compile definitions
 * (CMakeLists.txt:167-216) and the data contracts of its kernels.  Each entry point below names the
 * reference interface it stands in for.  All pointers are plain host or device addresses; `stream` is a
 * hipStream_t passed as void* (NULL = the null stream).  Every function returns a moe_status and never
 * exits the process (the reference prints and calls exit(1), util.cuh:24-36).
 *
 * Tensor conventions (row-major everywhere, K contiguous -- the (M,K) x (N,K) -> (M,N) convention of the
 * reference GEMM, mma.cuh:415-427):
 *   x        [S, H]        activations      f32 | bf16 | fp16
 *   gate_w   [E, H]        router weights   activation dtype
 *   w_up     [E, I, H]     expert up proj   f32 | bf16 | fp16 | e4m3 bytes
 *   w_gate   [E, I, H]     SwiGLU gate proj (hidden_act = 2 only)
 *   w_down   [E, H, I]     expert down proj
 *   b_*      [E, I] / [E, H]  optional biases, activation dtype
 *   s_*      [E, N/128, K/128] fp32 block scales (torch_dtype = 4 only)
 *   out      [S, H]        activation dtype
 */
#ifndef MOE355_H
#define MOE355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOE355_VERSION 1

typedef enum moe_status {
    MOE_OK = 0,
    MOE_ERR_BAD_CONFIG = 1,       /* a knob is outside its domain, or JSON is malformed / missing a key     */
    MOE_ERR_UNSUPPORTED = 2,      /* valid knob values this build has no kernel for (E > 512, H > 16384 ...) */
    MOE_ERR_WORKSPACE = 3,        /* workspace pointer NULL, misaligned or smaller than moe_workspace_bytes    */
    MOE_ERR_BAD_ARGUMENT = 4,     /* NULL where a tensor is required, or an extra tensor the config excludes   */
    MOE_ERR_HIP = 5,              /* a HIP call failed; moe_last_hip_error() returns its hipError_t            */
    MOE_ERR_NO_DEVICE = 6,        /* no gfx950 device is visible                                               */
    MOE_ERR_QUEUE_STALL = 7       /* the persistent kernel's bounded dependency wait expired                   */
} moe_status;

/* torch_dtype: the reference enum (aristos_config.schema.json:54-58) plus 4.  Activations are stored in the layer's
 * type, except: tf32 layers are fp32 in memory and are computed in full fp32 (gfx950 has no tf32 matrix instruction;
 * the reference's tf32 atoms, processor/tiling.cuh:131-143, keep fp32 storage too), e4m3 layers keep bf16 activations. */
enum { MOE_DTYPE_F32 = 0, MOE_DTYPE_TF32 = 1, MOE_DTYPE_BF16 = 2, MOE_DTYPE_FP16 = 3, MOE_DTYPE_FP8_E4M3_B128 = 4 };
/* hidden_act: the reference enum (aristos_config.schema.json:24-28) plus 2 */
enum { MOE_ACT_RELU = 0, MOE_ACT_GELU = 1, MOE_ACT_SWIGLU = 2, MOE_ACT_NONE = 3 /* moe_gemm_bias_act only */ };
enum { MOE_GATE_SOFTMAX = 0, MOE_GATE_SIGMOID = 1 };

/*
 * One field per key of aristos_config.schema.json:5-58, in the schema's order, then this build's extensions.
 * Relaxations of the schema (a file valid under the reference schema loads unchanged):
 *   capacity_factor  number > 0 (schema: integer >= 1)        hidden_act   adds 2 = SwiGLU
 *   torch_dtype      adds 4 = e4m3 weights + 128x128 scales   sequence_len any integer >= 1 (schema: x128)
 *   micro_batch      any integer >= 1 (schema: x2)            hidden_size / intermediate_size stay x64
 * Tokens per call: S = micro_batch * sequence_len.
 */
typedef struct moe_config {
    double capacity_factor;
    int32_t drop_tokens;
    int32_t expert_top_k;
    int32_t is_training;        /* parsed and kept; the forward path ignores it, as the reference does */
    int32_t hidden_act;
    int32_t hidden_size;
    int32_t intermediate_size;
    int32_t micro_batch;
    int32_t num_experts;
    int32_t sequence_len;
    int32_t torch_dtype;
    /* extensions */
    int32_t gate_fn;            /* MOE_GATE_*; default softmax */
    int32_t norm_topk_prob;     /* default: 1 when expert_top_k > 1, else 0 */
} moe_config;

/* Replaces the CMake JSON reader (CMakeLists.txt:167-203).  `err` (may be NULL) receives a message. */
int moe_config_default(moe_config* cfg);
int moe_config_from_json_string(const char* json, moe_config* cfg, char* err, size_t err_len);
int moe_config_from_json_file(const char* path, moe_config* cfg, char* err, size_t err_len);
int moe_config_validate(const moe_config* cfg, char* err, size_t err_len);
int64_t moe_config_tokens(const moe_config* cfg);                  /* S */
int moe_config_capacity(const moe_config* cfg, int64_t* capacity); /* ceil(capacity_factor * S * k / E) */

/* Replaces Hardware<Arch,maxRegs,Board>::blocks (arch.cuh:16-69): the resident-workgroup budget of the
 * device the handle was created on, queried at run time. */
typedef struct moe_arch {
    int32_t device;
    int32_t compute_units;
    int32_t xcds;
    int32_t wavefront_size;
    int32_t lds_bytes_per_cu;
    int32_t max_clock_khz;
    int32_t persistent_blocks;   /* workgroups the persistent FFN kernel is launched with */
    char name[64];
} moe_arch;

typedef struct moe_handle moe_handle;

/*
 * Tuning options of a handle: which tile, which kernel, which schedule -- everything the library would otherwise choose
 * from the layer's shape.  The reference has one knob surface, the JSON file turned into compile definitions
 * (CMakeLists.txt:204-216), and chooses tiles and schedulers at compile time (processor/tiling.cuh:97-159,
 * scheduling.cuh:170-200 against warpScheduler.cuh:167-265); these are the same choices as run-time values of a handle.
 * Every field is MOE_OPT_AUTO (the library chooses) or one of the values named beside it; a value outside its domain
 * makes moe_create_with_options return MOE_ERR_BAD_ARGUMENT, a value the layer's shape cannot take (the 256-row tile on
 * a layer with H % 256 != 0, say) falls back to the library's choice.  Results never depend on these options beyond
 * what is said here: schedules and tiles of one dtype agree bit for bit except where a field says otherwise.
 * Options are fixed when the handle is created; two handles of one process may differ in every one of them.
 */
#define MOE_OPT_AUTO (-1)
typedef struct moe_options {
    int32_t tile16;          /* bf16 / fp16 layers: 0 = 128x128 tile, 1 = 256x256 (hand-ordered), 2 = 128x256 (hand-ordered),
                                3 = 256x256 with the 128x256 tile for row blocks of at most 128 rows */
    int32_t block_rows;      /* bf16 / fp16 layers: 128 or 256 rows per row block (a coarser way to say tile16 = 0 / 1) */
    int32_t f32_tile;        /* fp32 / tf32 layers: 0 = 64x64 vector-ALU tile, 1 = 128x128 matrix-core tile; also read by the
                                backward entry points of an fp32 handle (there 1 means "where the shape allows") */
    int32_t fp8_tile;        /* e4m3 layers: 0 = weight streamer (decode), 1 = 128x128 tile GEMM */
    int32_t fp8_widen;       /* e4m3 layers: 1 = run the bf16 tiles on bf16 copies of the weights (widened into the workspace
                                by every call, or taken from moe_prepare_weights), 0 = never */
    int32_t queue_groups;    /* task queues of the FFN stage: 1, 2, 4 or 8 (never more than the device has XCDs) */
    int32_t queue_lag;       /* experts of up-projection work queued between an expert's two projections, >= 1 */
    int32_t queue_early;     /* 1 = the queue loop that starts the next task under the current one's epilogue (256x256 tile) */
    int32_t row_chunk;       /* order of the tasks of one expert and projection: 0 = row blocks fastest, R > 0 = R row
                                blocks at a time */
    int32_t blocks_per_cu;   /* resident workgroups per compute unit of the queue kernels, 1..16 */
    int32_t combine;         /* 0 = a launch of its own behind the FFN stage; 1 = inside the FFN kernels, by the workgroup
                                whose tile completes a token (arrival counters); 2 = as tasks of the FFN queue, taken by
                                workgroups that find no GEMM task left (task-queue mode only; the rest of the tokens is
                                combined by a short launch behind it).  All three give the same bits. */
    int32_t gate_kernel;     /* logits kernel: 0 = register-tiled, 1 = token rows in registers */
    int32_t gate_mfma;       /* 1 = the logits on the matrix cores where the shape allows (16-bit layers, H % 512 == 0), 0 = never */
    int32_t gate_tile;       /* register-tiled logits kernel: 0 = 4x8 pairs per wavefront, 1 = 4x4, 2 = 2x8 */
    int32_t gate_fused_topk; /* 1 = top-k inside the logits kernel where one exists for the shape (no logits round trip
                                through memory unless the caller asks for them), 0 = always a launch of its own */
    int32_t grouped_tile;    /* moe_expert_gemm on a 16-bit handle: 0 = 128x128, 1 = 256x256, 2 = 128x256 */
    int32_t tail_round;      /* task-queue mode: 1 (and AUTO) = the last up-projection segment of the queue is placed so that the
                                down-projection tasks behind it fill whole rounds of the resident workgroups (a permutation
                                of whole row blocks inside the queue: results and tables do not change), 0 = plain order */
    int32_t fp8_mfma;        /* e4m3 layers: 1 = the tile GEMM with both operands e4m3 on the fp8 matrix instructions: token rows and
                                intermediate rows are quantised to e4m3 with one fp32 scale per (row, 128 columns) by a pass in
                                front of each projection (moe_quant_rows128), weights are fed as stored; one launch per
                                projection; overrides fp8_tile and fp8_widen.  0 / AUTO = bf16 activations.  Opt-in because it
                                changes the arithmetic: e4m3 activations keep 3 mantissa bits, and results stand 2.4e-2 to
                                4.2e-2 of the output range away from the bf16-activation layer -- past the 3e-2 that the
                                other e4m3 plans keep. */
    int32_t prepared_weights;/* 1 = every moe_forward on the handle will carry moe_weights.prepared (moe_prepare_weights): the
                                workspace then holds no copies of the weights and a call without them is refused; 0 / AUTO =
                                prepared weights are used when given, else made per call in the workspace */
    int32_t tail_split;      /* 16-bit layers on the 256-column tiles (tile16 1, 2, 3): 2 or 4 = every down-projection tile of the last
                                row blocks -- the tasks the launch ends with -- is computed as that many tasks, each a partial sum
                                over its share of the intermediate dimension, kept in fp32 in the workspace and added up in a
                                fixed order by the task that finishes last: the launch's tail gets shorter tasks, the sums
                                of those tiles are associated differently (same tolerance, other bits; the same in both
                                ffn modes).  1 / AUTO = whole tiles.  Ignored where the intermediate size is not a multiple of
                                128 x parts, with combine != 0 and with queue_early. */
    int32_t reserved[6];     /* must be MOE_OPT_AUTO */
} moe_options;
/* Every field MOE_OPT_AUTO. */
int moe_options_default(moe_options* opt);
/* Overrides the fields of *opt for which a MOE355_<FIELD> environment variable (upper-case field name) is set to a value
 * of the field's domain.  This is the only place the library reads its environment, and it is never called from
 * moe_forward or any other per-step entry point: moe_create and moe_workspace_bytes (the entry points without an options
 * argument) call it once on defaults; moe_create_with_options and moe_workspace_bytes_with_options never do. */
int moe_options_from_env(moe_options* opt);
int moe_create_with_options(const moe_config* cfg, const moe_options* opt, moe_handle** out);
int moe_workspace_bytes_with_options(const moe_config* cfg, const moe_options* opt, size_t* bytes);
/* The options the handle runs with, every AUTO resolved to the value in force; and the workspace it needs -- the value to
 * trust when options and environment may have changed between moe_workspace_bytes and moe_create. */
int moe_get_options(const moe_handle* h, moe_options* opt);
int moe_get_workspace_bytes(const moe_handle* h, size_t* bytes);

int moe_create(const moe_config* cfg, moe_handle** out);
int moe_destroy(moe_handle* h);
int moe_get_arch(const moe_handle* h, moe_arch* out);
/* The tiling the handle chose: rows per row block, and column tiles of the up(/gate) and of the down projection.
 * Task totals follow the reference's bound tilesM*tilesNx + tilesM*tilesN (scheduling.cuh:212-222) per expert. */
int moe_get_plan(const moe_handle* h, int32_t* block_rows, int32_t* col_tiles_up, int32_t* col_tiles_down);
/* The dtype whose FFN kernels the handle runs: cfg.torch_dtype, except MOE_DTYPE_BF16 for an e4m3 layer whose experts
 * see so many rows (768 on average; option fp8_widen = 0 / 1 overrides) that every moe_forward first widens the weights
 * to bf16 in the workspace (moe_dequant_block128; moe_workspace_bytes then includes 2 bytes per weight) and runs
 * the bf16 tiles on them.  The reference fixes its element types at compile time (processor/tiling.cuh:97-159). */
int moe_get_kernel_dtype(const moe_handle* h, int32_t* dtype);
int moe_workspace_bytes(const moe_config* cfg, size_t* bytes);

typedef struct moe_weights {
    const void* gate_w;
    const float* gate_bias;   /* [E] fp32 or NULL */
    const void* w_up;
    const void* w_gate;       /* SwiGLU only, else NULL */
    const void* w_down;
    const void* b_up;         /* NULL = no bias */
    const void* b_gate;
    const void* b_down;
    const float* s_up;        /* fp8 only */
    const float* s_gate;
    const float* s_down;
    const void* prepared;     /* NULL, or what moe_prepare_weights wrote for these weights on this handle */
} moe_weights;

/* Optional device buffers receiving the routing result (any member may be NULL). */
typedef struct moe_routing_out {
    int32_t* topk_idx;        /* [S,k] expert of pair (t,r), ranks in descending score          */
    float*   topk_w;          /* [S,k] gate weight of the pair                                  */
    int32_t* slot;            /* [S,k] position inside the expert's row block, -1 = dropped     */
    int32_t* expert_count;    /* [E]   kept rows per expert                                     */
    int32_t* expert_offset;   /* [E]   exclusive scan of expert_count                           */
    int32_t* token_indices;   /* [S*k] token of each packed row, -1 past the last kept row      */
} moe_routing_out;

/*
 * Kernel-ready operands, made once.  The reference keeps its operands resident in one arena for the life of a run
 * (mma.cuh:385-391); here whatever a handle's plan would otherwise derive from the weights in every call is written
 * once into a buffer of the caller and handed back through moe_weights.prepared: today the bf16 copies of an e4m3
 * layer's expert weights on the widening plan (moe_get_kernel_dtype; 2 bytes per weight, moe_prepared_bytes says how
 * many, 0 when the plan prepares nothing -- then moe_prepare_weights does nothing and `prepared` may stay NULL).
 * The buffer is device memory, 256-byte aligned; its contents belong to (weights, handle plan) and stay valid as long as
 * both do; the original weights and scales are still passed with every call (the router and any plan change need
 * them).  Results are bit-identical to the per-call preparation.  Asynchronous on `stream`.
 */
int moe_prepared_bytes(const moe_handle* h, size_t* bytes);
int moe_prepare_weights(moe_handle* h, const moe_weights* w, void* prepared, size_t prepared_bytes, void* stream);

/* Variants of the FFN stage; MOE_FFN_AUTO lets the library choose. */
enum { MOE_FFN_AUTO = 0, MOE_FFN_TILED = 1 /* one launch per GEMM */, MOE_FFN_PERSISTENT = 2 /* task queue */ };
int moe_set_ffn_mode(moe_handle* h, int mode);
/* The variant a forward call on this handle runs (MOE_FFN_TILED or MOE_FFN_PERSISTENT), with AUTO resolved. */
int moe_get_ffn_mode(const moe_handle* h, int32_t* mode);

/*
 * The whole layer, asynchronous on `stream`, no host synchronisation, no allocation.  This is the path the
 * reference assembles from fGET (mma.cuh:46-179), its schedulers (scheduling.cuh:170-200,
 * warpScheduler.cuh:167-265) and Combine (combine.cuh:100-188).
 */
int moe_forward(moe_handle* h, const void* x, const moe_weights* w, void* out, const moe_routing_out* routing,
                void* workspace, size_t workspace_bytes, void* stream);

/*
 * moe_forward for callers that cannot allocate device memory at all -- code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc: the same layer, same kernels and same results, with the workspace taken
 * from an array that is part of the library's device code (MOE355_STATIC_WORKSPACE_BYTES per GPU, held from the moment
 * the library is loaded until the process ends) instead of from the caller.  It has no counterpart in the reference;
 * it is for callers that cannot allocate.  Calls no hipMalloc / hipFree or any other allocating routine.  Returns MOE_ERR_WORKSPACE when moe_workspace_bytes(config) exceeds the array (decode-sized and small
 * prefill layers fit; the Mixtral-shape intermediate does not; the bf16 weight copies of an e4m3 layer on the widening
 * plan count, see moe_get_kernel_dtype).  Every call on a GPU uses that GPU's one array: calls
 * that overlap in time on one GPU (two streams, two threads, two handles) race; calls in sequence on one stream are
 * safe, each call re-initialises what it needs.
 */
#define MOE355_STATIC_WORKSPACE_BYTES ((size_t)32 << 20)
int moe_forward_static(moe_handle* h, const void* x, const moe_weights* w, void* out, const moe_routing_out* routing,
                       void* stream);

/* ---- single stages, same kernels, for parity tests and callers that own the pipeline ---- */

/* Router: logits = x.gate_w^T (+bias), top-k on logits, softmax|sigmoid weights.  logits may be NULL. */
int moe_gate(moe_handle* h, const void* x, const void* gate_w, const float* gate_bias,
             float* logits, int32_t* topk_idx, float* topk_w, void* workspace, size_t workspace_bytes, void* stream);

/* Router statistics for a load-balancing loss (the training knob is_training, aristos_config.schema.json:20-23, has no
 * consumer in the reference).  From the fp32 logits [S,E] and topk_idx [S,k] that moe_gate returned:
 *   load[e]      = share of the S*k assignments the router gave expert e, before any capacity drop;
 *   mean_prob[e] = mean over tokens of expert e's gate score (softmax probability over all E, or sigmoid);
 *   aux_loss     = E * sum_e load[e] * mean_prob[e]   (1 for a uniform router).
 * Sums run in fp64 in a fixed order (reproducible); any of the three outputs may be NULL. */
int moe_router_stats(moe_handle* h, const float* logits, const int32_t* topk_idx, float* load, float* mean_prob,
                     float* aux_loss, void* workspace, size_t workspace_bytes, void* stream);

/* Slot assignment + capacity drop from topk_idx; the producer of the tokenIndices[] that the reference's
 * combine consumes (combine.cuh:115,134).  pair_row may be NULL. */
int moe_route(moe_handle* h, const int32_t* topk_idx, int32_t* slot, int32_t* expert_count, int32_t* expert_offset,
              int32_t* token_indices, int32_t* pair_row, void* workspace, size_t workspace_bytes, void* stream);

/* The reference tile GEMM contract, C = act(A.B^T + bias) (mma.cuh:46-179, processor/tiling.cuh:29-38).
 * dtype is MOE_DTYPE_F32 (TF32 is taken as F32), MOE_DTYPE_BF16 or MOE_DTYPE_FP16; act is RELU, GELU or NONE; bias [N] may be NULL. */
int moe_gemm_bias_act(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N, int64_t K,
                      int32_t dtype, int32_t act, void* stream);
/* The same with the tile named (the reference fixes its tile at compile time, processor/tiling.cuh:273-323): MOE_OPT_AUTO,
 * or for bf16 / fp16 0 = 128x128, 1 = 256x256, 2 = 128x256 (1 and 2 need N % 256 == 0 and K % 128 == 0, else the library's
 * choice runs), for fp32 0 = the vector-ALU tile, 1 = the matrix-core tile where the shape allows.  Same results as
 * moe_gemm_bias_act to the bit for the 16-bit tiles. */
int moe_gemm_bias_act_tile(const void* A, const void* B, const void* bias, void* C, int64_t M, int64_t N, int64_t K,
                           int32_t dtype, int32_t act, int32_t tile, void* stream);

/* out[t,:] = sum_r w[t,r] * y[pair_row[t,r],:]  (fp32, ascending r, one rounding); pair_row < 0 skipped.
 * With k = 1 and unit weights this is the reference's CombineMode::single row scatter
 * (combine.cuh:170-186). */
int moe_combine(const void* y_rows, const int32_t* pair_row, const float* topk_w, int32_t S, int32_t k, int32_t H,
                int32_t act_dtype, void* out, void* stream);

/* ---- measurement hooks ---- */
enum { MOE_STAGE_GATE = 0, MOE_STAGE_ROUTE = 1, MOE_STAGE_FFN = 2, MOE_STAGE_COMBINE = 3, MOE_STAGE_COUNT = 4 };
/* When enabled, moe_forward brackets each stage with hipEvents on the caller's stream (no synchronisation
 * is added).  Enabling or disabling restarts the count of recorded calls. */
int moe_set_stage_timing(moe_handle* h, int enable);
/* Mean milliseconds of stage `stage` over the moe_forward calls recorded since timing was enabled (the most
 * recent 64 at most); *calls (may be NULL) receives how many were averaged.  Synchronises on their events. */
int moe_get_stage_ms(moe_handle* h, int stage, float* ms, int32_t* calls);
/* The single measurements behind moe_get_stage_ms: milliseconds of `stage` (or, with stage = MOE_STAGE_COUNT, of the
 * whole call from its first to its last kernel) for each of the most recent recorded calls, oldest first, at most
 * `capacity` (and at most 64) of them; *count receives how many were written.  For medians and minima. */
int moe_get_stage_samples(moe_handle* h, int stage, float* ms, int32_t capacity, int32_t* count);

/* How evenly the task queue of the last moe_forward kept its workgroups busy (task-queue FFN only; MOE_ERR_UNSUPPORTED
 * in the two-launch mode).  Every workgroup stamps the device's constant-rate clock when it enters and when it leaves
 * the queue kernel: span_us = first entry to last exit, mean_active_us = mean of (exit - entry), mean_tail_idle_us =
 * mean of (last exit - own exit), i.e. the time a workgroup had nothing left to pop while others still worked.
 * Synchronises `stream`.  No counterpart in the reference, whose scheduler keeps no statistics. */
/* (Here and in moe_get_task_counts, workspace = NULL means this device's static array, i.e. the last moe_forward_static.) */
int moe_get_queue_balance(moe_handle* h, const void* workspace, void* stream, int32_t* workgroups, float* span_us,
                          float* mean_active_us, float* mean_tail_idle_us);
/* Per-task trace of the task-queue FFN kernel: with a trace buffer set, every task of a moe_forward on this handle
 * leaves a record -- which tile of which expert, which workgroup ran it, and the device's constant-rate clock before and
 * behind the tile (the dependency wait of a down-projection task lies in front of start_us).  The buffer is device
 * memory of the caller (moe_task_trace_bytes(max_tasks) bytes, 8-byte aligned; tasks beyond its capacity are counted
 * but not recorded); it holds the records of the most recent call.  moe_set_task_trace(h, NULL, 0) switches the trace
 * off.  Setting it copies 16 bytes to the device (synchronous; not for the serving loop); moe_get_task_trace copies
 * the records back, so it synchronises `stream`; times are microseconds since the earliest recorded start; *count
 * receives the number of records the call left (it may exceed `capacity`).  Cost with the trace on: two clock reads
 * and one atomic per task.  Counterpart in the reference: the clock stamps its kernels print (mma.cuh:51-57,162-169;
 * scheduling.cuh:261-263). */
typedef struct moe_task_record {
    int32_t phase;      /* 0: up(/gate) projection + activation, 1: down projection; a task that computed one of P partial
                           sums of its tile (option tail_split) has 1 + 4 * part + 16 * P here; 2: a combine sweep of
                           an idle workgroup (option combine = 2): expert = column slice, row_block = chunk of tokens,
                           col_tile = rows = (slice, token) units it combined */
    int32_t expert;
    int32_t row_block;  /* index into the layer's row-block table (expert-major) */
    int32_t col_tile;
    int32_t rows;       /* real rows of the block */
    int32_t workgroup;
    float start_us, end_us;
} moe_task_record;
size_t moe_task_trace_bytes(int64_t max_tasks);
int moe_set_task_trace(moe_handle* h, void* device_buffer, size_t bytes);
int moe_get_task_trace(moe_handle* h, void* stream, moe_task_record* out, int64_t capacity, int64_t* count);
/* Tile tasks the FFN stage of the last moe_forward issued to its queue (GEMM0 tasks, GEMM1 tasks); reads
 * back a few words from the workspace, so it synchronises the stream. */
int moe_get_task_counts(moe_handle* h, const void* workspace, void* stream, int64_t* gemm0_tasks, int64_t* gemm1_tasks);

/* A dependency wait of the task-queue kernel is bounded (the reference's spin waits are not: overlap.cuh:104,135,
 * warpScheduler.cuh:339).  When one expires, the kernel does not compute on unfinished rows: it fills the affected
 * output tile with NaN (which the combine carries into the affected rows of `out`), sets the stall word of the
 * workspace and a host-visible word of the handle, and every kernel still exits normally.  From then on moe_forward /
 * moe_forward_static / moe_get_task_counts on that handle return MOE_ERR_QUEUE_STALL (the handle's word, checked on the
 * host without synchronising) until moe_clear_stall.  moe_set_spin_limit sets the number of polls before a wait gives up
 * (0 = the default, about 2^24; negative = every wait expires at once, which exercises this path from the host). */
int moe_set_spin_limit(moe_handle* h, int32_t polls);
int moe_clear_stall(moe_handle* h);
/* Whether the handle's stall word is set: one read of host memory, no synchronisation.  A HIP graph that holds a captured
 * moe_forward runs no host code of this library when it is replayed, so a stall during a replay is reported by nothing
 * until the next eager call on the handle: callers that replay graphs poll this behind their own synchronisation. */
int moe_get_stall(const moe_handle* h, int32_t* stalled);

/* Ceilings measured on the current device, to be quoted beside the published peaks: bf16 MFMA issue rate with no
 * memory traffic (scratch: >= 2 MiB of device memory, overwritten; random_operands = 0: all-zero operands, the
 * clock stays at its maximum; 1: random bf16 operands, the board's power limit lowers the clock -- this is the
 * ceiling a GEMM on real data can approach), and streaming read bandwidth over `bytes` bytes
 * of `src` (>= 1 GiB, so the caches cannot serve it).  Both synchronise the stream.  No counterpart in the reference,
 * whose launch sizing is a hard-coded table (arch.cuh:22-69). */
int moe_measure_mfma_tflops(void* scratch, size_t scratch_bytes, void* stream, int random_operands, float* tflops);
int moe_measure_hbm_read_gbs(const void* src, size_t bytes, void* scratch, void* stream, float* gbs);

/* Weight preparation for torch_dtype = 4: `matrices` row-major [N,K] matrices (fp32 or bf16; N and K multiples of
 * 128) become OCP e4m3 bytes q[matrices,N,K] plus one fp32 scale per 128x128 block, scales[matrices,N/128,K/128]:
 * scale = amax/448 (1 for an all-zero block), q = e4m3(w/scale) rounded to nearest even, saturating.  Asynchronous on
 * `stream`.  No counterpart in the reference, whose dtypes stop at fp16 (aristos_config.schema.json:49-53). */
int moe_quant_block128(const void* w, int32_t src_dtype, int64_t matrices, int64_t N, int64_t K, void* q,
                       float* scales, void* stream);

/* Activation rows for the e4m3 x e4m3 plan (moe_options::fp8_mfma): x [rows, K] in bf16, K a multiple of 128, becomes
 * q [rows, K] e4m3 codes plus scales [rows, K / 128] fp32, scale = amax / 448 over that piece of the row (1 when it is all
 * zero), q = e4m3(x / scale) rounded to nearest even.  moe_forward runs this on the tokens and on the intermediate rows of
 * such a handle; exported so that the format can be checked and reused.  Asynchronous on `stream`.  No counterpart in the
 * reference (same reason). */
int moe_quant_rows128(const void* x, int64_t rows, int64_t K, void* q, float* scales, void* stream);

/* The inverse: out[matrices,N,K] (bf16) = e4m3(q) * scale of its block, rounded to nearest even once.  moe_forward
 * runs this on an e4m3 layer's weights, into its workspace, when the experts see enough rows for the bf16 tile GEMM
 * plus this pass to beat the e4m3 kernels (see moe_workspace_bytes).  Asynchronous on `stream`.  No counterpart in
 * the reference (same reason). */
int moe_dequant_block128(const void* q, const float* scales, int64_t matrices, int64_t N, int64_t K, void* out,
                         void* stream);

/* ---- Backward building blocks (fp32, tf32, bf16 and fp16 layers; e4m3 layers: MOE_ERR_UNSUPPORTED) ------------------
 * The reference declares a training knob (is_training, aristos_config.schema.json:20-23) that none of its code reads
 * and has no backward pass; these entry points are what a training step needs beyond the forward stages above.  All
 * of them work on packed expert-major rows as moe_route lays them out: rows [expert_offset[e], expert_offset[e] +
 * expert_count[e]) of a [S*k, *] buffer belong to expert e (expert_count / expert_offset as moe_route wrote them, on
 * the device).  (N, K) must be (H, I) or (I, H) of the handle's layer.  `scratch` is 256-byte aligned device memory of
 * at least moe_backward_scratch_bytes(); each call overwrites it.  Asynchronous on `stream`; fp32 accumulation.
 *
 * moe_transpose: dst[b][c][r] = src[b][r][c], elem_bytes 2 or 4.  Turns a weight [E,N,K] into its K-major view
 *   [E,K,N], which makes a data gradient an ordinary forward-shaped product:
 *     dX_rows = dY_rows . W        ==  moe_expert_gemm(dY_rows, transpose(W), no bias, MOE_ACT_NONE)
 * moe_expert_gemm: out_rows[r,:] = act(a_rows[r,:K] . w[e(r)]^T + bias[e(r)]) for every kept row r, w [E,N,K], bias
 *   [E,N] or null, act RELU / GELU / NONE; the grouped product of the forward FFN as a stage of its own.
 * moe_expert_wgrad: dw[e] [N,K] = sum over the rows r of expert e of dy_rows[r,:N]^T a_rows[r,:K]; an expert with no
 *   rows gets zeros.  dw is written in the layer's storage type (fp32, bf16 or fp16), like every operand here. */
int moe_backward_scratch_bytes(const moe_config* cfg, size_t* bytes);
int moe_transpose(const void* src, void* dst, int64_t batch, int64_t rows, int64_t cols, int32_t elem_bytes,
                  void* stream);
int moe_expert_gemm(moe_handle* h, const void* a_rows, const void* w, const void* bias, const int32_t* expert_count,
                    const int32_t* expert_offset, int32_t N, int32_t K, int32_t act, void* out_rows, void* scratch,
                    size_t scratch_bytes, void* stream);
int moe_expert_wgrad(moe_handle* h, const void* dy_rows, const void* a_rows, const int32_t* expert_count,
                     const int32_t* expert_offset, int32_t N, int32_t K, void* dw, void* scratch, size_t scratch_bytes,
                     void* stream);
/* The data gradient of the down projection with the activation's derivative in its epilogue -- the "fuse what is
 * elementwise" of a backward chain (is_training, aristos_config.schema.json:20-23, names the mode; the reference has no
 * backward code): du_rows = (dy_rows . w[e(r)]^T) * act'(u_rows) and, for SwiGLU, dg_rows beside it, i.e.
 * moe_expert_gemm(dy_rows, w = transpose(w_down), no bias, MOE_ACT_NONE) followed by moe_act_backward, in one kernel and
 * without dh ever reaching memory.  N = intermediate_size, K = hidden_size; the activation is the layer's hidden_act;
 * u_rows / g_rows / du_rows / dg_rows are [rows, N] (g_rows and dg_rows exactly when the layer is SwiGLU).  The product
 * is rounded to the storage type before the derivative, as the two calls do when they store dh, so both give the same
 * bits.  Exists for bf16 and fp16 layers whose shape meets the hand-ordered tiles' conditions (N % 256 == 0,
 * K % 128 == 0, operands below 4 GiB; option grouped_tile = 0 switches it off): moe_expert_gemm_act_backward_supported
 * tells, and the call returns MOE_ERR_UNSUPPORTED otherwise -- the two calls remain the general path. */
int moe_expert_gemm_act_backward_supported(const moe_handle* h, int32_t* supported);
int moe_expert_gemm_act_backward(moe_handle* h, const void* dy_rows, const void* w, const void* u_rows, const void* g_rows,
                                 const int32_t* expert_count, const int32_t* expert_offset, int32_t N, int32_t K,
                                 void* du_rows, void* dg_rows, void* scratch, size_t scratch_bytes, void* stream);
/* The elementwise and reduction steps between those products (same layers; fp32 arithmetic, one rounding on store):
 * moe_act_backward: for the first `rows` packed rows of width I, du = dh * act'(u) for hidden_act ReLU (1 where u > 0)
 *   and GELU (Phi(u) + u phi(u)); for SwiGLU, where h = silu(g) * u, du = dh * silu(g) and dg = dh * u * s * (1 + g (1 - s))
 *   with s = sigmoid(g).  u_rows / g_rows are the projections before the activation (moe_expert_gemm with
 *   MOE_ACT_NONE); g_rows and dg_rows are given exactly when the layer is SwiGLU.
 * moe_bias_grad: db[e, n] = sum over expert e's rows, in ascending row order, of dy_rows[r, n], stored in the layer's
 *   storage type like the bias it belongs to; N is H or I, db is [E, N].
 * moe_combine_backward: the adjoint of moe_combine: dy_rows[pair_row[t,r], :] = topk_w[t,r] * dout[t, :] and
 *   dw[t,r] = <dout[t, :], y_rows[pair_row[t,r], :]> (0 for a dropped pair); rows of dy_rows that no pair maps to are
 *   left untouched. */
int moe_act_backward(moe_handle* h, const void* dh_rows, const void* u_rows, const void* g_rows, int64_t rows,
                     void* du_rows, void* dg_rows, void* stream);
int moe_bias_grad(moe_handle* h, const void* dy_rows, const int32_t* expert_count, const int32_t* expert_offset, int32_t N,
                  void* db, void* stream);
int moe_combine_backward(moe_handle* h, const void* dout, const void* y_rows, const int32_t* pair_row, const float* topk_w,
                         void* dy_rows, float* dw, void* stream);

int moe_last_hip_error(const moe_handle* h);
const char* moe_status_string(int status);
int moe_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MOE355_H */
