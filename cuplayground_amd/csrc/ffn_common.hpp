// Task decoding and the phase-0 -> phase-1 dependency protocol shared by the FFN kernels.
//
// The reference distributes tilesM*tilesNx first-GEMM tasks and tilesM*tilesN second-GEMM tasks
// (scheduling.cuh:212-222): a scheduler thread (scheduling.cuh:170-200) or warp (warpScheduler.cuh:167-265)
// pops ready processors and rings their doorbells, and the second-GEMM tasks of a row block become
// schedulable when that block's first-GEMM row is complete (gtQHeads[m] = tilesN, scheduling.cuh:233-236).
// On gfx950 the doorbells are replaced by global atomic counters (one per XCD) that the persistent workgroups pop
// (no scheduler workgroup), and gtQHeads by done0[m]: each finished phase-0 tile adds one with release
// semantics, and a phase-1 task acquires done0[m] == nnt0 before it reads the intermediate rows.  Because the
// ids of a queue are popped in increasing order and every phase-0 task of a row block precedes its phase-1 tasks
// in every queue, the wait cannot deadlock as long as every queue has workgroups popping it from the start of the
// launch (see QueueCursor); the host guarantees that by building no more queues than the device partition has XCDs
// and launching at least one workgroup per queue.  The wait is bounded all the same.
#pragma once

#include "combine_core.hpp"

namespace moe355 {

struct Task {
    int phase;
    int expert;
    int mtile;     // index into the MTile table
    int ntile;     // column tile of this phase
    int row0;      // first packed row
    int rows;      // valid rows in the block
    int nnt0;      // phase-0 column tiles per row block (the dependency target)
    int kparts;    // 1, or F: the task is one of F partial sums of its tile over the contraction dimension ...
    int kpart;     // ... this one
    bool poison;   // such a task whose rows never became ready (its part is stored as NaN)
    bool valid;    // false: a hole of this group's id space, nothing to do
};

// The task behind id `id` of queue group `group` (queue_order.hpp: decode_id), with its rows from the MTile table.  All
// arguments are wavefront-uniform, so the loads are scalar.
__device__ __forceinline__ Task decode_task(const Segment* __restrict__ segs, int nseg, const MTile* __restrict__ mtiles,
                                            int id, int group, int groups, int nnt0, int row_chunk = 0) {
    const TaskId d = decode_id(segs, nseg, id, group, groups, row_chunk);
    Task t;
    t.phase = d.phase;
    t.expert = d.expert;
    t.mtile = d.mtile;
    t.ntile = d.ntile;
    t.kparts = d.kparts;
    t.kpart = d.kpart;
    t.poison = false;
    t.valid = d.valid;
    const MTile m = mtiles[t.mtile];
    t.row0 = m.row0;
    t.rows = m.rows;
    t.nnt0 = nnt0;
    return t;
}

// The three queue primitives below are deliberately NOT inlined.  Each contains a branch taken by thread 0
// only; inlined into the persistent loop, the compiler's control-flow structuriser merged the thread-0
// region at the end of one iteration with the one at the start of the next and let the other lanes run ahead
// through the next iteration's barriers with a stale task id.  As separate functions every divergent region
// reconverges before the function returns, and the loop itself only has wavefront-uniform branches.

// Pops the next task id for the whole workgroup (s_task is one int of LDS).
__device__ __noinline__ int pop_task(int32_t* head, int* s_task) {
    if (threadIdx.x == 0) *s_task = atomicAdd(head, 1);
    __syncthreads();
    const int id = __builtin_amdgcn_readfirstlane(*s_task);
    __syncthreads();   // s_task may be overwritten only after everyone has read it
    return id;
}

// The XCD this workgroup runs on (XCC_ID, bits 3:0 of hardware register 20).
__device__ __forceinline__ int xcd_id() { return __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 7; }

// Where a persistent workgroup takes its tasks from: the queue of its own XCD first (the workgroups of an XCD then
// walk the same few weight tiles and share them in that XCD's L2), and once that is empty the other groups' queues
// in turn.  Every group's ids are popped in increasing order, and in every group a row block's phase-0 tasks come
// before its phase-1 tasks; so the oldest phase-0 task not yet popped anywhere is only ever preceded, in its queue,
// by tasks that cannot block for ever, and a phase-1 wait always ends.
struct QueueCursor {
    int group, exhausted;
    int last_id;   // id of the task popped last (in `group`)
};
__device__ __forceinline__ QueueCursor queue_cursor(int groups) { return QueueCursor{groups > 1 ? xcd_id() % groups : 0, 0, 0}; }

// A pop that nothing waits for: lane 0 of the calling wavefront (call it from one wavefront of the workgroup, under a
// wavefront-uniform branch) adds one to the head and the old value arrives in its register some time later.
// pop_async_result waits for it and returns it in a scalar register.  Written in assembly so that the one-lane region
// is invisible to the compiler's control-flow structuriser (see the remark on pop_task above) and so that no wait is
// placed between the two.  The atomic is the wavefront's oldest outstanding vector memory operation until it returns.
__device__ __forceinline__ int pop_async(int32_t* head) {
    int rid;
    unsigned long long saved_exec;
    const int one = 1;
    asm volatile("s_mov_b64 %1, exec\n\ts_mov_b64 exec, 1\n\tglobal_atomic_add %0, %2, %3, off sc0\n\ts_mov_b64 exec, %1"
                 : "=&v"(rid), "=&s"(saved_exec)
                 : "v"(head), "v"(one)
                 : "memory");
    return rid;
}
__device__ __forceinline__ int pop_async_result(int rid) {
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(rid)::"memory");
    return __builtin_amdgcn_readfirstlane(rid);
}

// Next task of the workgroup; false when every queue is empty.  Holes are skipped here.
__device__ __forceinline__ bool next_task(const FfnArgs& a, QueueCursor& c, int* s_task, int ids, int nseg, int nnt0,
                                          Task& t) {
    for (;;) {
        const int id = __builtin_amdgcn_readfirstlane(pop_task(&a.q->heads[c.group], s_task));
        if (id >= ids) {
            if (++c.exhausted >= a.groups) return false;
            c.group = c.group + 1 == a.groups ? 0 : c.group + 1;
            continue;
        }
        t = decode_task(a.seg_queue, nseg, a.mtiles, id, c.group, a.groups, nnt0, a.row_chunk);
        c.last_id = id;
        if (t.valid) return true;
    }
}

// Tiled mode: workgroup b of the launch for `phase` (the dispatcher deals workgroups to the XCDs round robin, so
// b % groups is the XCD).  False: nothing to do.
__device__ __forceinline__ bool tiled_task(const FfnArgs& a, int phase, int b, Task& t) {
    const int group = b % a.groups, id = b / a.groups;
    if (id >= (phase ? a.q->ids_phase1 : a.q->ids_phase0)) return false;
    t = decode_task(phase ? a.seg_phase1 : a.seg_phase0, phase ? a.q->nseg_phase1 : a.E, a.mtiles, id, group, a.groups, a.seg_phase0[0].nnt, a.row_chunk);
    return t.valid;
}

// Visibility of the intermediate rows between workgroups that may sit on different XCDs (one L2 each):
//   producer: every intermediate store is an agent-scope store (publish8 / publish4: written through to
//             memory); each wavefront waits for its own stores (an explicit s_waitcnt vmcnt(0)),
//             the workgroup meets at a barrier, one lane adds to done0[m] with an agent-scope atomic;
//   consumer: one lane polls done0[m] with agent-scope atomic loads, the workgroup meets at a barrier, and
//             only then issues its first load of the block's rows.  Those lines cannot already sit in the
//             consumer's L1 or L2: within a launch every intermediate row is written once, before it is ever
//             read, and the agent-scope acquire at kernel entry (queue_kernel_entry) drops what an earlier
//             launch left behind.
// No cache-wide write-back or invalidate happens per task: with agent-scope release/acquire fences around
// every task those two operations cost more than the GEMMs they protected (4.3 ms of a 13 ms layer).
__device__ __forceinline__ void queue_kernel_entry() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent"); }

// Entry and exit times of every workgroup of a queue kernel, on the constant-rate clock (100 MHz): what the host
// needs to tell how evenly the queue kept the workgroups busy (moe_get_queue_balance).  Two stores per workgroup.
__device__ __forceinline__ void queue_clock_stamp(int64_t* wg_clock, int which) {
    if (wg_clock && threadIdx.x == 0 && blockIdx.x < (unsigned)kMaxQueueWorkgroups)
        wg_clock[2 * blockIdx.x + which] = (int64_t)wall_clock64();
}

// One record per task of a queue kernel, when the caller has handed over a trace buffer (moe_set_task_trace): which
// task, which workgroup, and the constant-rate clock before and behind the tile (the dependency wait of a
// down-projection task lies in front of `start`).  The reference's kernels print such stamps (mma.cuh:51-57,162-169).
// Four words per record: phase << 56 | expert << 40 | row block << 20 | column tile; workgroup << 32 | rows; start; end.
__device__ __forceinline__ long long trace_clock(const int64_t* trace) { return trace ? (long long)wall_clock64() : 0; }
__device__ __noinline__ void trace_task(int64_t* trace, int cap, int phase, int expert, int mtile, int ntile, int rows,
                                        long long start) {
    if (threadIdx.x != 0) return;
    const int slot = atomicAdd(reinterpret_cast<int*>(trace), 1);
    if (slot >= cap) return;
    int64_t* e = trace + 2 + 4 * (int64_t)slot;
    e[0] = ((int64_t)phase << 56) | ((int64_t)expert << 40) | ((int64_t)mtile << 20) | (int64_t)ntile;
    e[1] = ((int64_t)blockIdx.x << 32) | (uint32_t)rows;
    e[2] = start;
    e[3] = (int64_t)wall_clock64();
}

__device__ __forceinline__ void publish8(void* p, uint32_t lo, uint32_t hi) {
    __hip_atomic_store(reinterpret_cast<uint64_t*>(p), ((uint64_t)hi << 32) | lo, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void publish4(void* p, uint32_t v) {
    __hip_atomic_store(reinterpret_cast<uint32_t*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Called by every thread of the workgroup after its phase-0 stores.  The explicit vmcnt(0) is the release: it
// completes this wavefront's published (write-through) stores before the barrier and the counter increment.  A
// workgroup-scope fence alone emits no wait for global stores here, so the hand-off must not depend on it.
__device__ __noinline__ void signal_phase0_done(int32_t* done0, int mtile) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_fetch_add(done0 + mtile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Called by every thread of the workgroup before a phase-1 task reads the intermediate rows.  Returns 1 when the
// rows are complete.  Returns 0 (to every thread) when the bounded wait expired: the stall is recorded in the
// workspace and in the handle's host-visible word, and the caller must not compute on the rows -- it poisons its
// output tile instead (poison_tile), so a wrong result cannot pass for a right one.  spin_limit < 0 makes every wait
// expire at once without polling: the host-forceable way to exercise this path with every kernel exiting normally.
__device__ __noinline__ int wait_phase0_done(const int32_t* done0, int mtile, int target, int spin_limit,
                                             QueueState* q, int32_t* host_stall, int* s_ok) {
    if (threadIdx.x == 0) {
        int spins = 0, ok = spin_limit >= 0;
        while (ok && __hip_atomic_load(done0 + mtile, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
            __builtin_amdgcn_s_sleep(8);
            if (++spins > spin_limit) ok = 0;   // never hang the device
        }
        if (!ok) {
            __hip_atomic_store(&q->stall, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (host_stall) __hip_atomic_store(host_stall, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        *s_ok = ok;
    }
    __syncthreads();
    const int ok = __builtin_amdgcn_readfirstlane(*s_ok);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");   // keeps the block's loads behind the barrier
    return ok;
}

// Fills rows [0, rows) x columns [n0, min(n0 + ncols, N)) of a row-major output block with NaN (elem_bytes 2: bf16
// 0x7FC0, 4: fp32 0x7FC00000).  Run by the whole workgroup in place of a tile whose inputs never became ready.
__device__ __noinline__ void poison_tile(void* c_base, int rows, int N, int n0, int ncols, int elem_bytes) {
    const int n1 = min(n0 + ncols, N);
    // 4-byte agent-scope stores (two bf16 / fp16 NaNs or one fp32 NaN): the combine may read these rows from another
    // XCD within this launch.  Column counts are even (H and I are multiples of 64).
    const int per = elem_bytes == 2 ? 2 : 1, w = (n1 - n0) / per;
    if (w <= 0) return;
    const uint32_t nan = elem_bytes == 2 ? 0x7FC07FC0u : 0x7FC00000u;
    for (int i = threadIdx.x; i < rows * w; i += blockDim.x) {
        const int r = i / w, c = n0 + (i % w) * per;
        publish4(static_cast<char*>(c_base) + ((int64_t)r * N + c) * elem_bytes, nan);
    }
}

// ---- Combine inside the FFN kernels ----
// The reference applies its combine to a finished tile while the tile is still on chip (combine.cuh:105-188: vector
// copy for top-1, unordered vector atomic adds for top-k).  Here the result must not depend on who finishes first, so
// the FFN kernels keep writing the expert rows y and count arrivals instead: when a down-projection tile is stored,
// one thread per row adds one to arrive[token, column tile]; the workgroup whose increment completes a token -- all
// of the token's kept (token, expert) rows now hold this column tile -- combines that token's columns right there, in
// rank order, with the very function the separate combine kernel uses.  Which workgroup does it varies, what it
// computes does not.
// Visibility: y is written with agent-scope (write-through) stores; every wavefront waits for its stores, the
// workgroup meets at a barrier, then come the increments; the combining reads are agent-scope loads issued behind
// the increment that returned the completing count.  A line of y is written once per launch, entirely by one tile.
struct CombineArgs {
    int32_t* arrive;
    const int32_t* token_indices;
    const int32_t* pair_row;
    const float* topk_w;
    const void* y;
    void* out;
    int32_t k, nnt1, H, drop;
};
__device__ __forceinline__ CombineArgs combine_args(const FfnArgs& a) {
    return CombineArgs{a.arrive, a.token_indices, a.pair_row, a.topk_w, a.y, a.out, a.k, a.nnt1, a.H, a.drop};
}

// Called by every thread of the workgroup behind the stores of the down-projection tile rows [row0, row0 + rows) x
// columns [n0, n0 + ncols).  ET: bf16_s, f16_s or float.  s_list: 1 + (row-block height) ints of LDS.
template <class ET>
__device__ __noinline__ void combine_arrivals(CombineArgs c, int row0, int rows, int ntile, int n0, int ncols,
                                              int* s_list) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // this wavefront's stores of y have reached memory
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if (threadIdx.x == 0) s_list[0] = 0;
    __syncthreads();
    for (int r = threadIdx.x; r < rows; r += blockDim.x) {
        const int t = c.token_indices[row0 + r];
        int kept = c.k;
        if (c.drop) {
            kept = 0;
            for (int q = 0; q < c.k; ++q) kept += c.pair_row[(size_t)t * c.k + q] >= 0;
        }
        const int before = __hip_atomic_fetch_add(c.arrive + (size_t)t * c.nnt1 + ntile, 1, __ATOMIC_RELAXED,
                                                  __HIP_MEMORY_SCOPE_AGENT);
        if (before == kept - 1) s_list[1 + atomicAdd(&s_list[0], 1)] = t;
    }
    __syncthreads();
    const int n = s_list[0];
    constexpr int kPerThread = sizeof(ET) == 4 ? 4 : 8;   // elements in 16 bytes
    const int lanes = ncols / kPerThread;                 // threads that share a token
    const int per_pass = blockDim.x / lanes;
    const int sub = threadIdx.x / lanes, col = n0 + (threadIdx.x % lanes) * kPerThread;
    if (sub < per_pass && col < c.H) {
        for (int i = sub; i < n; i += per_pass) {
            const int t = s_list[1 + i];
            if constexpr (sizeof(ET) == 4)
                combine_token_f32<true>((const float*)c.y, c.pair_row, c.topk_w, t, c.k, c.H, col, (float*)c.out);
            else
                combine_token_16<ET, true>((const uint16_t*)c.y, c.pair_row, c.topk_w, t, c.k, c.H, col, (uint16_t*)c.out);
        }
    }
    __syncthreads();                                      // the list may be rewritten by the next tile
}

// Tokens that lost every pair to the capacity limit have no tile that would complete them: their output rows are
// zeroed here, one wavefront per token, by the workgroups of the launch that runs the up projection.
__device__ __forceinline__ void zero_unrouted_rows(const FfnArgs& a, int elem_bytes) {
    if (!a.arrive || !a.drop) return;
    const int lane = threadIdx.x & 63;
    const int waves = (int)(gridDim.x * blockDim.x) >> 6, wave = (int)(blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int row_vec = a.H * elem_bytes / 16;
    for (int t = wave; t < a.S; t += waves) {
        const bool kept = lane < a.k && a.pair_row[(size_t)t * a.k + lane] >= 0;
        if (__ballot(kept) != 0ull) continue;
        uint4* row = reinterpret_cast<uint4*>(static_cast<char*>(a.out) + (size_t)t * a.H * elem_bytes);
        for (int i = lane; i < row_vec; i += 64) row[i] = uint4{0u, 0u, 0u, 0u};
    }
}

// ---- Combine as tasks of the queue ----
// The third way to run the combine (moe_options::combine = 2), the one that keeps it off the critical path where the
// routing allows: a workgroup that finds every GEMM queue empty does not leave the kernel; as long as other workgroups
// are still busy with their last tiles -- the idle tail of a task-queue launch -- it combines the tokens that are
// already complete.  The reference's processor likewise applies the combine on chip as part of its task loop
// (combine.cuh:105-188, overlap.cuh:94-153), there with unordered atomic adds.  Here:
//   * every finished down-projection tile adds one to done1[row block] behind its written-through stores (the
//     signal_phase0_done protocol on a second counter array); pair_mt[token, rank] names the row block of a pair;
//   * a unit is (token, slice): the columns one pass of the workgroup covers (blockDim.x threads x 16 bytes); a combine
//     task is kCombineChunk consecutive tokens of one slice; every workgroup walks the tasks in a stride of its own
//     (no shared counter: hundreds of idle workgroups on one atomic hold up the queue pops of the busy ones, as does
//     anything in the queue state's cache line -- the combine state has its own): the units whose token is complete
//     (every kept pair's row block has done1 == nnt1) and that nobody has taken yet are claimed in combined[] and
//     combined, the others are left alone, and a workgroup that finds nothing backs off before it looks again;
//   * nobody ever waits: when the last down-projection tile is finished (cs->down_done == q->tasks_phase1; every one of
//     them has been popped by then, so each is running on a workgroup that needs nothing from this one) everybody
//     leaves, and the combine launch behind the kernel takes the units whose flag is still clear -- at the occupancy and cache
//     hit rate of a kernel of its own, which a queue kernel with one to three workgroups per compute unit cannot match
//     (measured: a blocking second sweep inside the kernel cost 47 to 140 us more than it saved).
// Same arithmetic as the combine kernel (combine_core.hpp), so not a bit changes.
constexpr int kCombineChunk = 16;      // tokens per combine task (one lane each checks readiness)
constexpr int kCombineLds = kCombineChunk + 4;   // ints of LDS the combine tasks need

// What the combine tasks need of FfnArgs, small enough to travel in registers: a function that is not inlined and takes
// the whole argument block by reference makes the kernel copy it to scratch memory first.
struct SweepArgs {
    const QueueState* q;
    CombineState* cs;
    const int32_t* pair_mt;
    const int32_t* done1;
    int32_t* combined;
    const int32_t* pair_row;
    const float* topk_w;
    const void* y;
    void* out;
    int64_t* task_trace;
    int32_t task_trace_cap;
    int32_t S, k, H, nnt1;
};
__device__ __forceinline__ SweepArgs sweep_args(const FfnArgs& a) {
    return SweepArgs{a.q, a.cs, a.pair_mt, a.done1, a.combined, a.pair_row, a.topk_w, a.y, a.out, a.task_trace, a.task_trace_cap,
                     a.S, a.k, a.H, a.nnt1};
}

// U tokens x R ranks: the rows a thread has in flight together.  s_lds: kCombineLds ints -- [0, 16) the tokens to
// combine, [16] their number, [17] finished down-projection tiles.
template <class ET, int U, int R>
__device__ __forceinline__ void combine_while_idle_body(const SweepArgs a, int* s_task, int* s_lds) {
    constexpr int N = CmbElem<ET>::N;
    const int cols = (int)blockDim.x * N;                 // columns of a slice
    const int nslice = (a.H + cols - 1) / cols;
    const int per_slice = (a.S + kCombineChunk - 1) / kCombineChunk;   // tasks per slice
    const int nchunks = per_slice * nslice;
    const int tid = threadIdx.x;
    const int down_tasks = a.q->tasks_phase1;
    int backoff = 0;
    unsigned c = blockIdx.x % (unsigned)nchunks;
    const unsigned stride = gridDim.x % (unsigned)nchunks;
    for (int polls = 0; polls < (1 << 22); ++polls) {     // bounded like every loop here that looks at other workgroups' progress
        if (tid == 0) s_lds[kCombineChunk + 1] = __hip_atomic_load(&a.cs->down_done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        const int done = __builtin_amdgcn_readfirstlane(s_lds[kCombineChunk + 1]);
        __syncthreads();
        if (done >= down_tasks) break;                    // every GEMM task is done: the launch behind us takes the rest
        const long long started = trace_clock(a.task_trace);
        const int slice = (int)c / per_slice, t0 = ((int)c - slice * per_slice) * kCombineChunk;
        if (tid < kWave) {                                // the first wavefront, whole: lane i looks at token t0 + i
            const int t = t0 + tid;
            bool take = false;
            if (tid < kCombineChunk && t < a.S) {
                int32_t* flag = a.combined + (size_t)slice * a.S + t;
                if (!__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
                    take = true;
                    for (int j = 0; j < a.k && take; ++j) {
                        const int mt = a.pair_mt[(size_t)t * a.k + j];
                        if (mt >= 0 && __hip_atomic_load(a.done1 + mt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < a.nnt1) take = false;
                    }
                    // complete: ours if nobody was faster
                    if (take) take = __hip_atomic_exchange(flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0;
                }
            }
            const unsigned long long go = __ballot(take);
            if (take) s_lds[__popcll(go & ((1ull << tid) - 1ull))] = t;
            if (tid == 0) s_lds[kCombineChunk] = __popcll(go);
        }
        __syncthreads();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");   // keeps the rows' loads behind the barrier
        const int n = s_lds[kCombineChunk];
        const int col = slice * cols + tid * N;
        for (int g = 0; g < n; g += U) {                  // uniform: every thread reads the same list
            int tok[U];
#pragma unroll
            for (int u = 0; u < U; ++u) tok[u] = g + u < n ? s_lds[g + u] : 0;
            if (col < a.H) combine_tokens_fresh<ET, U, R>(a.y, a.pair_row, a.topk_w, tok, min(U, n - g), a.k, a.H, col, a.out);
        }
        if (n > 0) {
            backoff = 0;
            if (a.task_trace) trace_task(a.task_trace, a.task_trace_cap, 2, slice, (int)c, n, n, started);
        } else {                                          // nothing complete here: look again later, and later still
            backoff = min(backoff + 1, 2);                // (the kernel ends when the last sleeper has woken up: keep it short)
            for (int i = 0; i < backoff; ++i) __builtin_amdgcn_s_sleep(127);   // 127 x 64 cycles, about 3.5 us
        }
        c += stride + 1;                                  // (stride + 1 and nchunks need not be coprime: every task is
        if (c >= (unsigned)nchunks) c -= (unsigned)nchunks;   // some workgroup's, and the launch behind takes the rest)
        if (c >= (unsigned)nchunks) c %= (unsigned)nchunks;
    }
}

// The forms the kernels call.  The kernels that keep one workgroup per compute unit (the 16-bit tiles) have registers to
// spare and nothing but the code itself to keep requests in flight: 32 rows at a time (16 tokens with up to 2 ranks, 8
// with up to 4, 4 with more), in a function of its own so that the slab loop's register allocation never sees it.  The
// kernels that keep two to four workgroups per compute unit get their overlap from that: two tokens at a time, inlined --
// a function that is not inlined is compiled without regard to the occupancy its callers were written for, and a
// kernel's register count is the larger of its own and its callees'.
template <class ET>
__device__ __noinline__ void combine_while_idle(const SweepArgs a, int* s_task, int* s_lds) {
    if (a.k <= 2) combine_while_idle_body<ET, 16, 2>(a, s_task, s_lds);
    else if (a.k <= 4) combine_while_idle_body<ET, 8, 4>(a, s_task, s_lds);
    else combine_while_idle_body<ET, 4, 8>(a, s_task, s_lds);
}
template <class ET>
__device__ __forceinline__ void combine_while_idle_narrow(const SweepArgs& a, int* s_task, int* s_lds) {
    combine_while_idle_body<ET, 2, 4>(a, s_task, s_lds);
}

// What follows a stored down-projection tile: nothing (separate combine launch), the arrival counters, or the row
// block's counter of finished tiles for the combine tasks of the queue.
template <class ET>
__device__ __forceinline__ void after_down_tile(const FfnArgs& a, int row0, int rows, int mtile, int ntile, int n0, int ncols,
                                                int* s_list) {
    if (a.arrive) {
        combine_arrivals<ET>(combine_args(a), row0, rows, ntile, n0, ncols, s_list);
    } else if (a.combined) {
        signal_phase0_done(a.done1, mtile);
        if (threadIdx.x == 0) __hip_atomic_fetch_add(&a.cs->down_done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
// Rows of y must be written through when another workgroup of the same launch will read them.
__device__ __forceinline__ bool publish_y(const FfnArgs& a) { return a.arrive != nullptr || a.combined != nullptr; }

// Workgroups of a tiled launch: every group's id space, holes included.
inline int tiled_grid(int max_mtiles, int nnt, int groups) { return groups * max_mtiles * ((nnt + groups - 1) / groups); }

// Two fp32 values rounded to bf16 (nearest even, NaN quieted) by the packed conversion instruction of gfx950.
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }

__device__ __forceinline__ float act_apply(float v, int act) {
    if (act == MOE_ACT_RELU) return v < 0.0f ? 0.0f : v;   // a NaN stays a NaN
    if (act == MOE_ACT_GELU) return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f));
    return v;
}
__device__ __forceinline__ float silu(float v) { return v / (1.0f + expf(-v)); }

}  // namespace moe355
