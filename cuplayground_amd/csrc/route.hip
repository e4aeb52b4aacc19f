// Slot assignment, capacity drop, and construction of the tile-task tables.
//
// The reference only shows the consumer of this stage: a tile of expert rows arrives with tokenIndices[]
// and a valid-row count (combine.cuh:115,121-122,134,170), and its warp scheduler assigns queue slices with
// a warp-wide inclusive scan (warpScheduler.cuh:84-88,110).  Here that prefix-sum idea produces the slots:
// pairs are numbered p = t*k + r, and slot[p] = number of earlier pairs routed to the same expert.
//   1. count:    each wavefront ranks its 64 pairs with ballot match masks and mbcnt-style popcounts; the four
//                wavefronts of a workgroup are chained through per-wave counters in LDS; the workgroup emits
//                its per-expert histogram.
//   2. scan:     one workgroup turns the histograms into exclusive prefixes over workgroups, applies the
//                capacity, scans the kept counts over experts, and writes the row-block (MTile) and task
//                segment tables the FFN stage consumes -- the analogue of the reference's task-bound
//                bookkeeping, tasks = tilesM*tilesNx + tilesM*tilesN (scheduling.cuh:212-222).
//   3. finalize: slot = prefix + local rank; dropped when slot >= capacity; packed row = offset + slot.
// Every step is integer arithmetic with a fixed order, so results do not depend on scheduling.
#include "moe_internal.hpp"
#include "queue_order.hpp"

namespace moe355 {
namespace {

// Pairs [blk * 256, blk * 256 + 256): ranks within the chunk and the chunk's histogram.  `tid` in [0, 256); wcount is
// this chunk's [4][kMaxExperts] counters in LDS.  Called by whole workgroups (it holds barriers); `active` false:
// the caller only keeps the barriers company.
__device__ __forceinline__ void route_count_body(const RouteArgs& a, int blk, int tid, int (*wcount)[kMaxExperts],
                                                 bool active) {
    const int wave = tid >> 6, lane = tid & 63;
    for (int i = tid; i < (kRouteBlock / kWave) * kMaxExperts; i += kRouteBlock) (&wcount[0][0])[i] = 0;
    __syncthreads();
    const int p = blk * kRouteBlock + tid;
    // an expert id outside [0, E) (only a caller-supplied topk_idx can hold one) is counted nowhere: the pair is dropped
    const int e_in = (active && p < a.A) ? a.topk_idx[p] : -1;
    const bool valid = (unsigned)e_in < (unsigned)a.E;
    const int e = valid ? e_in : 0;
    unsigned long long mask = __ballot(valid);
    int nbits = 0;
    while ((1 << nbits) < a.E) ++nbits;
    for (int b = 0; b < nbits; ++b) {
        const bool bit = (e >> b) & 1;
        const unsigned long long bal = __ballot(bit);
        mask &= bit ? bal : ~bal;
    }
    const unsigned long long below = (1ull << lane) - 1ull;
    const int rank_w = __popcll(mask & below);
    if (valid && rank_w == 0) wcount[wave][e] = __popcll(mask);
    __syncthreads();
    if (valid) {
        int base = 0;
        for (int w = 0; w < wave; ++w) base += wcount[w][e];
        a.rank_local[p] = base + rank_w;
    }
    if (active) {
        for (int i = tid; i < a.E; i += kRouteBlock) {
            int s = 0;
#pragma unroll
            for (int w = 0; w < kRouteBlock / kWave; ++w) s += wcount[w][i];
            a.block_hist[(size_t)blk * a.E + i] = s;
        }
    }
}

// The arrival counters of the fused combine start every call at zero.
__device__ __forceinline__ void clear_arrivals(const RouteArgs& a, int first, int stride) {
    if (!a.arrive) return;
    const int n = a.arrive_n;
    for (int i = first; i < n; i += stride) a.arrive[i] = 0;
}

__global__ __launch_bounds__(kRouteBlock) void route_count_kernel(RouteArgs a) {
    __shared__ int wcount[kRouteBlock / kWave][kMaxExperts];
    clear_arrivals(a, blockIdx.x * kRouteBlock + threadIdx.x, gridDim.x * kRouteBlock);
    route_count_body(a, blockIdx.x, threadIdx.x, wcount, true);
}

__device__ __forceinline__ void write_segment(Segment* s, int begin, int phase, int expert, int mt0, int nmt, int nnt,
                                              int groups) {
    s->begin = begin; s->phase = phase; s->expert = expert; s->mt0 = mt0; s->nmt = nmt; s->nnt = nnt;
    s->rot = (int)(((int64_t)expert * nnt) % groups); s->split = 0;
}

// Exclusive prefix sum of one int per thread over a workgroup of kMaxExperts threads (wave shuffles, then the
// eight wave totals through LDS).  *total receives the sum.  Every thread must call it.
__device__ __forceinline__ int block_exclusive_scan(int v, int* s_wave, int* total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int inc = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const int o = __shfl_up(inc, off, kWave);
        if (lane >= off) inc += o;
    }
    __syncthreads();                      // s_wave may still be read by a previous call
    if (lane == kWave - 1) s_wave[wave] = inc;
    __syncthreads();
    int base = 0, sum = 0;
#pragma unroll
    for (int w = 0; w < kMaxExperts / kWave; ++w) {
        const int t = s_wave[w];
        if (w < wave) base += t;
        sum += t;
    }
    *total = sum;
    return base + inc - v;
}

// One workgroup of kMaxExperts threads: thread e owns expert e.
struct ScanShared {
    int wave[kMaxExperts / kWave];
    int nmt[kMaxExperts];
    int mt0[kMaxExperts];
    int part[kMaxExperts];
    int total[kMaxExperts];
    // the segment tables while one thread rearranges them (split_tail): in LDS, where its dependent accesses cost cycles,
    // not memory round trips
    Segment segq[2 * kMaxExperts + 1];
    Segment seg1[kMaxExperts + 1];
    int nseg_out[2], ids_out[2];
};
__device__ __forceinline__ void route_scan_body(const RouteArgs& a, ScanShared& sh) {
    int* s_wave = sh.wave;
    int* s_nmt = sh.nmt;
    int* s_mt0 = sh.mt0;
    int* s_part = sh.part;
    int* s_total = sh.total;
    const int e = threadIdx.x;
    // per-expert exclusive prefix over the workgroups' histograms: the kMaxExperts threads split into
    // `parts` groups that each take a contiguous run of workgroups (two passes over block_hist)
    int epad = 1;
    while (epad < a.E) epad <<= 1;
    const int parts = kMaxExperts / epad;
    const int pe = threadIdx.x % epad, part = threadIdx.x / epad;
    const int chunk = (a.nblk + parts - 1) / parts;
    const int b0 = min(a.nblk, part * chunk), b1 = min(a.nblk, b0 + chunk);
    int sum = 0;
    if (pe < a.E) {
#pragma unroll 4
        for (int b = b0; b < b1; ++b) sum += a.block_hist[(size_t)b * a.E + pe];
    }
    s_part[threadIdx.x] = sum;
    __syncthreads();
    if (pe < a.E) {
        int run = 0, total = 0;
        for (int q = 0; q < parts; ++q) {
            const int v = s_part[q * epad + pe];
            if (q < part) run += v;
            total += v;
        }
        if (part == 0) s_total[pe] = total;
#pragma unroll 4
        for (int b = b0; b < b1; ++b) {
            const size_t i = (size_t)b * a.E + pe;
            const int v = a.block_hist[i];
            a.block_hist[i] = run;
            run += v;
        }
    }
    __syncthreads();
    int kept = 0;
    if (e < a.E) {
        const int run = s_total[e];
        kept = (a.drop && run > a.capacity) ? a.capacity : run;
    }
    const int nmt = (kept + a.block_m - 1) / a.block_m;
    int total_rows, total_mt, total_tasks;
    const int off = block_exclusive_scan(kept, s_wave, &total_rows);
    const int mt0 = block_exclusive_scan(nmt, s_wave, &total_mt);
    s_nmt[e] = nmt;
    s_mt0[e] = mt0;
    __syncthreads();
    // the merged queue: thread t owns segments 2t and 2t+1.  A phase-1 task must not be popped while the
    // phase-0 tasks it depends on are still running, or its workgroup idles: `lag` experts of phase-0 work
    // (at least a couple of tasks per resident workgroup) sit between the two.
    const int nseg = 2 * a.E;
    const int npg0 = (a.nnt0 + a.groups - 1) / a.groups, npg1 = (a.nnt1 + a.groups - 1) / a.groups;   // ids per row block and group
    int ph[2] = {0, 0}, ex[2] = {0, 0}, size[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int sidx = 2 * e + j;
        if (sidx < nseg) {
            queue_slot(sidx, a.E, a.lag, &ph[j], &ex[j]);
            size[j] = s_nmt[ex[j]] * (ph[j] ? npg1 : npg0);
        }
    }
    const int begin = block_exclusive_scan(size[0] + size[1], s_wave, &total_tasks);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int sidx = 2 * e + j;
        if (sidx < nseg)
            write_segment(a.seg_queue + sidx, begin + (j ? size[0] : 0), ph[j], ex[j], s_mt0[ex[j]], s_nmt[ex[j]],
                          ph[j] ? a.nnt1 : a.nnt0, a.groups);
    }
    if (e < a.E) {
        a.expert_count[e] = kept;
        a.expert_offset[e] = off;
        write_segment(a.seg_phase0 + e, mt0 * npg0, 0, e, mt0, nmt, a.nnt0, a.groups);
        write_segment(a.seg_phase1 + e, mt0 * npg1, 1, e, mt0, nmt, a.nnt1, a.groups);
    }
    // Down-projection tiles of the last tail_blocks row blocks as tail_split partial sums each (queue_order.hpp:
    // split_tail); a tail of short tasks needs no rounding.
    const int F = a.tail_split > 1 ? a.tail_split : 1;
    const int split_mt0 = F > 1 ? max(total_mt - a.tail_blocks, 0) : total_mt;
    int nseg_final = nseg, nseg_phase1 = a.E, ids_phase1 = total_mt * npg1;
    if (F > 1) {
        __syncthreads();                                  // the segment tables are complete
        for (int i = threadIdx.x; i < nseg; i += blockDim.x) sh.segq[i] = a.seg_queue[i];
        for (int i = threadIdx.x; i < a.E; i += blockDim.x) sh.seg1[i] = a.seg_phase1[i];
        __syncthreads();
        if (e == 0) {
            sh.nseg_out[0] = split_tail(sh.segq, nseg, split_mt0, F, npg0, npg1, &sh.ids_out[0]);
            sh.nseg_out[1] = split_tail(sh.seg1, a.E, split_mt0, F, npg0, npg1, &sh.ids_out[1]);
        }
        __syncthreads();
        nseg_final = sh.nseg_out[0];
        nseg_phase1 = sh.nseg_out[1];
        total_tasks = sh.ids_out[0];
        ids_phase1 = sh.ids_out[1];
        for (int i = threadIdx.x; i < nseg_final; i += blockDim.x) a.seg_queue[i] = sh.segq[i];
        for (int i = threadIdx.x; i < nseg_phase1; i += blockDim.x) a.seg_phase1[i] = sh.seg1[i];
    } else if (a.tail_workgroups > 0) {
        __syncthreads();                                  // the segment table is complete
        if (e == 0) {
            const TailParams tp{a.E, a.lag, a.nnt0, a.nnt1, a.groups, a.tail_workgroups};
            nseg_final = round_tail(a.seg_queue, nseg, tp, &total_tasks);
        }
    }
    if (e == 0) {
        a.q->groups = a.groups;
        for (int g = 0; g < kMaxQueueGroups; ++g) a.q->heads[g] = 0;
        if (a.cs) a.cs->down_done = 0;
        if (a.task_trace) a.task_trace[0] = 0;
        a.q->ids_queue = total_tasks;
        a.q->ids_phase0 = total_mt * npg0;
        a.q->ids_phase1 = ids_phase1;
        a.q->nseg_phase1 = nseg_phase1;
        a.q->split_mt0 = split_mt0;
        a.q->total_tasks = total_mt * (a.nnt0 + a.nnt1);
        a.q->tasks_phase0 = total_mt * a.nnt0;
        a.q->tasks_phase1 = total_mt * a.nnt1;
        a.q->num_mtiles = total_mt;
        a.q->kept_rows = total_rows;
        a.q->stall = 0;
        a.q->nseg = nseg_final;
        a.expert_offset[a.E] = total_rows;
    }
    if (e < a.E) {          // (behind the tail's one-thread section: the other threads get on with this meanwhile)
        for (int i = 0; i < nmt; ++i) {
            MTile t;
            t.expert = e;
            t.row0 = off + i * a.block_m;
            t.rows = min(a.block_m, kept - i * a.block_m);
            t.pad = 0;
            a.mtiles[mt0 + i] = t;
        }
    }
    for (int i = threadIdx.x; i < a.max_mtiles; i += blockDim.x) a.done0[i] = 0;
    if (a.done1)
        for (int i = threadIdx.x; i < a.max_mtiles; i += blockDim.x) a.done1[i] = 0;
    if (a.split_cnt)
        for (int i = threadIdx.x; i < a.tail_blocks * a.nnt1; i += blockDim.x) a.split_cnt[i] = 0;
}

__global__ __launch_bounds__(kMaxExperts) void route_scan_kernel(RouteArgs a) {
    __shared__ ScanShared sh;
    route_scan_body(a, sh);
}

// Pair p of chunk blk = p / 256.
__device__ __forceinline__ void route_finalize_pair(const RouteArgs& a, int p) {
    const int blk = p / kRouteBlock;
    const int e_in = a.topk_idx[p];
    const bool known = (unsigned)e_in < (unsigned)a.E;   // see route_count_kernel
    const int e = known ? e_in : 0;
    const int s = known ? a.block_hist[(size_t)blk * a.E + e] + a.rank_local[p] : 0;
    const bool dropped = !known || (a.drop && s >= a.capacity);
    const int row = dropped ? -1 : a.expert_offset[e] + s;
    a.slot[p] = dropped ? -1 : s;
    a.pair_row[p] = row;
    if (a.pair_mt) a.pair_mt[p] = dropped ? -1 : a.seg_phase0[e].mt0 + s / a.block_m;
    if (!dropped) a.token_indices[row] = p / a.k;
    if (p >= a.expert_offset[a.E]) a.token_indices[p] = -1;   // rows past the last kept one
}

__global__ __launch_bounds__(kRouteBlock) void route_finalize_kernel(RouteArgs a) {
    const int p = blockIdx.x * kRouteBlock + threadIdx.x;
    if (p < a.A) route_finalize_pair(a, p);
}

// Decode-sized layers: counting, scan and finalize in ONE workgroup of kMaxExperts threads, i.e. one launch instead of
// three -- with a few hundred pairs the launches and the gaps between dependent launches cost more than the work.
// Same bodies as the separate kernels, so the results are the same bit for bit.  Global memory written by one step is
// read by other wavefronts of the same workgroup in the next: a workgroup barrier orders that.  (Top-k stays a launch
// of its own: one wavefront per token in parallel beats a single workgroup walking the tokens, 10 against 70 us.)
__global__ __launch_bounds__(kMaxExperts) void router_small_kernel(RouteArgs a) {
    __shared__ int wcount[kMaxExperts / kRouteBlock][kRouteBlock / kWave][kMaxExperts];
    __shared__ ScanShared sh;
    const int tid = threadIdx.x;
    clear_arrivals(a, tid, kMaxExperts);
    constexpr int kChunksAtOnce = kMaxExperts / kRouteBlock;
    for (int b0 = 0; b0 < a.nblk; b0 += kChunksAtOnce) {      // uniform trip count: every thread meets every barrier
        const int blk = b0 + tid / kRouteBlock;
        route_count_body(a, blk, tid % kRouteBlock, wcount[tid / kRouteBlock], blk < a.nblk);
    }
    __syncthreads();
    route_scan_body(a, sh);
    __syncthreads();
    for (int p = tid; p < a.A; p += kMaxExperts) route_finalize_pair(a, p);
}

}  // namespace

// Pairs up to which the single-workgroup router is used.
constexpr int kSmallRouterPairs = 4096;

hipError_t launch_route(const RouteArgs& a, hipStream_t st) {
    if (a.A <= kSmallRouterPairs) {
        router_small_kernel<<<1, kMaxExperts, 0, st>>>(a);
        return hipGetLastError();
    }
    route_count_kernel<<<a.nblk, kRouteBlock, 0, st>>>(a);
    route_scan_kernel<<<1, kMaxExperts, 0, st>>>(a);
    route_finalize_kernel<<<a.nblk, kRouteBlock, 0, st>>>(a);
    return hipGetLastError();
}

}  // namespace moe355
