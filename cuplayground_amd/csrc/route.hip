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

namespace moe355 {
namespace {

__global__ __launch_bounds__(kRouteBlock) void route_count_kernel(RouteArgs a) {
    __shared__ int wcount[kRouteBlock / kWave][kMaxExperts];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    for (int i = tid; i < (kRouteBlock / kWave) * kMaxExperts; i += kRouteBlock) (&wcount[0][0])[i] = 0;
    __syncthreads();
    const int p = blockIdx.x * kRouteBlock + tid;
    const bool valid = p < a.A;
    const int e = valid ? a.topk_idx[p] : 0;
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
    for (int i = tid; i < a.E; i += kRouteBlock) {
        int s = 0;
#pragma unroll
        for (int w = 0; w < kRouteBlock / kWave; ++w) s += wcount[w][i];
        a.block_hist[(size_t)blockIdx.x * a.E + i] = s;
    }
}

__device__ __forceinline__ void write_segment(Segment* s, int begin, int phase, int expert, int mt0, int nmt, int nnt) {
    s->begin = begin; s->phase = phase; s->expert = expert; s->mt0 = mt0; s->nmt = nmt; s->nnt = nnt;
    s->pad0 = 0; s->pad1 = 0;
}

// One workgroup of kMaxExperts threads: thread e owns expert e.
__global__ __launch_bounds__(kMaxExperts) void route_scan_kernel(RouteArgs a) {
    __shared__ int s_kept[kMaxExperts];
    __shared__ int s_off[kMaxExperts + 1];
    __shared__ int s_mt0[kMaxExperts + 1];
    const int e = threadIdx.x;
    int kept = 0;
    if (e < a.E) {
        int run = 0;
        for (int b = 0; b < a.nblk; ++b) {
            const size_t i = (size_t)b * a.E + e;
            const int v = a.block_hist[i];
            a.block_hist[i] = run;
            run += v;
        }
        kept = (a.drop && run > a.capacity) ? a.capacity : run;
    }
    s_kept[e] = kept;
    __syncthreads();
    if (e == 0) {
        int off = 0, mt = 0;
        for (int i = 0; i < a.E; ++i) {
            s_off[i] = off;
            s_mt0[i] = mt;
            off += s_kept[i];
            mt += (s_kept[i] + a.block_m - 1) / a.block_m;
        }
        s_off[a.E] = off;
        s_mt0[a.E] = mt;
        // queue order: phase-0 tasks of expert e are followed by phase-1 tasks of expert e-1, so a phase-1
        // task never has to wait long for the phase-0 tasks it depends on
        int begin = 0;
        const int nseg = 2 * a.E;
        for (int s = 0; s < nseg; ++s) {
            int phase, ex;
            if (s == 0) { phase = 0; ex = 0; }
            else if (s == nseg - 1) { phase = 1; ex = a.E - 1; }
            else if (s & 1) { phase = 0; ex = (s + 1) >> 1; }
            else { phase = 1; ex = (s - 2) >> 1; }
            const int nmt = s_mt0[ex + 1] - s_mt0[ex];
            const int nnt = phase ? a.nnt1 : a.nnt0;
            write_segment(a.seg_queue + s, begin, phase, ex, s_mt0[ex], nmt, nnt);
            begin += nmt * nnt;
        }
        a.q->head = 0;
        a.q->total_tasks = begin;
        a.q->tasks_phase0 = mt * a.nnt0;
        a.q->tasks_phase1 = mt * a.nnt1;
        a.q->num_mtiles = mt;
        a.q->kept_rows = off;
        a.q->stall = 0;
        a.q->nseg = nseg;
    }
    __syncthreads();
    if (e < a.E) {
        a.expert_count[e] = kept;
        a.expert_offset[e] = s_off[e];
        const int mt0 = s_mt0[e], nmt = s_mt0[e + 1] - s_mt0[e];
        write_segment(a.seg_phase0 + e, mt0 * a.nnt0, 0, e, mt0, nmt, a.nnt0);
        write_segment(a.seg_phase1 + e, mt0 * a.nnt1, 1, e, mt0, nmt, a.nnt1);
        for (int i = 0; i < nmt; ++i) {
            MTile t;
            t.expert = e;
            t.row0 = s_off[e] + i * a.block_m;
            t.rows = min(a.block_m, kept - i * a.block_m);
            t.pad = 0;
            a.mtiles[mt0 + i] = t;
        }
    }
    if (e == 0) a.expert_offset[a.E] = s_off[a.E];
    for (int i = threadIdx.x; i < a.max_mtiles; i += blockDim.x) a.done0[i] = 0;
}

__global__ __launch_bounds__(kRouteBlock) void route_finalize_kernel(RouteArgs a) {
    const int p = blockIdx.x * kRouteBlock + threadIdx.x;
    if (p >= a.A) return;
    const int e = a.topk_idx[p];
    const int s = a.block_hist[(size_t)blockIdx.x * a.E + e] + a.rank_local[p];
    const bool dropped = a.drop && s >= a.capacity;
    const int row = dropped ? -1 : a.expert_offset[e] + s;
    a.slot[p] = dropped ? -1 : s;
    a.pair_row[p] = row;
    if (!dropped) a.token_indices[row] = p / a.k;
    if (p >= a.expert_offset[a.E]) a.token_indices[p] = -1;   // rows past the last kept one
}

}  // namespace

hipError_t launch_route(const RouteArgs& a, hipStream_t st) {
    route_count_kernel<<<a.nblk, kRouteBlock, 0, st>>>(a);
    route_scan_kernel<<<1, kMaxExperts, 0, st>>>(a);
    route_finalize_kernel<<<a.nblk, kRouteBlock, 0, st>>>(a);
    return hipGetLastError();
}

}  // namespace moe355
