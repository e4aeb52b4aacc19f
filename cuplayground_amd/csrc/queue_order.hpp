// The order of the merged task queue of the FFN stage, as plain C++: route.hip builds the table on the device with
// these functions, and a host program (tests/host/queue_order.cpp) runs the same functions under sanitizers and checks
// that every order they produce keeps a row block's up-projection tasks in front of its down-projection tasks.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define MOE_HD __host__ __device__
#else
#define MOE_HD
#endif

namespace moe355 {

// A run of consecutive task ids that share (phase, expert).
//
// The queue exists once per queue group (one group per XCD when the kernels ask for it, else a single group), and
// every group sees the same id space: in a segment, group g owns the column tiles c with (c + rot) % groups == g,
// i.e. c = (g - rot) mod groups + groups * j for j < ceil(nnt / groups), and id - begin = j * nmt + mtile_local
// (row blocks fastest, so neighbouring ids share the weight tile).  An id whose c falls behind nnt is a hole:
// popped and skipped.  rot = expert * nnt mod groups continues the round robin over the experts, so groups stay
// balanced when nnt is not a multiple of the group count.
struct Segment {
    int32_t begin;    // first task id (in the id space of one group)
    int32_t phase;    // 0 = up(/gate) projection + activation, 1 = down projection
    int32_t expert;
    int32_t mt0;      // index of the first MTile of the run (an expert's row blocks are consecutive)
    int32_t nmt;      // row blocks of the run
    int32_t nnt;      // column tiles of this phase
    int32_t rot;      // rotation of the column-tile round robin over the groups
    int32_t split;    // 0 or 1: whole tiles; F > 1 (down projection only): every tile of the run is F tasks, each a partial
                      // sum over a 1/F of the contraction dimension -- ids then run (j * nmt + mtile_local) * F + part
};

// What a task id of one queue group stands for.
struct TaskId {
    int32_t phase, expert;
    int32_t mtile;    // index into the MTile table
    int32_t ntile;    // column tile of this phase
    int32_t kparts;   // 1, or F: the task is one of F partial sums of its tile over the contraction dimension ...
    int32_t kpart;    // ... this one
    bool valid;       // false: a hole of this group's id space, nothing to do
};

// Finds the segment holding id `id` of queue group `group` (segments are sorted by begin, possibly empty; 0 <= id < the
// table's total) and decodes it.
//
// Order inside a segment (ids of one group): row blocks fastest -- consecutive ids, popped by workgroups that run side by
// side, share one column tile's weights.  With row_chunk R > 0 the run's row blocks are taken R at a time: all
// column tiles of the first R row blocks, then of the next R, ...; the workgroups of an XCD then hold fewer row blocks
// and more column tiles at a time (for kernels whose token rows cost more L2 space than their weight rows).  In a run
// of partial sums the parts of a tile are consecutive ids: they run side by side and meet again soon.
MOE_HD inline TaskId decode_id(const Segment* __restrict__ segs, int nseg, int id, int group, int groups, int row_chunk) {
    int lo = 0, hi = nseg - 1;
    while (lo < hi) {   // last segment with begin <= id
        const int mid = (lo + hi + 1) >> 1;
        if (segs[mid].begin <= id) lo = mid; else hi = mid - 1;
    }
    const Segment s = segs[lo];
    int local = id - s.begin;
    TaskId t;
    t.phase = s.phase;
    t.expert = s.expert;
    t.kparts = s.split > 1 ? s.split : 1;
    t.kpart = 0;
    if (t.kparts > 1) {
        t.kpart = local % t.kparts;
        local /= t.kparts;
    }
    int j, mb;
    if (row_chunk > 0 && row_chunk < s.nmt) {
        const int per_chunk = row_chunk * ((s.nnt + groups - 1) / groups);   // ids of a full chunk
        const int c = local / per_chunk, rem = local - c * per_chunk;
        const int left = s.nmt - c * row_chunk;
        const int rc = row_chunk < left ? row_chunk : left;                  // the last chunk may be shorter
        j = rem / rc;
        mb = c * row_chunk + (rem - j * rc);
    } else {
        j = local / s.nmt;
        mb = local - j * s.nmt;
    }
    int first = group - s.rot;
    if (first < 0) first += groups;
    t.ntile = first + groups * j;
    t.valid = t.ntile < s.nnt;
    t.mtile = s.mt0 + mb;
    return t;
}

struct TailParams {
    int32_t E, lag, nnt0, nnt1, groups, tail_workgroups;
};

// Queue order with lag L: phase-0 segments of experts 0..L-1, then (phase-0 of e, phase-1 of e-L) for
// e = L..E-1, then the phase-1 segments of the last L experts.
MOE_HD inline void queue_slot(int s, int E, int L, int* phase, int* ex) {
    if (s < L) { *phase = 0; *ex = s; }
    else if (s < 2 * E - L) { const int r = s - L; *phase = r & 1; *ex = (r & 1) ? (r >> 1) : L + (r >> 1); }
    else { *phase = 1; *ex = E - L + (s - (2 * E - L)); }
}

// The end of the merged queue, rounded to the workgroups that pop it.
//
// Behind the last up-projection segment, P0(E-1), the queue holds nothing but down-projection tasks, the longest of the
// layer (K = I), and the launch ends when the last of them does.  If their number is a little more than a multiple of
// the resident workgroups W, the last round is nearly empty: the Mixtral shape leaves 408 such tasks for 256
// workgroups, so 104 of them idle for the length of a whole task (a third of a millisecond) at the end.  P0(E-1) may
// stand anywhere in front of P1(E-1) -- it depends on nothing -- and a down-projection segment may be cut at any row
// block, so P0(E-1) is moved, by whole row blocks of its neighbours P1(E-2-L) in front and P1(E-1-L) behind, to where
// the tasks behind it fill whole rounds: the number of row blocks behind it becomes the largest k W / nnt1 within reach
// that still leaves a round of tasks between P0(E-1) and P1(E-1).  One segment more, the same tasks, the same bits;
// in every queue a row block's up-projection tasks still precede its down-projection tasks.
// Run by one thread behind the segment table's barrier (q has room for nseg + 1 segments).  Returns the new segment count.
MOE_HD inline int round_tail(Segment* q, int nseg, const TailParams& a, int* total_ids) {
    if (a.tail_workgroups <= 0 || a.E < 2 || a.lag >= a.E) return nseg;      // all up projections first: nothing to slide
    const int p = 2 * a.E - a.lag - 2;                                      // P0(E-1); p + 1 .. nseg - 1 are P1 segments
    if (p < 1 || p + 1 >= nseg) return nseg;
    if (q[p].phase != 0 || q[p + 1].phase != 1) return nseg;
    const bool prev_is_down = q[p - 1].phase == 1;
    int after = 0;
    for (int i = p + 1; i < nseg; ++i) after += q[i].nmt;
    const int last = q[nseg - 1].nmt;                                       // P1(E-1)
    const int per_round_x = a.tail_workgroups;                              // tasks per round
    const int lo = after - q[p + 1].nmt, hi = after + (prev_is_down ? q[p - 1].nmt : 0);
    const int floor_blocks = last + (per_round_x + a.nnt1 - 1) / a.nnt1;    // a round of tasks in front of P1(E-1)
    int target = -1;
    for (int k = 1; k < 64; ++k) {
        const int blocks = (int)(((int64_t)k * per_round_x) / a.nnt1);      // row blocks whose tasks fill k rounds (or just under)
        if (blocks > hi) break;
        if (blocks >= lo && blocks >= floor_blocks) target = blocks;
    }
    if (target < 0 || target == after) return nseg;
    // segments p-1 (or p) .. end are rebuilt: [prev_a] P0(E-1) [moved part] ...
    const int npg0 = (a.nnt0 + a.groups - 1) / a.groups, npg1 = (a.nnt1 + a.groups - 1) / a.groups;
    for (int i = nseg - 1; i > p; --i) q[i + 1] = q[i];                     // room for one more segment behind p
    if (target > after) {           // P0(E-1) moves forward over the last d row blocks of the segment in front of it
        const int d = target - after;
        const Segment up = q[p], prev = q[p - 1];
        q[p - 1].nmt = prev.nmt - d;
        q[p] = up;
        q[p + 1] = prev;
        q[p + 1].mt0 = prev.mt0 + prev.nmt - d;
        q[p + 1].nmt = d;
    } else {                        // the first d row blocks of the segment behind it go in front of P0(E-1)
        const int d = after - target;
        const Segment up = q[p], next = q[p + 2];                           // (already shifted by one)
        q[p] = next;
        q[p].nmt = d;
        q[p + 1] = up;
        q[p + 2].mt0 = next.mt0 + d;
        q[p + 2].nmt = next.nmt - d;
    }
    int begin = q[p - 1].begin;
    for (int i = p - 1; i <= nseg; ++i) {
        q[i].begin = begin;
        begin += q[i].nmt * (q[i].phase ? npg1 : npg0) * (q[i].split > 1 ? q[i].split : 1);
    }
    *total_ids = begin;
    return nseg + 1;
}

// The down-projection tiles of the last row blocks as partial sums.
//
// Row blocks [split_mt0, ...) -- the end of the last experts' runs, hence the end of the queue -- have each of their
// down-projection tiles computed as F tasks over a 1/F of the contraction dimension each (Segment::split): the tasks a
// workgroup ends its launch with are then a 1/F as long, and so is the time the others idle behind the last of them.
// Segments of phase 1 that lie wholly in that range are marked, one that straddles its start is cut in two (an
// expert's row blocks are consecutive and the experts' runs follow each other, so at most one does), and every begin
// is recomputed.  The order of the tasks does not change, so in every queue a row block's up-projection tasks still
// precede its down-projection tasks.  Takes the merged queue or the table of phase 1 alone.
// Run by one thread behind the segment table's barrier (q has room for nseg + 1 segments).  Returns the new segment count.
MOE_HD inline int split_tail(Segment* q, int nseg, int split_mt0, int F, int npg0, int npg1, int* total_ids) {
    if (F > 1) {
        int cut = -1;
        for (int i = 0; i < nseg; ++i)
            if (q[i].phase == 1 && q[i].mt0 < split_mt0 && q[i].mt0 + q[i].nmt > split_mt0) cut = i;
        if (cut >= 0) {
            for (int i = nseg; i > cut + 1; --i) q[i] = q[i - 1];
            const int keep = split_mt0 - q[cut].mt0;
            q[cut + 1] = q[cut];
            q[cut + 1].mt0 = split_mt0;
            q[cut + 1].nmt = q[cut].nmt - keep;
            q[cut].nmt = keep;
            ++nseg;
        }
        for (int i = 0; i < nseg; ++i)
            if (q[i].phase == 1 && q[i].nmt > 0 && q[i].mt0 >= split_mt0) q[i].split = F;
    }
    int begin = 0;
    for (int i = 0; i < nseg; ++i) {
        q[i].begin = begin;
        begin += q[i].nmt * (q[i].phase ? npg1 : npg0) * (q[i].split > 1 ? q[i].split : 1);
    }
    *total_ids = begin;
    return nseg;
}

}  // namespace moe355
