// The order of the FFN task queue on the host: builds the merged segment table the way the routing kernel does
// (queue_slot per slot, then round_tail) for many random layers and checks what every consumer of the table relies on:
// the segments tile the id space without gaps; every row block of every expert is covered by exactly one up-projection
// and one down-projection run; the up-projection run stands in front of the down-projection run (the dependency wait of
// a queue kernel can only end if that holds); and where round_tail moved the last up-projection segment, the tasks behind
// it fill whole rounds of the workgroups.  With split_tail the down-projection tiles of the last row blocks become F tasks
// each: then, besides the above, every id of every queue group is decoded (decode_id, the function the kernels use) and
// every (row block, column tile, part) must come out exactly once, with parts only where the table says so -- the index a
// kernel derives from it (row block - first split row block) stays inside the partial-sum buffers.
// Built with g++ under AddressSanitizer + UndefinedBehaviorSanitizer.
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "queue_order.hpp"

using namespace moe355;

static int failed = 0;
#define CHECK(cond, ...)                                   \
    do {                                                   \
        if (!(cond)) {                                     \
            ++failed;                                      \
            std::printf("FAILED %s: ", #cond);             \
            std::printf(__VA_ARGS__);                      \
            std::printf("\n");                             \
        }                                                  \
    } while (0)

struct Layer {
    int E, lag, nnt0, nnt1, groups, workgroups;
    std::vector<int> nmt;
};

// returns the number of row blocks behind P0(E-1), or -1 when the table is broken
static int build_and_check(const Layer& L, bool round, int* moved) {
    const int E = L.E, nseg0 = 2 * E;
    const int npg0 = (L.nnt0 + L.groups - 1) / L.groups, npg1 = (L.nnt1 + L.groups - 1) / L.groups;
    std::vector<int> mt0(E);
    int total_mt = 0;
    for (int e = 0; e < E; ++e) { mt0[e] = total_mt; total_mt += L.nmt[e]; }
    std::vector<Segment> q(nseg0 + 1);
    int begin = 0;
    for (int s = 0; s < nseg0; ++s) {
        int ph, ex;
        queue_slot(s, E, L.lag, &ph, &ex);
        q[s] = Segment{begin, ph, ex, mt0[ex], L.nmt[ex], ph ? L.nnt1 : L.nnt0, (int)(((long long)ex * (ph ? L.nnt1 : L.nnt0)) % L.groups), 0};
        begin += L.nmt[ex] * (ph ? npg1 : npg0);
    }
    int total_ids = begin, nseg = nseg0;
    const TailParams tp{E, L.lag, L.nnt0, L.nnt1, L.groups, round ? L.workgroups : 0};
    nseg = round_tail(q.data(), nseg0, tp, &total_ids);
    *moved = nseg != nseg0;
    CHECK(nseg == nseg0 || nseg == nseg0 + 1, "nseg %d", nseg);
    // id space: contiguous
    int expect = 0;
    for (int i = 0; i < nseg; ++i) {
        CHECK(q[i].begin == expect, "segment %d begins at %d, expected %d", i, q[i].begin, expect);
        CHECK(q[i].nmt >= 0, "segment %d has %d row blocks", i, q[i].nmt);
        expect += q[i].nmt * (q[i].phase ? npg1 : npg0);
    }
    CHECK(expect == total_ids && total_ids == begin, "ids %d / %d / %d", expect, total_ids, begin);
    // coverage and order
    std::vector<int> pos0(total_mt, -1), pos1(total_mt, -1);
    for (int i = 0; i < nseg; ++i) {
        const Segment& s = q[i];
        CHECK(s.expert >= 0 && s.expert < E, "expert %d", s.expert);
        CHECK(s.mt0 >= mt0[s.expert] && s.mt0 + s.nmt <= mt0[s.expert] + L.nmt[s.expert], "segment %d leaves its expert's row blocks", i);
        CHECK(s.nnt == (s.phase ? L.nnt1 : L.nnt0), "segment %d nnt", i);
        for (int b = s.mt0; b < s.mt0 + s.nmt; ++b) {
            std::vector<int>& pos = s.phase ? pos1 : pos0;
            CHECK(pos[b] == -1, "row block %d covered twice in phase %d", b, s.phase);
            pos[b] = i;
        }
    }
    int last_up = -1;
    for (int b = 0; b < total_mt; ++b) {
        CHECK(pos0[b] >= 0 && pos1[b] >= 0, "row block %d not covered", b);
        CHECK(pos0[b] < pos1[b], "row block %d: down projection (segment %d) in front of up projection (segment %d)", b, pos1[b], pos0[b]);
    }
    for (int i = 0; i < nseg; ++i)
        if (q[i].phase == 0) last_up = i;
    int behind = 0;
    for (int i = last_up + 1; i < nseg; ++i) behind += q[i].nmt;
    return failed ? -1 : behind;
}

// Builds the merged queue and the phase-1 table, applies split_tail to both, decodes every id.
static void split_and_check(const Layer& L, int F, int tail_blocks, int row_chunk) {
    const int E = L.E, nseg0 = 2 * E;
    const int npg0 = (L.nnt0 + L.groups - 1) / L.groups, npg1 = (L.nnt1 + L.groups - 1) / L.groups;
    std::vector<int> mt0(E);
    int total_mt = 0;
    for (int e = 0; e < E; ++e) { mt0[e] = total_mt; total_mt += L.nmt[e]; }
    const int split_mt0 = F > 1 ? (total_mt > tail_blocks ? total_mt - tail_blocks : 0) : total_mt;
    for (int table = 0; table < 2; ++table) {          // 0: the merged queue, 1: the table of phase 1 alone
        const int n0 = table ? E : nseg0;
        std::vector<Segment> q(n0 + 1);
        int begin = 0;
        for (int s = 0; s < n0; ++s) {
            int ph = 1, ex = s;
            if (!table) queue_slot(s, E, L.lag, &ph, &ex);
            q[s] = Segment{begin, ph, ex, mt0[ex], L.nmt[ex], ph ? L.nnt1 : L.nnt0, (int)(((long long)ex * (ph ? L.nnt1 : L.nnt0)) % L.groups), 0};
            begin += L.nmt[ex] * (ph ? npg1 : npg0);
        }
        int total_ids = -1;
        const int nseg = split_tail(q.data(), n0, split_mt0, F, npg0, npg1, &total_ids);
        CHECK(nseg == n0 || nseg == n0 + 1, "nseg %d", nseg);
        int expect = 0;
        std::vector<int> pos0(total_mt, -1), pos1(total_mt, -1);
        for (int i = 0; i < nseg; ++i) {
            const Segment& s = q[i];
            CHECK(s.begin == expect, "segment %d begins at %d, expected %d", i, s.begin, expect);
            const bool split = s.split > 1;
            CHECK(!split || (s.phase == 1 && s.split == F), "segment %d split %d", i, s.split);
            if (s.nmt > 0 && s.phase == 1) {
                CHECK(split == (s.mt0 >= split_mt0), "segment %d: row blocks %d.. split %d, first split row block %d", i, s.mt0, s.split, split_mt0);
                CHECK(s.mt0 >= split_mt0 || s.mt0 + s.nmt <= split_mt0, "segment %d straddles the first split row block", i);
            }
            CHECK(s.nmt >= 0 && s.mt0 >= mt0[s.expert] && s.mt0 + s.nmt <= mt0[s.expert] + L.nmt[s.expert], "segment %d leaves its expert's row blocks", i);
            expect += s.nmt * (s.phase ? npg1 : npg0) * (split ? F : 1);
            for (int b = s.mt0; b < s.mt0 + s.nmt; ++b) {
                std::vector<int>& pos = s.phase ? pos1 : pos0;
                CHECK(pos[b] == -1, "row block %d covered twice in phase %d", b, s.phase);
                pos[b] = i;
            }
        }
        CHECK(expect == total_ids, "ids %d / %d", expect, total_ids);
        for (int b = 0; b < total_mt; ++b) {
            CHECK(pos1[b] >= 0, "row block %d has no down projection", b);
            if (!table) CHECK(pos0[b] >= 0 && pos0[b] < pos1[b], "row block %d: up projection (segment %d) not in front of down projection (segment %d)", b, pos0[b], pos1[b]);
        }
        if (failed) return;
        // every id of every group
        std::vector<int> seen0((size_t)total_mt * L.nnt0, 0), seen1((size_t)total_mt * L.nnt1 * F, 0);
        for (int g = 0; g < L.groups; ++g)
            for (int id = 0; id < total_ids; ++id) {
                const TaskId t = decode_id(q.data(), nseg, id, g, L.groups, row_chunk);
                CHECK(t.mtile >= 0 && t.mtile < total_mt, "id %d group %d: row block %d", id, g, t.mtile);
                if (failed) return;
                if (!t.valid) continue;
                CHECK(t.ntile >= 0 && t.ntile < (t.phase ? L.nnt1 : L.nnt0), "id %d group %d: column tile %d", id, g, t.ntile);
                const bool split = t.phase == 1 && t.mtile >= split_mt0;
                CHECK(t.kparts == (split ? F : 1) && t.kpart >= 0 && t.kpart < t.kparts, "id %d group %d: part %d of %d", id, g, t.kpart, t.kparts);
                if (split) CHECK(t.mtile - split_mt0 < tail_blocks, "row block %d is outside the %d the buffers hold", t.mtile, tail_blocks);
                if (failed) return;
                int& n = t.phase ? seen1[((size_t)t.mtile * L.nnt1 + t.ntile) * F + t.kpart] : seen0[(size_t)t.mtile * L.nnt0 + t.ntile];
                ++n;
            }
        if (!table)
            for (size_t i = 0; i < seen0.size(); ++i) CHECK(seen0[i] == 1, "up-projection task %zu decoded %d times", i, seen0[i]);
        for (int b = 0; b < total_mt; ++b)
            for (int c = 0; c < L.nnt1; ++c)
                for (int k = 0; k < F; ++k) {
                    const int want = (b >= split_mt0 || k == 0) ? 1 : 0;
                    const int got = seen1[((size_t)b * L.nnt1 + c) * F + k];
                    CHECK(got == want, "down-projection tile (%d, %d) part %d decoded %d times, expected %d", b, c, k, got, want);
                    if (failed) return;
                }
    }
}

int main() {
    std::mt19937 rng(12345);
    int moved_count = 0, trials = 0;
    for (int it = 0; it < 20000; ++it) {
        Layer L;
        L.E = 1 + (int)(rng() % 24);
        L.lag = 1 + (int)(rng() % (unsigned)L.E);
        if (rng() % 8 == 0) L.lag = L.E;
        L.nnt0 = 1 + (int)(rng() % 120);
        L.nnt1 = 1 + (int)(rng() % 40);
        const int gs[4] = {1, 2, 4, 8};
        L.groups = gs[rng() % 4];
        L.workgroups = 1 + (int)(rng() % 1024);
        L.nmt.resize(L.E);
        for (int& n : L.nmt) n = (rng() % 5 == 0) ? 0 : (int)(rng() % 20);
        int moved = 0, moved_plain = 0;
        const int plain = build_and_check(L, false, &moved_plain);
        const int behind = build_and_check(L, true, &moved);
        CHECK(!moved_plain, "the plain order must not be touched");
        ++trials;
        if (failed) { std::printf("layer: E %d lag %d nnt %d/%d groups %d workgroups %d\n", L.E, L.lag, L.nnt0, L.nnt1, L.groups, L.workgroups); break; }
        if (moved) {
            ++moved_count;
            // the tasks behind the last up-projection segment fill whole rounds, or fall short of one by less than a row block's tasks
            const long long tasks = (long long)behind * L.nnt1;
            const long long k = (tasks + L.workgroups - 1) / L.workgroups;
            CHECK(k >= 1 && k * L.workgroups - tasks < L.nnt1, "%lld tasks behind the last up projection for %d workgroups", tasks, L.workgroups);
            CHECK(behind >= L.nmt[L.E - 1], "the last expert's down projection must stay behind its up projection");
            CHECK(behind != plain, "moved without a change");
        }
    }
    // partial sums in the tail
    int split_trials = 0;
    for (int it = 0; it < 3000 && !failed; ++it) {
        Layer L;
        L.E = 1 + (int)(rng() % 12);
        L.lag = 1 + (int)(rng() % (unsigned)L.E);
        L.nnt0 = 1 + (int)(rng() % 30);
        L.nnt1 = 1 + (int)(rng() % 20);
        const int gs[4] = {1, 2, 4, 8};
        L.groups = gs[rng() % 4];
        L.workgroups = 256;
        L.nmt.resize(L.E);
        for (int& n : L.nmt) n = (rng() % 5 == 0) ? 0 : (int)(rng() % 12);
        const int F = (rng() % 3 == 0) ? 1 : (rng() % 2 ? 2 : 4);
        const int tail_blocks = 1 + (int)(rng() % 40);
        const int row_chunk = (rng() % 3 == 0) ? 1 + (int)(rng() % 4) : 0;
        split_and_check(L, F, tail_blocks, row_chunk);
        ++split_trials;
        if (failed) std::printf("layer: E %d lag %d nnt %d/%d groups %d F %d tail_blocks %d row_chunk %d\n", L.E, L.lag, L.nnt0, L.nnt1, L.groups, F, tail_blocks, row_chunk);
    }
    std::printf("%d layers with partial sums decoded id by id\n", split_trials);
    // the Mixtral shape: 8 experts of 8 or 9 row blocks, lag 2, 16 column tiles, 256 workgroups -> 32 row blocks behind
    {
        Layer L{8, 2, 112, 16, 8, 256, {9, 8, 9, 8, 9, 8, 9, 8}};
        int moved = 0;
        const int behind = build_and_check(L, true, &moved);
        CHECK(moved && behind == 32, "Mixtral shape: %d row blocks behind the last up projection (moved %d)", behind, moved);
    }
    std::printf("%d layers, %d with a rounded tail, %d failed checks\n", trials, moved_count, failed);
    return failed ? 1 : 0;
}
