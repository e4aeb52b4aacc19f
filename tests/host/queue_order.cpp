// The order of the FFN task queue on the host: builds the merged segment table the way the routing kernel does
// (queue_slot per slot, then round_tail) for many random layers and checks what every consumer of the table relies on:
// the segments tile the id space without gaps; every row block of every expert is covered by exactly one up-projection
// and one down-projection run; the up-projection run stands in front of the down-projection run (the dependency wait of
// a queue kernel can only end if that holds); and where round_tail moved the last up-projection segment, the tasks behind
// it fill whole rounds of the workgroups.  Built with g++ under AddressSanitizer + UndefinedBehaviorSanitizer.
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
