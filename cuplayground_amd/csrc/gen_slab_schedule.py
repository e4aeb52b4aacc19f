"""Writes ffn_bf16_slab_steady.inc: the instruction order of one 64-wide K slab of the 256x256 bf16 tile.

Run from this directory after changing the schedule: `python gen_slab_schedule.py`.  The .inc files are committed;
the build does not run this script.

One wavefront owns 128 x 128 outputs: 8 token fragments A[i] x 8 weight fragments B[j] of v_mfma_f32_16x16x32_bf16 per
32-wide k half, 128 MFMAs per slab in 16 rows (k half s, token fragment i) of 8.  Both k halves of a slab's fragments
are double buffered in registers (af[s][i], bfr[s][j]):

  rows 0..2    the 16 fragments of k half 1 are read from LDS (6,5,5 per row)
  before row 4 BAR1: every wavefront has read all of this slab -> its LDS stage is free
  rows 4..15   the 16 global->LDS loads of slab kt+2 go into that stage, one or two per row
  before row 13 BAR2(n): this wavefront's loads of slab kt+1 have landed (only the n loads of slab kt+2 issued so
               far may be outstanding); after the barrier the other stage may be read
  rows 13..15  the 16 fragments of k half 0 of slab kt+1 are read (B first: row 0 of the next slab needs all of them)

The positions are measured, not derived: releasing the stage at row 8 with two loads per row over rows 8..15 is
2.6 % slower on the Mixtral-shaped layer, four loads per row 7 % slower, all sixteen at once 12 % slower -- the
L2 -> LDS fill wants the loads spread as thinly as the double buffering allows; releasing the stage before row 4
(all k-half-1 reads in rows 0..1) costs more in LDS-read stalls than it gains.

An MFMA needs no wait of its own for fragments read in an earlier half; the s_waitcnt lgkmcnt(n) in front of the
others is computed here from the read order (LDS returns in order), so that only what the MFMA needs has to have landed.
The kernel runs this one body for every slab, the last two included (their loads fetch nothing): the variants
without the loads ("pen", "last", still buildable here) are shorter, but in the code between differently shaped
bodies the compiler spills and copies accumulators, and it does not know that the asm statements in front of such a
copy are MFMAs whose results are still in flight.  For the same reason the body ends in TAIL: wait states behind
the last MFMA, which cover whatever the compiler places at the loop's exit (with the wait states behind the loop
instead, it placed accumulator spills in front of them); a test of the build checks both that and that the loop
itself holds nothing but this schedule and scalar bookkeeping.
"""
import os

BAR1_ROW = 4                          # MFMA row in front of which the slab's LDS stage is released
PER_ROW = [6, 5, 5, 0, 0, 0, 0, 0]    # fragment reads of k half 1 behind the MFMAs of rows 0..7
BAR2_ROW = 13                         # MFMA row in front of which the next slab's stage may be read

# The half tiles (128 x 256 on wavefronts of 128 x 64, 256 x 128 likewise): 8 token fragments x 4 weight fragments,
# 64 MFMAs per slab in 16 rows of 4, 12 fragment reads per k half, 12 global->LDS loads per slab.  A row lasts half
# as long, so the reads and loads are spread over more rows.
HALF = dict(nb=4, bar1=7, per_row=[3, 3, 2, 2, 2, 0, 0, 0], bar2=11, next_per_row=[3, 3, 2, 2, 2])
FULL = dict(nb=8, bar1=BAR1_ROW, per_row=PER_ROW, bar2=BAR2_ROW, next_per_row=[6, 6, 4])


def build(variant, shape=FULL):
    nb, bar1, bar2 = shape["nb"], shape["bar1"], shape["bar2"]
    nloads = 8 + nb
    seq = []
    if nb == 8:
        half1 = []
        for i in range(8):
            half1 += [("RA", "st", 1, i), ("RB", "st", 1, i)]
    else:   # the first row of k half 1 needs token fragment 0 and every weight fragment
        half1 = [("RA", "st", 1, 0)] + [("RB", "st", 1, j) for j in range(nb)] + [("RA", "st", 1, i) for i in range(1, 8)]
    per_row = shape["per_row"]
    nxt = [("RA", "sn", 0, 0)] + [("RB", "sn", 0, j) for j in range(nb)] + [("RA", "sn", 0, i) for i in range(1, 8)]
    next_per_row = list(shape["next_per_row"])
    assert sum(per_row) == len(half1) and sum(next_per_row) == len(nxt) and len(next_per_row) == 16 - bar2
    for g in range(16):
        s, i = divmod(g, 8)
        ops = []
        if g < 8:
            ops = half1[:per_row[i]]
            half1 = half1[per_row[i]:]
        if g >= bar1:
            if g == bar1:
                seq.append(("BAR1",))
            if variant == "steady":
                nrows = 16 - bar1
                k0 = (g - bar1) * nloads // nrows
                k1 = (g - bar1 + 1) * nloads // nrows
                ops = ops + [("GL", q) for q in range(k0, k1)]
            if g == bar2 and variant != "last":
                seq.append(("BAR2", (bar2 - bar1) * nloads // (16 - bar1) if variant == "steady" else 0))
            if g >= bar2 and variant != "last":
                n = next_per_row[g - bar2]
                ops = ops + nxt[:n]
                nxt = nxt[n:]
        n = len(ops)
        slots = [[] for _ in range(4)]
        for k, o in enumerate(ops):
            slots[(k * 4 // n) if n > 4 else k].append(o)
        per_slot = nb // 4
        for p in range(4):
            for q in range(per_slot):
                seq.append(("MF", i, per_slot * p + q, s))
            seq.extend(slots[p])
    return seq


def emit(variant, shape=FULL):
    steady, cur = build("steady", shape), build(variant, shape)
    issued, last = 0, {}

    def run(seq, out):
        nonlocal issued
        for op in seq:
            if op[0] == "RA":
                issued += 1
                last[("a", op[2], op[3])] = issued
            elif op[0] == "RB":
                issued += 1
                last[("b", op[2], op[3])] = issued
            if out is None:
                continue
            if op[0] == "MF":
                need = max(last.get(("a", op[3], op[1]), 0), last.get(("b", op[3], op[2]), 0))
                out.append(("WL", min(issued - need, 15)))
            out.append(op)

    run(steady, None)          # the slab before: its reads behind BAR2 are outstanding when this slab starts
    out = []
    run(cur, out)
    lines, prev, since = [], None, 0
    for op in out:
        if op[0] in ("RA", "RB"):
            since += 1
        if op[0] == "WL":
            if prev is not None and op[1] >= prev + since:
                continue       # already implied by the previous wait
            prev, since = op[1], 0
            lines.append("WL(%d);" % op[1])
        elif op[0] == "MF":
            lines.append("MF(%d, %d, %d);" % op[1:])
        elif op[0] == "RA":
            lines.append("RA(%s, %d, %d);" % op[1:])
        elif op[0] == "RB":
            lines.append("RB(%s, %d, %d);" % op[1:])
        elif op[0] == "GL":
            lines.append("GL(%d);" % op[1])
        elif op[0] == "BAR1":
            lines.append("BAR1;")
            prev, since = 0, 0
        elif op[0] == "BAR2":
            lines.append("BAR2(%d);" % op[1])
    lines.append("TAIL;")
    return "\n".join(lines) + "\n"


if __name__ == "__main__":
    here = os.path.dirname(os.path.abspath(__file__))
    for name, shape in (("steady", FULL), ("half", HALF)):
        with open(os.path.join(here, "ffn_bf16_slab_%s.inc" % name), "w") as f:
            f.write("// generated by gen_slab_schedule.py -- do not edit\n" + emit("steady", shape))
