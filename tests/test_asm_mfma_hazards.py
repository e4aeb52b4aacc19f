"""The bf16 slab loop issues its MFMAs as inline asm, so the compiler neither knows their latency nor that the
accumulator registers they write are still in flight.  This test compiles the kernels to assembly and checks what the
compiler placed behind every such MFMA: no read, copy or spill of the accumulator registers it writes may follow
within the MFMA's latency unless the wait states that end a slab body (s_nop 15) come first."""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

from cuplayground_amd import build as moe_build

WINDOW = 12   # instructions; a 16x16x32 bf16 / fp16 MFMA takes 8 passes of 4 cycles
MFMA = ("v_mfma_f32_16x16x32_bf16", "v_mfma_f32_16x16x32_f16")


_ASM = {}


def _assembly(name="ffn_bf16.hip"):
    if name not in _ASM:
        src = os.path.join(moe_build.CSRC, name)
        flags = [f for f in moe_build.FLAGS if f not in ("-fPIC",)]
        with tempfile.TemporaryDirectory() as tmp:
            out = os.path.join(tmp, os.path.splitext(name)[0] + ".s")
            r = subprocess.run(["hipcc", *flags, "-S", "--cuda-device-only", "-I",
                                os.path.join(moe_build.HERE, "..", "include"), "-o", out, src],
                               capture_output=True, text=True)
            assert r.returncode == 0, r.stderr[-2000:]
            _ASM[name] = open(out).read()
    return _ASM[name]


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_slab_loop_holds_nothing_but_the_schedule():
    """Between the asm statements of the slab loop the compiler may only place scalar bookkeeping: a vector-ALU
    instruction, a spill or an accumulator move there would sit between a ds_read and the wait that covers it, or
    behind an MFMA still in flight."""
    text = _assembly()
    loops, half_loops = 0, 0
    for kernel in re.split(r"\n(?=_Z\w+:)", text):
        lines = kernel.split("\n")
        labels = {m.group(1): k for k, l in enumerate(lines) for m in [re.match(r"^(\.LBB\d+_\d+):", l)] if m}
        for k, l in enumerate(lines):
            m = re.search(r"s_cbranch_\w+ (\.LBB\d+_\d+)", l)
            if not (m and m.group(1) in labels and labels[m.group(1)] < k):
                continue
            body = [x.strip() for x in lines[labels[m.group(1)]:k + 1]]
            body = [x for x in body if x and not x.startswith((";", "."))]
            mfmas = sum(x.startswith(MFMA) for x in body)
            if mfmas not in (256, 128) or len(body) > 1000:
                continue
            full = mfmas == 256            # two slabs of the 128 x 128 wavefront tile, or of the 128 x 64 one
            loops += full
            half_loops += not full
            other = [x for x in body if x.startswith(("v_", "scratch_", "global_", "flat_")) and not x.startswith(MFMA)]
            assert not other, "unexpected instructions in the slab loop: %s" % other[:5]
            assert sum(x.startswith("ds_read_b128") for x in body) == (64 if full else 48)
            assert sum(x.startswith("buffer_load_dwordx4") for x in body) == (32 if full else 24)
            assert sum(x.startswith("s_barrier") for x in body) == 4
    assert loops >= 8, "expected the slab loop in the two-launch, both queue and the plain-GEMM kernels, bf16 and fp16, found %d" % loops
    assert half_loops >= 8, "expected the half-width slab loop in the two-launch and queue kernels, alone and beside the full one, bf16 and fp16, found %d" % half_loops


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_no_accumulator_access_behind_asm_mfma():
    text = _assembly()
    lines = [x for x in text.split("\n")
             if x.strip() and (not x.strip().startswith(";") or "ASMSTART" in x or "ASMEND" in x)]
    access = re.compile(r"(v_accvgpr_read_b32 v\d+, a(\d+)|v_accvgpr_mov_b32 a\d+, a(\d+)|"
                        r"scratch_store_dword\w* \w+, a\[?(\d+)|v_accvgpr_write_b32 a(\d+))")
    labels = {m.group(1): k for k, l in enumerate(lines) for m in [re.match(r"^(\.LBB\d+_\d+):", l)] if m}
    asm_mfmas, bad = 0, []
    for k, line in enumerate(lines):
        m = re.search(r"v_mfma_f32_16x16x32_b?f16 a\[(\d+):(\d+)\]", line)
        if not m or "ASMSTART" not in lines[k - 1]:
            continue
        asm_mfmas += 1
        lo, hi = int(m.group(1)), int(m.group(2))
        pos, seen = k, 0
        while seen < WINDOW and pos + 1 < len(lines):
            pos += 1
            x = lines[pos].strip()
            if x.startswith(";") or x.endswith(":"):
                continue
            jump = re.match(r"s_branch (\.LBB\d+_\d+)", x)
            if jump:                          # follow the control flow, not the layout of the file
                pos = labels[jump.group(1)]
                continue
            seen += 1
            if "s_nop 15" in x:
                break
            a = access.search(x)
            if a:
                reg = int([g for g in a.groups()[1:] if g][0])
                if lo <= reg <= hi:
                    bad.append((line.strip(), seen, x))
    assert asm_mfmas >= 8 * 256, "the slab loop's inline-asm MFMAs were not found: has the kernel changed?"
    assert not bad, "accumulators touched behind an in-flight MFMA:\n" + "\n".join("%s -> +%d %s" % b for b in bad[:10])


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
@pytest.mark.parametrize("source", ["ffn_bf16.hip", "ffn_f32.hip", "ffn_f32_tile.hip", "ffn_fp8.hip", "ffn_fp8_tile.hip"])
def test_phase0_results_are_complete_before_they_are_signalled(source):
    """The hand-off of the intermediate rows between workgroups: in signal_phase0_done every wavefront must wait for
    its own stores (s_waitcnt vmcnt(0)) before the workgroup barrier and the counter increment that publishes the
    row block.  A workgroup-scope fence alone emits no such wait, so the wait is written out and checked here."""
    text = _assembly(source)
    m = re.search(r"\n(_ZN6moe355\w*signal_phase0_done\w*):[^\n]*\n(.*?)\n\s*s_setpc_b64", text, re.S)
    assert m, "signal_phase0_done is no longer a function of its own (it must not be inlined)"
    body = [x.strip() for x in m.group(2).split("\n") if x.strip() and not x.strip().startswith((";", "."))]
    barrier = next(i for i, x in enumerate(body) if x.startswith("s_barrier"))
    atomic = next(i for i, x in enumerate(body) if "atomic_add" in x)
    # the wait written out in the source (the calling convention's wait at the function's entry does not count)
    waits = [i for i, x in enumerate(body) if x == "s_waitcnt vmcnt(0)"]
    assert waits and waits[0] < barrier < atomic, body[:20]


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_fp8_tile_barriers_sit_behind_their_waits():
    """The e4m3 tile GEMM (ffn_fp8_tile.hip) meets at a bare s_barrier and spells its waits out in front of it: between
    the wait that covers the direct-to-LDS loads and this wavefront's LDS traffic (s_waitcnt vmcnt(<=2) lgkmcnt(0)) and
    the barrier the compiler may not have placed an LDS access or a load of either kind; its slab loops hold no spill;
    and the weight bytes are awaited with the count that leaves only the token-row loads issued since (vmcnt(4))."""
    text = _assembly("ffn_fp8_tile.hip")
    kernels = re.findall(r"\n(_ZN6moe355\w*fp8_tile_kernel\w*):[^\n]*\n(.*?)\n\s*s_endpgm", text, re.S)
    assert len(kernels) == 2
    for name, body in kernels:
        lines = [x.strip() for x in body.split("\n") if x.strip() and not x.strip().startswith(";")]
        mfma = [i for i, x in enumerate(lines) if x.startswith("v_mfma")]
        assert len(mfma) >= 6 * 32, name
        checked = 0
        for i, x in enumerate(lines):
            if not x.startswith("s_barrier") or not any(abs(i - m) < 60 for m in mfma):
                continue
            between = []
            for back in range(i - 1, max(i - 40, 0), -1):
                w = re.match(r"s_waitcnt vmcnt\((\d+)\) lgkmcnt\(0\)", lines[back])
                if w:
                    assert int(w.group(1)) <= 2, (name, lines[back])
                    break
                between.append(lines[back])
            else:
                continue        # a barrier of the queue bookkeeping (pop, dependency wait), not of the slab pipeline
            assert not [b for b in between if b.startswith(("ds_", "global_load", "buffer_load", "scratch_"))], (name, between)
            checked += 1
        assert checked >= 6, (name, checked)      # prologue + two per steady-state block + two of the peeled block, twice
        assert any(x == "s_waitcnt vmcnt(4)" for x in lines), name
        # no spill traffic between the first and the last MFMA of a slab loop: loops are the label .. back-branch ranges
        labels = {x.split(":")[0]: i for i, x in enumerate(lines) if re.match(r"\.LBB\d+_\d+:", x)}
        slab_loops = 0
        for i, x in enumerate(lines):
            j = re.match(r"s_cbranch_\w+ (\.LBB\d+_\d+)", x)
            if j and j.group(1) in labels and labels[j.group(1)] < i:
                loop = lines[labels[j.group(1)]:i]
                if sum(y.startswith("v_mfma") for y in loop) >= 32 and sum(y.startswith("s_barrier") for y in loop) == 2:
                    assert not [y for y in loop if y.startswith("scratch_")], (name, "spill in the slab loop")
                    slab_loops += 1
        assert slab_loops >= 2, name      # the full-block loop and the partial-block loops


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_f32_tile_barriers_sit_behind_their_waits():
    """The fp32 tile GEMM (ffn_f32_tile.hip) fills both LDS stages with direct-to-LDS loads and meets once per slab at a
    bare s_barrier behind s_waitcnt vmcnt(0) lgkmcnt(0): between that wait and the barrier the compiler may not have
    placed an LDS access or a load, and each slab loop holds its 64 fp32 MFMAs, its 8 loads and no spill."""
    text = _assembly("ffn_f32_tile.hip")
    kernels = re.findall(r"\n(_ZN6moe355\w*f32_tile_kernel\w*):[^\n]*\n(.*?)\n\s*s_endpgm", text, re.S)
    assert len(kernels) == 5      # the two FFN schedules, the dense product, the grouped product, the weight gradient
    for name, body in kernels:
        lines = [x.strip() for x in body.split("\n") if x.strip() and not x.strip().startswith(";")]
        labels = {x.split(":")[0]: i for i, x in enumerate(lines) if re.match(r"\.LBB\d+_\d+:", x)}
        # loops = label .. back-branch ranges; of nested ranges around the same MFMAs the innermost is the slab loop
        loops = {}
        for i, x in enumerate(lines):
            j = re.match(r"s_c?branch\w* (\.LBB\d+_\d+)", x)
            if not (j and j.group(1) in labels and labels[j.group(1)] < i):
                continue
            first = labels[j.group(1)]
            mf = [k for k in range(first, i) if lines[k].startswith("v_mfma_f32_32x32x2_f32")]
            if len(mf) == 64 and (mf[0] not in loops or i - first < len(loops[mf[0]])):
                loops[mf[0]] = lines[first:i]
        slab_loops = 0
        for loop in loops.values():
            bars = [k for k, y in enumerate(loop) if y.startswith("s_barrier")]
            assert len(bars) == 1, (name, bars)
            back = bars[0] - 1
            while re.match(r"\.LBB\d+_\d+:", loop[back]) or loop[back].startswith(("s_or_b64 exec", "s_mov_b64 exec")):
                back -= 1
            assert loop[back] == "s_waitcnt vmcnt(0) lgkmcnt(0)", (name, loop[back - 2:bars[0] + 1])
            assert not [y for y in loop if y.startswith("scratch_")], (name, "spill in the slab loop")
            assert sum(y.startswith("global_load_lds_dwordx4") for y in loop) == 8, name
            slab_loops += 1
        assert slab_loops == 2, (name, slab_loops)      # the full-block and the partial-block loop


def _vregs(text):
    """Vector registers an instruction line names: v7 -> {7}, v[4:7] -> {4..7}."""
    regs = set()
    for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", text):
        regs.update(range(int(a), int(b) + 1))
    regs.update(int(a) for a in re.findall(r"\bv(\d+)\b", text))
    return regs


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_fp8_tile_weight_bytes_are_not_touched_in_flight():
    """The e4m3 tile GEMM fetches its weight bytes with a load written in assembly, so the compiler does not know that
    the destination registers are pending until the wait that names them (s_waitcnt vmcnt(4)).  Inside the slab loops
    nothing between such a load and that wait may read, copy or spill those registers."""
    text = _assembly("ffn_fp8_tile.hip")
    kernels = re.findall(r"\n(_ZN6moe355\w*fp8_tile_kernel\w*):[^\n]*\n(.*?)\n\s*s_endpgm", text, re.S)
    assert len(kernels) == 2
    for name, body in kernels:
        lines = [x.strip() for x in body.split("\n") if x.strip() and not x.strip().startswith(";")]
        labels = {x.split(":")[0]: i for i, x in enumerate(lines) if re.match(r"\.LBB\d+_\d+:", x)}
        checked = 0
        for i, x in enumerate(lines):
            j = re.match(r"s_cbranch_\w+ (\.LBB\d+_\d+)", x)
            if not (j and j.group(1) in labels and labels[j.group(1)] < i):
                continue
            loop = [y for y in lines[labels[j.group(1)]:i] if not re.match(r"\.LBB\d+_\d+:", y)]
            if sum(y.startswith("v_mfma") for y in loop) < 32 or sum(y.startswith("s_barrier") for y in loop) != 2:
                continue
            n = len(loop)
            for k, y in enumerate(loop):
                m = re.match(r"global_load_dwordx4 v\[(\d+):(\d+)\], v\[\d+:\d+\], off", y)
                if not m:
                    continue
                pending = set(range(int(m.group(1)), int(m.group(2)) + 1))
                for step in range(1, n + 1):           # the wait may sit behind the loop's back edge
                    z = loop[(k + step) % n]
                    if z == "s_waitcnt vmcnt(4)":
                        break
                    assert not (_vregs(z) & pending), (name, y, z)
                else:
                    raise AssertionError("no wait for " + y)
                checked += 1
        assert checked >= 4, (name, checked)       # two loads per slab, two slabs per loop iteration


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_asm_stores_keep_their_data_registers():
    """A store of more than 8 bytes reads its data registers over the cycles behind its issue; whoever writes one of
    them must keep two wait states' distance.  The compiler pads the stores it emits itself but does not look inside an
    asm statement -- and it does reuse the data registers right away (the partial-sum stores of the queue kernel came
    out as store v[0:3]; v_accvgpr_read v0 and lost a dword in a quarter of the lanes).  So every 16-byte store that
    comes from an asm statement must bring its wait states along."""
    text = _assembly()
    stores = 0
    lines = [l.strip() for l in text.split("\n")]
    for k, l in enumerate(lines):
        if l.startswith(";;#ASMSTART") and k + 1 < len(lines) and lines[k + 1].startswith(("global_store_dwordx3", "global_store_dwordx4")):
            stores += 1
            assert lines[k + 2].startswith("s_nop 1"), "asm store without wait states: %s / %s" % (lines[k + 1], lines[k + 2])
    assert stores > 100      # the published rows of the hand-ordered tiles and the partial sums
